"""Pins of the oracle's ray functions (restating ash/src/sampler.cu) by cases
worked out by hand from the reference's loops: all quantities are chosen
exactly representable in fp32, so the expected numbers are exact."""
import torch

G = 8.0  # cells per block edge


def _map(oracle, blocks):
    cap = max(len(blocks), 1) + 8
    m = oracle.HashMap(3, cap, torch.arange(cap, dtype=torch.int32))
    if len(blocks):
        m.insert_keys(torch.tensor(blocks, dtype=torch.int32))
    return m


def _row(x0, y=16.25, z=16.5):
    return torch.tensor([[x0, y, z]]), torch.tensor([[1.0, 0.0, 0.0]])


BOX = (torch.zeros(3), torch.full((3,), 32.0))


def test_near_far_hand_case(oracle):
    """Blocks 1 and 2 along x active (cells 8..24), ray from x = 1.5 along +x,
    half-block steps of 4: hits at t = 8, 12, 16, 20.  The reference's update
    `near = near < 0 ? t : max(near - step, t_min)` walks near back to 0, far
    ends one step after the last hit; the march stops when x leaves the box."""
    m = _map(oracle, [[1, 2, 2], [2, 2, 2]])
    o, d = _row(1.5)
    near, far = oracle.ray_find_near_far(m, o, d, *BOX, 0.0, 100.0, 1.0, G)
    assert near.tolist() == [0.0] and far.tolist() == [24.0]
    # a single hit keeps near at the hit and far one step later
    m1 = _map(oracle, [[2, 2, 2]])
    near, far = oracle.ray_find_near_far(m1, *_row(3.0), *BOX, 1.0, 100.0, 1.0, G)
    # t = 1, 5, 9, 13 (x = 16 -> block 2), 17 (x = 20), 21 (x = 24 -> block 3) ...
    assert near.tolist() == [9.0] and far.tolist() == [21.0]
    # t_max cuts far
    near, far = oracle.ray_find_near_far(m1, *_row(3.0), *BOX, 1.0, 15.0, 1.0, G)
    assert near.tolist() == [13.0] and far.tolist() == [15.0]


def test_near_far_misses(oracle):
    empty = _map(oracle, [])
    o, d = _row(1.5)
    near, far = oracle.ray_find_near_far(empty, o, d, *BOX, 0.0, 50.0, 1.0, G)
    assert near.tolist() == [-1.0] and far.tolist() == [50.0]
    # origin outside the box: the march ends before the first lookup
    m = _map(oracle, [[0, 2, 2], [1, 2, 2], [2, 2, 2], [3, 2, 2]])
    near, far = oracle.ray_find_near_far(m, *_row(-3.0), *BOX, 0.0, 50.0, 1.0, G)
    assert near.tolist() == [-1.0] and far.tolist() == [50.0]
    # t_min >= t_max: nothing to march
    near, far = oracle.ray_find_near_far(m, *_row(1.0), *BOX, 9.0, 9.0, 1.0, G)
    assert near.tolist() == [-1.0] and far.tolist() == [9.0]


def test_ray_sample_dense_run_is_a_uniform_tiling(oracle):
    m = _map(oracle, [[b, 2, 2] for b in range(4)])
    o, d = _row(0.5)
    # (far - near) / 9 = 2 > 0.7: nine samples [2,4], ..., [18,20]
    idx, tn, tf, prefix = oracle.ray_sample(
        m, o, d, torch.tensor([2.0]), torch.tensor([20.0]), *BOX, 9, G)
    assert prefix.tolist() == [9] and idx.tolist() == [0] * 9
    assert tn.tolist() == [2.0 + 2 * k for k in range(9)]
    assert tf.tolist() == [4.0 + 2 * k for k in range(9)]
    # many samples allowed: the step is clamped to 0.7 from below
    idx, tn, tf, prefix = oracle.ray_sample(
        m, o, d, torch.tensor([2.0]), torch.tensor([4.0]), *BOX, 1000, G)
    step = torch.tensor(0.7)
    expect, t = [], torch.tensor(2.0)
    while t < 4.0:
        expect.append(float(t))
        t = t + step
    assert tn.tolist() == expect and prefix.tolist() == [len(expect)] and len(expect) == 3


def test_ray_sample_skips_empty_blocks_by_whole_steps(oracle):
    """Block 1 missing: at t = 8 (x = 8.5) the march jumps by step * G = 16 to
    t = 24 (block 3); the next interval starts where the last one ended."""
    m = _map(oracle, [[0, 2, 2], [2, 2, 2], [3, 2, 2]])
    o, d = _row(0.5)
    idx, tn, tf, prefix = oracle.ray_sample(
        m, o, d, torch.tensor([2.0]), torch.tensor([30.0]), *BOX, 14, G)
    assert tn.tolist() == [2.0, 4.0, 6.0, 8.0, 26.0, 28.0]
    assert tf.tolist() == [4.0, 6.0, 8.0, 26.0, 28.0, 30.0]
    assert prefix.tolist() == [6]


def test_ray_sample_batches_and_prefix(oracle):
    m = _map(oracle, [[b, 2, 2] for b in range(4)])
    o = torch.tensor([[0.5, 16.25, 16.5], [0.5, 100.0, 16.5], [0.5, 17.0, 17.0]])
    d = torch.tensor([[1.0, 0.0, 0.0]] * 3)
    nears, fars = torch.tensor([2.0, 2.0, 10.0]), torch.tensor([20.0, 20.0, 14.0])
    idx, tn, tf, prefix = oracle.ray_sample(m, o, d, nears, fars, *BOX, 9, G)
    # ray 1 runs outside every block; ray 2: step max(0.7, 4/9) = 0.7
    assert prefix.tolist() == [9, 9, 15]
    assert idx.tolist() == [0] * 9 + [2] * 6
    assert tn[9].item() == 10.0 and abs(tf[-1].item() - 14.2) < 1e-5
    # no rays at all
    e = torch.zeros(0, 3)
    idx, tn, tf, prefix = oracle.ray_sample(m, e, e, torch.zeros(0), torch.zeros(0), *BOX, 4, G)
    assert idx.numel() == tn.numel() == tf.numel() == prefix.numel() == 0
