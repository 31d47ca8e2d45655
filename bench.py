"""Benchmark of the two hot paths on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-trilinear] [--no-fusion] [--no-cpu]

Headline (`value`): configuration 2 of the baseline -- HashMap with values
{color: fp32[3], depth: fp32[1]}, 16 M distinct voxel keys into capacity 24 M,
16 M queries (70 % hits), full items(return_indices=True, return_values=True) enumeration.  One step is
clear + insert + find + items through the public Python API (including its
host read-backs), inputs resident in HBM; `value` counts the 32 M keys that
were inserted or looked up per step.

Beside it, on the same JSON line:
  roofline      the step's longest operation (for an insert of this size the
                three kernels of the streaming path together), timed alone with
                HIP events on the stream it runs on (raw C-ABI call, no host
                read-back inside), priced with the algorithmic bytes per key of
                that operation;
  kernels       the same figures for every hash kernel, for the trilinear query
                kernels of configurations 3 and 4, and the frame rate of the
                fusion loop of configuration 5;
  ceilings      what the device delivers for random line reads / updates and
                for a plain copy, measured in the same run;
  cpu_baseline  the CPU oracle (OpenMP) on a bounded sample of the same
                workload, on this machine's host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for sub in ("torch-ash_amd", "oracle", ""):
    path = os.path.join(ROOT, sub) if sub else ROOT
    if path not in sys.path:
        sys.path.insert(0, path)

HBM_PEAK_GBPS = 8000.0  # MI355X, published

PROBES_SRC = os.path.join(ROOT, "bench_probes.hip")
PROBES_LIB = os.path.join(ROOT, "bench_probes.so")


def build_probes(force: bool = False) -> str:
    """Compiles bench_probes.hip (the random-line probes behind `ceilings`) for
    gfx950 into bench_probes.so beside this file.  The probes belong to the
    benchmark, not to libash_hip.so."""
    import shutil
    import subprocess

    if not force and os.path.exists(PROBES_LIB) and \
            os.path.getmtime(PROBES_LIB) >= os.path.getmtime(PROBES_SRC):
        return PROBES_LIB
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    tmp = PROBES_LIB + ".tmp"
    subprocess.check_call([
        hipcc, "-O3", "-std=c++17", "-fPIC", "-shared", "--offload-arch=gfx950",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", PROBES_SRC, "-o", tmp])
    os.replace(tmp, PROBES_LIB)
    return PROBES_LIB


def load_probes():
    lib = ctypes.CDLL(build_probes())
    lib.bench_probe_last_error.restype = ctypes.c_char_p
    lib.bench_probe_random_lines.restype = ctypes.c_int
    lib.bench_probe_random_lines.argtypes = [
        ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
        ctypes.c_uint64, ctypes.c_void_p]
    return lib

# Algorithmic bytes per unit of work.  A stored slot counts as 16 B (12 B key +
# 4 B index) whatever the physical layout; E = embedding width; fp32.
FIND_BYTES = 12 + 16 + 8 + 1                 # key in, slot, index out, mask out
INSERT_KEY_BYTES = 12 + 16 + 16 + 4          # key in, probe, slot write, heap pop (all unique)
VALUE_ROW_BYTES = 2 * (12 + 4)               # color + depth, read and written


# Counters per launch at the default sizes, from rocprofv3 --pmc runs of this
# file (one counter set per run; the summaries are in profiles/).  Only attached
# when the run uses those sizes.
#   traffic: bytes that cross the far side of the L2s (read + written), i.e.
#     HBM plus what the Infinity Cache answers: FETCH_SIZE x 1024 / 0.50 +
#     WRITE_SIZE x 1024 / 1.00, the factors being what the same counters read
#     for kernels that move a known number of bytes;
#   l2_hit_rate: TCC_HIT / (TCC_HIT + TCC_MISS);
#   atomic_requests: TCC_ATOMIC (all of them are forwarded to the memory side:
#     TCC_EA0_ATOMIC reads the same).
MEASURED_COUNTERS = {
    "insert_values": (2_564_000_000 + 1_947_000_000, 0.343, 16_405_000),
    "insert_keys": (2_336_000_000 + 1_688_000_000, 0.265, 16_422_000),
    "find": (2_231_000_000 + 146_000_000, 0.064, 0),
    "erase": (2_234_000_000 + 1_217_000_000, 0.448, 16_031_000),
    # the two keys-only split passes and the range pass
    "erase_bulk": (192_000_000 + 128_000_000 + 641_000_000
                   + 144_000_000 + 135_000_000 + 1_094_000_000, 0.212, 279_000),
    "items": (128_000_000 + 320_000_000, 0.417, 0),
    "items_values_by_index": (528_000_000 + 256_000_000, 0.247, 0),
    # sums over the split, build and row-copy kernels
    "insert_values_bulk": (835_000_000 + 1_327_000_000, 0.413, 259_000),
    "insert_keys_bulk": (449_000_000 + 920_000_000, 0.426, 271_000),
    "cfg3_forward_linear": (3_508_000_000 + 282_000_000, 0.172, 0),
    "cfg3_forward_smooth_step": (3_508_000_000 + 282_000_000, 0.172, 0),
    "cfg4_forward": (377_000_000 + 67_000_000, 0.257, 0),
    # kernel only: the zero fill of the dense gradient adds 1.64 GB written
    "cfg4_backward": (439_000_000 + 149_000_000 + 1_638_400_000, 0.098, 2_344_000),
    "cfg4_double_backward": (486_000_000 + 166_000_000 + 1_638_400_000, 0.109, 2_344_000),
    "cfg4_grid_query": (71_000_000 + 122_000_000, 0.399, 0),
    "cfg4_module_forward": (325_000_000 + 72_000_000, 0.398, 0),
    "cfg4_module_forward_for_training": (325_000_000 + 190_000_000, 0.428, 0),
}


# The figures above were not measured by the run that prints them: they come
# from separate rocprofv3 --pmc runs (counters cannot be collected together with
# timings) whose summaries are the files below, taken on the kernel sources with
# the fingerprint below.  A run on other kernel sources, or at other sizes, does
# not attach them (`traffic` is then null).
COUNTERS_SOURCE = {
    "profiles": ["profiles/bench_hbm_traffic_pmc.md",
                 "profiles/bench_l2_hit_rate_and_atomics_pmc.md"],
    "csrc_sha256": "c6faef7718351d8d76b6af8431f0d453eaf253c59e8058507d7d4a72540cd714",
}


def csrc_fingerprint() -> str:
    """SHA-256 over the kernel sources of libash_hip.so (names and contents),
    as the build computes it and compiles it into the library."""
    import importlib.util

    spec = importlib.util.spec_from_file_location(
        "ash_build", os.path.join(ROOT, "torch-ash_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    return build.source_fingerprint()


def attach_counters(kernels, default_sizes: bool, library: str):
    """Adds the separately collected counter figures to the kernel entries when
    they describe this run; returns what the JSON line says about them.
    `library`: the fingerprint compiled into the library that ran."""
    current = csrc_fingerprint()
    note = dict(COUNTERS_SOURCE, measured_in_this_run=False, csrc_sha256_of_this_run=current,
                csrc_sha256_of_the_library=library)
    note["attached"] = bool(default_sizes and library == current == COUNTERS_SOURCE["csrc_sha256"])
    if not note["attached"]:
        note["why_not"] = (
            "other sizes than the counters were collected at" if not default_sizes
            else "the library was not built from the kernel sources beside it" if library != current
            else "the kernel sources changed since the counters were collected")
        return note
    for name, (traffic, hit_rate, atomics) in MEASURED_COUNTERS.items():
        entry = kernels.get(name)
        if not isinstance(entry, dict) or "ms" not in entry:
            continue
        entry["traffic"] = traffic
        entry["l2_hit_rate"] = hit_rate
        entry["atomic_requests"] = atomics
        entry["counters_from"] = "separate rocprofv3 --pmc runs, see `counters`"
    return note


def items_bytes(scanned: int, n: int) -> int:
    """items(): the key log is scanned (8 B per index, `scanned` indices: the
    size while the heap is in its initial order, else the capacity), 12 B key +
    8 B index written per live entry."""
    return 8 * scanned + 20 * n


def fwd_bytes(e: int) -> int:
    return 29 + 36 * e


def bwd_bytes(e: int) -> int:
    return 41 + 100 * e


def bwd2_bytes(e: int) -> int:
    return 41 + 104 * e


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--keys", type=int, default=16_000_000, help="distinct keys (configuration 2)")
    ap.add_argument("--capacity", type=int, default=24_000_000)
    ap.add_argument("--no-trilinear", action="store_true", help="skip the trilinear kernel figures")
    ap.add_argument("--no-fusion", action="store_true", help="skip the configuration 5 figure")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-keys", type=int, default=0,
                    help="CPU baseline size (0 = the configuration itself: --keys into --capacity)")
    ap.add_argument("--csrc-fingerprint", action="store_true",
                    help="print the fingerprint of the kernel sources (COUNTERS_SOURCE) and exit")
    ap.add_argument("--calibrate", action="store_true",
                    help="run a 1 GiB device copy first (reference point for HBM counters)")
    return ap.parse_args()


class EventTimer:
    """Average duration of a region on torch's current stream, in ms."""

    def __init__(self, torch):
        self.torch = torch
        self.pairs = []

    def __call__(self, fn):
        start = self.torch.cuda.Event(enable_timing=True)
        end = self.torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        self.pairs.append((start, end))

    def mean_ms(self):
        self.torch.cuda.synchronize()
        times = [s.elapsed_time(e) for s, e in self.pairs]
        return sum(times) / max(len(times), 1)


def roofline_entry(name, alg_bytes, ms, traffic=None):
    achieved = alg_bytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
    return {
        "kernel": name,
        "bound": "hbm",
        "achieved": round(achieved, 2),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 5),
        "traffic": traffic,
        "ms": round(ms, 4),
    }


def measure_ceilings(torch, ash, dev, table_bytes, n):
    """What this device's memory system delivers for the two access patterns
    that bound the table kernels, measured with the probes of bench_probes.hip on a
    buffer of the table's size: random 128-byte line reads (a probe) and random
    line read + compare-and-swap + dword store (an insert); float adds without
    a result, alone and sixteen to a 64-byte half-line (gradient accumulation);
    plus a plain device-to-device copy for the streaming rate."""
    lib = load_probes()
    stream = torch.cuda.current_stream(dev).cuda_stream
    buf = torch.empty(table_bytes // 128 * 128, dtype=torch.uint8, device=dev).fill_(255)
    sink = torch.empty(n, dtype=torch.int32, device=dev)
    out = {}
    for mode, name in ((0, "random_line_reads"), (1, "random_line_updates"),
                       (2, "random_half_line_reads")):
        timer = EventTimer(torch)
        for it in range(6):
            call = lambda: lib.bench_probe_random_lines(
                mode, buf.data_ptr(), buf.numel(), n, sink.data_ptr(), 7919 * it, stream)
            if it == 0:
                assert call() == 0, lib.bench_probe_last_error().decode()
            else:
                timer(call)
        ms = timer.mean_ms()
        out[name] = {"Glines_per_s": round(n / ms / 1e6, 2), "ms": round(ms, 4)}
    # float adds without a result: one lane per line against sixteen lanes per
    # 64-byte half-line -- the memory side charges per request, not per float
    for mode, name, lanes in ((3, "float_adds_one_lane_per_line", 1),
                              (4, "float_adds_16_lanes_per_half_line", 16)):
        timer = EventTimer(torch)
        for it in range(6):
            call = lambda: lib.bench_probe_random_lines(
                mode, buf.data_ptr(), buf.numel(), n, sink.data_ptr(), 7919 * it, stream)
            if it == 0:
                assert call() == 0, lib.bench_probe_last_error().decode()
            else:
                timer(call)
        ms = timer.mean_ms()
        out[name] = {"Grequests_per_s": round(n / lanes / ms / 1e6, 2),
                     "Gfloats_per_s": round(n / ms / 1e6, 2), "ms": round(ms, 4)}
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    timer = EventTimer(torch)
    for it in range(6):
        if it == 0:
            dst.copy_(src)
        else:
            timer(lambda: dst.copy_(src))
    ms = timer.mean_ms()
    out["copy_1GiB"] = {"GB_per_s_read_plus_write": round(2 * src.numel() * 4 / ms / 1e6, 1),
                        "ms": round(ms, 4)}
    del buf, sink, src, dst
    torch.cuda.empty_cache()
    return out


def bench_hash(torch, ash, workloads, args, dev):
    w = workloads.hashmap_sphere_voxels(num_keys=args.keys, device=dev)
    n = args.keys
    hm = ash.HashMap(3, {"color": 3, "depth": 1}, args.capacity, dev)
    values = {"color": w["color"], "depth": w["depth"]}

    def step():
        hm.clear()
        hm.insert(w["keys"], values)
        masks, indices = hm.find(w["query_keys"])
        keys_out, idx_out, values_out = hm.items(return_indices=True, return_values=True)
        return masks, keys_out

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        masks, keys_out = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert keys_out.shape[0] == n
    hits = int(masks.sum())
    ms_per_step = elapsed / args.steps * 1e3

    # The same step with one key erased and put back after the insert: the
    # heap is no longer 0, 1, 2, ..., so the listing goes by ranks, the value
    # rows are gathered by index and the next clear rewrites heap and key log
    # -- the general case of which the step above is the best one.
    def step_after_erase():
        hm.clear()
        hm.insert(w["keys"], values)
        hm.erase(w["keys"][:1])
        hm.insert(w["keys"][:1], {name: rows[:1] for name, rows in values.items()})
        masks, indices = hm.find(w["query_keys"])
        return hm.items(return_indices=True, return_values=True)

    for _ in range(args.warmup):
        step_after_erase()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        keys_out, _, _ = step_after_erase()
    torch.cuda.synchronize()
    ms_per_step_after_erase = (time.perf_counter() - t0) / args.steps * 1e3
    assert keys_out.shape[0] == n and not hm.engine.backend.last_items_in_index_order
    hm.clear()

    # Kernel-only timings through the raw C ABI (no host read-back inside).
    backend = hm.engine.backend
    lib, handle = backend._lib, backend._handle
    stream = torch.cuda.current_stream(dev).cuda_stream
    keys, queries = w["keys"], w["query_keys"]
    k = 2
    c_rows = (ctypes.c_int64 * k)(12, 4)
    c_src = (ctypes.c_void_p * k)(w["color"].data_ptr(), w["depth"].data_ptr())
    c_dst = (ctypes.c_void_p * k)(hm.values["color"].data_ptr(), hm.values["depth"].data_ptr())
    idx_out = torch.empty(n, dtype=torch.int64, device=dev)
    mask_out = torch.empty(n, dtype=torch.bool, device=dev)
    items_keys = torch.empty((n, 3), dtype=torch.int32, device=dev)
    items_idx = torch.empty(n, dtype=torch.int64, device=dev)

    def check(rc):
        if rc != 0:
            raise RuntimeError(lib.ash_last_error().decode())

    # The streaming insert path (what hm.insert takes for a batch of this size
    # when the library calls it worthwhile) next to the per-key kernel.
    ws_bytes, worthwhile = ctypes.c_int64(0), ctypes.c_int(0)
    check(lib.ash_map_bulk_workspace_bytes(
        handle, n, k, c_rows, ctypes.byref(ws_bytes), ctypes.byref(worthwhile)))
    bulk = ws_bytes.value > 0
    api_uses_bulk = bool(bulk and worthwhile.value and ash.common.BULK_INSERT != "never")
    workspace = torch.empty(max(ws_bytes.value, 256), dtype=torch.uint8, device=dev)
    t_bulk, t_bulk_keys = EventTimer(torch), EventTimer(torch)

    t_clear, t_insert, t_insert_keys, t_find, t_items, t_erase, t_erase_bulk = (
        EventTimer(torch) for _ in range(7))
    erase_bytes, erase_worthwhile = ctypes.c_int64(0), ctypes.c_int(0)
    check(lib.ash_map_erase_bulk_query(
        handle, n, ctypes.byref(erase_bytes), ctypes.byref(erase_worthwhile)))
    erase_ws = (torch.empty(erase_bytes.value, dtype=torch.uint8, device=dev)
                if erase_bytes.value > 0 else None)

    def settle():
        check(lib.ash_map_find(handle, queries.data_ptr(), 1, idx_out.data_ptr(),
                               mask_out.data_ptr(), stream))

    for it in range(args.warmup + args.steps):
        timed = it >= args.warmup
        run = (lambda timer, fn: timer(fn)) if timed else (lambda timer, fn: fn())
        if bulk:
            check(lib.ash_map_clear(handle, stream))
            run(t_bulk_keys, lambda: check(lib.ash_map_insert_bulk(
                handle, keys.data_ptr(), n, 0, None, None, None,
                workspace.data_ptr(), workspace.numel(), stream)))
            check(lib.ash_map_clear(handle, stream))
            run(t_bulk, lambda: check(lib.ash_map_insert_bulk(
                handle, keys.data_ptr(), n, k, c_src, c_dst, c_rows,
                workspace.data_ptr(), workspace.numel(), stream)))
        # clear() leaves the fill of the bucket array to the next call that
        # needs the table (a streaming insert rewrites all of it and skips the
        # fill); a one-key look-up makes it happen where it is to be timed
        run(t_clear, lambda: (check(lib.ash_map_clear(handle, stream)), settle()))
        run(t_insert_keys, lambda: check(lib.ash_map_insert_keys(handle, keys.data_ptr(), n, stream)))
        check(lib.ash_map_clear(handle, stream))
        settle()
        run(t_insert, lambda: check(lib.ash_map_insert(
            handle, keys.data_ptr(), n, k, c_src, c_dst, c_rows, None, stream)))
        run(t_find, lambda: check(lib.ash_map_find(
            handle, queries.data_ptr(), n, idx_out.data_ptr(), mask_out.data_ptr(), stream)))
        run(t_items, lambda: check(lib.ash_map_items(
            handle, items_keys.data_ptr(), items_idx.data_ptr(), n, stream)))
        run(t_erase, lambda: check(lib.ash_map_erase(handle, keys.data_ptr(), n, stream)))
        if erase_ws is not None:
            # the same erase through the streaming path, on a map filled again
            check(lib.ash_map_insert_keys(handle, keys.data_ptr(), n, stream))
            run(t_erase_bulk, lambda: check(lib.ash_map_erase_bulk(
                handle, keys.data_ptr(), n, erase_ws.data_ptr(), erase_ws.numel(), stream)))
    assert int(mask_out.sum()) == hits
    assert backend.size() == 0
    c_count = (ctypes.c_int64 * k)(args.capacity, args.capacity)
    gathered = [torch.empty((n, 3), device=dev), torch.empty((n, 1), device=dev)]
    c_out = (ctypes.c_void_p * k)(gathered[0].data_ptr(), gathered[1].data_ptr())
    t_gather = EventTimer(torch)
    for it in range(args.warmup + args.steps):
        fn = lambda: check(lib.ash_gather_rows(k, c_dst, c_out, c_rows, c_count,
                                               items_idx.data_ptr(), n, stream))
        if it >= args.warmup:
            t_gather(fn)
        else:
            fn()
    # what HashMap.items(return_values=True) does while the listing is in index
    # order (nothing erased or loaded since the clear): the first n rows, copied
    t_rows = EventTimer(torch)
    for it in range(args.warmup + args.steps):
        fn = lambda: check(lib.ash_gather_rows(k, c_dst, c_out, c_rows, c_count, None, n, stream))
        if it >= args.warmup:
            t_rows(fn)
        else:
            fn()
    kernels = {
        "insert_values": roofline_entry(
            "insert_kernel<3,fused>", (INSERT_KEY_BYTES + VALUE_ROW_BYTES) * n, t_insert.mean_ms()),
        "insert_keys": roofline_entry("insert_kernel<3,keys>", INSERT_KEY_BYTES * n, t_insert_keys.mean_ms()),
        "find": roofline_entry("find_kernel<3>", FIND_BYTES * n, t_find.mean_ms()),
        # the heap is in its initial order when items() runs here: n indices scanned
        "items": roofline_entry("items_dense_kernel<3>", items_bytes(n, n), t_items.mean_ms()),
        # value rows of the enumerated entries while the listing is in index
        # order: 16 B read and written per entry (one launch for both tensors)
        "items_values": roofline_entry("copy_first_rows_kernel (first n rows of color and depth)",
                                       VALUE_ROW_BYTES * n, t_rows.mean_ms()),
        # ... and by index (after an erase or a load): index in, 16 B read and written
        "items_values_by_index": roofline_entry(
            "gather_rows_kernel (color + depth by items() index)",
            (8 + VALUE_ROW_BYTES) * n, t_gather.mean_ms()),
        # the heap array is rewritten only after an erase or a load wrote to it,
        # and the key log emptied only then; none did before the clear timed
        # here: what is written is the bucket array
        "clear": roofline_entry("reset counters + deferred fill16 (+ a one-key find)",
                                backend._table.numel() - 256 - (args.capacity + 1) // 2 * 16,
                                t_clear.mean_ms()),
        "erase": roofline_entry("erase_kernel<3> (every key stored)", INSERT_KEY_BYTES * n,
                                t_erase.mean_ms()),
    }
    if bulk:
        chain = "split_keys_kernel<3> + split_records_kernel + build_kernel"
        kernels["insert_values_bulk"] = roofline_entry(
            chain + " (ash_map_insert_bulk, fused values)",
            (INSERT_KEY_BYTES + VALUE_ROW_BYTES) * n, t_bulk.mean_ms())
        kernels["insert_keys_bulk"] = roofline_entry(
            chain + " (ash_map_insert_bulk, keys)", INSERT_KEY_BYTES * n, t_bulk_keys.mean_ms())
        for name in ("insert_values_bulk", "insert_keys_bulk"):
            kernels[name]["Mkeys_per_s"] = round(n / kernels[name]["ms"] / 1e3, 1)
            kernels[name]["workspace_bytes"] = ws_bytes.value
    kernels["api_insert_path"] = "insert_values_bulk" if api_uses_bulk else "insert_values"
    if erase_ws is not None:
        kernels["erase_bulk"] = roofline_entry(
            "split_keys_kernel<3> + split_records_kernel + erase_range_kernel "
            "(ash_map_erase_bulk, every key stored)", INSERT_KEY_BYTES * n, t_erase_bulk.mean_ms())
        kernels["erase_bulk"]["Mkeys_per_s"] = round(n / kernels["erase_bulk"]["ms"] / 1e3, 1)
    kernels["api_erase_path"] = (
        "erase_bulk" if erase_ws is not None and erase_worthwhile.value
        and ash.common.BULK_ERASE != "never" else "erase")
    for name in ("insert_values", "insert_keys", "find", "erase"):
        kernels[name]["Mkeys_per_s"] = round(n / kernels[name]["ms"] / 1e3, 1)
    kernels["items"]["Mkeys_per_s"] = round(n / kernels["items"]["ms"] / 1e3, 1)
    del hm, w, workspace, erase_ws
    torch.cuda.empty_cache()
    kernels["step_after_erase_ms"] = round(ms_per_step_after_erase, 3)
    return ms_per_step, hits, kernels


def bench_config1(torch, ash, workloads, dev, reps=5):
    """Configuration 1 on the device (the configuration the CPU baseline also
    runs at full size): HashSet, 1 M inserts with 50 % duplicates into
    capacity 2 M, then 1 M finds; kernel times through the raw C ABI."""
    w = workloads.hashset_uniform_keys(device=dev)
    hs = ash.HashSet(3, 2_000_000, dev)
    backend = hs.engine.backend
    lib, handle = backend._lib, backend._handle
    stream = torch.cuda.current_stream(dev).cuda_stream
    keys, queries = w["insert_keys"], w["query_keys"]
    n_ins, n_q = keys.shape[0], queries.shape[0]
    idx = torch.empty(n_q, dtype=torch.int64, device=dev)
    msk = torch.empty(n_q, dtype=torch.bool, device=dev)
    t_ins, t_find = EventTimer(torch), EventTimer(torch)
    for it in range(2 + reps):
        run = (lambda timer, fn: timer(fn)) if it >= 2 else (lambda timer, fn: fn())
        assert lib.ash_map_clear(handle, stream) == 0
        assert lib.ash_map_find(handle, queries.data_ptr(), 1, idx.data_ptr(), msk.data_ptr(),
                                stream) == 0   # the deferred fill of the cleared table
        run(t_ins, lambda: lib.ash_map_insert_keys(handle, keys.data_ptr(), n_ins, stream))
        run(t_find, lambda: lib.ash_map_find(handle, queries.data_ptr(), n_q, idx.data_ptr(),
                                             msk.data_ptr(), stream))
    ms_i, ms_f = t_ins.mean_ms(), t_find.mean_ms()
    unique = backend.size()   # (the handle follows the raw launches above as well)
    # 38 B per input key: 12 + 16 for every key, 16 + 4 more for the unique half
    out = {
        "insert_keys": roofline_entry("insert_kernel<3,keys> 1 M keys, 50 % duplicates",
                                      28 * n_ins + 20 * unique, ms_i),
        "find": roofline_entry("find_kernel<3> 1 M queries", FIND_BYTES * n_q, ms_f),
        "unique_keys": unique,
        "hits": int(msk.sum()),
    }
    out["insert_keys"]["Mkeys_per_s"] = round(n_ins / ms_i / 1e3, 1)
    out["find"]["Mkeys_per_s"] = round(n_q / ms_f / 1e3, 1)
    # the same insert through the API, HashSet.insert on the cleared set: the
    # library chooses the path (a table that has not been used since it was
    # emptied is written whole by the streaming passes, which saves its fill)
    import ctypes
    need = ctypes.c_int64(0)
    assert lib.ash_map_clear(handle, stream) == 0
    assert lib.ash_map_insert_scratch_bytes(handle, n_ins, 0, None, 0, ctypes.byref(need)) == 0
    t_api = EventTimer(torch)
    for it in range(2 + reps):
        hs.clear()
        (t_api if it >= 2 else (lambda fn: fn()))(lambda: hs.insert(keys))
    assert backend.size() == unique
    out["insert_api"] = {
        "path": "streaming" if need.value > 0 else "per key",
        "ms": round(t_api.mean_ms(), 4),
        "Mkeys_per_s": round(n_ins / t_api.mean_ms() / 1e3, 1),
        "includes": "all the call queues -- with the table fill a clear leaves behind when the "
                    "per-key path runs -- and its look at the counters",
    }
    del hs, w
    return out


def demo_width_entry(torch, ash, workloads, x, radii, centres, reps, dev):
    """The queries of configuration 4 on rows of five channels, the width of
    the reference's demos (distance, colour, weight: demo/rgbd_fusion.py:283,
    demo/train_scene_recon.py:41): kernel times of the three query functions
    and the module forward, priced like the other widths."""
    backend = ash.grid_query.backend
    torch.cuda.empty_cache()
    grid, _, _ = workloads.build_grid(ash, 200_000, 5, device=dev)
    n = x.shape[0]
    gi, ci, off, mk = grid.query(grid.transform_world_to_cell(x))
    ops = (grid.embeddings.detach(), off, gi, ci, mk, grid.lut_grid_nb2grid_idx,
           grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb)
    n_live = int(mk.sum())
    masked = n - n_live
    z = torch.rand(n, 5, device=dev) - 0.5
    u = torch.rand(n, 3, device=dev) - 0.5
    dense = 4 * grid.embeddings.numel()
    timers = [EventTimer(torch) for _ in range(4)]
    for it in range(2 + reps):
        run = (lambda timer, fn: timer(fn)) if it >= 2 else (lambda timer, fn: fn())
        run(timers[0], lambda: backend.query_forward(*ops, 8, "smooth_step"))
        run(timers[1], lambda: backend.query_backward_forward(z, *ops, 8, "smooth_step"))
        run(timers[2], lambda: backend.query_backward_backward(None, u, z, *ops, 8, "smooth_step"))
        with torch.no_grad():
            run(timers[3], lambda: grid(x, "smooth_step"))
    entry = {
        "forward": roofline_entry("query_forward_kernel<f32,E5> (one lane per row)",
                                  fwd_bytes(5) * n_live + (29 + 20) * masked, timers[0].mean_ms()),
        "backward": roofline_entry("zero16 + query_backward_forward_kernel (E=5)",
                                   bwd_bytes(5) * n_live + (29 + 12) * masked + dense,
                                   timers[1].mean_ms()),
        "double_backward": roofline_entry("zero16 + query_backward_backward_kernel (E=5)",
                                          bwd2_bytes(5) * n_live + (29 + 20) * masked + dense,
                                          timers[2].mean_ms()),
        "module_forward": roofline_entry("grid_forward_kernel<f32,E5>",
                                         fwd_bytes(5) * n_live + (29 + 20) * masked,
                                         timers[3].mean_ms()),
    }
    for e in entry.values():
        e["Mqueries_per_s"] = round(n / e["ms"] / 1e3, 1)
    del grid, ops, z, u
    torch.cuda.empty_cache()
    return entry


def bench_trilinear(torch, ash, workloads, args, dev):
    """Kernel figures of configurations 3 (E=16 forward) and 4 (E=4 forward,
    backward, double backward) plus the module-level autograd step of
    configuration 4."""
    out = {}
    backend = ash.grid_query.backend
    reps = max(args.steps, 3)

    # configuration 3
    grid, _, _ = workloads.build_grid(ash, 200_000, 16, device=dev)
    x = workloads.uniform_queries(grid, 4_000_000)
    gi, ci, off, mk = grid.query(grid.transform_world_to_cell(x))
    ops = (grid.embeddings.detach(), off, gi, ci, mk, grid.lut_grid_nb2grid_idx,
           grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb)
    n3 = x.shape[0]
    for interp in ("linear", "smooth_step"):
        t = EventTimer(torch)
        for it in range(2 + reps):
            if it < 2:
                backend.query_forward(*ops, 8, interp)
            else:
                t(lambda: backend.query_forward(*ops, 8, interp))
        n_live = int(mk.sum())
        alg = fwd_bytes(16) * n_live + (29 + 64) * (n3 - n_live)
        e = roofline_entry(f"query_forward_kernel<f32,E16> {interp}", alg, t.mean_ms())
        e["Mqueries_per_s"] = round(n3 / e["ms"] / 1e3, 1)
        out[f"cfg3_forward_{interp}"] = e

    # sparse convolution over the same grid (3^3 window, per channel): every
    # row is read once per tap through the caches; the algorithmic figure
    # counts one read and one write of each active row
    cells = grid.engine.size() * 512
    for size in (3, 7):   # 7 is the window of the demos' gaussian_filter_
        weights = torch.rand(size, size, size, 16, device=dev)
        t = EventTimer(torch)
        for it in range(3):
            if it == 0:
                grid.convolution(grid.embeddings.detach(), weights)
            else:
                t(lambda: grid.convolution(grid.embeddings.detach(), weights))
        e = roofline_entry(f"convolution_tile_kernel<f32> {size**3} taps (incl. table construction)",
                           2 * 64 * cells, t.mean_ms())
        e["Gcells_per_s"] = round(cells / e["ms"] / 1e6, 2)
        # large windows are bound by the multiply-adds, not by HBM: one fp32 FMA
        # per tap, channel and cell against the 157.3 TFLOP/s vector peak
        e["fp32_TFLOP_per_s"] = round(2 * size**3 * 16 * cells / (e["ms"] * 1e-3) / 1e12, 2)
        e["fp32_frac"] = round(e["fp32_TFLOP_per_s"] / 157.3, 4)
        out["cfg3_convolution" if size == 3 else f"cfg3_convolution_{size}"] = e
    del grid, ops, x, weights
    torch.cuda.empty_cache()

    # configuration 4
    grid, radii, centres = workloads.build_grid(ash, 200_000, 4, device=dev)
    x = workloads.ray_queries(grid, radii, centres, 32768, 128)
    n4 = x.shape[0]
    gi, ci, off, mk = grid.query(grid.transform_world_to_cell(x))
    ops = (grid.embeddings.detach(), off, gi, ci, mk, grid.lut_grid_nb2grid_idx,
           grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb)
    n_live = int(mk.sum())
    z = torch.rand(n4, 4, device=dev) - 0.5
    u = torch.rand(n4, 3, device=dev) - 0.5
    dense = 4 * grid.embeddings.numel()
    t_f, t_b, t_bb = EventTimer(torch), EventTimer(torch), EventTimer(torch)
    for it in range(2 + reps):
        run = (lambda timer, fn: timer(fn)) if it >= 2 else (lambda timer, fn: fn())
        run(t_f, lambda: backend.query_forward(*ops, 8, "smooth_step"))
        run(t_b, lambda: backend.query_backward_forward(z, *ops, 8, "smooth_step"))
        run(t_bb, lambda: backend.query_backward_backward(None, u, z, *ops, 8, "smooth_step"))
    masked = n4 - n_live
    entries = {
        "cfg4_forward": roofline_entry(
            "query_forward_kernel<f32,E4>", fwd_bytes(4) * n_live + (29 + 16) * masked, t_f.mean_ms()),
        "cfg4_backward": roofline_entry(
            "zero16 + query_backward_forward_vec_kernel (E=4)",
            bwd_bytes(4) * n_live + (29 + 12) * masked + dense, t_b.mean_ms()),
        "cfg4_double_backward": roofline_entry(
            "zero16 + query_backward_backward_vec_kernel (E=4)",
            bwd2_bytes(4) * n_live + (29 + 16) * masked + dense, t_bb.mean_ms()),
    }
    for name, e in entries.items():
        e["Mqueries_per_s"] = round(n4 / e["ms"] / 1e3, 1)
        out[name] = e
    fb_ms = entries["cfg4_forward"]["ms"] + entries["cfg4_backward"]["ms"]
    fb_bytes = (fwd_bytes(4) + bwd_bytes(4)) * n_live + (58 + 28) * masked + dense
    e = roofline_entry("cfg4 forward + backward kernels", fb_bytes, fb_ms)
    e["Mqueries_per_s"] = round(n4 / fb_ms / 1e3, 1)
    out["cfg4_forward_plus_backward"] = e
    out["cfg4_live_fraction"] = round(n_live / n4, 4)

    # the front end that turns positions into the operands above
    # (ash/grid.py:183-199): 12 B read, 8 + 8 + 12 + 1 B written per position
    xc = grid.transform_world_to_cell(x).contiguous()
    t_q = EventTimer(torch)
    for it in range(2 + reps):
        if it < 2:
            grid.query(xc)
        else:
            t_q(lambda: grid.query(xc))
    e = roofline_entry("grid_query_kernel (positions -> block, cell, offset, mask)", 41 * n4,
                       t_q.mean_ms())
    e["Mqueries_per_s"] = round(n4 / e["ms"] / 1e3, 1)
    out["cfg4_grid_query"] = e
    del xc

    # the ray sampler that produces such queries (ash/grid.py:322-403)
    ro, rd = workloads.camera_rays(grid, radii, centres, 32768)
    extent = float((grid.bbox_max - grid.bbox_min).norm())
    t_nf, t_rs = EventTimer(torch), EventTimer(torch)
    for it in range(2 + reps):
        run = (lambda timer, fn: timer(fn)) if it >= 2 else (lambda timer, fn: fn())
        box = {}
        run(t_nf, lambda: box.update(nf=grid.ray_find_near_far(ro, rd, 0.0, extent, 0.01)))
        run(t_rs, lambda: box.update(rs=grid.ray_sample(ro, rd, *box["nf"], 128)))
    n_samples = int(box["rs"][0].numel())
    ms_nf, ms_rs = t_nf.mean_ms(), t_rs.mean_ms()
    out["cfg4_ray_sampler"] = {
        "rays": 32768,
        "samples": n_samples,
        "ray_find_near_far_ms": round(ms_nf, 4),
        "ray_sample_ms": round(ms_rs, 4),
        "Mrays_per_s": round(32768 / (ms_nf + ms_rs) / 1e3, 1),
        "Msamples_per_s": round(n_samples / (ms_nf + ms_rs) / 1e3, 1),
    }

    # surface extraction over the same blocks (ash/grid.py:628-711): the
    # algorithmic figure counts one read of field and weight per cell and one
    # write of every vertex and triangle
    field = workloads.sphere_distance_field(grid, radii, centres)
    ones = torch.ones_like(field)
    t_mesh, t_pts = EventTimer(torch), EventTimer(torch)
    for it in range(2 + reps):
        run = (lambda timer, fn: timer(fn)) if it >= 2 else (lambda timer, fn: fn())
        run(t_mesh, lambda: box.update(mesh=grid.surface_mesh(field, ones)))
        run(t_pts, lambda: box.update(pts=grid.isosurface_points(field, ones)))
    cells = grid.engine.size() * 512
    n_tri, n_vtx, n_pts = len(box["mesh"][0]), len(box["mesh"][1]), len(box["pts"])
    e = roofline_entry("marching cubes: classify + extract (6 kernels, one read-back)",
                       8 * cells + 12 * (n_tri + n_vtx), t_mesh.mean_ms())
    e.update(cells=cells, vertices=n_vtx, triangles=n_tri,
             Gcells_per_s=round(cells / e["ms"] / 1e6, 2))
    out["cfg4_surface_mesh"] = e
    e = roofline_entry("iso-surface points: classify + points (4 kernels, one read-back)",
                       8 * cells + 12 * n_pts, t_pts.mean_ms())
    e.update(cells=cells, points=n_pts, Gcells_per_s=round(cells / e["ms"] / 1e6, 2))
    out["cfg4_isosurface_points"] = e
    del field, ones, box

    # the module's forward, grid(x): positions -> features in one kernel
    # (ash_grid_forward); 12 B position + 16 B slot + 8 rows + 1 row out + mask
    # per live query -- the same 29 + 36 E as the operand-level forward; with
    # the operands of a backward pass written as well: + 28 B per query
    t_inf, t_trn = EventTimer(torch), EventTimer(torch)
    xg = x.clone().requires_grad_(True)
    for it in range(2 + reps):
        run = (lambda timer, fn: timer(fn)) if it >= 2 else (lambda timer, fn: fn())
        with torch.no_grad():
            run(t_inf, lambda: grid(x, "smooth_step"))
        run(t_trn, lambda: grid(xg, "smooth_step"))
    for name, timer, extra in (("cfg4_module_forward", t_inf, 0),
                               ("cfg4_module_forward_for_training", t_trn, 28)):
        e = roofline_entry("grid_forward_kernel<f32,E4> (SparseDenseGrid.forward, smooth_step)",
                           (fwd_bytes(4) + extra) * n_live + (29 + 16 + extra) * masked,
                           timer.mean_ms())
        e["Mqueries_per_s"] = round(n4 / e["ms"] / 1e3, 1)
        out[name] = e
    del xg

    # module-level training step: value loss + gradient-norm loss
    # (demo/train_scene_recon.py:326-341)
    xq = x.clone().requires_grad_(True)

    def train_step(contract):
        grid.embeddings.grad = None
        feats, _ = grid(xq, "smooth_step")
        (gx,) = torch.autograd.grad(feats[:, 0].sum(), xq, create_graph=True)
        loss = (feats[:, 1:] ** 2).mean() + (gx.norm(dim=-1) - 1).abs().mean()
        if contract:
            with ash.dense_grad(grid):
                loss.backward()
        else:
            loss.backward()

    # plain backward(): every backward node fills a dense gradient of its own
    # and autograd adds them (the reference's behaviour); inside
    # `with ash.dense_grad(grid):` the nodes add to embeddings.grad directly
    for label, contract in (("", False), ("_dense_grad", True)):
        for _ in range(2):
            train_step(contract)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            train_step(contract)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / reps * 1e3
        out["cfg4_module_train_step" + label] = {
            "ms": round(ms, 3), "Mqueries_per_s": round(n4 / ms / 1e3, 1)}
    out["cfg4_rows_of_five"] = demo_width_entry(torch, ash, workloads, x, radii, centres, reps, dev)
    if not args.no_cpu:
        # The CPU baseline runs after every section that is timed with the wall
        # clock: its OpenMP workers keep spinning for a while after a parallel
        # region and would compete with the thread that launches the GPU work.
        out["cfg4_cpu_job"] = cpu_trilinear_job(torch, ops, z, u, 1 << 18)
    return out


def bench_fusion(torch, ash, workloads, args, dev, frames=100):
    """Configuration 5 (secondary figure): depth frames of the synthetic scene
    fused into an unbounded grid, once with the library's fused activation and
    integration kernels and once in the reference's formulation (candidate
    expansion + scratch set, torch expressions around
    embeddings[grid_indices, cell_indices])."""
    # same allocator state whatever ran before: the reference formulation
    # allocates tens of MB per frame and is sensitive to what is cached
    torch.cuda.empty_cache()
    scene = workloads.FusionScene()
    intrinsic = scene.intrinsic.to(dev)
    data = []
    for f in range(frames):
        ext = scene.pose(f * (100 // frames))
        depth = scene.depth(ext)
        data.append((scene.unproject(depth, ext).to(dev), depth.to(dev), ext.to(dev)))
    points = sum(d[0].shape[0] for d in data) / frames
    out = {"frames": frames, "points_per_frame": round(points),
           "candidate_keys_per_frame": round(points * 27)}
    # "fused": the library's activation + integration kernels with the number of
    # touched blocks read back per frame (what spatial_init_ returns needs it);
    # "fused_no_readback": the same kernels with that number left on the device
    for name, fused, count in (("reference_formulation", False, True), ("fused", True, True),
                               ("fused_no_readback", True, False)):
        for rep in range(2):  # the first pass warms allocations up
            grid = ash.UnBoundedSparseDenseGrid(3, 80000, 2, 8, cell_size=0.015, device=dev)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            touched = 0
            for pts, depth, ext in data:
                touched += workloads.fuse_frame(grid, pts, depth, intrinsic, ext, trunc=0.04,
                                                fused=fused, count_blocks=count) or 0
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        out[name] = {
            "frames_per_s": round(frames / dt, 1),
            "ms_per_frame": round(dt / frames * 1e3, 3),
            "Mkeys_per_s": round(points * 27 * frames / dt / 1e6, 1),
            "active_blocks": grid.engine.size(),
            "touched_blocks_per_frame": round(touched / frames),
        }
        del grid
    # the same frames with the launches of a frame recorded once into a HIP
    # graph and replayed (ash_map_insert-style calls only queue launches on a
    # capturing stream): inputs are rewritten in place, the point lists padded
    # to one length with copies of their last point
    most = max(d[0].shape[0] for d in data)
    for rep in range(2):
        grid = ash.UnBoundedSparseDenseGrid(3, 80000, 2, 8, cell_size=0.015, device=dev)
        pts = torch.empty((most, 3), device=dev)
        depth, ext = torch.empty_like(data[0][1]), torch.empty_like(data[0][2])

        def load(frame):
            p = data[frame][0]
            pts[: len(p)] = p
            pts[len(p):] = p[-1]
            depth.copy_(data[frame][1])
            ext.copy_(data[frame][2])

        load(0)
        ash.fusion.fuse_frame(grid, pts, depth, intrinsic, ext, 0.04, 6.0, count_blocks=False)
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            ash.fusion.fuse_frame(grid, pts, depth, intrinsic, ext, 0.04, 6.0, count_blocks=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for frame in range(1, frames):
            load(frame)
            graph.replay()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        # the replays alone (inputs left as they are): what the graph costs
        t_replay = EventTimer(torch)
        for _ in range(20):
            t_replay(graph.replay)
        replay_ms = t_replay.mean_ms()
    out["fused_graph_replay"] = {
        "frames_per_s": round((frames - 1) / dt, 1),
        "ms_per_frame": round(dt / (frames - 1) * 1e3, 3),
        "ms_per_replay_alone": round(replay_ms, 4),
        "active_blocks": grid.engine.size(),
    }
    del grid
    torch.cuda.empty_cache()
    return out


def cpu_baseline(torch, workloads, args):
    """The oracle (OpenMP) on configuration 2 itself (same generator, the same
    keys, capacity, queries and value rows as the device run; `--cpu-keys`
    picks a smaller sample with capacity 1.5x): insert + find + items with the
    value rows gathered, as in the device step."""
    import ash_oracle

    oracle = ash_oracle.OracleBackend()
    n = args.cpu_keys or args.keys
    cap = n * 3 // 2 if args.cpu_keys else args.capacity
    w = workloads.hashmap_sphere_voxels(num_keys=n, device="cpu")
    heap = torch.arange(cap, dtype=torch.int32)
    omap = oracle.HashMap(3, cap, heap)
    stores = {"color": torch.zeros(cap, 3), "depth": torch.zeros(cap, 1)}
    values = {"color": w["color"], "depth": w["depth"]}
    best = None
    for _ in range(2):
        omap.clear()
        t0 = time.perf_counter()
        omap.insert(w["keys"], values, stores)
        t1 = time.perf_counter()
        omap.find(w["query_keys"])
        t2 = time.perf_counter()
        _, idx = omap.items()
        gathered = {name: rows[idx] for name, rows in stores.items()}
        t3 = time.perf_counter()
        if best is None or t3 - t0 < best[0]:
            best = (t3 - t0, t1 - t0, t2 - t1, t3 - t2)
    total, t_ins, t_find, t_items = best
    out = {
        "value": round(2 * n / total / 1e6, 2),
        "unit": "Mkeys/s",
        "cores": oracle.num_threads(),
        "kind": "port",
        "sample": f"configuration 2 at {n} keys, capacity {cap}: insert + find + items with "
                  "values, best of 2",
        "insert_Mkeys_per_s": round(n / t_ins / 1e6, 2),
        "find_Mkeys_per_s": round(n / t_find / 1e6, 2),
    }
    del omap, stores, values, w, gathered

    # configuration 1 at full size (HashSet, 1 M inserts with 50 % duplicates
    # into capacity 2 M, 1 M finds), all threads and one thread
    w1 = workloads.hashset_uniform_keys(device="cpu")
    threads = oracle.num_threads()
    for label, nthreads in (("config1", threads), ("config1_one_thread", 1)):
        oracle.set_num_threads(nthreads)
        oset = oracle.HashMap(3, 2_000_000, torch.arange(2_000_000, dtype=torch.int32))
        t0 = time.perf_counter()
        oset.insert_keys(w1["insert_keys"])
        t1 = time.perf_counter()
        oset.find(w1["query_keys"])
        t2 = time.perf_counter()
        out[label] = {
            "cores": nthreads,
            "insert_Mkeys_per_s": round(len(w1["insert_keys"]) / (t1 - t0) / 1e6, 2),
            "find_Mkeys_per_s": round(len(w1["query_keys"]) / (t2 - t1) / 1e6, 2),
        }
        del oset
    oracle.set_num_threads(threads)
    return out


def cpu_trilinear_job(torch, ops, z, u, n_sample):
    """Copies what the CPU baseline of the query functions needs to the host
    and returns the function that runs it."""
    emb, off, gi, ci, mk, lut_g, lut_c2c, lut_c2g = ops
    cops = (emb.cpu(), off[:n_sample].cpu(), gi[:n_sample].cpu(), ci[:n_sample].cpu(),
            mk[:n_sample].cpu(), lut_g.cpu(), lut_c2c.cpu(), lut_c2g.cpu())
    zc, uc = z[:n_sample].cpu(), u[:n_sample].cpu()
    return lambda: cpu_trilinear(cops, zc, uc, n_sample)


def cpu_trilinear(cops, zc, uc, n_sample):
    """The oracle's three query functions on the first `n_sample` queries of
    configuration 4 (whole rays), all host threads."""
    import ash_oracle

    oracle = ash_oracle.OracleBackend()
    t0 = time.perf_counter()
    oracle.query_forward(*cops, 8, "smooth_step")
    t1 = time.perf_counter()
    oracle.query_backward_forward(zc, *cops, 8, "smooth_step")
    t2 = time.perf_counter()
    oracle.query_backward_backward(None, uc, zc, *cops, 8, "smooth_step")
    t3 = time.perf_counter()
    return {
        "cores": oracle.num_threads(),
        "sample": f"first {n_sample} queries of configuration 4 (E=4); backward passes include the "
                  "dense zero fill of grad_embeddings",
        "forward_Mqueries_per_s": round(n_sample / (t1 - t0) / 1e6, 2),
        "backward_Mqueries_per_s": round(n_sample / (t2 - t1) / 1e6, 2),
        "double_backward_Mqueries_per_s": round(n_sample / (t3 - t2) / 1e6, 2),
    }


def main():
    args = parse_args()
    if args.csrc_fingerprint:
        print(csrc_fingerprint())
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has one GPU and the path "
              "has no multi-GPU part; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    import ash
    import workloads
    from ash.common import _Backend

    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    assert isinstance(ash.core.backend, _Backend), "libash_hip.so is not loaded"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate:
        # A plain 1 GiB device-to-device copy: the reference point for scaling
        # rocprofv3's FETCH_SIZE / WRITE_SIZE counters to bytes.
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    ms_per_step, hits, kernels = bench_hash(torch, ash, workloads, args, dev)
    if not args.no_trilinear:
        kernels.update(bench_trilinear(torch, ash, workloads, args, dev))
    kernels["cfg1_hashset"] = bench_config1(torch, ash, workloads, dev)
    if not args.no_fusion:
        kernels["cfg5_fusion"] = bench_fusion(torch, ash, workloads, args, dev)
    counters_note = attach_counters(
        kernels, args.keys == 16_000_000 and args.capacity == 24_000_000,
        ash.common.load_library().ash_source_fingerprint().decode())
    dominant = max((kernels["api_insert_path"], "find", "items"), key=lambda k: kernels[k]["ms"])
    roof = dict(kernels[dominant])
    table_bytes = (args.capacity + 5) // 6 * 128
    ceilings = measure_ceilings(torch, ash, dev, table_bytes, 16 << 20)
    kernels["find"]["of_random_line_read_rate"] = round(
        kernels["find"]["Mkeys_per_s"] / 1e3 / ceilings["random_line_reads"]["Glines_per_s"], 3)
    for name in ("insert_values", "insert_keys"):
        kernels[name]["of_random_line_update_rate"] = round(
            kernels[name]["Mkeys_per_s"] / 1e3 / ceilings["random_line_updates"]["Glines_per_s"], 3)
    value = 2 * args.keys / (ms_per_step * 1e-3) / 1e6
    line = {
        "metric": "Mkeys/s insert+find (16M int3); Mqueries/s trilinear fwd+bwd; % HBM roofline",
        "value": round(value, 1),
        "unit": "Mkeys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        # the same step once the map has seen an erase (plus one erase and one
        # one-key insert per step): listing by ranks, value rows by index
        "ms_per_step_after_erase": kernels.pop("step_after_erase_ms"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u64 keys / int32 indices; fp32 trilinear",
        "data": "synthetic",
        "config": {
            "workload": "configuration 2: HashMap{color fp32[3], depth fp32[1]}, "
                        f"{args.keys} distinct int3 voxel keys into capacity {args.capacity}, "
                        f"{args.keys} finds ({hits} hits), items(); step = clear+insert+find+items "
                        "through the Python API",
            "keys": args.keys,
            "capacity": args.capacity,
        },
        "roofline": roof,
        "counters": counters_note,
        "kernels": kernels,
        "ceilings": ceilings,
    }
    cpu_job = kernels.pop("cfg4_cpu_job", None)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(torch, workloads, args)
        if cpu_job is not None:
            line["cpu_baseline"]["trilinear"] = cpu_job()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
