"""Builds the marching-cubes case table that ash_mc_table.h holds.

The table is derived here from the geometry of the cube, not taken from a
published listing.  Conventions:

* corner c of a cell sits at offset (c & 1, (c >> 1) & 1, (c >> 2) & 1), which
  is also entry c of the 8-entry neighbour tables of a sparse-dense grid;
* bit c of a case is set when the field at corner c lies below the iso value
  (the "inside" corners; ash/src/grid.cu:646-666 of the reference builds its
  case the same way over its own corner numbering);
* edge e = 4 * axis + j runs along `axis` from the corner obtained by inserting
  a zero bit at position `axis` into the 2-bit number j; the cell at that
  corner stores the surface vertex of the edge in its slot `axis`.

Per case: on each face of the cube the inside corners form runs along the
face's corner cycle, and one segment joins the two crossed edges that bound a
run.  A face with two diagonal inside corners therefore isolates each of them
-- the same decision on both cells that share the face, so surfaces close
across cells.  The segments chain into closed loops, each loop is oriented so
that its normal points from the inside corners to the outside ones, and is cut
into a fan of triangles whose diagonals all run through the interior of the
cube.

Run as a script to rewrite ash_mc_table.h beside this file.
"""
import os
from typing import Dict, List, Tuple

HEADER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ash_mc_table.h")
MAX_TRIANGLES = 5


def corner_xyz(c: int) -> Tuple[int, int, int]:
    return (c & 1, (c >> 1) & 1, (c >> 2) & 1)


def edge_corners(e: int) -> Tuple[int, int]:
    axis, j = divmod(e, 4)
    low_bits = j & ((1 << axis) - 1)
    low = low_bits | ((j >> axis) << (axis + 1))
    return low, low | (1 << axis)


EDGE_OF: Dict[Tuple[int, int], int] = {}
for _e in range(12):
    _a, _b = edge_corners(_e)
    EDGE_OF[(_a, _b)] = _e
    EDGE_OF[(_b, _a)] = _e


def face_cycles() -> List[List[int]]:
    """The six faces as cycles of four corners."""
    faces = []
    for axis in range(3):
        u, v = [a for a in range(3) if a != axis]
        for side in (0, 1):
            base = side << axis
            ring = [base, base | (1 << u), base | (1 << u) | (1 << v), base | (1 << v)]
            faces.append(ring)
    return faces


def case_segments(case: int) -> List[Tuple[int, int]]:
    """Undirected segments between crossed edges, face by face."""
    segs = []
    for ring in face_cycles():
        inside = [(case >> c) & 1 for c in ring]
        if sum(inside) in (0, 4):
            continue
        for i in range(4):
            # a run of inside corners starts at i when i is inside and i-1 is not
            if not inside[i] or inside[(i - 1) % 4]:
                continue
            j = i
            while inside[(j + 1) % 4]:
                j = (j + 1) % 4
            first = EDGE_OF[(ring[(i - 1) % 4], ring[i])]
            last = EDGE_OF[(ring[j], ring[(j + 1) % 4])]
            segs.append((first, last))
    return segs


def _loops(segs: List[Tuple[int, int]]) -> List[List[int]]:
    links: Dict[int, List[int]] = {}
    for a, b in segs:
        links.setdefault(a, []).append(b)
        links.setdefault(b, []).append(a)
    assert all(len(v) == 2 for v in links.values()), "every crossed edge lies on two faces"
    loops, seen = [], set()
    for start in sorted(links):
        if start in seen:
            continue
        loop, prev, cur = [start], None, start
        seen.add(start)
        while True:
            a, b = links[cur]
            nxt = b if a == prev else a
            if nxt == start:
                break
            loop.append(nxt)
            seen.add(nxt)
            prev, cur = cur, nxt
        loops.append(loop)
    return loops


def _midpoint(e: int) -> Tuple[float, float, float]:
    a, b = edge_corners(e)
    pa, pb = corner_xyz(a), corner_xyz(b)
    return tuple((x + y) / 2 for x, y in zip(pa, pb))


def _oriented(loop: List[int], case: int) -> List[int]:
    """Orders the loop so that its normal points from inside to outside."""
    pts = [_midpoint(e) for e in loop]
    normal = [0.0, 0.0, 0.0]
    for i, p in enumerate(pts):  # Newell's formula
        q = pts[(i + 1) % len(pts)]
        normal[0] += (p[1] - q[1]) * (p[2] + q[2])
        normal[1] += (p[2] - q[2]) * (p[0] + q[0])
        normal[2] += (p[0] - q[0]) * (p[1] + q[1])
    outward = [0.0, 0.0, 0.0]
    for e in loop:
        a, b = edge_corners(e)
        if not (case >> a) & 1:
            a, b = b, a  # a inside, b outside
        for d in range(3):
            outward[d] += corner_xyz(b)[d] - corner_xyz(a)[d]
    dot = sum(n * o for n, o in zip(normal, outward))
    assert abs(dot) > 1e-9, "loop without a usable orientation"
    return loop if dot > 0 else [loop[0]] + loop[:0:-1]


def case_loops(case: int) -> List[List[int]]:
    return [_oriented(loop, case) for loop in _loops(case_segments(case))]


def _share_a_face(e1: int, e2: int) -> bool:
    def faces(e):
        low, _ = edge_corners(e)
        return {(a, (low >> a) & 1) for a in range(3) if a != e // 4}

    return bool(faces(e1) & faces(e2))


def _fan(loop: List[int]) -> List[int]:
    """The loop rotated so that the fan from its first corner has as few
    diagonals inside a face of the cube as possible (none, for every loop that
    occurs): such a diagonal could coincide with one of the neighbouring cell
    and give an edge shared by four triangles."""
    def flat_diagonals(start):
        r = loop[start:] + loop[:start]
        return sum(_share_a_face(r[0], r[i]) for i in range(2, len(r) - 1))

    best = min(range(len(loop)), key=lambda s: (flat_diagonals(s), s))
    return loop[best:] + loop[:best]


def case_triangles(case: int) -> List[Tuple[int, int, int]]:
    tris = []
    for loop in case_loops(case):
        loop = _fan(loop)
        for i in range(1, len(loop) - 1):
            tris.append((loop[0], loop[i], loop[i + 1]))
    return tris


def build_table() -> List[List[int]]:
    """256 rows of up to 5 triangles as edge triples, padded with -1 to 16."""
    table = []
    for case in range(256):
        tris = case_triangles(case)
        assert len(tris) <= MAX_TRIANGLES
        flat = [e for t in tris for e in t]
        table.append(flat + [-1] * (16 - len(flat)))
    return table


def triangle_counts() -> List[int]:
    return [sum(1 for v in row[::3] if v >= 0) for row in build_table()]


def header_text() -> str:
    table = build_table()
    counts = triangle_counts()
    lines = [
        "// Marching-cubes case table, written by gen_mc_table.py -- edit that file,",
        "// not this one.  Corner c sits at offset (c&1, c>>1&1, c>>2&1); bit c of a",
        "// case is set when the field at corner c is below the iso value; edge",
        "// e = 4*axis + j runs along `axis` from the corner made by inserting a zero",
        "// bit at position `axis` into j.  Row = triangles as edge triples, -1 padded.",
        "#pragma once",
        "#include <cstdint>",
        "",
        "namespace ash {",
        "",
        "__device__ const int8_t kMcTriangles[256][16] = {",
    ]
    for row in table:
        lines.append("    {" + ", ".join(f"{v:2d}" for v in row) + "},")
    lines.append("};")
    lines.append("")
    lines.append("__device__ const int8_t kMcTriangleCount[256] = {")
    for i in range(0, 256, 32):
        lines.append("    " + ", ".join(str(v) for v in counts[i : i + 32]) + ",")
    lines.append("};")
    lines.append("")
    lines.append("// The rows again, four bits per entry (15 = none), entry i in bits 4i..4i+3.")
    lines.append("__device__ const uint64_t kMcPackedRows[256] = {")
    packed = [sum(((v if v >= 0 else 15) << (4 * i)) for i, v in enumerate(row)) for row in table]
    for i in range(0, 256, 4):
        lines.append("    " + ", ".join(f"0x{v:016x}ull" for v in packed[i : i + 4]) + ",")
    lines.append("};")
    lines.append("")
    lines.append("}  // namespace ash")
    return "\n".join(lines) + "\n"


if __name__ == "__main__":
    with open(HEADER, "w") as f:
        f.write(header_text())
    print(f"wrote {HEADER}")
