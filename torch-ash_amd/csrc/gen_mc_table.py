"""Builds the marching-cubes case table that ash_mc_table.h holds.

The outline of every case's patch is derived here from the geometry of the
cube; how its polygons are cut into triangles follows the reference's table
(see below).  Conventions:

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
across cells.  The segments chain into closed loops and each loop is oriented
so that its normal points from the inside corners to the outside ones: that
fixes the outline of a case's patch, and it is the outline of the reference's
table (ash/src/mc_macros.h:32-288) for all 256 cases.

What the geometry leaves open is how a loop of more than three corners is cut
into triangles.  So that a cell gives the very triangles the reference gives,
the cut of every such loop is the reference's: `triangulations` enumerates the
cuts of a polygon in a fixed order and CUTS names, per case and loop, the
number of the one whose triangles are those of the reference's row.  CUTS is
written by tests/golden/make_mc_case_fixture.py (which reads the reference's
header as text) and pinned by tests/test_oracle_marching_cubes.py against the
fixture that script also writes.

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


def triangulations(polygon: List[int]) -> List[List[Tuple[int, int, int]]]:
    """Every way of cutting the polygon into triangles, in a fixed order: the
    triangle over the side (first, last) takes each other corner k in turn,
    with every cut of the part before k and of the part after it."""
    n = len(polygon)
    if n < 3:
        return [[]]
    if n == 3:
        return [[tuple(polygon)]]
    cuts = []
    for k in range(1, n - 1):
        for before in triangulations(polygon[: k + 1]):
            for after in triangulations(polygon[k:]):
                cuts.append(before + [(polygon[0], polygon[k], polygon[n - 1])] + after)
    return cuts


def from_lowest_edge(loop: List[int]) -> List[int]:
    """The loop's corners in the same cyclic order, starting at its lowest edge."""
    i = loop.index(min(loop))
    return loop[i:] + loop[:i]


# case -> for each of its loops with more than three corners (in the order of
# case_loops, each taken from its lowest edge), the number of the cut in
# triangulations() whose triangles the reference's table holds
CUTS: Dict[int, Tuple[int, ...]] = {
    3: (0,), 5: (1,), 7: (1,), 10: (0,), 11: (2,), 12: (1,), 13: (2,), 14: (1,), 15: (1,),
    17: (0,), 19: (2,), 21: (0,), 23: (10,), 25: (0,), 26: (0,), 27: (11,), 28: (1,), 29: (2,),
    30: (3,), 31: (3,), 34: (1,), 35: (1,), 37: (1,), 38: (1,), 39: (11,), 42: (0,), 43: (10,),
    44: (1,), 45: (0,), 46: (11,), 47: (0,), 48: (1,), 49: (1,), 50: (2,), 51: (1,), 52: (1,),
    53: (2,), 54: (0,), 55: (0,), 56: (1,), 57: (3,), 58: (2,), 59: (3,), 60: (1, 0), 61: (41,),
    62: (41,), 63: (0,), 67: (0,), 68: (1,), 69: (4,), 70: (1,), 71: (2,), 74: (0,), 75: (0,),
    76: (1,), 77: (3,), 78: (11,), 79: (0,), 80: (0,), 81: (3,), 82: (0,), 83: (2,), 84: (4,),
    85: (0,), 86: (2,), 87: (2,), 88: (0,), 89: (4,), 90: (0, 1), 91: (13,), 92: (2,), 93: (4,),
    94: (0,), 95: (1,), 98: (1,), 99: (3,), 100: (1,), 101: (2,), 102: (1, 0), 103: (20,),
    106: (1,), 107: (10,), 108: (3,), 109: (10,), 110: (20,), 111: (6,), 112: (2,), 113: (12,),
    114: (11,), 115: (3,), 116: (11,), 117: (2,), 118: (13,), 119: (0,), 120: (0,), 121: (8,),
    122: (23,), 123: (4,), 124: (41,), 125: (13,), 131: (0,), 133: (1,), 135: (3,), 136: (0,),
    137: (0,), 138: (3,), 139: (11,), 140: (2,), 141: (11,), 142: (8,), 143: (3,), 145: (0,),
    147: (0,), 149: (1,), 151: (10,), 152: (0,), 153: (0, 1), 154: (4,), 155: (23,), 156: (0,),
    157: (23,), 158: (8,), 159: (4,), 160: (1,), 161: (1,), 162: (4,), 163: (2,), 164: (1,),
    165: (0, 1), 166: (2,), 167: (0,), 168: (3,), 169: (4,), 170: (0,), 171: (4,), 172: (2,),
    173: (13,), 174: (2,), 175: (0,), 176: (1,), 177: (11,), 178: (1,), 179: (0,), 180: (3,),
    181: (20,), 182: (1,), 183: (0,), 184: (2,), 185: (0,), 186: (4,), 187: (1,), 188: (41,),
    190: (13,), 192: (0,), 193: (0,), 194: (0,), 195: (0, 1), 196: (2,), 197: (2,), 198: (0,),
    199: (41,), 200: (1,), 201: (3,), 202: (2,), 203: (41,), 204: (1,), 205: (3,), 206: (0,),
    207: (1,), 208: (1,), 209: (11,), 210: (3,), 211: (41,), 212: (5,), 213: (1,), 214: (1,),
    215: (13,), 216: (11,), 217: (18,), 218: (18,), 220: (0,), 221: (1,), 222: (6,), 224: (2,),
    225: (0,), 226: (2,), 227: (41,), 228: (11,), 229: (28,), 230: (28,), 232: (5,), 233: (1,),
    234: (1,), 235: (7,), 236: (3,), 237: (4,), 238: (0,), 240: (1,), 241: (0,), 242: (3,),
    243: (1,), 244: (3,), 245: (0,), 246: (4,), 248: (0,), 249: (0,), 250: (1,), 252: (0,),
}


def case_triangles(case: int) -> List[Tuple[int, int, int]]:
    tris = []
    cuts = iter(CUTS.get(case, ()))
    for loop in case_loops(case):
        loop = from_lowest_edge(loop)
        which = next(cuts) if len(loop) > 3 else 0
        tris.extend(triangulations(loop)[which])
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
