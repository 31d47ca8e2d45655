"""Writes mc_case_boundaries.json: for each of the 256 marching-cubes cases the
outline of the surface patch the reference emits, as a set of directed segments
between cube edges, plus its triangle count.

The outline is what the reference's case table (ash/src/mc_macros.h:32-288)
fixes about a cell's surface independently of how each polygon is cut into
triangles: which crossed edges are joined across each face of the cube, and on
which side the surface faces.  It is computed from the triangles the reference
writes (ash/src/grid.cu:818-841 stores each table triangle in reverse order):
a directed triangle side that is not cancelled by the opposite side of another
triangle of the same case lies on the outline.

Everything is expressed in this library's numbering (see
torch-ash_amd/csrc/gen_mc_table.py): corner c at offset (c&1, c>>1&1, c>>2&1),
case bit c set when corner c is below the iso value, edge 4*axis + j.  The
reference header is read as text and must be present at /root/reference; the
JSON this script writes is what the tests load.
"""
import json
import os
import re

REF = "/root/reference/ash/src/mc_macros.h"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mc_case_boundaries.json")


def _ints(body):
    return [int(t, 0) for t in re.findall(r"-?(?:0x[0-9a-fA-F]+|\d+)", body)]


def _array(text, name):
    m = re.search(name + r"(?:\[\d+\])+\s*=\s*\{(.*?)\};", text, re.S)
    body = re.sub(r"//[^\n]*", "", m.group(1))
    return _ints(body)


def main():
    text = open(REF).read()
    tri = _array(text, "tri_table")
    vtx = _array(text, "vtx_shifts")
    edg = _array(text, "edge_shifts")
    assert len(tri) == 256 * 16 and len(vtx) == 24 and len(edg) == 48
    corner = [vtx[3 * k] | vtx[3 * k + 1] << 1 | vtx[3 * k + 2] << 2 for k in range(8)]
    edge = []
    for e in range(12):
        x, y, z, axis = edg[4 * e : 4 * e + 4]
        low = x | y << 1 | z << 2
        j = (low & ((1 << axis) - 1)) | ((low >> (axis + 1)) << axis)
        edge.append(4 * axis + j)
    cases = {}
    for ref_case in range(256):
        mine = 0
        for k in range(8):
            if ref_case >> k & 1:
                mine |= 1 << corner[k]
        row = tri[16 * ref_case : 16 * ref_case + 16]
        sides = []
        count = 0
        for t in range(0, 15, 3):
            if row[t] < 0:
                break
            count += 1
            a, b, c = (edge[row[t + 2]], edge[row[t + 1]], edge[row[t]])
            sides += [(a, b), (b, c), (c, a)]
        outline = sorted(s for s in sides if (s[1], s[0]) not in sides)
        cases[str(mine)] = {"triangles": count, "outline": outline}
    with open(OUT, "w") as f:
        json.dump(cases, f, separators=(",", ":"), sort_keys=True)
    print(f"wrote {OUT}")


if __name__ == "__main__":
    main()
