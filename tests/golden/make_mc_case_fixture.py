"""Writes mc_case_boundaries.json: for each of the 256 marching-cubes cases the
triangles the reference emits ("set": oriented edge triples, each starting at
its lowest edge, sorted), their number, and the outline of the patch they form,
as a set of directed segments between cube edges.

With --cuts it also prints the CUTS dictionary of
torch-ash_amd/csrc/gen_mc_table.py: for every polygon of more than three
corners of that generator's loops, the number of the cut (in the generator's
enumeration) whose triangles are the reference's.

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
import importlib.util
import json
import os
import re
import sys

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
        triangles = []
        for t in range(0, 15, 3):
            if row[t] < 0:
                break
            a, b, c = (edge[row[t + 2]], edge[row[t + 1]], edge[row[t]])
            sides += [(a, b), (b, c), (c, a)]
            triangles.append(_from_lowest([a, b, c]))
        outline = sorted(s for s in sides if (s[1], s[0]) not in sides)
        cases[str(mine)] = {"triangles": len(triangles), "outline": outline,
                            "set": sorted(triangles)}
    with open(OUT, "w") as f:
        json.dump(cases, f, separators=(",", ":"), sort_keys=True)
    print(f"wrote {OUT}")
    if "--cuts" in sys.argv:
        print_cuts(cases)


def _from_lowest(t):
    i = t.index(min(t))
    return t[i:] + t[:i]


def print_cuts(cases):
    """The CUTS dictionary of the library's generator: per case, which cut of
    each polygon of more than three corners gives the reference's triangles."""
    here = os.path.dirname(os.path.abspath(__file__))
    path = os.path.join(here, os.pardir, os.pardir, "torch-ash_amd", "csrc", "gen_mc_table.py")
    spec = importlib.util.spec_from_file_location("gen_mc_table", path)
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    cuts = {}
    for case in range(256):
        want = {tuple(t) for t in cases[str(case)]["set"]}
        picked = []
        for loop in gen.case_loops(case):
            loop = gen.from_lowest_edge(loop)
            if len(loop) <= 3:
                continue
            mine = {t for t in want if set(t) <= set(loop)}
            which = [n for n, cut in enumerate(gen.triangulations(loop))
                     if {tuple(_from_lowest(list(t))) for t in cut} == mine]
            assert len(which) == 1, f"case {case}: no cut of {loop} gives {sorted(mine)}"
            picked.append(which[0])
        if picked:
            cuts[case] = tuple(picked)
    print("CUTS =", cuts)


if __name__ == "__main__":
    main()
