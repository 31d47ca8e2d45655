"""Builds libash_hip.so (gfx950) in-tree with hipcc.

    python torch-ash_amd/build.py            # rebuild when sources are newer
    python torch-ash_amd/build.py --force    # always rebuild

The library lands in torch-ash_amd/ash/lib/ so that it travels with the source
tree; nothing is installed into site-packages.
"""
import argparse
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "ash", "lib")
OUT = os.path.join(OUT_DIR, "libash_hip.so")
SOURCES = ["ash_map.hip", "ash_bulk.hip", "ash_query.hip", "ash_fusion.hip", "ash_mesh.hip"]
HEADERS = [
    os.path.join(CSRC, "ash_probe.h"),
    os.path.join(CSRC, "ash_dev.h"),
    os.path.join(CSRC, "ash_table.h"),
    os.path.join(CSRC, "ash_mc_table.h"),
    os.path.join(HERE, os.pardir, "include", "ash_hip.h"),
]
ARCH = "gfx950"


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def compile_flags():
    return [
        "-O3",
        "-std=c++17",
        "-fPIC",
        f"--offload-arch={ARCH}",
        "-Xclang",
        "-target-feature",
        "-Xclang",
        "-packed-fp32-ops",
        "-Wall",
        "-Wno-unused-function",
    ]


def source_fingerprint() -> str:
    """SHA-256 over the kernel sources (names and contents of csrc/*.hip and
    csrc/*.h).  It is compiled into the library (ash_source_fingerprint), so
    that a benchmark or a test can tell a library that was not built from the
    sources beside it."""
    import hashlib

    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def is_stale() -> bool:
    if not os.path.exists(OUT):
        return True
    built = os.path.getmtime(OUT)
    deps = [os.path.join(CSRC, s) for s in SOURCES] + HEADERS + [os.path.abspath(__file__)]
    return any(os.path.getmtime(d) > built for d in deps)


def build(force: bool = False, verbose: bool = True) -> str:
    if not force and not is_stale():
        return OUT
    os.makedirs(OUT_DIR, exist_ok=True)
    hipcc = hipcc_path()
    stamp = f'-DASH_SOURCE_FINGERPRINT="{source_fingerprint()}"'
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(OUT_DIR, src.replace(".hip", ".o"))
        cmd = [hipcc, *compile_flags(), "-c", os.path.join(CSRC, src), "-o", obj]
        if src == "ash_map.hip":
            cmd.insert(1, stamp)
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd)))
        objs.append(obj)
    for cmd, p in procs:
        if p.wait() != 0:
            raise RuntimeError("compile failed: " + " ".join(cmd))
    tmp = OUT + ".tmp"
    link = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    os.replace(tmp, OUT)
    for o in objs:
        os.remove(o)
    return OUT


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    args = ap.parse_args()
    print(build(force=args.force))
    sys.exit(0)
