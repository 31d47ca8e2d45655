"""Builds the CPU oracle (oracle/ash_oracle.c) into oracle/_build/libash_oracle.so.

    python oracle/build.py [--force]

The reference's own native code cannot be built here: its hash map needs
stdgpu (an empty, un-vendored submodule), CUDA and ATen, so there is no
oracle/_ref; the C restatement in this directory is the only CPU checker.
"""
import argparse
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "ash_oracle.c")
OUT_DIR = os.path.join(HERE, "_build")
OUT = os.path.join(OUT_DIR, "libash_oracle.so")


def is_stale() -> bool:
    if not os.path.exists(OUT):
        return True
    built = os.path.getmtime(OUT)
    return os.path.getmtime(SRC) > built or os.path.getmtime(__file__) > built


def build(force: bool = False, verbose: bool = True) -> str:
    if not force and not is_stale():
        return OUT
    os.makedirs(OUT_DIR, exist_ok=True)
    gcc = shutil.which("gcc") or "gcc"
    tmp = OUT + ".tmp"
    cmd = [gcc, "-O2", "-std=gnu11", "-ffp-contract=off", "-fopenmp", "-fPIC", "-shared", "-Wall", SRC,
           "-o", tmp, "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    os.replace(tmp, OUT)
    return OUT


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    print(build(force=ap.parse_args().force))
