"""Build libtlf_hip.so (gfx950) in-tree with hipcc.

Usage: python tinyllmforge_amd/csrc/build.py [--force]

Every ``*.hip`` file in this directory is compiled to an object under
``build/`` and linked into ``tinyllmforge_amd/libtlf_hip.so``.  The library is
built here (hipcc cross-compiles without a GPU) and travels to the GPU box as a
file; nothing is compiled at import time.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
ROOT = os.path.dirname(PKG)
OUT = os.path.join(PKG, "libtlf_hip.so")
OBJ_DIR = os.path.join(CSRC, "build")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-ignored-attributes",
    "-Wno-pass-failed",  # waves-per-eu is used as a register budget; LDS may cap the occupancy lower
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


# Extra flags per source file.  The attention kernels never compute with NaNs (masked scores are -inf and the
# -inf - -inf cases are handled explicitly): without NaNs to quiet, a maximum is one instruction instead of three.
EXTRA_FLAGS = {
    "prefill_attn.hip": ["-fno-honor-nans"],
    "decode_attn.hip": ["-fno-honor-nans"],
}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def build(force: bool = True, verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(ROOT, "include", "tlf_hip.h"))
    jobs = []
    objs = []
    for src in sources():
        obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
        objs.append(obj)
        if not force and _newer(obj, [os.path.join(CSRC, src)] + headers):
            continue
        jobs.append(["hipcc", *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj])

    def run(cmd):
        if verbose:
            print("[build]", os.path.basename(cmd[-3]), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        lines = [l for l in (r.stdout + r.stderr).splitlines()
                 if "packed-fp32-ops" not in l and l.strip()]
        return r.returncode, "\n".join(lines)

    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        results = list(ex.map(run, jobs))
    for rc, out in results:
        if out and (verbose or rc):
            print(out)
        if rc:
            raise RuntimeError("hipcc failed")
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", OUT]
    r = subprocess.run(link, capture_output=True, text=True)
    if r.returncode:
        print(r.stdout + r.stderr)
        raise RuntimeError("link failed")
    if verbose:
        print("[build] ->", OUT, flush=True)
    return OUT


if __name__ == "__main__":
    build(force="--force" in sys.argv or True)
