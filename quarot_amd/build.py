"""Build recipe for libquarot_hip.so: plain hipcc, gfx950 only, no torch headers.

    python -m quarot_amd.build                # compile every source, link in-tree (quarot_amd/libquarot_hip.so)
    python -m quarot_amd.build --incremental  # recompile only sources newer than their objects
"""
import concurrent.futures
import os
import pathlib
import subprocess
import sys

PKG = pathlib.Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libquarot_hip.so"
OBJ = PKG.parent / "build" / "obj"
SOURCES = ("api.hip", "quant.hip", "gemm.hip", "gemm_f6.hip", "hadamard.hip", "kv.hip", "attn.hip", "calib.hip", "decode_fused.hip",
           "paged_f16.hip")
FLAGS = ("--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fno-gpu-rdc",
         # every fp16/fp32 operation must round on its own (the reference's results are defined that
         # way): no fused multiply-add contraction unless a kernel spells fma out
         "-ffp-contract=off",
         # packed-fp32 VALU forms are kept out of the generated code on purpose
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless, filtered.
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose=True, incremental=False):
    """One object per source (compiled side by side), then one link.  incremental: a source is
    recompiled only if it, or any header beside it, is newer than its object."""
    OBJ.mkdir(parents=True, exist_ok=True)
    headers_mtime = max((h.stat().st_mtime for h in CSRC.glob("*.h")), default=0.0)
    jobs, objs = [], []
    for s in SOURCES:
        src, obj = CSRC / s, OBJ / (s[:-4] + ".o")
        objs.append(str(obj))
        fresh = incremental and obj.exists() and obj.stat().st_mtime > max(src.stat().st_mtime, headers_mtime)
        if not fresh:
            jobs.append(["hipcc", *FLAGS, "-c", str(src), "-o", str(obj)])
    workers = max(1, min(len(jobs), (os.cpu_count() or 2)))
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", str(LIB)], verbose)
    return LIB


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv)
