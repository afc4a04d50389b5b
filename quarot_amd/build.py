"""Build recipe for libquarot_hip.so: plain hipcc, gfx950 only, no torch headers.

    python -m quarot_amd.build          # compile in-tree (quarot_amd/libquarot_hip.so)
"""
import pathlib
import subprocess
import sys

PKG = pathlib.Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libquarot_hip.so"
SOURCES = ("api.hip", "quant.hip", "gemm.hip", "gemm_f6.hip", "hadamard.hip", "kv.hip", "attn.hip")
FLAGS = ("--offload-arch=gfx950", "-O3", "-fPIC", "-shared", "-std=c++17", "-fno-gpu-rdc",
         # every fp16/fp32 operation must round on its own (the reference's results are defined that
         # way): no fused multiply-add contraction unless a kernel spells fma out
         "-ffp-contract=off",
         # packed-fp32 VALU forms are kept out of the generated code on purpose
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument")


def build(verbose=True):
    srcs = [str(CSRC / s) for s in SOURCES if (CSRC / s).exists()]
    cmd = ["hipcc", *FLAGS, *srcs, "-o", str(LIB)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless, filtered.
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    build()
