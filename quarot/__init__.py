"""`quarot`: the reference's package name, served by quarot_amd.

Callers written for the reference run unchanged:

    import quarot
    from quarot.nn import Linear4bit, Quantizer, OnlineHadamard        # benchmarks/qlinear_benchmark.py:2
    from quarot.functional.hadamard import get_hadK
    from quarot.transformers.kv_cache import asym_quantize_and_pack_i4

Every submodule name below is the SAME module object as its quarot_amd counterpart (registered in
sys.modules), so classes, buffers and isinstance checks are shared between the two names.  The top
level carries the reference's four names (quarot/__init__.py:9-71) and quarot_amd's fused extras.
"""
import importlib
import sys

import quarot_amd
from quarot_amd import *                                   # noqa: F401,F403  (matmul, sym_quant, sym_dequant, PackedQuantizedTensor, ...)
from quarot_amd import __all__ as _names

_SUBMODULES = ("nn", "nn.linear", "nn.normalization", "nn.quantization", "nn.hadamard",
               "functional", "functional.hadamard", "functional.quantization",
               "transformers", "transformers.kv_cache")
for _sub in _SUBMODULES:
    sys.modules[f"{__name__}.{_sub}"] = importlib.import_module(f"quarot_amd.{_sub}")

nn = sys.modules[f"{__name__}.nn"]
functional = sys.modules[f"{__name__}.functional"]
transformers = sys.modules[f"{__name__}.transformers"]

__all__ = list(_names) + ["nn", "functional", "transformers"]
