"""Mirror of the reference's quarot.functional namespace (quarot/functional/__init__.py:1-5), plus
the hot path's entry points under this namespace as well: `hadamard_transform` (the call the
reference makes into fast_hadamard_transform) and the package-level `matmul`, `sym_quant`,
`sym_dequant` (quarot/__init__.py:37-52).  The torch-only primitives of the same names stay in
`functional.quantization`, as in the reference."""
from . import hadamard
from . import quantization
from .quantization import pack_i4, unpack_i4, asym_quant_dequant, sym_quant_dequant
from .hadamard import matmul_hadU_cuda, random_hadamard_matrix, apply_exact_had_to_linear, hadamard_transform

_TOP_LEVEL = ("matmul", "sym_quant", "sym_dequant")


def __getattr__(name):
    # resolved on first use: the package's top level imports this namespace before it defines them
    if name in _TOP_LEVEL:
        import quarot_amd
        return getattr(quarot_amd, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
