"""Mirror of quarot.nn (quarot/nn/__init__.py:1-4) plus the fused Hadamard+Quantizer module."""
from .linear import Linear4bit
from .normalization import RMSNorm
from .quantization import Quantizer
from .hadamard import OnlineHadamard, OnlineHadamardQuantizer
