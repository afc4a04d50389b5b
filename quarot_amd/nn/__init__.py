"""Mirror of quarot.nn (quarot/nn/__init__.py:1-4) plus the fused Hadamard+Quantizer, heads-Hadamard+Quantizer and RMSNorm+Quantizer modules."""
from .linear import Linear4bit, Linear4bitSequential, enable_fp6_prefill
from .normalization import RMSNorm, RMSNormQuantizer
from .quantization import Quantizer
from .hadamard import OnlineHadamard, OnlineHadamardQuantizer, HeadsHadamardQuantizer
