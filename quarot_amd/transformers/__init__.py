"""Mirror of quarot.transformers (quarot/transformers/__init__.py:1)."""
from .kv_cache import MultiLayerPagedKVCache4Bit
from . import kv_cache
