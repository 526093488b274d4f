"""MI355X-native (gfx950) implementation of the VAR-Q KV-cache quantization hot
path: quantize -> pack -> (append) -> unpack/dequant -> attention.

Python surface mirrors the reference package `VAR_Q` (quant.VAR_Q,
pack_unpack.*, config_loader.*); the arithmetic runs in hand-written HIP kernels
behind the C ABI of include/varq.h.
"""
from ._lib import VarqError, load as load_library  # noqa: F401
from .quant import VAR_Q  # noqa: F401
from .config_loader import VARQConfig, load_varq_config  # noqa: F401
from .kv_cache import PackedKVCache  # noqa: F401
from . import hooks, ops, schedules  # noqa: F401
