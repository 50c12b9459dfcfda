"""MI355X-native low-bit KV-cache decode engine (quantize-pack + split-KV decode attention).

Drop-in for the reference's `bit_decode` package: `kvcache_pack_int`, `fwd_kvcache_int`.
"""
__version__ = "1.0.0.post1"

from .interface import (  # noqa: F401
    DecodePlan,
    fwd_kvcache_int,
    fwd_kvcache_int_append,
    kvcache_pack_int,
    plan_fwd_kvcache_int,
    plan_fwd_kvcache_int_append,
)
from .cache import BitKVCache  # noqa: F401,E402
