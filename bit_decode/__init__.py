"""Drop-in alias so that `from bit_decode import kvcache_pack_int, fwd_kvcache_int` (the
reference's import, bit_decode/__init__.py:1-6) resolves to the MI355X implementation."""
from bitladder_amd import __version__, fwd_kvcache_int, kvcache_pack_int  # noqa: F401
