"""MI355X-native paged KV-cache attention path for the opt_prime inference runtime.

* ``ops``       - kv_append / paged_decode_attn / paged_prefill_attn on torch tensors
* ``kv_cache``  - drop-in ``CachedScaledDotProductAttention`` and ``KVCacheManager``
* ``workloads`` - the seeded synthetic benchmark shapes
"""
from . import _lib  # noqa: F401

__all__ = ["ops", "kv_cache", "workloads"]
__version__ = "0.2.0"
