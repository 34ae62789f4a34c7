"""MI355X-native paged KV-cache path of Falcon Perception.

Host-side mirror of the reference modules `falcon_perception.kv_cache`,
`falcon_perception.paged_attention` and `falcon_perception.attention`; the device
work is done by hand-written gfx950 kernels in libfp_paged_kv.so
(include/fp_paged_kv.h), reached through ctypes.
"""

from . import attention, kv_cache, ops, paged_attention  # noqa: F401
from .kv_cache import KVCacheBase  # noqa: F401
from .paged_attention import PagedKVCache  # noqa: F401

__all__ = ["KVCacheBase", "PagedKVCache", "attention", "kv_cache", "ops", "paged_attention", "install"]


def install() -> None:
    """Serve the reference's module names from this package.

    After `install()`, `import falcon_perception.paged_attention`,
    `falcon_perception.kv_cache` and `falcon_perception.attention` resolve to the
    modules here, so the reference's `model.py`, `paged_inference.py` and
    `paged_ocr_inference.py` bind these implementations at import time without
    any change to their source.  Call it before importing those modules.
    """
    import sys

    sys.modules["falcon_perception.kv_cache"] = kv_cache
    sys.modules["falcon_perception.paged_attention"] = paged_attention
    sys.modules["falcon_perception.attention"] = attention
