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


def install(kv_rep: int = 1, qk_norm: bool = False, fuse_decode_append: bool = True) -> None:
    """Serve the reference's module names from this package.

    After `install()`, `import falcon_perception.paged_attention`,
    `falcon_perception.kv_cache` and `falcon_perception.attention` resolve to the
    modules here, so the reference's `model.py`, `paged_inference.py` and
    `paged_ocr_inference.py` bind these implementations at import time without
    any change to their source.  Call it before importing those modules.

    `kv_rep` = n_heads // n_kv_heads of the model to be served (2 for every variant of the
    reference, `falcon_perception/__init__.py:36-40`) tells every cache created afterwards that
    the V heads it is given are that many identical copies per kv head, which is what the
    reference's `repeat_kv` hands to `insert_kv` (`model.py:112-116`): decode then reads V once
    per group.  The engine builds its cache with `n_heads` heads (`paged_inference.py:321-330`)
    and never says so itself; left at 1, every cached head is read in full.

    `qk_norm=True` states that the model RMS-normalises q and k without a weight before the rotary
    embedding, as every variant of the reference does (`model.py:110-116`): |q| = |k| = sqrt(head_dim),
    so the attention scores are bounded and the bf16 prefill kernel runs its softmax without a running
    maximum (`score_bound` of `fp_paged_prefill`).  Leave it off for a model with learned norm weights.

    `fuse_decode_append` (default on): the decode `insert_kv` of the caches created afterwards hands its rows
    to the attention call that follows it in the reference's model (`model.py:150-162`), which appends and
    attends in one launch; `PagedKVCache.flush` and every other entry of the cache append them first.  Turn
    it off for a model that reads the pool views `insert_kv` returns by any other means than the attention
    callables of this package.
    """
    import sys

    if kv_rep < 1:
        raise ValueError("kv_rep must be at least 1")
    PagedKVCache.default_kv_rep = int(kv_rep)
    PagedKVCache.default_qk_normalised = bool(qk_norm)
    PagedKVCache.default_fuse_decode_append = bool(fuse_decode_append)
    sys.modules["falcon_perception.kv_cache"] = kv_cache
    sys.modules["falcon_perception.paged_attention"] = paged_attention
    sys.modules["falcon_perception.attention"] = attention
