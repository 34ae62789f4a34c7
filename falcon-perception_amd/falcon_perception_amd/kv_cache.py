"""KV-cache interface the attention layers program against.

Mirrors the reference's `falcon_perception/kv_cache.py:12-31`: a cache owns the
`kv_cache` tensor and implements `insert_kv(layer_id, k, v, **kwargs)`, which
stores the new keys/values and returns the (K, V) the attention call should use.
"""

from __future__ import annotations

import abc

from torch import Tensor


class KVCacheBase(abc.ABC):
    """Base class of every KV cache (kv_cache.py:12-31 in the reference)."""

    kv_cache: Tensor | None

    @abc.abstractmethod
    def insert_kv(self, layer_id: int, k: Tensor, v: Tensor, **kwargs) -> tuple[Tensor, Tensor]:
        """Store k, v for `layer_id`; return the key/value tensors to attend over."""
        raise NotImplementedError
