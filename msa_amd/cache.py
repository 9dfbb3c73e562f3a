"""State container of the MSA layer: per-layer pooled K / V / K_r plus the ``cache_kwargs`` dictionary
the layer reads its stage from and writes its compact cache into.  Same attribute and method names
as the reference's ``CustomDynamicCache`` (src/utils/cache.py:14-172) without the transformers base
class; pooled tensors are kept in the reference's ``[1, Hkv, C, D]`` view convention."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch


class CustomDynamicCache:
    def __init__(self):
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        self.router_key_cache: List[torch.Tensor] = []
        self.cache_kwargs: Dict[int, dict] = {}
        self.group_cache: dict = {}
        self.meta: dict = {}

    # -- metadata (cache.py:30-44)
    def record_kwargs(self, layer_idx: int, kwargs: dict) -> None:
        if layer_idx in self.cache_kwargs:
            self.cache_kwargs[layer_idx].update(kwargs)
        else:
            self.cache_kwargs[layer_idx] = kwargs

    def get_layer_length(self) -> int:
        return len(self.cache_kwargs)

    # -- pooled K / V (DynamicCache.update semantics: first write stores, later writes append on dim -2)
    @staticmethod
    def _put(store: List[torch.Tensor], t: Optional[torch.Tensor], layer_idx: int) -> Optional[torch.Tensor]:
        if t is None:
            return store[layer_idx] if layer_idx < len(store) else None
        while len(store) <= layer_idx:
            store.append(torch.tensor([]))
        store[layer_idx] = t if not store[layer_idx].numel() else torch.cat([store[layer_idx], t], dim=-2)
        return store[layer_idx]

    def update(self, key_states, value_states, layer_idx: int, cache_kwargs=None) -> Tuple[torch.Tensor, torch.Tensor]:
        return self._put(self.key_cache, key_states, layer_idx), self._put(self.value_cache, value_states, layer_idx)

    def update_router_kcache(self, key_states, layer_idx: int):
        return self._put(self.router_key_cache, key_states, layer_idx)

    def get_kvcache(self, layer_idx: int):
        return self.key_cache[layer_idx], self.value_cache[layer_idx]

    def get_router_kcache(self, layer_idx: int):
        if layer_idx < len(self.router_key_cache) and self.router_key_cache[layer_idx].numel():
            return self.router_key_cache[layer_idx]
        return None

    def get_seq_length(self, layer_idx: int = 0) -> int:
        if len(self.key_cache) <= layer_idx or not self.key_cache[layer_idx].numel():
            return 0
        return self.key_cache[layer_idx].shape[-2]

    def clear_kvcache(self) -> None:
        self.key_cache, self.value_cache = [], []

    def clear_query(self):
        for v in self.cache_kwargs.values():
            for name in ("compacked_key_cache", "compacked_value_cache", "prefill_stage2_kvcache_size",
                         "prefill_stage1_kvcache_size", "recall_topk", "kv_lengths", "attention_mask"):
                v.pop(name, None)
        return self


class CustomDynamicCacheOnCPU(CustomDynamicCache):
    """Moves everything it is given to host memory (src/utils/cache.py:139-172)."""

    @staticmethod
    def _host(t):
        return t.cpu() if (t is not None and torch.is_tensor(t) and t.is_cuda) else t

    def record_kwargs(self, layer_idx, kwargs):
        super().record_kwargs(layer_idx, {k: self._host(v) for k, v in kwargs.items()})

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        return super().update(self._host(key_states), self._host(value_states), layer_idx, cache_kwargs)

    def update_router_kcache(self, key_states, layer_idx):
        return super().update_router_kcache(self._host(key_states), layer_idx)


def create_cache() -> CustomDynamicCache:
    return CustomDynamicCache()


def compact_cache_reference_layout(key_cache: torch.Tensor, value_cache: torch.Tensor, kv_lengths: torch.Tensor):
    """The compact decode cache in the layout the reference keeps it in (src/msa/memory_sparse_attention.py:344-357):
    ``key / value [B, Hkv, maxL, D]`` left-padded with zeros and ``attention_mask [B, maxL]`` (True on the valid,
    right-aligned rows), ``maxL = kv_lengths.max()``.  This build keeps ``[B, Lcap, Hkv, D]`` with rows valid from 0
    and appends in place; code that reads ``cache_kwargs["compacked_key_cache"]`` in the reference's layout takes this
    copy instead (a conversion for outside readers: the attention kernels never need it)."""
    B, _, Hkv, D = key_cache.shape
    lens = kv_lengths.to(torch.int64)
    max_len = int(lens.max()) if B else 0
    pos = torch.arange(max_len, device=key_cache.device).unsqueeze(0)
    mask = pos >= (max_len - lens.unsqueeze(1))                                   # [B, maxL]
    src = (pos - (max_len - lens.unsqueeze(1))).clamp(min=0)                      # row of the cache a position holds
    out = []
    for cache in (key_cache, value_cache):
        rows = torch.gather(cache[:, :max(max_len, 1)] if max_len else cache[:, :0], 1,
                            src.view(B, max_len, 1, 1).expand(B, max_len, Hkv, D)) if max_len else cache[:, :0]
        rows = rows * mask.view(B, max_len, 1, 1).to(rows.dtype)
        out.append(rows.permute(0, 2, 1, 3).contiguous())
    return out[0], out[1], mask
