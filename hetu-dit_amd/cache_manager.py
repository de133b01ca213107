"""Per-attention-layer stale K/V buffer.

Same surface as the reference's ``CacheManager``
(``hetu_dit/core/resource_manager/cache_manager.py:38-254``):
``register_cache_entry(layer, "attn", cache_type)`` at wrap time,
``update_and_get_kv_cache(new_kv=[k, v], layer=, slice_dim=, layer_type="attn")``
per call, keyed by the layer object.  K and V are packed on the last dim; with
patch mode off (or a single patch) the packed tensor replaces the entry, in
patch mode the rows of the current patch are overwritten in place and every
other row keeps what an earlier call left (``:117-149,:208-231``).  The two
returned tensors are strided views of the packed buffer (``:113``).

The fused blocks do not go through ``update_and_get_kv_cache``: they ask for
the packed buffer with ``kv_buffer`` and let the K|V projection GEMM write its
rows directly, which is the same state transition without the two copies.
"""
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from . import ops
from .runtime_state import get_runtime_state, runtime_state_is_initialized


class CacheEntry:
    def __init__(self, cache_type: str, num_cache_tensors: int = 1):
        self.cache_type = cache_type
        self.tensors: List[Optional[torch.Tensor]] = [None] * num_cache_tensors


class CacheManager:
    supported_layer = ["attn"]
    supported_cache_type = ["naive_cache", "sequence_parallel_attn_cache"]

    def __init__(self):
        self.cache: Dict[Tuple[str, Any], CacheEntry] = {}

    def register_cache_entry(self, layer, layer_type: str, cache_type: str = "naive_cache"):
        if layer_type not in self.supported_layer:
            raise ValueError(
                f"Layer type: {layer_type} is not supported. Supported layer type: {self.supported_layer}"
            )
        if cache_type not in self.supported_cache_type:
            raise ValueError(
                f"Cache type: {cache_type} is not supported. Supported cache type: {self.supported_cache_type}"
            )
        self.cache[layer_type, layer] = CacheEntry(cache_type)

    # -- state helpers ---------------------------------------------------------
    @staticmethod
    def _patch_range() -> Optional[Tuple[int, int]]:
        """None when the whole sequence is (re)written, else the token range of
        the current patch (cache_manager.py:126-140)."""
        if not runtime_state_is_initialized():
            return None
        rs = get_runtime_state()
        if rs.num_pipeline_patch == 1 or not rs.patch_mode:
            return None
        starts = rs.pp_patches_token_start_idx_local
        return starts[rs.pipeline_patch_idx], starts[rs.pipeline_patch_idx + 1]

    def _entry(self, layer, layer_type: str) -> CacheEntry:
        entry = self.cache.get((layer_type, layer))
        if entry is None:
            raise KeyError("no cache entry registered for this layer; call register_cache_entry at wrap time")
        return entry

    # -- reference-shaped API ----------------------------------------------------
    def update_and_get_kv_cache(
        self,
        new_kv: Union[torch.Tensor, List[torch.Tensor]],
        layer: Any,
        slice_dim: int = 1,
        layer_type: str = "attn",
        **kwargs,
    ):
        return_list = isinstance(new_kv, (list, tuple))
        if return_list:
            k, v = new_kv
            inner = k.shape[-1]
            packed_new = torch.empty(*k.shape[:-1], 2 * inner, dtype=k.dtype, device=k.device)
            self._copy(k, packed_new[..., :inner])
            self._copy(v, packed_new[..., inner:])
            new_kv = packed_new
        entry = self._entry(layer, layer_type)
        rng = self._patch_range()
        if rng is None:
            entry.tensors[0] = new_kv
        else:
            if entry.tensors[0] is None:
                raise RuntimeError("patch-mode KV update before a full-sequence pass filled the buffer")
            index = [slice(None)] * entry.tensors[0].dim()
            index[slice_dim] = slice(rng[0], rng[1])
            self._copy(new_kv, entry.tensors[0][tuple(index)])
        kv_cache = entry.tensors[0]
        if return_list:
            return torch.chunk(kv_cache, 2, dim=-1)
        return kv_cache

    @staticmethod
    def _copy(src: torch.Tensor, dst: torch.Tensor):
        """Strided row copy on the HIP kernel ([.., T, D] views, unit inner stride)."""
        s3 = src.reshape(-1, src.shape[-2], src.shape[-1]) if src.dim() != 3 else src
        d3 = dst
        if dst.dim() == 4:  # [B, H, T, 2d] layout: fold (B, H) only when it is a single stride
            if dst.stride(0) == dst.shape[1] * dst.stride(1) and src.is_contiguous():
                d3 = dst.as_strided((dst.shape[0] * dst.shape[1], dst.shape[2], dst.shape[3]),
                                    (dst.stride(1), dst.stride(2), 1))
                s3 = src.reshape(-1, src.shape[-2], src.shape[-1])
            else:
                for b in range(dst.shape[0]):
                    ops.copy_rows(src[b], dst[b])
                return
        ops.copy_rows(s3, d3)

    # -- fused-path API ------------------------------------------------------------
    def kv_buffer(self, layer, batch: int, tokens: int, inner: int, device, layer_type: str = "attn"):
        """Packed [batch, tokens, 2*inner] buffer the K|V projection writes into,
        and the row range to write: ``(buffer, start, end)``.  With patch mode
        off a fresh buffer of ``tokens`` rows replaces the entry; in patch mode
        the persistent buffer is returned with the current patch's range."""
        entry = self._entry(layer, layer_type)
        rng = self._patch_range()
        if rng is None:
            buf = torch.empty(batch, tokens, 2 * inner, dtype=torch.bfloat16, device=device)
            entry.tensors[0] = buf
            return buf, 0, tokens
        buf = entry.tensors[0]
        if buf is None:
            raise RuntimeError("patch-mode KV update before a full-sequence pass filled the buffer")
        if rng[1] - rng[0] != tokens or buf.shape[0] != batch or buf.shape[2] != 2 * inner:
            raise ValueError(
                f"patch of {tokens} tokens does not match the runtime state's range {rng} / buffer {tuple(buf.shape)}"
            )
        return buf, rng[0], rng[1]

    def _reset_cache(self):
        self.cache = {}


_CACHE_MGR = CacheManager()


def get_cache_manager() -> CacheManager:
    return _CACHE_MGR


def reset_cache_manager():
    _CACHE_MGR._reset_cache()
