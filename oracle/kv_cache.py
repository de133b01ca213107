"""Stale K/V buffer of one attention layer (test infrastructure, never shipped).

Restates ``CacheManager.update_and_get_kv_cache`` / ``_naive_cache_update`` /
``_update_kv_in_dim`` (``hetu_dit/core/resource_manager/cache_manager.py:64-149,
:208-231``) for one layer: K and V are packed on the last dim, kept whole when
patch mode is off (or there is one patch), and in patch mode the rows
``[start[patch], start[patch+1])`` along ``slice_dim`` are overwritten in place
while every other row keeps what an earlier call left there.
"""

from typing import List, Optional, Tuple

import torch


class StaleKVBuffer:
    def __init__(self):
        self.packed: Optional[torch.Tensor] = None
        self.patch_mode = False
        self.num_pipeline_patch = 1
        self.pipeline_patch_idx = 0
        self.pp_patches_token_start_idx_local: List[int] = [0]

    def set_patches(self, starts: List[int]):
        """starts has num_patches + 1 entries (``runtime_state.py:333-446``)."""
        self.pp_patches_token_start_idx_local = list(starts)
        self.num_pipeline_patch = len(starts) - 1

    def update_and_get(self, k: torch.Tensor, v: torch.Tensor, slice_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
        new_kv = torch.cat([k.float(), v.float()], dim=-1)
        if self.num_pipeline_patch == 1 or not self.patch_mode:
            self.packed = new_kv
        else:
            s = self.pp_patches_token_start_idx_local[self.pipeline_patch_idx]
            e = self.pp_patches_token_start_idx_local[self.pipeline_patch_idx + 1]
            index = [slice(None)] * self.packed.dim()
            index[slice_dim] = slice(s, e)
            self.packed[tuple(index)] = new_kv
        kk, vv = torch.chunk(self.packed, 2, dim=-1)
        return kk, vv
