"""Block-loop callers: the part of the reference's transformer wrappers'
``forward`` that sits between the embedders and ``norm_out`` -- "for block in
blocks" with each model family's call convention and patch-mode rules.

* SD3 (``models/transformers/transformer_sd3.py:107-152``): in patch mode,
  patch 0 stores every block's *input* text states; later patches feed those
  back and drop the block's text output.
* Flux (``transformer_flux.py:133-201``): double blocks, then
  ``cat([text, image])``, single blocks on the joint sequence, split.
* CogVideoX (``cogvideox_transformer_3d.py:99-127``).
"""
from typing import List, Optional, Tuple

import torch
from torch import nn

from .blocks import (CogVideoXBlock, FluxSingleTransformerBlock, FluxTransformerBlock, JointTransformerBlock,
                     StackModulation, use_fp32_residual_stream)
from .runtime_state import get_runtime_state


class SD3TransformerBlocks(nn.Module):
    def __init__(self, num_layers: int = 24, dim: int = 1536, num_attention_heads: int = 24,
                 attention_head_dim: int = 64):
        super().__init__()
        self.transformer_blocks = nn.ModuleList(
            [
                JointTransformerBlock(dim, num_attention_heads, attention_head_dim,
                                      context_pre_only=(i == num_layers - 1))
                for i in range(num_layers)
            ]
        )
        self.encoder_hidden_states_cache: List[Optional[torch.Tensor]] = [None] * num_layers
        self.modulation = StackModulation(self.transformer_blocks)
        use_fp32_residual_stream(self.transformer_blocks)

    @torch.no_grad()
    def forward(self, hidden_states, encoder_hidden_states, temb):
        rs = get_runtime_state()
        self.modulation.precompute(temb)
        for i, block in enumerate(self.transformer_blocks):
            if rs.patch_mode and rs.pipeline_patch_idx == 0:
                self.encoder_hidden_states_cache[i] = encoder_hidden_states
                encoder_hidden_states, hidden_states = block(
                    hidden_states=hidden_states, encoder_hidden_states=encoder_hidden_states, temb=temb
                )
            elif rs.patch_mode:
                # the text output of these calls is dropped: the block does not compute it
                _, hidden_states = block(
                    hidden_states=hidden_states, encoder_hidden_states=self.encoder_hidden_states_cache[i], temb=temb,
                    skip_text_output=True,
                )
            else:
                encoder_hidden_states, hidden_states = block(
                    hidden_states=hidden_states, encoder_hidden_states=encoder_hidden_states, temb=temb
                )
        return hidden_states


class FluxTransformerBlocks(nn.Module):
    def __init__(self, num_layers: int = 19, num_single_layers: int = 38, dim: int = 3072,
                 num_attention_heads: int = 24, attention_head_dim: int = 128):
        super().__init__()
        self.transformer_blocks = nn.ModuleList(
            [FluxTransformerBlock(dim, num_attention_heads, attention_head_dim) for _ in range(num_layers)]
        )
        self.single_transformer_blocks = nn.ModuleList(
            [FluxSingleTransformerBlock(dim, num_attention_heads, attention_head_dim) for _ in range(num_single_layers)]
        )
        self.modulation = StackModulation(list(self.transformer_blocks) + list(self.single_transformer_blocks))
        use_fp32_residual_stream(list(self.transformer_blocks) + list(self.single_transformer_blocks))

    @torch.no_grad()
    def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb):
        self.modulation.precompute(temb)
        for block in self.transformer_blocks:
            encoder_hidden_states, hidden_states = block(
                hidden_states=hidden_states, encoder_hidden_states=encoder_hidden_states, temb=temb,
                image_rotary_emb=image_rotary_emb,
            )
        n_txt = encoder_hidden_states.shape[1]
        hidden_states = torch.cat([encoder_hidden_states, hidden_states], dim=1)
        for block in self.single_transformer_blocks:
            hidden_states = block(hidden_states=hidden_states, temb=temb, image_rotary_emb=image_rotary_emb)
        encoder_hidden_states = hidden_states[:, :n_txt, ...]
        hidden_states = hidden_states[:, n_txt:, ...]
        return hidden_states, encoder_hidden_states


class CogVideoXTransformerBlocks(nn.Module):
    def __init__(self, num_layers: int = 42, dim: int = 3072, num_attention_heads: int = 48,
                 attention_head_dim: int = 64, time_embed_dim: int = 512):
        super().__init__()
        self.transformer_blocks = nn.ModuleList(
            [CogVideoXBlock(dim, num_attention_heads, attention_head_dim, time_embed_dim) for _ in range(num_layers)]
        )
        self.modulation = StackModulation(self.transformer_blocks)
        use_fp32_residual_stream(self.transformer_blocks)

    @torch.no_grad()
    def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None) -> Tuple[torch.Tensor, torch.Tensor]:
        self.modulation.precompute(temb)
        for block in self.transformer_blocks:
            hidden_states, encoder_hidden_states = block(
                hidden_states=hidden_states, encoder_hidden_states=encoder_hidden_states, temb=temb,
                image_rotary_emb=image_rotary_emb,
            )
        return hidden_states, encoder_hidden_states
