"""The Flux transformer around its double- and single-stream blocks, following the reference's
``hetuDiTFluxTransformer2DWrapper.forward`` (``models/transformers/transformer_flux.py:101-207``): ``x_embedder``,
the timestep (+ guidance) + pooled-text conditioning on ``timestep * 1000``, ``context_embedder``, the rotary
table from ``cat(txt_ids, img_ids)``, the blocks, ``norm_out`` and ``proj_out``.  The latent arrives packed as
tokens ([B, N_img, 64]); packing is the pipeline's business."""
from typing import Optional

import torch
from torch import nn

from . import ops
from ._lib import eager_only
from .layers.embeddings import conditioning_embedding, norm_out_project, project
from .layers.modules import (AdaLayerNormContinuous, CombinedTimestepGuidanceTextProjEmbeddings,
                             CombinedTimestepTextProjEmbeddings, FluxPosEmbed)
from .runtime_state import get_runtime_state
from .transformer import FluxTransformerBlocks


class FluxTransformer2DModel(nn.Module):
    def __init__(self, patch_size: int = 1, in_channels: int = 64, num_layers: int = 19, num_single_layers: int = 38,
                 attention_head_dim: int = 128, num_attention_heads: int = 24, joint_attention_dim: int = 4096,
                 pooled_projection_dim: int = 768, guidance_embeds: bool = True, axes_dims_rope=(16, 56, 56)):
        super().__init__()
        D = num_attention_heads * attention_head_dim
        if sum(axes_dims_rope) != attention_head_dim:
            raise ValueError(f"rotary axes {tuple(axes_dims_rope)} do not add up to the head dim {attention_head_dim}")
        self.inner_dim, self.out_channels = D, in_channels
        self.pos_embed = FluxPosEmbed(10000.0, axes_dims_rope)
        embed_cls = CombinedTimestepGuidanceTextProjEmbeddings if guidance_embeds else CombinedTimestepTextProjEmbeddings
        self.time_text_embed = embed_cls(D, pooled_projection_dim)
        self.context_embedder = nn.Linear(joint_attention_dim, D)
        self.x_embedder = nn.Linear(in_channels, D)
        # the block runner stays off the module tree: parameter paths are ``transformer_blocks.N...`` /
        # ``single_transformer_blocks.N...``
        object.__setattr__(self, "_runner", FluxTransformerBlocks(num_layers, num_single_layers, D, num_attention_heads,
                                                                  attention_head_dim))
        self.transformer_blocks = self._runner.transformer_blocks
        self.single_transformer_blocks = self._runner.single_transformer_blocks
        self.norm_out = AdaLayerNormContinuous(D, D, eps=1e-6)
        self.proj_out = nn.Linear(D, patch_size * patch_size * self.out_channels)

    def conditioning(self, timestep: torch.Tensor, pooled_projections: torch.Tensor,
                     guidance: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The reference scales in the model's dtype: ``timestep.to(bf16) * 1000`` (and the same for guidance)."""
        t = timestep.to(torch.bfloat16) * 1000
        if isinstance(self.time_text_embed, CombinedTimestepGuidanceTextProjEmbeddings):
            if guidance is None:
                raise ValueError("this model embeds the guidance scale: pass guidance")
            g = guidance.to(torch.bfloat16) * 1000
        else:
            g = None
        return conditioning_embedding(self.time_text_embed, t, pooled_projections, g)

    def rotary_table(self, txt_ids: torch.Tensor, img_ids: torch.Tensor):
        if txt_ids.dim() == 3:
            txt_ids = txt_ids[0]
        if img_ids.dim() == 3:
            img_ids = img_ids[0]
        ids = torch.cat((txt_ids, img_ids), dim=0).to(torch.float32).contiguous()
        return ops.rope_table(ids, self.pos_embed.axes_dim, self.pos_embed.theta)

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, pooled_projections: torch.Tensor,
                timestep: torch.Tensor, img_ids: torch.Tensor, txt_ids: torch.Tensor,
                guidance: Optional[torch.Tensor] = None) -> torch.Tensor:
        """packed latent bf16 [B, N_img, C], text states bf16 [B, N_txt, joint_dim], pooled bf16 [B, pooled_dim],
        timestep / guidance [B] (timestep in [0, 1]), ids [N, 3] -> bf16 [B, N_img, C]."""
        B, n_img, _ = hidden_states.shape
        n_txt = encoder_hidden_states.shape[1]
        get_runtime_state().max_condition_sequence_length = n_txt
        x = hidden_states.contiguous()
        x = project(x.view(B * n_img, -1), self.x_embedder).view(B, n_img, -1)
        temb = self.conditioning(timestep, pooled_projections, guidance)
        enc = encoder_hidden_states.contiguous()
        enc = project(enc.view(B * n_txt, -1), self.context_embedder).view(B, n_txt, -1)
        rope = self.rotary_table(txt_ids, img_ids)
        x, _ = self._runner(x, enc, temb, rope)
        return norm_out_project(self.norm_out, self.proj_out, x.contiguous(), temb)
