"""The SD3 transformer around the block stack: what the reference's ``hetuDiTSD3Transformer2DWrapper.forward``
does between the latent and the predicted noise (``models/transformers/transformer_sd3.py:92-185``) --
patch embedding with position table, timestep + pooled-text conditioning, context projection, the joint
blocks, ``norm_out`` / ``proj_out`` and unpatchify -- plus the guidance and scheduler update that follow it in
the pipeline (``pipeline_stable_diffusion_3.py:1703-1713``,
``schedulers/scheduling_flow_match_euler_discrete.py:74-118``).  Every projection is a launch of the grouped
GEMM; the small glue steps have their own kernels (``csrc/embed.hip``)."""
from typing import Optional

import torch
from torch import nn

from . import ops
from .blocks import _adaln
from .layers.embeddings import hetuDiTPatchEmbedWrapper
from .layers.modules import AdaLayerNormContinuous, CombinedTimestepTextProjEmbeddings, PatchEmbed
from .transformer import SD3TransformerBlocks


class SD3Transformer2DModel(nn.Module):
    def __init__(self, sample_size: int = 128, patch_size: int = 2, in_channels: int = 16, num_layers: int = 24,
                 attention_head_dim: int = 64, num_attention_heads: int = 24, joint_attention_dim: int = 4096,
                 caption_projection_dim: int = 1536, pooled_projection_dim: int = 2048, out_channels: int = 16,
                 pos_embed_max_size: int = 192):
        super().__init__()
        D = num_attention_heads * attention_head_dim
        self.inner_dim, self.patch_size, self.out_channels = D, patch_size, out_channels
        self.pos_embed = hetuDiTPatchEmbedWrapper(
            PatchEmbed(sample_size, sample_size, patch_size, in_channels, D, pos_embed_max_size))
        self.time_text_embed = CombinedTimestepTextProjEmbeddings(D, pooled_projection_dim)
        self.context_embedder = nn.Linear(joint_attention_dim, caption_projection_dim)
        # the block runner is kept off the module tree so that parameter paths stay ``transformer_blocks.N...``
        object.__setattr__(self, "_runner", SD3TransformerBlocks(num_layers, D, num_attention_heads, attention_head_dim))
        self.transformer_blocks = self._runner.transformer_blocks
        self.norm_out = AdaLayerNormContinuous(D, D, eps=1e-6)
        self.proj_out = nn.Linear(D, patch_size * patch_size * out_channels)
        self._ones: Optional[torch.Tensor] = None

    def _linear(self, x2: torch.Tensor, lin: nn.Linear, **epilogue) -> torch.Tensor:
        out = torch.empty(x2.shape[0], lin.weight.shape[0], dtype=torch.bfloat16, device=x2.device)
        ops.gemm_launch([ops.gemm_problem(x2, lin.weight.data, out, lin.bias.data, **epilogue)])
        return out

    def conditioning(self, timestep: torch.Tensor, pooled_projections: torch.Tensor) -> torch.Tensor:
        """bf16 [B, D]: timestep_embedder(sincos(t)) + text_embedder(pooled); the sum rides the last GEMM's
        residual epilogue."""
        tte = self.time_text_embed
        B = timestep.shape[0]
        if self._ones is None or self._ones.device != timestep.device:
            self._ones = torch.ones(1, self.inner_dim, dtype=torch.float32, device=timestep.device)
        t_proj = ops.timestep_embedding(timestep.to(torch.float32), tte.frequency_dim)
        t_emb = self._linear(ops.silu(self._linear(t_proj, tte.timestep_embedder.linear_1)), tte.timestep_embedder.linear_2)
        h = ops.silu(self._linear(pooled_projections.contiguous(), tte.text_embedder.linear_1))
        return self._linear(h, tte.text_embedder.linear_2, epilogue=ops.EPI_GATE_RESIDUAL, resid=t_emb, gate=self._ones,
                            rows_per_batch=B)

    @torch.no_grad()
    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, pooled_projections: torch.Tensor,
                timestep: torch.Tensor) -> torch.Tensor:
        """latent bf16 [B, C, H, W], text states bf16 [B, N_t, joint_dim], pooled bf16 [B, pooled_dim], timestep
        f32 [B] -> predicted noise bf16 [B, C_out, H, W]."""
        B, _, H, W = hidden_states.shape
        tokens = self.pos_embed(hidden_states)
        temb = self.conditioning(timestep, pooled_projections)
        enc = encoder_hidden_states.contiguous()
        enc = self._linear(enc.view(-1, enc.shape[-1]), self.context_embedder).view(B, enc.shape[1], -1)
        tokens = self._runner(tokens, enc, temb)
        scale, shift = _adaln(self.norm_out, temb)  # AdaLayerNormContinuous: scale first
        x = ops.layernorm_modulate(tokens, shift, scale, self.norm_out.norm.eps)
        x = self._linear(x.view(-1, self.inner_dim), self.proj_out).view(B, tokens.shape[1], -1)
        return ops.unpatchify(x, self.out_channels, H, W, self.patch_size)

    @torch.no_grad()
    def denoise_step(self, latents: torch.Tensor, encoder_hidden_states: torch.Tensor, pooled_projections: torch.Tensor,
                     timestep: torch.Tensor, guidance_scale: float, sigma: float, sigma_next: float) -> torch.Tensor:
        """One guided step on one GPU: the CFG pair as a batch of two per latent (unconditional first, as
        ``noise_pred.chunk(2)`` expects), guidance and the Euler update fused in one kernel."""
        n = latents.shape[0]
        noise = self.forward(torch.cat([latents, latents], 0), encoder_hidden_states, pooled_projections,
                             timestep.expand(2 * n) if timestep.numel() == 1 else timestep)
        return ops.cfg_euler_step(noise[:n].contiguous(), noise[n:].contiguous(), latents.contiguous(), guidance_scale, sigma,
                                  sigma_next)
