"""The SD3 transformer around the block stack: what the reference's ``hetuDiTSD3Transformer2DWrapper.forward``
does between the latent and the predicted noise (``models/transformers/transformer_sd3.py:92-185``) --
patch embedding with position table, timestep + pooled-text conditioning, context projection, the joint
blocks, ``norm_out`` / ``proj_out`` and unpatchify -- plus the guidance and scheduler update that follow it in
the pipeline (``pipeline_stable_diffusion_3.py:1703-1713``,
``schedulers/scheduling_flow_match_euler_discrete.py:74-118``).  Every projection is a launch of the grouped
GEMM; the small glue steps have their own kernels (``csrc/embed.hip``)."""
import torch
from torch import nn

from . import ops
from ._lib import eager_only
from .layers.embeddings import conditioning_embedding, hetuDiTPatchEmbedWrapper, norm_out_project, project
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

    def conditioning(self, timestep: torch.Tensor, pooled_projections: torch.Tensor) -> torch.Tensor:
        return conditioning_embedding(self.time_text_embed, timestep, pooled_projections)

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, pooled_projections: torch.Tensor,
                timestep: torch.Tensor) -> torch.Tensor:
        """latent bf16 [B, C, H, W], text states bf16 [B, N_t, joint_dim], pooled bf16 [B, pooled_dim], timestep
        f32 [B] -> predicted noise bf16 [B, C_out, H, W]."""
        B, _, H, W = hidden_states.shape
        tokens = self.pos_embed(hidden_states)
        temb = self.conditioning(timestep, pooled_projections)
        enc = encoder_hidden_states.contiguous()
        enc = project(enc.view(-1, enc.shape[-1]), self.context_embedder).view(B, enc.shape[1], -1)
        tokens = self._runner(tokens, enc, temb)
        x = norm_out_project(self.norm_out, self.proj_out, tokens, temb)
        return ops.unpatchify(x, self.out_channels, H, W, self.patch_size)

    @torch.no_grad()
    @eager_only
    def denoise_step(self, latents: torch.Tensor, encoder_hidden_states: torch.Tensor, pooled_projections: torch.Tensor,
                     timestep: torch.Tensor, guidance_scale: float, sigma: float, sigma_next: float) -> torch.Tensor:
        """One guided step on one GPU: the CFG pair as a batch of two per latent (unconditional first, as
        ``noise_pred.chunk(2)`` expects), guidance and the Euler update fused in one kernel."""
        n = latents.shape[0]
        noise = self.forward(torch.cat([latents, latents], 0), encoder_hidden_states, pooled_projections,
                             timestep.expand(2 * n) if timestep.numel() == 1 else timestep)
        return ops.cfg_euler_step(noise[:n].contiguous(), noise[n:].contiguous(), latents.contiguous(), guidance_scale, sigma,
                                  sigma_next)
