"""The CogVideoX-5B transformer around its blocks, following the reference's
``hetuDiTCogVideoXTransformer3DWrapper.forward`` (``models/transformers/cogvideox_transformer_3d.py:72-160``):
timestep embedding, patch embedding of text + video into one joint sequence, the blocks, ``norm_final`` over the
joint sequence, ``norm_out`` (AdaLayerNorm, shift first) + ``proj_out``, and the channel-major unpatchify."""
import torch
from torch import nn

from . import ops
from ._lib import eager_only
from .blocks import _adaln
from .layers.embeddings import hetuDiTCogVideoXPatchEmbedWrapper, project
from .layers.modules import AdaLayerNorm, CogVideoXPatchEmbed, TimestepEmbedding
from .transformer import CogVideoXTransformerBlocks


class CogVideoXTransformer3DModel(nn.Module):
    def __init__(self, num_attention_heads: int = 48, attention_head_dim: int = 64, in_channels: int = 16,
                 out_channels: int = 16, time_embed_dim: int = 512, text_embed_dim: int = 4096, num_layers: int = 42,
                 patch_size: int = 2):
        super().__init__()
        D = num_attention_heads * attention_head_dim
        self.inner_dim, self.patch_size, self.out_channels = D, patch_size, out_channels
        self.patch_embed = hetuDiTCogVideoXPatchEmbedWrapper(
            CogVideoXPatchEmbed(patch_size, in_channels, D, text_embed_dim))
        self.time_embedding = TimestepEmbedding(D, time_embed_dim)  # fed by the sinusoidal projection of width D
        object.__setattr__(self, "_runner", CogVideoXTransformerBlocks(num_layers, D, num_attention_heads,
                                                                       attention_head_dim, time_embed_dim))
        self.transformer_blocks = self._runner.transformer_blocks
        self.norm_final = nn.LayerNorm(D, eps=1e-5, elementwise_affine=True)
        self.norm_out = AdaLayerNorm(time_embed_dim, 2 * D, eps=1e-5)
        self.proj_out = nn.Linear(D, patch_size * patch_size * out_channels)

    def conditioning(self, timestep: torch.Tensor) -> torch.Tensor:
        """bf16 [B, time_embed_dim]: linear_2(silu(linear_1(sincos_D(t))))."""
        t_proj = ops.timestep_embedding(timestep.to(torch.float32), self.inner_dim)
        return project(ops.silu(project(t_proj, self.time_embedding.linear_1)), self.time_embedding.linear_2)

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, timestep: torch.Tensor,
                image_rotary_emb=None) -> torch.Tensor:
        """video latent bf16 [B, F, C, H, W], text states bf16 [B, N_t, text_dim], timestep [B], rotary table
        (cos, sin) f32 [F h w, head_dim] -> bf16 [B, F, C_out, H, W]."""
        B, F, _, H, W = hidden_states.shape
        n_txt = encoder_hidden_states.shape[1]
        emb = self.conditioning(timestep)
        joint = self.patch_embed(encoder_hidden_states, hidden_states)
        enc, hid = joint[:, :n_txt], joint[:, n_txt:]
        hid, enc = self._runner(hid, enc, emb, image_rotary_emb)
        # norm_final over cat([text, video]) is row-wise: only the video rows are kept, so only they are normalised
        nf = self.norm_final
        hid = ops.layernorm_modulate(hid.contiguous(), None, None, nf.eps, nf.weight.data, nf.bias.data)
        shift, scale = _adaln(self.norm_out, emb)  # AdaLayerNorm: shift first
        no = self.norm_out.norm
        hid = ops.layernorm_modulate(hid, shift, scale, no.eps, no.weight.data, no.bias.data)
        D = self.inner_dim
        x = project(hid.view(-1, D), self.proj_out).view(B * F, hid.shape[1] // F, -1)
        out = ops.unpatchify(x, self.out_channels, H, W, self.patch_size, channel_major=True)
        return out.view(B, F, self.out_channels, H, W)
