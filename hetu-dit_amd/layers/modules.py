"""Parameter containers with the module structure and parameter names of the
third-party (diffusers) layers the reference wraps -- ``Attention``,
``FeedForward``/``GELU``, ``AdaLayerNormZero`` and friends, ``RMSNorm`` -- plus
marker classes for the attention processors the reference's registry keys on
(``layers/attention_processor.py:9-16``).  diffusers itself is not a dependency:
only the attribute names the reference's wrappers, weight hot-swap
(``hetu_dit/utils.py:561-582``) and block call sites rely on are reproduced.
None of these modules computes anything; computation lives in the wrappers and
blocks, on the HIP kernels."""
from typing import Optional

import torch
from torch import nn


class JointAttnProcessor2_0:
    """Marker for the SD3 joint attention processor."""


class FluxAttnProcessor2_0:
    """Marker for the Flux attention processor."""


class CogVideoXAttnProcessor2_0:
    """Marker for the CogVideoX attention processor."""


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float, elementwise_affine: bool = True):
        super().__init__()
        self.eps = eps
        self.dim = dim
        self.weight = nn.Parameter(torch.ones(dim)) if elementwise_affine else None


class Attention(nn.Module):
    def __init__(
        self,
        query_dim: int,
        heads: int,
        dim_head: int,
        added_kv_proj_dim: Optional[int] = None,
        bias: bool = True,
        out_bias: bool = True,
        context_pre_only: Optional[bool] = None,
        pre_only: bool = False,
        qk_norm: Optional[str] = None,
        eps: float = 1e-6,
        processor=None,
    ):
        super().__init__()
        self.inner_dim = heads * dim_head
        self.query_dim = query_dim
        self.heads = heads
        self.dim_head = dim_head
        self.scale = dim_head ** -0.5
        self.context_pre_only = context_pre_only
        self.pre_only = pre_only
        self.added_kv_proj_dim = added_kv_proj_dim
        self.is_cross_attention = False
        self.to_q = nn.Linear(query_dim, self.inner_dim, bias=bias)
        self.to_k = nn.Linear(query_dim, self.inner_dim, bias=bias)
        self.to_v = nn.Linear(query_dim, self.inner_dim, bias=bias)
        if qk_norm is None:
            self.norm_q = self.norm_k = None
        elif qk_norm == "rms_norm":
            self.norm_q = RMSNorm(dim_head, eps=eps)
            self.norm_k = RMSNorm(dim_head, eps=eps)
        elif qk_norm == "layer_norm":
            self.norm_q = nn.LayerNorm(dim_head, eps=eps)
            self.norm_k = nn.LayerNorm(dim_head, eps=eps)
        else:
            raise ValueError(f"unknown qk_norm: {qk_norm}")
        self.norm_added_q = self.norm_added_k = None
        if added_kv_proj_dim is not None:
            self.add_q_proj = nn.Linear(added_kv_proj_dim, self.inner_dim, bias=bias)
            self.add_k_proj = nn.Linear(added_kv_proj_dim, self.inner_dim, bias=bias)
            self.add_v_proj = nn.Linear(added_kv_proj_dim, self.inner_dim, bias=bias)
            if qk_norm == "rms_norm":
                self.norm_added_q = RMSNorm(dim_head, eps=eps)
                self.norm_added_k = RMSNorm(dim_head, eps=eps)
        if not pre_only:
            self.to_out = nn.ModuleList([nn.Linear(self.inner_dim, query_dim, bias=out_bias), nn.Dropout(0.0)])
        if context_pre_only is not None and not context_pre_only:
            self.to_add_out = nn.Linear(self.inner_dim, query_dim, bias=out_bias)
        self.processor = processor


class GELU(nn.Module):
    def __init__(self, dim_in: int, dim_out: int, approximate: str = "tanh", bias: bool = True):
        super().__init__()
        self.proj = nn.Linear(dim_in, dim_out, bias=bias)
        self.approximate = approximate


class GEGLU(nn.Module):
    """``proj`` to twice the width; value half times exact GELU of the gate half."""

    def __init__(self, dim_in: int, dim_out: int, bias: bool = True):
        super().__init__()
        self.proj = nn.Linear(dim_in, dim_out * 2, bias=bias)


class LinearActivation(nn.Module):
    """``proj`` followed by SiLU."""

    def __init__(self, dim_in: int, dim_out: int, bias: bool = True, activation: str = "silu"):
        super().__init__()
        if activation != "silu":
            raise ValueError("LinearActivation: only 'silu' is built")
        self.proj = nn.Linear(dim_in, dim_out, bias=bias)
        self.activation = activation


class FeedForward(nn.Module):
    """``net = [activation(proj), Dropout, Linear]``; ``activation_fn`` as in diffusers: "gelu-approximate" (what
    every model here uses), "gelu", "geglu", "linear-silu"."""

    def __init__(self, dim: int, dim_out: Optional[int] = None, mult: int = 4, inner_dim: Optional[int] = None,
                 bias: bool = True, activation_fn: str = "gelu-approximate"):
        super().__init__()
        inner_dim = inner_dim or dim * mult
        dim_out = dim_out or dim
        if activation_fn == "gelu-approximate":
            act = GELU(dim, inner_dim, approximate="tanh", bias=bias)
        elif activation_fn == "gelu":
            act = GELU(dim, inner_dim, approximate="none", bias=bias)
        elif activation_fn == "geglu":
            act = GEGLU(dim, inner_dim, bias=bias)
        elif activation_fn == "linear-silu":
            act = LinearActivation(dim, inner_dim, bias=bias)
        else:
            raise ValueError(f"activation_fn {activation_fn!r} is not built")
        self.net = nn.ModuleList([act, nn.Dropout(0.0), nn.Linear(inner_dim, dim_out, bias=bias)])


class AdaLayerNormZero(nn.Module):
    """emb -> (shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp)."""

    chunks = 6

    def __init__(self, embedding_dim: int):
        super().__init__()
        self.silu = nn.SiLU()
        self.linear = nn.Linear(embedding_dim, 6 * embedding_dim, bias=True)
        self.norm = nn.LayerNorm(embedding_dim, elementwise_affine=False, eps=1e-6)


class AdaLayerNormZeroSingle(nn.Module):
    """emb -> (shift, scale, gate)."""

    chunks = 3

    def __init__(self, embedding_dim: int):
        super().__init__()
        self.silu = nn.SiLU()
        self.linear = nn.Linear(embedding_dim, 3 * embedding_dim, bias=True)
        self.norm = nn.LayerNorm(embedding_dim, elementwise_affine=False, eps=1e-6)


class AdaLayerNormContinuous(nn.Module):
    """emb -> (scale, shift)  -- scale first."""

    chunks = 2

    def __init__(self, embedding_dim: int, conditioning_embedding_dim: int, eps: float = 1e-6):
        super().__init__()
        self.silu = nn.SiLU()
        self.linear = nn.Linear(conditioning_embedding_dim, 2 * embedding_dim, bias=True)
        self.norm = nn.LayerNorm(embedding_dim, elementwise_affine=False, eps=eps)


class CogVideoXLayerNormZero(nn.Module):
    """emb -> (shift, scale, gate, enc_shift, enc_scale, enc_gate); one affine LayerNorm for both streams."""

    chunks = 6

    def __init__(self, conditioning_dim: int, embedding_dim: int, eps: float = 1e-5):
        super().__init__()
        self.silu = nn.SiLU()
        self.linear = nn.Linear(conditioning_dim, 6 * embedding_dim, bias=True)
        self.norm = nn.LayerNorm(embedding_dim, eps=eps, elementwise_affine=True)


def sincos_pos_embed_2d(embed_dim: int, grid_size: int, base_size: int, interpolation_scale: float = 1.0) -> torch.Tensor:
    """diffusers ``get_2d_sincos_pos_embed``: [grid_size^2, embed_dim] fp32, first half of the channels from
    the column coordinate, second half from the row coordinate, each [sin | cos] of pos * 10000^(-2i/d);
    positions are scaled by base_size / grid_size."""
    coord = torch.arange(grid_size, dtype=torch.float64) * (base_size / grid_size) / interpolation_scale
    omega = 1.0 / 10000.0 ** (torch.arange(embed_dim // 4, dtype=torch.float64) / (embed_dim / 4.0))

    def one_axis(pos):
        ang = pos.reshape(-1)[:, None] * omega[None]
        return torch.cat([ang.sin(), ang.cos()], dim=1)

    cols = coord[None, :].expand(grid_size, grid_size)
    rows = coord[:, None].expand(grid_size, grid_size)
    return torch.cat([one_axis(cols), one_axis(rows)], dim=1).float()


class PatchEmbed(nn.Module):
    """diffusers ``PatchEmbed`` as SD3 configures it: p x p stride-p convolution, flatten, and a fixed sin-cos
    position table of ``pos_embed_max_size``^2 entries that is centre-cropped to the latent's token grid."""

    def __init__(self, height: int = 128, width: int = 128, patch_size: int = 2, in_channels: int = 16,
                 embed_dim: int = 1536, pos_embed_max_size: int = 192):
        super().__init__()
        self.patch_size, self.height, self.width = patch_size, height // patch_size, width // patch_size
        self.base_size = height // patch_size
        self.pos_embed_max_size = pos_embed_max_size
        self.flatten, self.layer_norm = True, False
        self.proj = nn.Conv2d(in_channels, embed_dim, kernel_size=patch_size, stride=patch_size, bias=True)
        table = sincos_pos_embed_2d(embed_dim, pos_embed_max_size, self.base_size)
        self.register_buffer("pos_embed", table[None], persistent=True)

    def cropped_pos_embed(self, height: int, width: int) -> torch.Tensor:
        """[1, tokens, D] centre crop of the table for a latent of height x width pixels."""
        height, width = height // self.patch_size, width // self.patch_size
        m = self.pos_embed_max_size
        if height > m or width > m:
            raise ValueError(f"token grid {height}x{width} exceeds pos_embed_max_size {m}")
        top, left = (m - height) // 2, (m - width) // 2
        t = self.pos_embed.reshape(1, m, m, -1)[:, top : top + height, left : left + width]
        return t.reshape(1, height * width, -1)


class TimestepEmbedding(nn.Module):
    def __init__(self, in_channels: int, time_embed_dim: int):
        super().__init__()
        self.linear_1 = nn.Linear(in_channels, time_embed_dim)
        self.act = nn.SiLU()
        self.linear_2 = nn.Linear(time_embed_dim, time_embed_dim)


class PixArtAlphaTextProjection(nn.Module):
    def __init__(self, in_features: int, hidden_size: int):
        super().__init__()
        self.linear_1 = nn.Linear(in_features, hidden_size)
        self.act_1 = nn.SiLU()
        self.linear_2 = nn.Linear(hidden_size, hidden_size)


class CombinedTimestepTextProjEmbeddings(nn.Module):
    """temb = timestep_embedder(sincos_256(t)) + text_embedder(pooled_projection)."""

    def __init__(self, embedding_dim: int, pooled_projection_dim: int, frequency_dim: int = 256):
        super().__init__()
        self.frequency_dim = frequency_dim
        self.timestep_embedder = TimestepEmbedding(frequency_dim, embedding_dim)
        self.text_embedder = PixArtAlphaTextProjection(pooled_projection_dim, embedding_dim)


class CombinedTimestepGuidanceTextProjEmbeddings(nn.Module):
    """temb = timestep_embedder(sincos_256(t)) + guidance_embedder(sincos_256(g)) + text_embedder(pooled)."""

    def __init__(self, embedding_dim: int, pooled_projection_dim: int, frequency_dim: int = 256):
        super().__init__()
        self.frequency_dim = frequency_dim
        self.timestep_embedder = TimestepEmbedding(frequency_dim, embedding_dim)
        self.guidance_embedder = TimestepEmbedding(frequency_dim, embedding_dim)
        self.text_embedder = PixArtAlphaTextProjection(pooled_projection_dim, embedding_dim)


class FluxPosEmbed(nn.Module):
    """Rotary table from (text | image) position ids, one rotary axis per id column."""

    def __init__(self, theta: float = 10000.0, axes_dim=(16, 56, 56)):
        super().__init__()
        self.theta, self.axes_dim = theta, tuple(axes_dim)


class CogVideoXPatchEmbed(nn.Module):
    """diffusers ``CogVideoXPatchEmbed`` as CogVideoX-5B configures it: a p x p stride-p convolution per frame,
    a text projection, no learned or sin-cos position table (the model uses rotary embeddings)."""

    def __init__(self, patch_size: int = 2, in_channels: int = 16, embed_dim: int = 3072, text_embed_dim: int = 4096,
                 bias: bool = True):
        super().__init__()
        self.patch_size, self.patch_size_t = patch_size, None
        self.use_positional_embeddings = False
        self.use_learned_positional_embeddings = False
        self.proj = nn.Conv2d(in_channels, embed_dim, kernel_size=patch_size, stride=patch_size, bias=bias)
        self.text_proj = nn.Linear(text_embed_dim, embed_dim)


class AdaLayerNorm(nn.Module):
    """temb -> (shift, scale) -- shift first (``chunk_dim=1``); the LayerNorm carries affine weights."""

    chunks = 2

    def __init__(self, embedding_dim: int, output_dim: int, eps: float = 1e-5):
        super().__init__()
        self.silu = nn.SiLU()
        self.linear = nn.Linear(embedding_dim, output_dim)
        self.norm = nn.LayerNorm(output_dim // 2, eps=eps, elementwise_affine=True)
