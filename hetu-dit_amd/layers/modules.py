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


class FeedForward(nn.Module):
    """``net = [GELU(proj), Dropout, Linear]`` (activation_fn="gelu-approximate")."""

    def __init__(self, dim: int, dim_out: Optional[int] = None, mult: int = 4, inner_dim: Optional[int] = None,
                 bias: bool = True):
        super().__init__()
        inner_dim = inner_dim or dim * mult
        dim_out = dim_out or dim
        self.net = nn.ModuleList([GELU(dim, inner_dim, approximate="tanh", bias=bias), nn.Dropout(0.0),
                                  nn.Linear(inner_dim, dim_out, bias=bias)])


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
