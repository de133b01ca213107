"""fp32 primitives of the oracle (test infrastructure, never shipped).

Every function takes and returns fp32 ``torch.Tensor`` on the CPU and is written
as an explicit formula, so that the tests can pin it against PyTorch's library
routine for the same operation without comparing a formula with itself.
"""

import math
from typing import Optional, Sequence, Tuple

import torch


def _f32(x: torch.Tensor) -> torch.Tensor:
    return x.detach().to(torch.float32)


def silu(x: torch.Tensor) -> torch.Tensor:
    """x * sigmoid(x): the activation in front of every adaLN linear
    (diffusers ``AdaLayerNormZero``: ``self.linear(self.silu(emb))``)."""
    x = _f32(x)
    return x / (1.0 + torch.exp(-x))


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))).

    The FeedForward the reference wraps is built with
    ``activation_fn="gelu-approximate"``; its structure ``net[0].proj`` /
    ``net[2]`` is relied on at ``layers/feedforward.py:25-61``."""
    x = _f32(x)
    c = math.sqrt(2.0 / math.pi)
    return 0.5 * x * (1.0 + torch.tanh(c * (x + 0.044715 * x * x * x)))


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    """x Phi(x) = 0.5 x (1 + erf(x / sqrt 2)): ``F.gelu`` without approximation, what diffusers' ``GELU(approximate=
    "none")`` and the gate of ``GEGLU`` compute -- first-layer classes the reference's FeedForward wrapper accepts
    (``layers/feedforward.py:25-46``)."""
    x = _f32(x)
    return 0.5 * x * (1.0 + torch.erf(x * (1.0 / math.sqrt(2.0))))


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x W^T + b (``nn.Linear``; the projections at
    ``layers/attention_processor.py:688-695,:844-846,:1054-1056``)."""
    y = _f32(x) @ _f32(weight).transpose(-1, -2)
    if bias is not None:
        y = y + _f32(bias)
    return y


def layer_norm(
    x: torch.Tensor,
    eps: float,
    weight: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """LayerNorm over the last dim with biased variance."""
    x = _f32(x)
    mu = x.mean(dim=-1, keepdim=True)
    xc = x - mu
    var = (xc * xc).mean(dim=-1, keepdim=True)
    y = xc / torch.sqrt(var + eps)
    if weight is not None:
        y = y * _f32(weight)
    if bias is not None:
        y = y + _f32(bias)
    return y


def rms_norm(x: torch.Tensor, eps: float, weight: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * w  (diffusers ``RMSNorm``; applied as
    ``attn.norm_q`` / ``attn.norm_k`` at ``attention_processor.py:859-862``)."""
    x = _f32(x)
    ms = (x * x).mean(dim=-1, keepdim=True)
    y = x / torch.sqrt(ms + eps)
    if weight is not None:
        y = y * _f32(weight)
    return y


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None) -> torch.Tensor:
    """Non-causal softmax(q k^T * scale) v on ``[B, H, S, d]`` tensors.

    ``scale`` defaults to 1/sqrt(d): the reference calls
    ``F.scaled_dot_product_attention`` / ``flash_attn_func`` without a scale
    (``attention_processor.py:752-779``), so ``attn.scale`` is ignored.
    ``S_q`` may differ from ``S_kv`` (a PipeFusion query patch against the
    full K/V buffer)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    s = (q @ k.transpose(-1, -2)) * scale
    s = s - s.amax(dim=-1, keepdim=True)
    p = torch.exp(s)
    p = p / p.sum(dim=-1, keepdim=True)
    return p @ v


def apply_rotary_emb(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate adjacent pairs: follows ``attention_processor.py:88-113`` with
    ``use_real=True, use_real_unbind_dim=-1``.

    x ``[B, H, S, d]``; cos, sin ``[S, d]`` (each angle repeated for the pair).
    out[2i]   = x[2i] cos[2i]   - x[2i+1] sin[2i]
    out[2i+1] = x[2i+1] cos[2i+1] + x[2i] sin[2i+1]
    """
    x = _f32(x)
    cos = _f32(cos)[None, None]
    sin = _f32(sin)[None, None]
    even = x[..., 0::2]
    odd = x[..., 1::2]
    rot = torch.empty_like(x)
    rot[..., 0::2] = -odd
    rot[..., 1::2] = even
    return x * cos + rot * sin


def _axis_angles(pos: torch.Tensor, dim: int, theta: float) -> torch.Tensor:
    """angles[p, i] = pos[p] * theta^(-2i/dim), i < dim/2, in float64."""
    i = torch.arange(0, dim, 2, dtype=torch.float64)[: dim // 2]
    inv = 1.0 / (theta ** (i / dim))
    return pos.to(torch.float64)[:, None] * inv[None, :]


def flux_rope_table(
    ids: torch.Tensor, axes_dim: Sequence[int] = (16, 56, 56), theta: float = 10000.0
) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin tables ``[S, sum(axes_dim)]`` of Flux's positional embedding.

    ids ``[S, 3]``; text rows are all zero, image rows are (0, row, col)
    (the wrapper concatenates ``txt_ids, img_ids`` at ``transformer_flux.py:130-131``).
    Per axis the angle table is computed in float64, each angle is repeated for
    its pair, the axes are concatenated on the last dim and cast to fp32."""
    cos_parts, sin_parts = [], []
    for a, dim in enumerate(axes_dim):
        ang = _axis_angles(ids[:, a], dim, theta)
        cos_parts.append(torch.cos(ang).repeat_interleave(2, dim=1))
        sin_parts.append(torch.sin(ang).repeat_interleave(2, dim=1))
    return torch.cat(cos_parts, dim=-1).float(), torch.cat(sin_parts, dim=-1).float()


def cogvideox_rope_table(
    frames: int, height: int, width: int, head_dim: int = 64, theta: float = 10000.0
) -> Tuple[torch.Tensor, torch.Tensor]:
    """3-D RoPE tables ``[frames*height*width, head_dim]`` for CogVideoX-5B.

    head_dim splits into t: d/4, h: 3d/8, w: 3d/8 (64 -> 16, 24, 24); token
    order is t-major, then h, then w.  The pipeline builds the table once per
    request (``pipeline_cogvideox.py:303-309``) from integer grid positions."""
    dt, dh, dw = head_dim // 4, head_dim // 8 * 3, head_dim // 8 * 3
    gt = torch.arange(frames)
    gh = torch.arange(height)
    gw = torch.arange(width)
    parts_cos, parts_sin = [], []
    for pos, dim, shape in ((gt, dt, (frames, 1, 1)), (gh, dh, (1, height, 1)), (gw, dw, (1, 1, width))):
        ang = _axis_angles(pos, dim, theta).float()
        c = torch.cos(ang).repeat_interleave(2, dim=1)
        s = torch.sin(ang).repeat_interleave(2, dim=1)
        c = c.reshape(*shape, dim).expand(frames, height, width, dim)
        s = s.reshape(*shape, dim).expand(frames, height, width, dim)
        parts_cos.append(c)
        parts_sin.append(s)
    cos = torch.cat(parts_cos, dim=-1).reshape(frames * height * width, head_dim)
    sin = torch.cat(parts_sin, dim=-1).reshape(frames * height * width, head_dim)
    return cos.contiguous(), sin.contiguous()


def adaln_modulation(temb: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, chunks: int):
    """``linear(silu(temb)).chunk(chunks, dim=1)`` -- the adaLN projection
    shared by AdaLayerNormZero (6), ZeroSingle (3), Continuous (2) and
    CogVideoXLayerNormZero (6)."""
    return linear(silu(temb), weight, bias).chunk(chunks, dim=1)


def modulate(x_normed: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """x * (1 + scale[:, None]) + shift[:, None]."""
    return x_normed * (1.0 + scale[:, None, :]) + shift[:, None, :]
