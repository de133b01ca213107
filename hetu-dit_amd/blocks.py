"""The four transformer blocks of the denoise hot path as ``nn.Module``s that
live in ``transformer.transformer_blocks`` / ``.single_transformer_blocks`` and
keep the call conventions the reference's transformer wrappers use:

* SD3   ``block(hidden_states=, encoder_hidden_states=, temb=) -> (enc, hid)``
  (``models/transformers/transformer_sd3.py:136-152``)
* Flux double, same + ``image_rotary_emb=``   (``transformer_flux.py:160-165``)
* Flux single ``block(hidden_states=, temb=, image_rotary_emb=) -> hid`` (``:194-198``)
* CogVideoX ``block(hidden_states=, encoder_hidden_states=, temb=, image_rotary_emb=)
  -> (hid, enc)``                      (``cogvideox_transformer_3d.py:122-127``)

Sub-module names and parameter paths are those of the diffusers blocks with
the reference's wrappers applied (``attn.module.to_q``, ``attn.output_bias``,
``ff.module.net.0.proj``, ``norm1.linear`` ...), which is what the reference's
weight hot-swap addresses (``hetu_dit/utils.py:561-582``).

Per block the device work is: adaLN projections (weight streaming), fused
LayerNorm+modulate, ONE grouped GEMM per projection stage covering both
streams with bias / GELU-tanh / gated-residual epilogues, QK-norm+RoPE in
place, and the joint flash attention.  Inputs are never modified.
"""
from typing import Optional, Tuple

import torch
from torch import nn

from . import ops
from ._lib import eager_only
from .base_model import wrap_layer
from .layers.attention_processor import _PackedProjection, _rows2d, hetuDiTAttentionWrapper
from .layers.feedforward import hetuDiTFeedForwardWrapper
from .layers.modules import (
    AdaLayerNormContinuous,
    AdaLayerNormZero,
    AdaLayerNormZeroSingle,
    Attention,
    CogVideoXAttnProcessor2_0,
    CogVideoXLayerNormZero,
    FeedForward,
    FluxAttnProcessor2_0,
    JointAttnProcessor2_0,
)
from .runtime_state import get_runtime_state


def _wrap(layer: nn.Module) -> nn.Module:
    """What ``_wrap_layers`` + ``_register_cache`` do for one sub-module
    (``models/base_model.py:59-112,:162-178``): registry lookup, construct, and
    register the K/V cache entry under the *wrapper*."""
    return wrap_layer(layer)


def _adaln(norm: nn.Module, temb: torch.Tensor):
    """f32 [B, chunks*D] = linear(silu(temb)); chunk views.  Taken from the stack-wide launch of
    ``StackModulation`` when that ran on this very ``temb``."""
    cached = getattr(norm, "_stack_emb", None)
    # the cache holds the tensor itself: a later, different temb cannot alias it by address
    if cached is not None and cached[0] is temb and cached[1] == temb._version:
        return cached[2].chunk(norm.chunks, dim=1)
    emb = ops.adaln_gemv(temb.contiguous(), norm.linear.weight.data, norm.linear.bias.data)
    return emb.chunk(norm.chunks, dim=1)


class StackModulation:
    """``linear(silu(temb))`` of every adaLN module of a block stack in one launch.

    Within a denoise step all blocks are conditioned on the same ``temb``
    (``transformer_sd3.py:107-152`` passes it unchanged to every block), so the
    per-block weight streams (56.6 MB per SD3 block) can be read by one
    bandwidth-bound GEMV over the concatenated weights instead of 48 short ones.
    The ``nn.Linear`` modules stay addressable: their ``.data`` are row slices of
    the packed weight, re-packed if a hot-swap re-assigns them."""

    def __init__(self, blocks):
        kinds = (AdaLayerNormZero, AdaLayerNormZeroSingle, AdaLayerNormContinuous, CogVideoXLayerNormZero)
        self.norms = [m for b in blocks for m in b.modules() if isinstance(m, kinds)]
        self.packed = _PackedProjection([n.linear for n in self.norms])
        self._gather = {}  # (batch, device) -> element indices that regroup [B, all rows] by module

    def precompute(self, temb: torch.Tensor):
        w, b = self.packed.get()
        emb = ops.adaln_gemv(temb.contiguous(), w, b)
        off = 0
        for norm, rows in zip(self.norms, self.packed.splits):
            norm._stack_emb = (temb, temb._version, emb[:, off : off + rows])
            off += rows
        return emb

    def precompute_by_module(self, temb: torch.Tensor):
        """``precompute`` plus the same numbers regrouped so that every module's [batch, rows] block is
        contiguous (what the whole-block entry points take): returns ``(flat f32 tensor, {module: element
        offset of its block})``; batch element b of a module starts ``b * rows`` elements into its block."""
        emb = self.precompute(temb)
        B, total = emb.shape
        key = (B, emb.device)
        cached = self._gather.get(key)
        if cached is None:
            parts, offsets, off = [], {}, 0
            cols = torch.arange(total, device=emb.device)
            for norm, rows in zip(self.norms, self.packed.splits):
                offsets[norm] = B * off
                parts.append((torch.arange(B, device=emb.device)[:, None] * total + cols[off : off + rows][None, :]).reshape(-1))
                off += rows
            cached = self._gather[key] = (torch.cat(parts), offsets)
        index, offsets = cached
        return emb.reshape(-1).index_select(0, index), offsets


def _stream_out(resid: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Where a residual update of ``resid`` (a tensor this block owns) goes: in place when the stream keeps
    its element type, else into a new tensor of the requested type."""
    return resid if resid.dtype == dtype else torch.empty(resid.shape, dtype=dtype, device=resid.device)


def _mlp_both_streams(ff, x2, resid, gate, ff_c=None, xc2=None, resid_c=None, gate_c=None,
                      out_dtype: torch.dtype = torch.bfloat16):
    """gated-residual MLP of one or two streams: two grouped launches.  ``resid`` (and ``resid_c``) are the
    block's own intermediates (the fp32 stream after the attention residual); the result has ``out_dtype``.
    Returns ``(out, out_c_or_None)``."""
    p_in, h = ff.in_problem(x2)
    probs = [p_in]
    if ff_c is not None:
        pc_in, hc = ff_c.in_problem(xc2)
        probs.append(pc_in)
    ops.gemm_launch(probs)
    out, out_c = _stream_out(resid, out_dtype), None
    probs = [ff.out_problem(h, _rows2d(out), _rows2d(resid), gate, rows_per_batch=resid.shape[1])]
    if ff_c is not None:
        out_c = _stream_out(resid_c, out_dtype)
        probs.append(ff_c.out_problem(hc, _rows2d(out_c), _rows2d(resid_c), gate_c, rows_per_batch=resid_c.shape[1]))
    ops.gemm_launch(probs)
    return out, out_c


def use_fp32_residual_stream(blocks, last_block_bf16: bool = True):
    """Carry the residual stream between the blocks of a stack in fp32: every block but the last returns f32
    ``hidden_states`` / ``encoder_hidden_states`` (each block accepts bf16 or f32 inputs), the last one
    returns bf16 for whatever follows the stack (``norm_out`` / ``proj_out``).  Rounding the stream to bf16
    at every residual costs about 2.3e-3 relative error per block, i.e. 1.1e-2 after the 24 blocks of an
    SD3-shape step; with the stream in fp32 the same step stays below 4e-3."""
    blocks = list(blocks)
    for i, b in enumerate(blocks):
        b.stream_dtype = torch.bfloat16 if (last_block_bf16 and i == len(blocks) - 1) else torch.float32


class JointTransformerBlock(nn.Module):
    """SD3 MMDiT joint block (diffusers ``JointTransformerBlock``)."""

    def __init__(self, dim: int, num_attention_heads: int, attention_head_dim: int, context_pre_only: bool = False):
        super().__init__()
        self.context_pre_only = context_pre_only
        # element type of the returned streams: bf16 as the reference's blocks, or f32 (use_fp32_residual_stream)
        self.stream_dtype = torch.bfloat16
        self.norm1 = AdaLayerNormZero(dim)
        self.norm1_context = AdaLayerNormContinuous(dim, dim, eps=1e-6) if context_pre_only else AdaLayerNormZero(dim)
        self.attn = _wrap(
            Attention(dim, num_attention_heads, attention_head_dim, added_kv_proj_dim=dim,
                      context_pre_only=context_pre_only, bias=True, processor=JointAttnProcessor2_0())
        )
        self.norm2 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.ff = _wrap(FeedForward(dim))
        if not context_pre_only:
            self.norm2_context = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
            self.ff_context = _wrap(FeedForward(dim))
        else:
            self.norm2_context = None
            self.ff_context = None

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, temb: torch.Tensor,
                skip_text_output: bool = False, pending=None, defer: bool = False):
        """``skip_text_output``: the caller drops this block's text output (the SD3 block loop does for every
        pipeline patch after the first, ``transformer_sd3.py:131-146``), so the text stream stops after its
        q|k|v projection -- no out-projection, ``norm2_context`` or ``ff_context`` -- and ``None`` is returned
        for it.  The image output is unchanged bit for bit.

        ``pending`` / ``defer`` (block stacks, f32 streams): the launches of ``hdit_block_sd3`` with
        ``lazy_residual`` -- see ``_forward_lazy``."""
        if pending is not None or defer:
            return self._forward_lazy(hidden_states, encoder_hidden_states, temb, skip_text_output,
                                      pending or (None, None), defer)
        eps = 1e-6
        sh_a, sc_a, g_a, sh_m, sc_m, g_m = _adaln(self.norm1, temb)
        if self.context_pre_only:
            c_sc, c_sh = _adaln(self.norm1_context, temb)  # AdaLayerNormContinuous: scale first
            n, nc = ops.layernorm_modulate_many([(hidden_states, sh_a, sc_a), (encoder_hidden_states, c_sh, c_sc)], eps)
            hidden, _ = self.attn.forward_gated(n, nc, hidden_states, g_a)
        else:
            c_sh_a, c_sc_a, c_g_a, c_sh_m, c_sc_m, c_g_m = _adaln(self.norm1_context, temb)
            n, nc = ops.layernorm_modulate_many([(hidden_states, sh_a, sc_a), (encoder_hidden_states, c_sh_a, c_sc_a)], eps)
            hidden, encoder = self.attn.forward_gated(n, nc, hidden_states, g_a, encoder_hidden_states, c_g_a,
                                                      skip_txt=skip_text_output)
        # between the two residuals of a block the stream is always fp32
        if self.context_pre_only or skip_text_output:
            n2 = ops.layernorm_modulate(hidden, sh_m, sc_m, eps)
            hidden, _ = _mlp_both_streams(self.ff, _rows2d(n2), hidden, g_m, out_dtype=self.stream_dtype)
            return None, hidden
        n2, nc2 = ops.layernorm_modulate_many([(hidden, sh_m, sc_m), (encoder, c_sh_m, c_sc_m)], eps)
        hidden, encoder = _mlp_both_streams(self.ff, _rows2d(n2), hidden, g_m, self.ff_context, _rows2d(nc2), encoder,
                                            c_g_m, out_dtype=self.stream_dtype)
        return encoder, hidden


    def _forward_lazy(self, hidden_states, encoder_hidden_states, temb, skip_text_output, pending, defer):
        """The block with its gated residuals taken out of the GEMM epilogues: a projection writes
        ``y = bf16(A W^T + bias)`` and the normalisation that reads the f32 stream next adds ``gate * y`` (and
        writes the updated stream), which spares the GEMM the read-modify-write of the stream.  ``pending``:
        ``(img, txt)``, each ``(y, gate)`` or None -- the MLP residual the previous block left to this block's
        norm1.  ``defer``: this block leaves its own MLP residuals the same way; ``self.deferred`` is then the
        ``pending`` of the next block and the returned streams are the ones after the attention residual.  A
        stream that arrives in bf16 (the first block of a stack) keeps the fused epilogue for its attention
        residual.  Sums are fma(gate, y, x) in fp32 wherever they are made, so the bits are the ones of
        ``forward`` without these arguments."""
        eps = 1e-6
        f32 = torch.float32
        pre_only = self.context_pre_only
        text_out = not pre_only and not skip_text_output
        sh_a, sc_a, g_a, sh_m, sc_m, g_m = _adaln(self.norm1, temb)
        if pre_only:
            c_sc_a, c_sh_a = _adaln(self.norm1_context, temb)  # AdaLayerNormContinuous: scale first
            c_g_a = c_sh_m = c_sc_m = c_g_m = None
        else:
            c_sh_a, c_sc_a, c_g_a, c_sh_m, c_sc_m, c_g_m = _adaln(self.norm1_context, temb)
        pend_img, pend_txt = pending

        def first_norm(x, shift, scale, pend, keep):
            """norm1 item of one stream; returns (item, the stream the rest of the block works on)."""
            if pend is None:
                return (x, shift, scale), x
            x0 = torch.empty_like(x) if keep else None
            return (x, shift, scale, None, (pend[0], pend[1], x0)), x0

        item_i, x0_img = first_norm(hidden_states, sh_a, sc_a, pend_img, True)
        item_t, x0_txt = first_norm(encoder_hidden_states, c_sh_a, c_sc_a, pend_txt, text_out)
        n, nc = ops.layernorm_modulate_many([item_i, item_t], eps)
        kwargs = {"skip_text_queries": True} if skip_text_output and not pre_only else {}
        o_img, o_txt = self.attn.processor(self.attn, n, encoder_hidden_states=nc, **kwargs)
        lazy_img = x0_img.dtype == f32
        lazy_txt = text_out and x0_txt.dtype == f32
        problems, outs = self.attn.out_proj_problems(
            o_img, o_txt, None if lazy_img else x0_img, None if lazy_img else g_a,
            None if lazy_txt else x0_txt, None if lazy_txt else c_g_a, skip_txt=not text_out)
        ops.gemm_launch(problems)
        # norm2 (+ the attention residual of the lazily updated streams)
        items = [(x0_img, sh_m, sc_m, None, (outs[0], g_a, x0_img if x0_img is not hidden_states else torch.empty_like(x0_img)))
                 if lazy_img else (outs[0], sh_m, sc_m)]
        if text_out:
            items.append((x0_txt, c_sh_m, c_sc_m, None,
                          (outs[1], c_g_a, x0_txt if x0_txt is not encoder_hidden_states else torch.empty_like(x0_txt)))
                         if lazy_txt else (outs[1], c_sh_m, c_sc_m))
        normed = ops.layernorm_modulate_many(items, eps)
        x1_img = items[0][4][2] if lazy_img else outs[0]
        x1_txt = (items[1][4][2] if lazy_txt else outs[1]) if text_out else None
        # MLP
        p_in, h = self.ff.in_problem(_rows2d(normed[0]))
        probs = [p_in]
        if text_out:
            pc_in, hc = self.ff_context.in_problem(_rows2d(normed[1]))
            probs.append(pc_in)
        ops.gemm_launch(probs)
        self.deferred = None
        if defer:
            if self.stream_dtype != f32:
                raise ValueError("residuals can only be left to the next block on an f32 stream")
            y_img = torch.empty(x1_img.shape, dtype=torch.bfloat16, device=x1_img.device)
            probs = [self.ff.out_problem(h, _rows2d(y_img))]
            y_txt = None
            if text_out:
                y_txt = torch.empty(x1_txt.shape, dtype=torch.bfloat16, device=x1_txt.device)
                probs.append(self.ff_context.out_problem(hc, _rows2d(y_txt)))
            ops.gemm_launch(probs)
            self.deferred = ((y_img, g_m), (y_txt, c_g_m) if text_out else None)
            return x1_txt, x1_img
        out = _stream_out(x1_img, self.stream_dtype)
        probs = [self.ff.out_problem(h, _rows2d(out), _rows2d(x1_img), g_m, rows_per_batch=x1_img.shape[1])]
        out_c = None
        if text_out:
            out_c = _stream_out(x1_txt, self.stream_dtype)
            probs.append(self.ff_context.out_problem(hc, _rows2d(out_c), _rows2d(x1_txt), c_g_m, rows_per_batch=x1_txt.shape[1]))
        ops.gemm_launch(probs)
        return out_c, out


class FluxTransformerBlock(nn.Module):
    """Flux double-stream block (diffusers ``FluxTransformerBlock``)."""

    def __init__(self, dim: int, num_attention_heads: int, attention_head_dim: int):
        super().__init__()
        self.stream_dtype = torch.bfloat16
        self.norm1 = AdaLayerNormZero(dim)
        self.norm1_context = AdaLayerNormZero(dim)
        self.attn = _wrap(
            Attention(dim, num_attention_heads, attention_head_dim, added_kv_proj_dim=dim, context_pre_only=False,
                      bias=True, qk_norm="rms_norm", eps=1e-6, processor=FluxAttnProcessor2_0())
        )
        self.norm2 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.ff = _wrap(FeedForward(dim))
        self.norm2_context = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.ff_context = _wrap(FeedForward(dim))

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None):
        eps = 1e-6
        sh_a, sc_a, g_a, sh_m, sc_m, g_m = _adaln(self.norm1, temb)
        c_sh_a, c_sc_a, c_g_a, c_sh_m, c_sc_m, c_g_m = _adaln(self.norm1_context, temb)
        n, nc = ops.layernorm_modulate_many([(hidden_states, sh_a, sc_a), (encoder_hidden_states, c_sh_a, c_sc_a)], eps)
        hidden, encoder = self.attn.forward_gated(n, nc, hidden_states, g_a, encoder_hidden_states, c_g_a,
                                                  image_rotary_emb=image_rotary_emb)
        n2, nc2 = ops.layernorm_modulate_many([(hidden, sh_m, sc_m), (encoder, c_sh_m, c_sc_m)], eps)
        hidden, encoder = _mlp_both_streams(self.ff, _rows2d(n2), hidden, g_m, self.ff_context, _rows2d(nc2), encoder,
                                            c_g_m, out_dtype=self.stream_dtype)
        return encoder, hidden


class FluxSingleTransformerBlock(nn.Module):
    """Flux single-stream block (diffusers ``FluxSingleTransformerBlock``): the
    q|k|v projection and the MLP-in projection share one launch, attention
    output and GELU(MLP) are produced side by side in one [B, S, 5D] buffer
    (no concatenation), ``proj_out`` carries the gated residual."""

    def __init__(self, dim: int, num_attention_heads: int, attention_head_dim: int, mlp_ratio: float = 4.0):
        super().__init__()
        self.mlp_hidden_dim = int(dim * mlp_ratio)
        self.stream_dtype = torch.bfloat16
        self.norm = AdaLayerNormZeroSingle(dim)
        self.proj_mlp = nn.Linear(dim, self.mlp_hidden_dim)
        self.act_mlp = nn.GELU(approximate="tanh")
        self.proj_out = nn.Linear(dim + self.mlp_hidden_dim, dim)
        self.attn = _wrap(
            Attention(dim, num_attention_heads, attention_head_dim, bias=True, qk_norm="rms_norm", eps=1e-6,
                      pre_only=True, processor=FluxAttnProcessor2_0())
        )

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states, temb, image_rotary_emb=None):
        B, S, D = hidden_states.shape
        sh, sc, g = _adaln(self.norm, temb)
        n = ops.layernorm_modulate(hidden_states, sh, sc, 1e-6)
        cat = torch.empty(B, S, D + self.mlp_hidden_dim, dtype=torch.bfloat16, device=hidden_states.device)
        mlp_problem = ops.gemm_problem(_rows2d(n), self.proj_mlp.weight.data, cat.view(-1, cat.shape[-1])[:, D:],
                                       self.proj_mlp.bias.data, ops.EPI_BIAS_GELU)
        self.attn.processor(self.attn, n, encoder_hidden_states=None, image_rotary_emb=image_rotary_emb,
                            out=cat[:, :, :D], extra_problems=[mlp_problem])
        out = torch.empty(B, S, D, dtype=self.stream_dtype, device=hidden_states.device)
        ops.gemm_launch([
            ops.gemm_problem(cat.view(-1, cat.shape[-1]), self.proj_out.weight.data, out.view(-1, D),
                             self.proj_out.bias.data, ops.EPI_GATE_RESIDUAL, resid=_rows2d(hidden_states), gate=g,
                             rows_per_batch=S)
        ])
        return out


class CogVideoXBlock(nn.Module):
    """CogVideoX block (diffusers ``CogVideoXBlock``): one weight set over the
    joint [text, video] rows; the two streams differ only in their modulation
    and gates.  Returns ``(hidden_states, encoder_hidden_states)``."""

    def __init__(self, dim: int, num_attention_heads: int, attention_head_dim: int, time_embed_dim: int = 512):
        super().__init__()
        self.stream_dtype = torch.bfloat16
        self.norm1 = CogVideoXLayerNormZero(time_embed_dim, dim, eps=1e-5)
        self.attn1 = _wrap(
            Attention(dim, num_attention_heads, attention_head_dim, bias=True, out_bias=True, qk_norm="layer_norm",
                      eps=1e-6, processor=CogVideoXAttnProcessor2_0())
        )
        self.norm2 = CogVideoXLayerNormZero(time_embed_dim, dim, eps=1e-5)
        self.ff = _wrap(FeedForward(dim))

    def _norm_joint(self, norm, hidden, encoder, temb):
        """Both streams' LayerNorm(affine)+modulate written into one joint
        [B, n_txt + n_img, D] buffer in [text, video] order."""
        sh, sc, g, e_sh, e_sc, e_g = _adaln(norm, temb)
        B, N, D = hidden.shape
        Nt = encoder.shape[1]
        joint = torch.empty(B, Nt + N, D, dtype=torch.bfloat16, device=hidden.device)
        w, b = norm.norm.weight.data, norm.norm.bias.data
        ops.layernorm_modulate_many([(encoder, e_sh, e_sc, joint[:, :Nt]), (hidden, sh, sc, joint[:, Nt:])],
                                    norm.norm.eps, w, b)
        return joint, g, e_g

    @staticmethod
    def _gated_out_problems(a_joint, weight, bias, hidden, encoder, gate, e_gate, out_h, out_e):
        """out_stream = stream + gate_stream * (a_joint[rows of stream] @ W^T + b), per batch."""
        B, N, D = hidden.shape
        Nt = encoder.shape[1]
        probs = []
        for bi in range(B):
            probs.append(ops.gemm_problem(a_joint[bi, :Nt], weight, out_e[bi], bias, ops.EPI_GATE_RESIDUAL,
                                          resid=encoder[bi], gate=e_gate[bi:bi + 1], rows_per_batch=Nt))
            probs.append(ops.gemm_problem(a_joint[bi, Nt:], weight, out_h[bi], bias, ops.EPI_GATE_RESIDUAL,
                                          resid=hidden[bi], gate=gate[bi:bi + 1], rows_per_batch=N))
        return probs

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None):
        hidden_states = hidden_states.contiguous()
        encoder_hidden_states = encoder_hidden_states.contiguous()
        attn = self.attn1
        joint, g, e_g = self._norm_joint(self.norm1, hidden_states, encoder_hidden_states, temb)
        o = attn.processor(attn, hidden_states, encoder_hidden_states, image_rotary_emb=image_rotary_emb,
                           joint_input=joint)
        hidden = torch.empty(hidden_states.shape, dtype=torch.float32, device=hidden_states.device)
        encoder = torch.empty(encoder_hidden_states.shape, dtype=torch.float32, device=hidden_states.device)
        ops.gemm_launch(self._gated_out_problems(
            o, attn.module.to_out[0].weight.data, attn.output_bias.data if attn.has_output_bias else None,
            hidden_states, encoder_hidden_states, g, e_g, hidden, encoder))
        joint, g, e_g = self._norm_joint(self.norm2, hidden, encoder, temb)
        p_in, h = self.ff.in_problem(joint.view(-1, joint.shape[-1]))
        ops.gemm_launch([p_in])
        h = h.view(joint.shape[0], joint.shape[1], -1)
        out_h, out_e = _stream_out(hidden, self.stream_dtype), _stream_out(encoder, self.stream_dtype)
        ops.gemm_launch(self._gated_out_problems(
            h, self.ff.module.net[2].weight.data, self.ff.output_bias.data if self.ff.has_output_bias else None,
            hidden, encoder, g, e_g, out_h, out_e))
        return out_h, out_e
