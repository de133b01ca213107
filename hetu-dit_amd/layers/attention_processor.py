"""Attention wrapper and attention processors with the interface of the
reference's ``layers/attention_processor.py`` -- same class names, call
signatures, return conventions and registries -- computing on the gfx950
kernels:

* the q|k|v (and add_q|k|v) projections of both streams are ONE grouped GEMM
  launch over packed weights; K|V rows land directly in the layer's stale K/V
  buffer (``CacheManager.kv_buffer``), so the cat / slice-assign / chunk copies
  of ``cache_manager.py:88-113`` disappear;
* QK-RMSNorm / QK-LayerNorm and RoPE run as one in-place pass;
* the joint sequence is never concatenated: the attention kernel reads image
  and text segments from their own buffers.
"""
import inspect
from typing import List, Optional, Tuple

import torch
from torch import nn

from .. import ops
from .._lib import eager_only
from ..cache_manager import get_cache_manager
from ..parallel_state import (
    get_pipeline_parallel_world_size,
    get_sequence_parallel_world_size,
    get_tensor_model_parallel_rank,
    get_tensor_model_parallel_world_size,
    get_tp_group,
)
from ..registry import hetuDiTAttentionProcessorRegister, hetuDiTLayerWrappersRegister
from ..runtime_state import get_runtime_state
from .base_layer import hetuDiTDiffusionLayerBaseWrapper
from .modules import Attention, CogVideoXAttnProcessor2_0, FluxAttnProcessor2_0, JointAttnProcessor2_0, RMSNorm

# the reference probes these at import (attention_processor.py:50-52); neither
# third-party backend exists here and neither is needed
HAS_LONG_CTX_ATTN = False
HAS_FLASH_ATTN = False


def _cat_params(layers: List[nn.Linear]) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    w = torch.cat([l.weight.data for l in layers], dim=0).contiguous()
    b = None
    if layers[0].bias is not None:
        b = torch.cat([l.bias.data for l in layers], dim=0).contiguous()
    return w, b


class _PackedProjection:
    """Several nn.Linear sharing an input, fused into one [sum(out), in] weight.
    The original modules are kept addressable (the reference's weight hot-swap
    reaches them by path): their ``.data`` become row-slices of the packed
    tensor; if someone re-assigns ``.data`` the pack is rebuilt on next use."""

    def __init__(self, layers: List[nn.Linear]):
        if len({l.bias is None for l in layers}) != 1:
            raise ValueError("the layers of one packed projection must all have a bias or all have none")
        self.layers = layers
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.splits = [l.weight.shape[0] for l in layers]

    def _stale(self) -> bool:
        """True when a weight or a bias no longer is the row slice of the pack it was made (a hot-swap
        re-assigned its ``.data``)."""
        if self.weight is None:
            return True
        off = 0
        for l, n in zip(self.layers, self.splits):
            if l.weight.data_ptr() != self.weight.data_ptr() + off * self.weight.shape[1] * self.weight.element_size():
                return True
            if l.bias is not None and (self.bias is None or
                                       l.bias.data_ptr() != self.bias.data_ptr() + off * self.bias.element_size()):
                return True
            off += n
        return False

    def get(self) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        if self._stale():
            self.splits = [l.weight.shape[0] for l in self.layers]
            self.weight, self.bias = _cat_params(self.layers)
            off = 0
            for l, n in zip(self.layers, self.splits):
                l.weight.data = self.weight[off : off + n]
                if l.bias is not None:
                    l.bias.data = self.bias[off : off + n]
                off += n
        return self.weight, self.bias

    def rows(self, start: int, count: int) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        w, b = self.get()
        return w[start : start + count], (None if b is None else b[start : start + count])


def _patch_range():
    return get_cache_manager()._patch_range()


def _rows2d(x: torch.Tensor) -> torch.Tensor:
    """[B, T, D] -> contiguous [B*T, D] view."""
    if not x.is_contiguous():
        x = x.contiguous()
    return x.view(-1, x.shape[-1])


def _qkv_problems(x: torch.Tensor, packed: _PackedProjection, layer, inner: int, use_cache: bool):
    """Problems projecting one stream to q and k|v.

    Returns (problems, q [B,T,I] view, kv [B,T_kv,2I] view).  Without the cache
    (or with patch mode off) one GEMM writes a [B, T, 3I] tensor whose column
    ranges are q and k|v, and -- if cached -- that k|v view becomes the layer's
    buffer.  In patch mode q gets its own tensor and k|v goes straight into the
    rows of the current patch of the persistent buffer."""
    B, T, _ = x.shape
    x2 = _rows2d(x)
    rng = _patch_range() if use_cache else None
    if rng is None:
        w, b = packed.get()
        qkv = torch.empty(B, T, 3 * inner, dtype=torch.bfloat16, device=x.device)
        kv = qkv[:, :, inner:]
        if use_cache:
            get_cache_manager()._entry(layer, "attn").tensors[0] = kv
        return [ops.gemm_problem(x2, w, qkv.view(-1, 3 * inner), b)], qkv[:, :, :inner], kv
    buf, start, end = get_cache_manager().kv_buffer(layer, B, T, inner, x.device)
    wq, bq = packed.rows(0, inner)
    wkv, bkv = packed.rows(inner, 2 * inner)
    q = torch.empty(B, T, inner, dtype=torch.bfloat16, device=x.device)
    problems = [ops.gemm_problem(x2, wq, q.view(-1, inner), bq)]
    for bi in range(B):
        problems.append(ops.gemm_problem(x2[bi * T : (bi + 1) * T], wkv, buf[bi, start:end], bkv))
    return problems, q, buf


def _heads(x: torch.Tensor, heads: int) -> torch.Tensor:
    """[B, T, H*d] (any row stride) -> [B, T, H, d] view."""
    return x.unflatten(2, (heads, x.shape[2] // heads))


class hetuDiTAttentionBaseWrapper(hetuDiTDiffusionLayerBaseWrapper):
    """Weight slicing by tensor-parallel rank and re-homing of the output
    biases, as ``attention_processor.py:123-193``: ``to_out[0].bias`` moves to
    ``self.output_bias`` and ``to_add_out.bias`` to ``self.encoder_output_bias``
    (added after the tensor-parallel reduce, which is skipped at one GPU)."""

    def __init__(self, attention: Attention):
        super().__init__(module=attention)
        to_k, to_v = self.module.to_k, self.module.to_v
        assert isinstance(to_k, nn.Linear) and isinstance(to_v, nn.Linear)
        assert (to_k.bias is None) == (to_v.bias is None)
        assert to_k.weight.shape == to_v.weight.shape
        tp_degree = get_tensor_model_parallel_world_size()
        tp_rank = get_tensor_model_parallel_rank()
        for name in ["to_q", "to_k", "to_v", "add_k_proj", "add_v_proj", "add_q_proj"]:
            proj = getattr(self.module, name, None)
            if proj is not None:
                proj.weight.data = proj.weight.data.chunk(tp_degree, dim=0)[tp_rank].clone()
                if proj.bias is not None:
                    proj.bias.data = proj.bias.data.chunk(tp_degree, dim=0)[tp_rank].clone()
        self.has_output_bias = False
        if not self.module.pre_only:
            proj = self.module.to_out[0]
            proj.weight.data = proj.weight.data.chunk(tp_degree, dim=1)[tp_rank].clone()
            if proj.bias is not None:
                self.register_parameter("output_bias", nn.Parameter(proj.bias.data.clone(), requires_grad=False))
                proj.bias = None
                self.has_output_bias = True
        self.has_encoder_output_bias = False
        if self.module.context_pre_only is not None and not self.module.context_pre_only:
            proj = getattr(self.module, "to_add_out", None)
            if proj is not None:
                proj.weight.data = proj.weight.data.chunk(tp_degree, dim=1)[tp_rank].clone()
                if proj.bias is not None:
                    self.register_parameter(
                        "encoder_output_bias", nn.Parameter(proj.bias.data.clone(), requires_grad=False)
                    )
                    proj.bias = None
                    self.has_encoder_output_bias = True
        self.heads_per_device = self.module.heads // tp_degree
        m = self.module
        self._qkv = _PackedProjection([m.to_q, m.to_k, m.to_v])
        self._add_qkv = None
        if getattr(m, "add_q_proj", None) is not None:
            self._add_qkv = _PackedProjection([m.add_q_proj, m.add_k_proj, m.add_v_proj])


@hetuDiTLayerWrappersRegister.register(Attention)
class hetuDiTAttentionWrapper(hetuDiTAttentionBaseWrapper):
    def __init__(self, attention: Attention):
        super().__init__(attention=attention)
        self.processor = hetuDiTAttentionProcessorRegister.get_processor(attention.processor)()
        self._proc_params = set(inspect.signature(self.processor.__call__).parameters.keys())

    # -- out-projection as GEMM problems (optionally with the gated residual) ------
    def out_proj_problems(self, o_img, o_txt, resid_img=None, gate_img=None, resid_txt=None, gate_txt=None,
                          skip_txt: bool = False):
        """Problems for ``to_out[0]`` (+ ``output_bias``) and ``to_add_out``
        (+ ``encoder_output_bias`` unless ``encoder_bias`` is off for this
        family).  With ``resid``/``gate`` the epilogue is the gated residual and
        the result is f32: the residual stream inside a block is carried in fp32."""
        m = self.module
        problems, outs = [], []

        def one(o, weight, bias, resid, gate):
            B, T, _ = o.shape
            out = torch.empty(B, T, weight.shape[0], dtype=torch.bfloat16 if resid is None else torch.float32,
                              device=o.device)
            if resid is None:
                problems.append(ops.gemm_problem(_rows2d(o), weight, out.view(-1, out.shape[-1]), bias))
            else:
                problems.append(
                    ops.gemm_problem(_rows2d(o), weight, out.view(-1, out.shape[-1]), bias, ops.EPI_GATE_RESIDUAL,
                                     resid=_rows2d(resid), gate=gate, rows_per_batch=T)
                )
            outs.append(out)

        one(o_img, m.to_out[0].weight.data, self.output_bias.data if self.has_output_bias else None, resid_img, gate_img)
        if o_txt is not None and not skip_txt and not m.context_pre_only and getattr(m, "to_add_out", None) is not None:
            bias = None
            if self.has_encoder_output_bias and self.processor.adds_encoder_output_bias:
                bias = self.encoder_output_bias.data
            one(o_txt, m.to_add_out.weight.data, bias, resid_txt, gate_txt)
        return problems, outs

    def forward(
        self,
        hidden_states: torch.Tensor,
        encoder_hidden_states: Optional[torch.Tensor] = None,
        attention_mask: Optional[torch.Tensor] = None,
        **cross_attention_kwargs,
    ):
        """Same dispatch and return conventions as the reference's
        ``hetuDiTAttentionWrapper.forward`` (``attention_processor.py:207-449``):
        SD3 / Flux-double -> ``(hidden, encoder)`` after the out-projections;
        Flux-single (``encoder_hidden_states is None``) -> joint attention output
        without out-projection; CogVideoX -> ``(hidden, encoder)`` split from the
        projected joint tensor."""
        if attention_mask is not None:
            raise NotImplementedError("the DiT blocks on this path never pass an attention mask")
        kwargs = {k: v for k, v in cross_attention_kwargs.items() if k in self._proc_params}
        proc = self.processor
        if isinstance(proc, hetuDiTCogVideoXAttnProcessor2_0):
            n_txt = encoder_hidden_states.size(1)
            joint = proc(self, hidden_states, encoder_hidden_states=encoder_hidden_states, **kwargs)
            problems, outs = self.out_proj_problems(joint, None)
            ops.gemm_launch(problems)
            out = outs[0]
            return out[:, n_txt:], out[:, :n_txt]
        if isinstance(proc, hetuDiTFluxAttnProcessor2_0) and encoder_hidden_states is None:
            return proc(self, hidden_states, encoder_hidden_states=None, **kwargs)
        # [B, C, H, W] inputs are token sequences in channel-major layout (attention_processor.py:672-683); the
        # outputs go back to that layout (:436-443), each with its own height and width
        shape_img = hidden_states.shape if hidden_states.ndim == 4 else None
        shape_txt = encoder_hidden_states.shape if encoder_hidden_states is not None and encoder_hidden_states.ndim == 4 else None
        if shape_img is not None:
            hidden_states = hidden_states.flatten(2).transpose(1, 2).contiguous()
        if shape_txt is not None:
            encoder_hidden_states = encoder_hidden_states.flatten(2).transpose(1, 2).contiguous()
        o_img, o_txt = proc(self, hidden_states, encoder_hidden_states=encoder_hidden_states, **kwargs)
        problems, outs = self.out_proj_problems(o_img, o_txt)
        ops.gemm_launch(problems)
        out_img = outs[0]
        out_txt = outs[1] if len(outs) == 2 else o_txt  # context_pre_only: raw attention slice (:420-421)
        if shape_img is not None:
            out_img = out_img.transpose(-1, -2).reshape(shape_img[0], -1, shape_img[2], shape_img[3])
        if shape_txt is not None and out_txt is not None:
            out_txt = out_txt.transpose(-1, -2).reshape(shape_txt[0], -1, shape_txt[2], shape_txt[3])
        return out_img, out_txt

    def forward_gated(self, hidden_states, encoder_hidden_states, resid_img, gate_img, resid_txt=None, gate_txt=None,
                      skip_txt: bool = False, **kwargs):
        """``resid + gate * attn(...)`` for both streams with the gated residual
        fused into the out-projection epilogue (what the diffusers block does
        with the wrapper's outputs right after the call).  Returns
        ``(hidden_new, encoder_new_or_None)``.  ``skip_txt`` leaves the text
        stream's out-projection out (its result would be dropped by the caller)."""
        kwargs = {k: v for k, v in kwargs.items() if k in self._proc_params}
        if skip_txt and "skip_text_queries" in self._proc_params:
            kwargs["skip_text_queries"] = True
        o_img, o_txt = self.processor(self, hidden_states, encoder_hidden_states=encoder_hidden_states, **kwargs)
        problems, outs = self.out_proj_problems(o_img, o_txt, resid_img, gate_img, resid_txt, gate_txt, skip_txt=skip_txt)
        ops.gemm_launch(problems)
        return outs[0], (outs[1] if len(outs) == 2 else None)


# ---------------------------------------------------------------------------
# processors
# ---------------------------------------------------------------------------

@hetuDiTAttentionProcessorRegister.register(JointAttnProcessor2_0)
class hetuDiTJointAttnProcessor2_0(JointAttnProcessor2_0):
    """SD3: no QK-norm, joint order [image, text], image K/V through the stale
    buffer (``attention_processor.py:657-793``)."""

    adds_encoder_output_bias = True

    def __init__(self):
        super().__init__()
        self.use_long_ctx_attn_kvcache = HAS_LONG_CTX_ATTN and get_sequence_parallel_world_size() > 1

    @eager_only
    def __call__(self, attn, hidden_states, encoder_hidden_states=None, attention_mask=None, *args,
                 skip_text_queries: bool = False, **kwargs):
        """``skip_text_queries``: the caller drops the text rows of the attention output (the SD3 block loop
        does for pipeline patches after the first), so the text stream only contributes keys and values: its
        q projection and its query rows are left out and ``None`` is returned for them."""
        H = attn.heads_per_device
        inner = attn.module.to_k.weight.shape[0]
        p_img, q_img, kv_img = _qkv_problems(hidden_states, attn._qkv, attn, inner, use_cache=True)
        B, N, _ = hidden_states.shape
        Nt = encoder_hidden_states.shape[1]
        dev = hidden_states.device
        o_img = torch.empty(B, N, inner, dtype=torch.bfloat16, device=dev)
        if skip_text_queries:
            wkv, bkv = attn._add_qkv.rows(inner, 2 * inner)
            kv_txt = torch.empty(B, Nt, 2 * inner, dtype=torch.bfloat16, device=dev)
            ops.gemm_launch(p_img + [ops.gemm_problem(_rows2d(encoder_hidden_states), wkv, kv_txt.view(-1, 2 * inner), bkv)])
            ops.attention(
                [_heads(q_img, H)],
                [_heads(kv_img[:, :, :inner], H), _heads(kv_txt[:, :, :inner], H)],
                [_heads(kv_img[:, :, inner:], H), _heads(kv_txt[:, :, inner:], H)],
                out=[_heads(o_img, H)],
                fp8=getattr(attn, "fp8_attention", False),
            )
            return o_img, None
        p_txt, q_txt, kv_txt = _qkv_problems(encoder_hidden_states, attn._add_qkv, attn, inner, use_cache=False)
        ops.gemm_launch(p_img + p_txt)
        o_txt = torch.empty(B, Nt, inner, dtype=torch.bfloat16, device=dev)
        ops.attention(
            [_heads(q_img, H), _heads(q_txt, H)],
            [_heads(kv_img[:, :, :inner], H), _heads(kv_txt[:, :, :inner], H)],
            [_heads(kv_img[:, :, inner:], H), _heads(kv_txt[:, :, inner:], H)],
            out=[_heads(o_img, H), _heads(o_txt, H)],
            fp8=getattr(attn, "fp8_attention", False),
        )
        return o_img, o_txt


def _norm_kind(norm) -> int:
    if norm is None:
        return 0
    return 1 if isinstance(norm, RMSNorm) else 2


def _norm_eps(attn) -> float:
    n = attn.module.norm_q
    return float(n.eps) if n is not None else 1e-6


def _norm_wb(norm):
    if norm is None:
        return None, None
    w = norm.weight.data if norm.weight is not None else None
    b = getattr(norm, "bias", None)
    return w, (b.data if b is not None else None)


@hetuDiTAttentionProcessorRegister.register(FluxAttnProcessor2_0)
class hetuDiTFluxAttnProcessor2_0(FluxAttnProcessor2_0):
    """Flux: RMSNorm on q, k of both streams, joint order [text, image], RoPE on
    every joint token, image K/V through the stale buffer
    (``attention_processor.py:824-987``).  The wrapper's Flux branch never adds
    ``encoder_output_bias`` (``:284-305``), so neither does this path."""

    adds_encoder_output_bias = False

    def __init__(self):
        super().__init__()
        self.use_long_ctx_attn_kvcache = HAS_LONG_CTX_ATTN and get_sequence_parallel_world_size() > 1

    @eager_only
    def __call__(self, attn, hidden_states, encoder_hidden_states=None, attention_mask=None, image_rotary_emb=None,
                 *args, out=None, extra_problems=None, **kwargs):
        """``image_rotary_emb`` = (cos, sin) f32 [S_call, head_dim] over this call's
        joint [text, image] rows.  ``out`` (single-stream only) lets the caller
        place the attention output inside a wider buffer; ``extra_problems`` are
        GEMM problems launched together with the q|k|v projection (the
        single-stream block's MLP-in shares its input)."""
        extra_problems = list(extra_problems or [])
        m = attn.module
        H = attn.heads_per_device
        inner = m.to_k.weight.shape[0]
        hd = inner // H
        B = hidden_states.shape[0]
        dev = hidden_states.device
        cos, sin = image_rotary_emb if image_rotary_emb is not None else (None, None)
        eps = _norm_eps(attn)
        wq, _ = _norm_wb(m.norm_q)
        wk, _ = _norm_wb(m.norm_k)
        rng = _patch_range()
        jobs = []
        if encoder_hidden_states is not None:
            n_txt = encoder_hidden_states.shape[1]
            N = hidden_states.shape[1]
            if cos is not None and cos.shape[0] != n_txt + N:
                raise ValueError(f"image_rotary_emb has {cos.shape[0]} rows, this call's joint [text, image] "
                                 f"sequence has {n_txt + N}")
            p_img, q_img, kv_img = _qkv_problems(hidden_states, attn._qkv, attn, inner, use_cache=True)
            p_txt, q_txt, kv_txt = _qkv_problems(encoder_hidden_states, attn._add_qkv, attn, inner, use_cache=False)
            ops.gemm_launch(p_img + p_txt)
            waq, _ = _norm_wb(m.norm_added_q)
            wak, _ = _norm_wb(m.norm_added_k)
            k_new = kv_img[:, rng[0]:rng[1], :inner] if rng else kv_img[:, :, :inner]
            tc = (cos[:n_txt], sin[:n_txt]) if cos is not None else (None, None)
            ic = (cos[n_txt:n_txt + N], sin[n_txt:n_txt + N]) if cos is not None else (None, None)
            jobs = [
                ops.qk_norm_rope_job(_heads(q_txt, H), _norm_kind(m.norm_added_q), waq, None, *tc),
                ops.qk_norm_rope_job(_heads(kv_txt[:, :, :inner], H), _norm_kind(m.norm_added_k), wak, None, *tc),
                ops.qk_norm_rope_job(_heads(q_img, H), _norm_kind(m.norm_q), wq, None, *ic),
                ops.qk_norm_rope_job(_heads(k_new, H), _norm_kind(m.norm_k), wk, None, *ic),
            ]
            ops.qk_norm_rope(jobs, B, H, hd, eps)
            o_img = torch.empty(B, N, inner, dtype=torch.bfloat16, device=dev)
            o_txt = torch.empty(B, n_txt, inner, dtype=torch.bfloat16, device=dev)
            ops.attention(
                [_heads(q_txt, H), _heads(q_img, H)],
                [_heads(kv_txt[:, :, :inner], H), _heads(kv_img[:, :, :inner], H)],
                [_heads(kv_txt[:, :, inner:], H), _heads(kv_img[:, :, inner:], H)],
                out=[_heads(o_txt, H), _heads(o_img, H)],
                fp8=getattr(attn, "fp8_attention", False),
            )
            return o_img, o_txt

        # single-stream block: hidden_states is the joint [text, image] sequence
        n_txt = get_runtime_state().max_condition_sequence_length
        S = hidden_states.shape[1]
        N = S - n_txt
        if cos is not None and cos.shape[0] != S:
            raise ValueError(f"image_rotary_emb has {cos.shape[0]} rows, this call's joint sequence has {S}")
        x2 = _rows2d(hidden_states)
        w, b = attn._qkv.get()
        if rng is None:
            qkv = torch.empty(B, S, 3 * inner, dtype=torch.bfloat16, device=dev)
            ops.gemm_launch([ops.gemm_problem(x2, w, qkv.view(-1, 3 * inner), b)] + extra_problems)
            q = qkv[:, :, :inner]
            get_cache_manager()._entry(attn, "attn").tensors[0] = qkv[:, n_txt:, inner:]
            k_segs = [_heads(qkv[:, :, inner:2 * inner], H)]
            v_segs = [_heads(qkv[:, :, 2 * inner:], H)]
            jobs = [
                ops.qk_norm_rope_job(_heads(q, H), _norm_kind(m.norm_q), wq, None, cos, sin),
                ops.qk_norm_rope_job(k_segs[0], _norm_kind(m.norm_k), wk, None, cos, sin),
            ]
        else:
            # patch mode: text rows and the image patch rows form this call's joint input
            # The queries of all rows go to one [B, S, inner] tensor, the text rows' K|V to a small tensor of their
            # own, and the image rows' K|V straight into this patch's rows of the stale buffer (one problem per batch
            # element and destination: the destinations differ in batch stride) -- no copy afterwards.
            buf, start, end = get_cache_manager().kv_buffer(attn, B, N, inner, dev)
            q = torch.empty(B, S, inner, dtype=torch.bfloat16, device=dev)
            kv_txt = torch.empty(B, n_txt, 2 * inner, dtype=torch.bfloat16, device=dev)
            x3 = x2.view(B, S, -1)
            wq_, bq_ = attn._qkv.rows(0, inner)
            wkv, bkv = attn._qkv.rows(inner, 2 * inner)
            problems = [ops.gemm_problem(x2, wq_, q.view(-1, inner), bq_)]
            for bi in range(B):
                problems.append(ops.gemm_problem(x3[bi, :n_txt], wkv, kv_txt[bi], bkv))
                problems.append(ops.gemm_problem(x3[bi, n_txt:], wkv, buf[bi, start:end], bkv))
            ops.gemm_launch(problems + extra_problems)
            if cos is not None:
                qc, qs = cos, sin
                kc, ks = cos[n_txt:], sin[n_txt:]
                tc, ts = cos[:n_txt], sin[:n_txt]
            else:
                qc = qs = kc = ks = tc = ts = None
            k_txt = kv_txt[:, :, :inner]
            jobs = [
                ops.qk_norm_rope_job(_heads(q, H), _norm_kind(m.norm_q), wq, None, qc, qs),
                ops.qk_norm_rope_job(_heads(k_txt, H), _norm_kind(m.norm_k), wk, None, tc, ts),
                ops.qk_norm_rope_job(_heads(buf[:, start:end, :inner], H), _norm_kind(m.norm_k), wk, None, kc, ks),
            ]
            k_segs = [_heads(k_txt, H), _heads(buf[:, :, :inner], H)]
            v_segs = [_heads(kv_txt[:, :, inner:], H), _heads(buf[:, :, inner:], H)]
        ops.qk_norm_rope(jobs, B, H, hd, eps)
        if out is None:
            out = torch.empty(B, S, inner, dtype=torch.bfloat16, device=dev)
        ops.attention([_heads(q, H)], k_segs, v_segs, out=[_heads(out, H)], fp8=getattr(attn, "fp8_attention", False))
        return out


@hetuDiTAttentionProcessorRegister.register(CogVideoXAttnProcessor2_0)
class hetuDiTCogVideoXAttnProcessor2_0(CogVideoXAttnProcessor2_0):
    """CogVideoX: one projection set over the joint [text, video] rows,
    LayerNorm on q, k per head, RoPE on the video rows only, no KV-cache call;
    returns the joint attention output (``attention_processor.py:1022-1158``).
    The branch at ``:1085-1094`` is dead at one GPU because
    ``split_text_embed_in_sp`` is forced False."""

    adds_encoder_output_bias = False

    def __init__(self):
        super().__init__()
        self.use_long_ctx_attn_kvcache = HAS_LONG_CTX_ATTN and get_sequence_parallel_world_size() > 1

    @eager_only
    def __call__(self, attn, hidden_states, encoder_hidden_states, attention_mask=None, image_rotary_emb=None,
                 *args, joint_input: Optional[torch.Tensor] = None, **kwargs):
        """``joint_input``: optionally the already-assembled [B, S, D] joint rows
        (the fused block writes its two norm outputs into one buffer), in which
        case ``hidden_states`` / ``encoder_hidden_states`` are only read for
        their lengths."""
        assert not (get_pipeline_parallel_world_size() == 1 and get_runtime_state().split_text_embed_in_sp)
        m = attn.module
        H = attn.heads_per_device
        inner = m.to_k.weight.shape[0]
        hd = inner // H
        n_txt = encoder_hidden_states.size(1)
        n_img = hidden_states.size(1)
        B = hidden_states.shape[0]
        dev = hidden_states.device
        S = n_txt + n_img
        w, b = attn._qkv.get()
        qkv = torch.empty(B, S, 3 * inner, dtype=torch.bfloat16, device=dev)
        if joint_input is not None:
            problems = [ops.gemm_problem(_rows2d(joint_input), w, qkv.view(-1, 3 * inner), b)]
        else:
            problems = []
            xe, xh = encoder_hidden_states.contiguous(), hidden_states.contiguous()
            for bi in range(B):
                problems.append(ops.gemm_problem(xe[bi], w, qkv[bi, :n_txt], b))
                problems.append(ops.gemm_problem(xh[bi], w, qkv[bi, n_txt:], b))
        ops.gemm_launch(problems)
        q, k, v = qkv[:, :, :inner], qkv[:, :, inner:2 * inner], qkv[:, :, 2 * inner:]
        cos, sin = image_rotary_emb if image_rotary_emb is not None else (None, None)
        wq, bq = _norm_wb(m.norm_q)
        wk, bk = _norm_wb(m.norm_k)
        kcos, ksin = (cos, sin) if not m.is_cross_attention else (None, None)
        jobs = [
            ops.qk_norm_rope_job(_heads(q, H), _norm_kind(m.norm_q), wq, bq, cos, sin, rope_row0=n_txt),
            ops.qk_norm_rope_job(_heads(k, H), _norm_kind(m.norm_k), wk, bk, kcos, ksin, rope_row0=n_txt),
        ]
        if m.norm_q is not None or cos is not None:
            ops.qk_norm_rope(jobs, B, H, hd, _norm_eps(attn))
        out = torch.empty(B, S, inner, dtype=torch.bfloat16, device=dev)
        ops.attention([_heads(q, H)], [_heads(k, H)], [_heads(v, H)], out=[_heads(out, H)],
                      fp8=getattr(attn, "fp8_attention", False))
        assert n_txt + n_img == out.shape[1]
        return out
