"""Tensor-level entry to the C ABI: checks dtypes/devices, extracts pointers and
strides, enqueues on PyTorch's current HIP stream.  PyTorch is only the owner
of device memory and streams here; every computation happens in ``libhdit.so``.

The same functions are registered as ``torch.ops.hdit.*`` custom ops (with
fake/meta kernels) in ``torch_ops.py`` for callers that trace the model.
"""
import ctypes as C
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import EPI_BIAS, EPI_BIAS_GELU, EPI_GATE_RESIDUAL, AttnArgs, GemmProblem, QkNormJob, check

bf16 = torch.bfloat16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class KernelTimer:
    """Optional per-launch HIP-event timing on the launch stream.  When a timer
    is installed (``set_timer``) every C-ABI launch is bracketed by a pair of
    events on PyTorch's current stream -- the stream the kernel runs on -- and
    logged as (kernel class, algorithmic work, events).  ``work`` is flops for
    the MFMA kernels and bytes for the bandwidth-bound ones."""

    def __init__(self):
        self.records = []

    def summary(self):
        """class -> (launches, total ms, total work)"""
        out = {}
        for kind, work, e0, e1 in self.records:
            n, ms, w = out.get(kind, (0, 0.0, 0.0))
            out[kind] = (n + 1, ms + e0.elapsed_time(e1), w + work)
        return out


_TIMER: Optional[KernelTimer] = None


def set_timer(timer: Optional[KernelTimer]):
    global _TIMER
    _TIMER = timer


def _run(kind: str, work: float, call):
    t = _TIMER
    if t is None:
        return call()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    rc = call()
    e1.record()
    t.records.append((kind, work, e0, e1))
    return rc


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, dtype, name: str):
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")


# ---------------------------------------------------------------------------
# grouped GEMM
# ---------------------------------------------------------------------------

def gemm_problem(
    a: torch.Tensor,
    w: torch.Tensor,
    out: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    epilogue: int = EPI_BIAS,
    resid: Optional[torch.Tensor] = None,
    gate: Optional[torch.Tensor] = None,
    rows_per_batch: int = 0,
) -> GemmProblem:
    """Describe out[m, n] = epilogue(a[m, k] @ w[n, k]^T + bias).

    a, out (and resid) are 2-D views with unit inner stride (row stride free);
    gate is an f32 [batch, n] view with unit inner stride.  In the gated-residual
    epilogue ``resid`` and ``out`` may each be f32 instead of bf16 (the residual
    stream of a block stack carried in fp32)."""
    _need(a, bf16, "a"), _need(w, bf16, "w")
    if epilogue == EPI_GATE_RESIDUAL and out.dtype == torch.float32:
        _need(out, torch.float32, "out")
        epilogue |= _lib.EPI_OUT_F32
    else:
        _need(out, bf16, "out")
    m, k = a.shape
    n, k2 = w.shape
    if k2 != k or tuple(out.shape) != (m, n):
        raise ValueError(f"gemm shapes do not agree: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(1) != 1:
        raise ValueError("gemm operands need a unit inner stride")
    p = GemmProblem()
    p.a, p.b, p.c = a.data_ptr(), w.data_ptr(), out.data_ptr()
    p.lda, p.ldb, p.ldc = a.stride(0) if m > 1 else k, w.stride(0), out.stride(0) if m > 1 else n
    p.m, p.n, p.k = m, n, k
    p.epilogue = epilogue
    if bias is not None:
        _need(bias, bf16, "bias")
        if bias.numel() != n or not bias.is_contiguous():
            raise ValueError("bias must be a contiguous [n] vector")
        p.bias = bias.data_ptr()
    if epilogue & 0xF == EPI_GATE_RESIDUAL:
        if resid is not None and resid.dtype == torch.float32:
            epilogue |= _lib.EPI_RESID_F32
        _need(resid, torch.float32 if epilogue & _lib.EPI_RESID_F32 else bf16, "resid"), _need(gate, torch.float32, "gate")
        p.epilogue = epilogue
        if tuple(resid.shape) != (m, n) or resid.stride(1) != 1:
            raise ValueError("resid must be [m, n] with unit inner stride")
        if gate.dim() != 2 or gate.shape[1] != n or gate.stride(1) != 1:
            raise ValueError("gate must be [batch, n] with unit inner stride")
        if rows_per_batch <= 0 or m > rows_per_batch * gate.shape[0]:
            raise ValueError("rows_per_batch does not cover m")
        p.resid, p.gate = resid.data_ptr(), gate.data_ptr()
        p.ldr = resid.stride(0) if m > 1 else n
        p.rows_per_batch, p.gate_stride = rows_per_batch, gate.stride(0) if gate.shape[0] > 1 else n
    p._keep = (a, w, out, bias, resid, gate)  # the struct only holds raw pointers
    return p


def gemm_launch(problems: Sequence[GemmProblem]):
    """One call of the grouped GEMM per HDIT_GEMM_MAX_PROBLEMS problems (a call plans its problems together)."""
    for first in range(0, len(problems), _lib.HDIT_GEMM_MAX_PROBLEMS):
        chunk = problems[first : first + _lib.HDIT_GEMM_MAX_PROBLEMS]
        n = len(chunk)
        arr = (GemmProblem * n)(*chunk)
        flops = sum(2.0 * p.m * p.n * p.k for p in chunk) if _TIMER is not None else 0.0
        check(_run("gemm", flops, lambda: _lib.lib().hdit_gemm_bf16(arr, n, _stream())), "hdit_gemm_bf16")


def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, gelu: bool = False,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w^T + bias (optionally GELU-tanh) on [..., k] bf16 input."""
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    if out is None:
        out = torch.empty(*lead, w.shape[0], dtype=bf16, device=x.device)
    gemm_launch([gemm_problem(x2, w, out.view(-1, w.shape[0]), bias, EPI_BIAS_GELU if gelu else EPI_BIAS)])
    return out


# ---------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------

def _fill_segments(dst, tensors: Sequence[torch.Tensor], name: str) -> Tuple[int, int, int, int]:
    """tensors: 1 or 2 views [B, S, H, d] with unit stride on d."""
    if not 1 <= len(tensors) <= 2:
        raise ValueError(f"{name}: one or two segments expected")
    B, _, H, D = tensors[0].shape
    total = 0
    for i, t in enumerate(tensors):
        _need(t, bf16, name)
        if t.dim() != 4 or t.shape[0] != B or t.shape[2] != H or t.shape[3] != D:
            raise ValueError(f"{name}: segment shapes disagree")
        if t.stride(3) != 1:
            raise ValueError(f"{name}: head_dim must be contiguous")
        dst[i].ptr = t.data_ptr()
        dst[i].stride_b, dst[i].stride_s, dst[i].stride_h = t.stride(0), t.stride(1), t.stride(2)
        dst[i].len = t.shape[1]
        total += t.shape[1]
    return B, total, H, D


def attention_args(q, k, v, o, scale: float = 0.0) -> AttnArgs:
    a = AttnArgs()
    B, sq, H, D = _fill_segments(a.q, q, "q")
    Bk, skv, Hk, Dk = _fill_segments(a.k, k, "k")
    Bv, skv2, Hv, Dv = _fill_segments(a.v, v, "v")
    Bo, so, Ho, Do = _fill_segments(a.o, o, "o")
    if (Bk, Hk, Dk) != (B, H, D) or (Bv, Hv, Dv) != (B, H, D) or (Bo, Ho, Do) != (B, H, D) or so != sq or skv2 != skv:
        raise ValueError("attention operand shapes disagree")
    a.batch, a.heads, a.head_dim, a.scale = B, H, D, scale
    a._keep = (tuple(q), tuple(k), tuple(v), tuple(o))
    return a


def attention(q: Sequence[torch.Tensor], k: Sequence[torch.Tensor], v: Sequence[torch.Tensor],
              out: Optional[Sequence[torch.Tensor]] = None, scale: float = 0.0, fp8: bool = False):
    """Joint non-causal attention.  q/k/v are lists of one or two [B, S, H, d]
    bf16 views (the segments of the joint sequence).  Returns the list of
    output segments (allocated [B, S, H, d] contiguous when not given)."""
    if out is None:
        out = [torch.empty(t.shape, dtype=bf16, device=t.device) for t in q]
    args = attention_args(q, k, v, out, scale)
    lib = _lib.lib()
    sq, skv = sum(t.shape[1] for t in q), sum(t.shape[1] for t in k)
    flops = 4.0 * args.batch * args.heads * sq * skv * args.head_dim
    if fp8:
        absmax = torch.empty(3, args.batch, args.heads, dtype=torch.float32, device=q[0].device)
        nbytes = 2.0 * args.batch * args.heads * args.head_dim * (sq + 2 * skv)
        check(_run("attn_absmax", nbytes, lambda: lib.hdit_attn_absmax(C.byref(args), absmax.data_ptr(), _stream())),
              "hdit_attn_absmax")
        ws = torch.empty(lib.hdit_attn_fp8_workspace_bytes(C.byref(args)), dtype=torch.uint8, device=q[0].device)
        check(_run("attn_fp8", flops,
                   lambda: lib.hdit_attn_fwd_fp8(C.byref(args), absmax.data_ptr(), ws.data_ptr(), _stream())),
              "hdit_attn_fwd_fp8")
    else:
        check(_run("attn_bf16", flops, lambda: lib.hdit_attn_fwd_bf16(C.byref(args), _stream())), "hdit_attn_fwd_bf16")
    return list(out)


def attention_fp8_absmax(args: AttnArgs) -> torch.Tensor:
    """f32 [3, batch, heads] absmax of q, k, v per (batch, head): the scales of the fp8 path."""
    dev = args._keep[0][0].device
    absmax = torch.empty(3, args.batch, args.heads, dtype=torch.float32, device=dev)
    check(_lib.lib().hdit_attn_absmax(C.byref(args), absmax.data_ptr(), _stream()), "hdit_attn_absmax")
    return absmax


def attention_fp8_static(args: AttnArgs, absmax: torch.Tensor):
    """fp8 attention through the entry point that allocates nothing: the quantised K / V copy lives in a
    fixed array inside the library (``HDIT_ATTN_FP8_STATIC_MAX_BYTES`` per GPU) instead of a workspace.
    Calls on one GPU share that array and must not overlap."""
    _need(absmax, torch.float32, "absmax")
    if tuple(absmax.shape) != (3, args.batch, args.heads) or not absmax.is_contiguous():
        raise ValueError("absmax must be a contiguous f32 [3, batch, heads] tensor")
    check(_lib.lib().hdit_attn_fwd_fp8_static(C.byref(args), absmax.data_ptr(), _stream()), "hdit_attn_fwd_fp8_static")


# ---------------------------------------------------------------------------
# whole-block entry point
# ---------------------------------------------------------------------------

def block_sd3(block, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, temb: torch.Tensor,
              out_dtype=bf16, skip_text_output: bool = False, kv_buffer: Optional[torch.Tensor] = None, kv_row0: int = 0):
    """One SD3 joint block through ``hdit_block_sd3`` -- the single C-ABI call a non-Python host would make --
    with the weights of a ``JointTransformerBlock``.  Returns ``(encoder_or_None, hidden)`` like the block.
    ``kv_buffer``: bf16 [B, rows, 2*dim] stale K|V buffer of a PipeFusion patch whose rows
    ``[kv_row0, kv_row0 + n_img)`` this call overwrites."""
    attn, m = block.attn, block.attn.module
    B, Ni, D = hidden_states.shape
    Nt = encoder_hidden_states.shape[1]
    for t, name in ((hidden_states, "hidden_states"), (encoder_hidden_states, "encoder_hidden_states")):
        if not t.is_cuda or t.dtype not in (bf16, torch.float32) or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous bf16 or f32 GPU tensor")
    _need(temb, bf16, "temb")
    qkv_w, qkv_b = attn._qkv.get()
    aqkv_w, aqkv_b = attn._add_qkv.get()
    pre_only = bool(block.context_pre_only)
    a = _lib.Sd3BlockArgs()
    keep = [qkv_w, qkv_b, aqkv_w, aqkv_b]

    def ptr(t):
        if t is None:
            return None
        keep.append(t)
        return t.data_ptr()

    w = a.w
    w.norm1_w, w.norm1_b = ptr(block.norm1.linear.weight.data), ptr(block.norm1.linear.bias.data)
    w.norm1_context_w, w.norm1_context_b = ptr(block.norm1_context.linear.weight.data), ptr(block.norm1_context.linear.bias.data)
    w.qkv_w, w.qkv_b, w.add_qkv_w, w.add_qkv_b = ptr(qkv_w), ptr(qkv_b), ptr(aqkv_w), ptr(aqkv_b)
    w.to_out_w = ptr(m.to_out[0].weight.data)
    w.to_out_b = ptr(attn.output_bias.data) if attn.has_output_bias else None
    if not pre_only:
        w.to_add_out_w = ptr(m.to_add_out.weight.data)
        w.to_add_out_b = ptr(attn.encoder_output_bias.data) if attn.has_encoder_output_bias else None
    ff = block.ff
    w.ff_in_w, w.ff_in_b = ptr(ff.module.net[0].proj.weight.data), ptr(ff.module.net[0].proj.bias.data)
    w.ff_out_w = ptr(ff.module.net[2].weight.data)
    w.ff_out_b = ptr(ff.output_bias.data) if ff.has_output_bias else None
    if block.ff_context is not None:
        fc = block.ff_context
        w.ff_context_in_w, w.ff_context_in_b = ptr(fc.module.net[0].proj.weight.data), ptr(fc.module.net[0].proj.bias.data)
        w.ff_context_out_w = ptr(fc.module.net[2].weight.data)
        w.ff_context_out_b = ptr(fc.output_bias.data) if fc.has_output_bias else None
    text_out = not pre_only and not skip_text_output
    hidden_out = torch.empty(B, Ni, D, dtype=out_dtype, device=hidden_states.device)
    encoder_out = torch.empty(B, Nt, D, dtype=out_dtype, device=hidden_states.device) if text_out else None
    temb = temb.contiguous()  # bound to a name and kept below: a temporary's memory could be handed to the workspace
    a.hidden, a.encoder, a.temb = hidden_states.data_ptr(), encoder_hidden_states.data_ptr(), temb.data_ptr()
    a.hidden_out, a.encoder_out = hidden_out.data_ptr(), (encoder_out.data_ptr() if text_out else None)
    a.batch, a.n_img, a.n_txt, a.dim, a.heads = B, Ni, Nt, D, attn.heads_per_device
    a.ff_dim, a.temb_dim = ff.module.net[0].proj.weight.shape[0], temb.shape[1]
    a.hidden_f32, a.encoder_f32 = int(hidden_states.dtype == torch.float32), int(encoder_hidden_states.dtype == torch.float32)
    a.out_f32 = int(out_dtype == torch.float32)
    a.context_pre_only, a.skip_text_output = int(pre_only), int(skip_text_output)
    if kv_buffer is not None:
        _need(kv_buffer, bf16, "kv_buffer")
        if tuple(kv_buffer.shape[::2]) != (B, 2 * D) or not kv_buffer.is_contiguous():
            raise ValueError("kv_buffer must be a contiguous bf16 [batch, rows, 2 * dim] tensor")
        a.kv_buffer, a.kv_rows, a.kv_row0 = kv_buffer.data_ptr(), kv_buffer.shape[1], kv_row0
    lib = _lib.lib()
    nbytes = lib.hdit_block_sd3_workspace_bytes(C.byref(a))
    if nbytes < 0:
        raise _lib.HditError("hdit_block_sd3_workspace_bytes refused the arguments")
    ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=hidden_states.device)
    base = (ws.data_ptr() + 255) // 256 * 256
    a.workspace, a.workspace_bytes = base, nbytes
    check(lib.hdit_block_sd3(C.byref(a), _stream()), "hdit_block_sd3")
    a._keep = (keep, ws, hidden_states, encoder_hidden_states, temb, kv_buffer)
    return encoder_out, hidden_out


def timer_installed() -> bool:
    """True while ``set_timer`` has a per-launch timer in place (the whole-block calls launch from C and are
    not seen by it, so callers that want per-kernel times take the per-kernel path)."""
    return _TIMER is not None


class Sd3BlockCall:
    """A reusable ``hdit_block_sd3`` call for one ``JointTransformerBlock``.

    The weight pointers and the block's geometry are written into the argument struct once (``refresh``
    re-reads them, e.g. after a weight hot-swap re-assigned a ``.data``); a call only sets the stream tensors,
    the modulation and K/V buffer pointers and the flags, which keeps the host cost of a block at one foreign
    call -- what a block stack launched eagerly on several streams needs.  The struct is rewritten by every call
    (the library copies it before returning), so one object serves any number of streams from ONE host thread at
    a time."""

    def __init__(self, block):
        self.block = block
        self.args = _lib.Sd3BlockArgs()
        self._ws_bytes = {}
        self.refresh()

    @staticmethod
    def describes(block) -> bool:
        """Whether ``block`` has the sub-modules the entry point's weight table is filled from (an explicit
        check of the structure, so that a genuine ``AttributeError`` in ``refresh`` is not mistaken for it)."""
        from .layers.attention_processor import hetuDiTAttentionWrapper
        from .layers.feedforward import hetuDiTFeedForwardWrapper

        def adaln(n):
            return isinstance(getattr(n, "linear", None), torch.nn.Linear) and n.linear.bias is not None

        attn = getattr(block, "attn", None)
        if not isinstance(attn, hetuDiTAttentionWrapper) or getattr(attn, "_add_qkv", None) is None:
            return False
        if not (adaln(getattr(block, "norm1", None)) and adaln(getattr(block, "norm1_context", None))):
            return False
        ffs = [getattr(block, "ff", None)]
        if not getattr(block, "context_pre_only", False):
            ffs.append(getattr(block, "ff_context", None))
            if getattr(attn.module, "to_add_out", None) is None:
                return False
        return all(isinstance(f, hetuDiTFeedForwardWrapper) and f.module.net[0].proj.bias is not None for f in ffs)

    def refresh(self):
        block, a = self.block, self.args
        fill = _ArgFiller()
        _fill_sd3_weights(a.w, block, fill)
        self._weights = fill.keep
        a.dim = block.norm1.linear.weight.shape[1]
        a.heads = block.attn.heads_per_device
        a.ff_dim = block.ff.module.net[0].proj.weight.shape[0]
        a.temb_dim = block.norm1.linear.weight.shape[1]
        a.context_pre_only = int(bool(block.context_pre_only))
        a.fp8_attention = int(bool(getattr(block.attn, "fp8_attention", False)))

    def __call__(self, *args, **kwargs):
        """Fill the argument struct (``prepare``) and launch the block on the current stream."""
        encoder_out, hidden_out, ws = self.prepare(*args, **kwargs)
        self.launch()
        # stream-ordered reuse: the workspace may be freed as soon as the launches are queued
        del ws
        return encoder_out, hidden_out

    def launch(self):
        """Enqueue the block described by ``self.args`` (filled by ``prepare``) on the current stream."""
        check(_lib.lib().hdit_block_sd3(C.byref(self.args), _stream()), "hdit_block_sd3")

    def prepare(self, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor, temb: torch.Tensor,
                out_dtype=bf16, skip_text_output: bool = False, kv_buffer: Optional[torch.Tensor] = None,
                kv_row0: int = 0, modulation_img: Optional[int] = None, modulation_txt: Optional[int] = None,
                hidden_out: Optional[torch.Tensor] = None, text_kv: Optional[torch.Tensor] = None,
                text_kv_mode: int = _lib.TEXT_KV_NONE, pending_img=None, pending_txt=None, defer: bool = False,
                lazy: bool = False):
        """Fills ``self.args`` for one call without launching; returns ``(encoder_out_or_None, hidden_out,
        workspace tensor)`` -- the caller launches (``hdit_block_sd3`` or, with other blocks' structs,
        ``sd3_blocks_launch``) and keeps the workspace alive until then.
        Same contract as ``block_sd3``.  ``modulation_img`` / ``modulation_txt``: device addresses of the f32
        [batch, 6 dim] (text stream of a ``context_pre_only`` block: [batch, 2 dim]) adaLN projections of this
        block for this ``temb`` (the caller keeps their tensor alive), or None to have the call compute them.
        ``hidden_out``: a contiguous [batch, n_img, dim] tensor of ``out_dtype`` to write the image stream to.
        ``text_kv`` / ``text_kv_mode``: bf16 [batch, n_txt, 2 dim] buffer of the text stream's keys | values that
        this call fills (``TEXT_KV_STORE``) or, with ``skip_text_output``, takes as they are (``TEXT_KV_REUSE``).
        ``pending_img`` / ``pending_txt``: ``(y, gate address, gate batch stride)`` -- an update ``gate * y`` the
        previous block of the chain left owing to the f32 stream it hands over; this block's first normalisation
        adds it.  ``defer`` (f32 output, modulation given): the MLP residuals of this block are left owing in the
        same way; ``self.deferred`` is then ``(pending_img, pending_txt_or_None)`` for the next block.  ``lazy``:
        inside the block the attention residual of an f32 stream is added by norm2 rather than by the out-projection."""
        a = self.args
        B, Ni, D = hidden_states.shape
        Nt = encoder_hidden_states.shape[1]
        if D != a.dim or encoder_hidden_states.shape[2] != D or encoder_hidden_states.shape[0] != B:
            raise ValueError("stream shapes do not match the block")
        a.hidden_f32 = _stream_tensor(hidden_states, "hidden_states")
        a.encoder_f32 = _stream_tensor(encoder_hidden_states, "encoder_hidden_states")
        _need(temb, bf16, "temb")
        if temb.shape != (B, a.temb_dim) or not temb.is_contiguous():
            raise ValueError("temb must be a contiguous [batch, dim] tensor")
        dev = hidden_states.device
        text_out = not a.context_pre_only and not skip_text_output
        if hidden_out is None:
            hidden_out = torch.empty(B, Ni, D, dtype=out_dtype, device=dev)
        elif hidden_out.shape != (B, Ni, D) or hidden_out.dtype != out_dtype or not hidden_out.is_contiguous():
            raise ValueError("hidden_out must be a contiguous [batch, n_img, dim] tensor of out_dtype")
        encoder_out = torch.empty(B, Nt, D, dtype=out_dtype, device=dev) if text_out else None
        a.hidden, a.encoder, a.temb = hidden_states.data_ptr(), encoder_hidden_states.data_ptr(), temb.data_ptr()
        a.hidden_out, a.encoder_out = hidden_out.data_ptr(), (encoder_out.data_ptr() if text_out else None)
        a.modulation_img, a.modulation_txt = modulation_img, modulation_txt
        a.batch, a.n_img, a.n_txt = B, Ni, Nt
        a.out_f32, a.skip_text_output = int(out_dtype == torch.float32), int(skip_text_output)
        if kv_buffer is not None:
            if kv_buffer.dtype != bf16 or kv_buffer.dim() != 3 or tuple(kv_buffer.shape[::2]) != (B, 2 * D) \
                    or not kv_buffer.is_contiguous():
                raise ValueError("kv_buffer must be a contiguous bf16 [batch, rows, 2 * dim] tensor")
            a.kv_buffer, a.kv_rows, a.kv_row0 = kv_buffer.data_ptr(), kv_buffer.shape[1], kv_row0
        else:
            a.kv_buffer, a.kv_rows, a.kv_row0 = None, 0, 0
        if text_kv_mode != _lib.TEXT_KV_NONE:
            if text_kv is None or text_kv.dtype != bf16 or tuple(text_kv.shape) != (B, Nt, 2 * D) or not text_kv.is_contiguous():
                raise ValueError("text_kv must be a contiguous bf16 [batch, n_txt, 2 * dim] tensor")
            a.text_kv, a.text_kv_mode = text_kv.data_ptr(), text_kv_mode
        else:
            a.text_kv, a.text_kv_mode = None, _lib.TEXT_KV_NONE
        for name, pend, rows, f32 in (("img", pending_img, Ni, a.hidden_f32), ("txt", pending_txt, Nt, a.encoder_f32)):
            if pend is None:
                setattr(a, f"pending_{name}", None), setattr(a, f"pending_{name}_gate", None)
                setattr(a, f"pending_{name}_gate_stride", 0)
                continue
            y, gate, stride = pend
            if not f32 or y.dtype != bf16 or tuple(y.shape) != (B, rows, D) or not y.is_contiguous():
                raise ValueError("a pending update is a contiguous bf16 tensor of the shape of its f32 stream")
            setattr(a, f"pending_{name}", y.data_ptr()), setattr(a, f"pending_{name}_gate", gate)
            setattr(a, f"pending_{name}_gate_stride", stride)
        self._pending = (pending_img, pending_txt)
        self.deferred = None
        a.defer_img = a.defer_txt = None
        a.lazy_residual = int(bool(defer or lazy))
        if defer:
            if out_dtype != torch.float32 or modulation_img is None or (text_out and modulation_txt is None):
                raise ValueError("residuals can only be left to the next block on an f32 stream with the modulation given")
            d_img = torch.empty(B, Ni, D, dtype=bf16, device=dev)
            d_txt = torch.empty(B, Nt, D, dtype=bf16, device=dev) if text_out else None
            a.defer_img, a.defer_txt = d_img.data_ptr(), (d_txt.data_ptr() if text_out else None)
            # gate_mlp is the sixth chunk of a stream's modulation
            self.deferred = ((d_img, modulation_img + 4 * 5 * D, 6 * D), (d_txt, modulation_txt + 4 * 5 * D, 6 * D) if text_out else None)
        lib = _lib.lib()
        key = (B, Ni, Nt, bool(skip_text_output), a.kv_rows, text_kv_mode, a.fp8_attention)
        nbytes = self._ws_bytes.get(key)
        if nbytes is None:
            nbytes = lib.hdit_block_sd3_workspace_bytes(C.byref(a))
            if nbytes < 0:
                raise _lib.HditError("hdit_block_sd3_workspace_bytes refused the arguments")
            self._ws_bytes[key] = nbytes
        ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=dev)
        a.workspace, a.workspace_bytes = (ws.data_ptr() + 255) // 256 * 256, nbytes
        return encoder_out, hidden_out, ws


def sd3_blocks_launch(calls: Sequence["Sd3BlockCall"]):
    """The prepared calls -- blocks that do not depend on each other -- as one ``hdit_block_sd3_multi`` call per
    ``HDIT_BLOCK_MAX_MULTI``: every stage of the blocks (normalise, q|k|v, attention, ...) is one merged launch."""
    lib = _lib.lib()
    for first in range(0, len(calls), _lib.HDIT_BLOCK_MAX_MULTI):
        chunk = calls[first : first + _lib.HDIT_BLOCK_MAX_MULTI]
        arr = (_lib.Sd3BlockArgs * len(chunk))(*(c.args for c in chunk))
        check(lib.hdit_block_sd3_multi(arr, len(chunk), _stream()), "hdit_block_sd3_multi")


class _ArgFiller:
    """Pointer bookkeeping for the whole-block argument structs: keeps every tensor alive whose address went in."""

    def __init__(self):
        self.keep = []

    def __call__(self, t):
        if t is None:
            return None
        self.keep.append(t)
        return t.data_ptr()


def _stream_tensor(t: torch.Tensor, name: str) -> int:
    if not t.is_cuda or t.dtype not in (bf16, torch.float32) or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous bf16 or f32 GPU tensor")
    return int(t.dtype == torch.float32)


def _run_block(a, size_fn, run_fn, what: str, device, keep):
    nbytes = size_fn(C.byref(a))
    if nbytes < 0:
        raise _lib.HditError(f"{what}_workspace_bytes refused the arguments")
    ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=device)
    a.workspace, a.workspace_bytes = (ws.data_ptr() + 255) // 256 * 256, nbytes
    check(run_fn(C.byref(a), _stream()), what)
    a._keep = (keep, ws)


def _norm_kind_of(norm) -> int:
    if norm is None:
        return 0
    return 2 if isinstance(norm, torch.nn.LayerNorm) else 1


def _fill_sd3_weights(w, block, ptr):
    attn, m = block.attn, block.attn.module
    qkv_w, qkv_b = attn._qkv.get()
    aqkv_w, aqkv_b = attn._add_qkv.get()
    w.norm1_w, w.norm1_b = ptr(block.norm1.linear.weight.data), ptr(block.norm1.linear.bias.data)
    w.norm1_context_w, w.norm1_context_b = ptr(block.norm1_context.linear.weight.data), ptr(block.norm1_context.linear.bias.data)
    w.qkv_w, w.qkv_b, w.add_qkv_w, w.add_qkv_b = ptr(qkv_w), ptr(qkv_b), ptr(aqkv_w), ptr(aqkv_b)
    w.to_out_w = ptr(m.to_out[0].weight.data)
    w.to_out_b = ptr(attn.output_bias.data) if attn.has_output_bias else None
    if getattr(m, "to_add_out", None) is not None and not m.context_pre_only:
        w.to_add_out_w = ptr(m.to_add_out.weight.data)
        w.to_add_out_b = ptr(attn.encoder_output_bias.data) if attn.has_encoder_output_bias else None
    for prefix, ff in (("ff", block.ff), ("ff_context", getattr(block, "ff_context", None))):
        if ff is None:
            continue
        setattr(w, prefix + "_in_w", ptr(ff.module.net[0].proj.weight.data))
        setattr(w, prefix + "_in_b", ptr(ff.module.net[0].proj.bias.data))
        setattr(w, prefix + "_out_w", ptr(ff.module.net[2].weight.data))
        setattr(w, prefix + "_out_b", ptr(ff.output_bias.data) if ff.has_output_bias else None)


def _kv_buffer_args(a, kv_buffer, kv_row0: int, batch: int, rows: int, dim: int, keep):
    """``kv_buffer``: contiguous bf16 [batch, kv_rows, 2 dim] K|V buffer of the layer whose rows
    ``[kv_row0, kv_row0 + rows)`` the call writes."""
    if kv_buffer is None:
        return
    _need(kv_buffer, bf16, "kv_buffer")
    if kv_buffer.dim() != 3 or tuple(kv_buffer.shape[::2]) != (batch, 2 * dim) or not kv_buffer.is_contiguous():
        raise ValueError("kv_buffer must be a contiguous bf16 [batch, rows, 2 * dim] tensor")
    if kv_row0 < 0 or kv_row0 + rows > kv_buffer.shape[1]:
        raise ValueError("kv_row0 + rows exceeds the K/V buffer")
    a.kv_buffer, a.kv_rows, a.kv_row0 = kv_buffer.data_ptr(), kv_buffer.shape[1], kv_row0
    keep.append(kv_buffer)


def block_flux_double(block, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None, out_dtype=bf16,
                      kv_buffer=None, kv_row0: int = 0, modulation_img: Optional[int] = None,
                      modulation_txt: Optional[int] = None):
    """One Flux double-stream block through ``hdit_block_flux_double``; returns ``(encoder, hidden)``.
    ``kv_buffer`` / ``kv_row0``: the image stream's K|V buffer of the layer and the first row this call writes
    (a pipeline patch attends to all its rows).  ``modulation_*``: device addresses of precomputed f32
    [batch, 6 dim] adaLN projections (the caller keeps their tensor alive)."""
    attn, m = block.attn, block.attn.module
    B, Ni, D = hidden_states.shape
    Nt = encoder_hidden_states.shape[1]
    _need(temb, bf16, "temb")
    a, ptr = _lib.FluxDoubleBlockArgs(), _ArgFiller()
    _fill_sd3_weights(a.w, block, ptr)
    for name in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"):
        n = getattr(m, name)
        setattr(a, name + "_w", ptr(n.weight.data) if n is not None and n.weight is not None else None)
    a.qk_norm_kind, a.qk_norm_eps = _norm_kind_of(m.norm_q), float(m.norm_q.eps) if m.norm_q is not None else 1e-6
    a.hidden_f32, a.encoder_f32 = _stream_tensor(hidden_states, "hidden_states"), _stream_tensor(encoder_hidden_states, "encoder_hidden_states")
    if image_rotary_emb is not None:
        cos, sin = image_rotary_emb
        _need(cos, torch.float32, "cos"), _need(sin, torch.float32, "sin")
        if tuple(cos.shape) != (Nt + Ni, D // attn.heads_per_device) or cos.shape != sin.shape or not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("image_rotary_emb must be contiguous f32 [n_txt + n_img, head_dim] tables")
        a.rope_cos, a.rope_sin = ptr(cos), ptr(sin)
    hidden_out = torch.empty(B, Ni, D, dtype=out_dtype, device=hidden_states.device)
    encoder_out = torch.empty(B, Nt, D, dtype=out_dtype, device=hidden_states.device)
    a.hidden, a.encoder, a.temb = ptr(hidden_states), ptr(encoder_hidden_states), ptr(temb.contiguous())
    a.hidden_out, a.encoder_out, a.out_f32 = hidden_out.data_ptr(), encoder_out.data_ptr(), int(out_dtype == torch.float32)
    a.batch, a.n_img, a.n_txt, a.dim, a.heads = B, Ni, Nt, D, attn.heads_per_device
    a.ff_dim, a.temb_dim = block.ff.module.net[0].proj.weight.shape[0], temb.shape[1]
    a.modulation_img, a.modulation_txt = modulation_img, modulation_txt
    _kv_buffer_args(a, kv_buffer, kv_row0, B, Ni, D, ptr.keep)
    lib = _lib.lib()
    _run_block(a, lib.hdit_block_flux_double_workspace_bytes, lib.hdit_block_flux_double, "hdit_block_flux_double",
               hidden_states.device, ptr.keep)
    return encoder_out, hidden_out


def block_flux_single(block, hidden_states, temb, image_rotary_emb=None, out_dtype=bf16, kv_buffer=None, kv_row0: int = 0,
                      n_txt: int = 0, modulation: Optional[int] = None):
    """One Flux single-stream block through ``hdit_block_flux_single`` on the joint [text, image] rows.
    ``kv_buffer`` / ``kv_row0`` / ``n_txt``: the layer's K|V buffer for the image rows (the rows behind the first
    ``n_txt``); ``modulation``: device address of the precomputed f32 [batch, 3 dim] adaLN projection."""
    attn, m = block.attn, block.attn.module
    B, S, D = hidden_states.shape
    _need(temb, bf16, "temb")
    a, ptr = _lib.FluxSingleBlockArgs(), _ArgFiller()
    qkv_w, qkv_b = attn._qkv.get()
    a.norm_w, a.norm_b = ptr(block.norm.linear.weight.data), ptr(block.norm.linear.bias.data)
    a.qkv_w, a.qkv_b = ptr(qkv_w), ptr(qkv_b)
    a.proj_mlp_w, a.proj_mlp_b = ptr(block.proj_mlp.weight.data), ptr(block.proj_mlp.bias.data)
    a.proj_out_w, a.proj_out_b = ptr(block.proj_out.weight.data), ptr(block.proj_out.bias.data)
    for name in ("norm_q", "norm_k"):
        n = getattr(m, name)
        setattr(a, name + "_w", ptr(n.weight.data) if n is not None and n.weight is not None else None)
    a.qk_norm_kind, a.qk_norm_eps = _norm_kind_of(m.norm_q), float(m.norm_q.eps) if m.norm_q is not None else 1e-6
    a.hidden_f32 = _stream_tensor(hidden_states, "hidden_states")
    if image_rotary_emb is not None:
        cos, sin = image_rotary_emb
        _need(cos, torch.float32, "cos"), _need(sin, torch.float32, "sin")
        if tuple(cos.shape) != (S, D // attn.heads_per_device) or cos.shape != sin.shape or not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("image_rotary_emb must be contiguous f32 [seq, head_dim] tables")
        a.rope_cos, a.rope_sin = ptr(cos), ptr(sin)
    hidden_out = torch.empty(B, S, D, dtype=out_dtype, device=hidden_states.device)
    a.hidden, a.temb, a.hidden_out, a.out_f32 = ptr(hidden_states), ptr(temb.contiguous()), hidden_out.data_ptr(), int(out_dtype == torch.float32)
    a.batch, a.seq, a.dim, a.heads, a.ff_dim, a.temb_dim = B, S, D, attn.heads_per_device, block.mlp_hidden_dim, temb.shape[1]
    a.modulation, a.n_txt = modulation, n_txt
    _kv_buffer_args(a, kv_buffer, kv_row0, B, S - n_txt, D, ptr.keep)
    lib = _lib.lib()
    _run_block(a, lib.hdit_block_flux_single_workspace_bytes, lib.hdit_block_flux_single, "hdit_block_flux_single",
               hidden_states.device, ptr.keep)
    return hidden_out


def block_cogvideox(block, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None, out_dtype=bf16,
                    modulation1: Optional[int] = None, modulation2: Optional[int] = None):
    """One CogVideoX block through ``hdit_block_cogvideox``; returns ``(hidden, encoder)`` like the block.
    ``modulation1`` / ``modulation2``: device addresses of the precomputed f32 [batch, 6 dim] projections of
    ``norm1`` / ``norm2``."""
    attn, m = block.attn1, block.attn1.module
    B, N, D = hidden_states.shape
    Nt = encoder_hidden_states.shape[1]
    _need(temb, bf16, "temb")
    a, ptr = _lib.CogVideoXBlockArgs(), _ArgFiller()
    qkv_w, qkv_b = attn._qkv.get()
    for i, norm in ((1, block.norm1), (2, block.norm2)):
        setattr(a, f"norm{i}_w", ptr(norm.linear.weight.data)), setattr(a, f"norm{i}_b", ptr(norm.linear.bias.data))
        setattr(a, f"norm{i}_ln_w", ptr(norm.norm.weight.data)), setattr(a, f"norm{i}_ln_b", ptr(norm.norm.bias.data))
    a.norm_eps = float(block.norm1.norm.eps)
    a.qkv_w, a.qkv_b = ptr(qkv_w), ptr(qkv_b)
    a.to_out_w = ptr(m.to_out[0].weight.data)
    a.to_out_b = ptr(attn.output_bias.data) if attn.has_output_bias else None
    for name in ("norm_q", "norm_k"):
        n = getattr(m, name)
        if n is not None:
            setattr(a, name + "_w", ptr(n.weight.data) if n.weight is not None else None)
            b = getattr(n, "bias", None)
            setattr(a, name + "_b", ptr(b.data) if b is not None else None)
    a.qk_norm_kind, a.qk_norm_eps = _norm_kind_of(m.norm_q), float(m.norm_q.eps) if m.norm_q is not None else 1e-6
    ff = block.ff
    a.ff_in_w, a.ff_in_b = ptr(ff.module.net[0].proj.weight.data), ptr(ff.module.net[0].proj.bias.data)
    a.ff_out_w = ptr(ff.module.net[2].weight.data)
    a.ff_out_b = ptr(ff.output_bias.data) if ff.has_output_bias else None
    a.hidden_f32, a.encoder_f32 = _stream_tensor(hidden_states, "hidden_states"), _stream_tensor(encoder_hidden_states, "encoder_hidden_states")
    if image_rotary_emb is not None:
        cos, sin = image_rotary_emb
        _need(cos, torch.float32, "cos"), _need(sin, torch.float32, "sin")
        if tuple(cos.shape) != (N, D // attn.heads_per_device) or cos.shape != sin.shape or not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("image_rotary_emb must be contiguous f32 [n_img, head_dim] tables")
        a.rope_cos, a.rope_sin = ptr(cos), ptr(sin)
    hidden_out = torch.empty(B, N, D, dtype=out_dtype, device=hidden_states.device)
    encoder_out = torch.empty(B, Nt, D, dtype=out_dtype, device=hidden_states.device)
    a.hidden, a.encoder, a.temb = ptr(hidden_states), ptr(encoder_hidden_states), ptr(temb.contiguous())
    a.hidden_out, a.encoder_out, a.out_f32 = hidden_out.data_ptr(), encoder_out.data_ptr(), int(out_dtype == torch.float32)
    a.batch, a.n_img, a.n_txt, a.dim, a.heads = B, N, Nt, D, attn.heads_per_device
    a.ff_dim, a.temb_dim = ff.module.net[0].proj.weight.shape[0], temb.shape[1]
    a.fp8_attention = int(bool(getattr(attn, "fp8_attention", False)))
    a.modulation1, a.modulation2 = modulation1, modulation2
    lib = _lib.lib()
    _run_block(a, lib.hdit_block_cogvideox_workspace_bytes, lib.hdit_block_cogvideox, "hdit_block_cogvideox",
               hidden_states.device, ptr.keep)
    return hidden_out, encoder_out


# ---------------------------------------------------------------------------
# glue
# ---------------------------------------------------------------------------

def _as3d(x: torch.Tensor, name: str, dtype=bf16) -> Tuple[int, int, int, int, int]:
    """[B, T, D] view with unit inner stride; returns (B, T, D, batch stride, token stride)."""
    _need(x, dtype, name)
    if x.dim() != 3 or x.stride(2) != 1:
        raise ValueError(f"{name} must be [batch, tokens, dim] with unit inner stride")
    B, T, D = x.shape
    st = x.stride(1) if T > 1 else D
    sb = x.stride(0) if B > 1 else T * st
    return B, T, D, sb, st


def _mod(v: Optional[torch.Tensor], B: int, D: int, name: str):
    if v is None:
        return None, 0
    _need(v, torch.float32, name)
    if tuple(v.shape) != (B, D) or v.stride(1) != 1:
        raise ValueError(f"{name} must be f32 [batch, dim] with unit inner stride")
    return v.data_ptr(), (v.stride(0) if B > 1 else D)


def layernorm_modulate(x, shift=None, scale=None, eps: float = 1e-6, ln_weight=None, ln_bias=None, out=None):
    """bf16 out = LayerNorm(x) * (1 + scale) + shift; x bf16, or f32 (the fp32 residual stream)."""
    if x.dtype == torch.float32:
        return layernorm_modulate_many([(x, shift, scale, out) if out is not None else (x, shift, scale)], eps, ln_weight,
                                       ln_bias)[0]
    B, T, D, xsb, xst = _as3d(x, "x")
    if out is None:
        out = torch.empty(B, T, D, dtype=bf16, device=x.device)
    Bo, To, Do, ysb, yst = _as3d(out, "out")
    if (Bo, To, Do) != (B, T, D):
        raise ValueError("out shape differs from x")
    sh, st1 = _mod(shift, B, D, "shift")
    sc, st2 = _mod(scale, B, D, "scale")
    if sh is not None and sc is not None and st1 != st2:
        raise ValueError("shift and scale must share a batch stride")
    for w in (ln_weight, ln_bias):
        if w is not None:
            _need(w, bf16, "ln affine")
    check(
        _run("ln_modulate", 4.0 * B * T * D,
             lambda: _lib.lib().hdit_layernorm_modulate(x.data_ptr(), out.data_ptr(), sh, sc, _ptr(ln_weight),
                                                        _ptr(ln_bias), B, T, D, xsb, xst, ysb, yst, st1 or st2, eps,
                                                        _stream())),
        "hdit_layernorm_modulate",
    )
    return out


def layernorm_modulate_many(items, eps: float = 1e-6, ln_weight=None, ln_bias=None):
    """LayerNorm + modulate of several tensors of one width in one launch.

    ``items`` is a list of ``(x, shift, scale)``, ``(x, shift, scale, out)`` or ``(x, shift, scale, out, delta)``
    with ``delta = (y bf16 like x, gate f32 [batch, dim], x_out f32 like x or None)``: the f32 stream ``x`` is
    first updated to ``x + gate * y`` (and written to ``x_out``, which may be ``x``).  Returns the outputs in order."""
    jobs = (_lib.LnJob * len(items))()
    outs, keep, D0, nbytes = [], [], None, 0.0
    for i, it in enumerate(items):
        x, shift, scale = it[0], it[1], it[2]
        out = it[3] if len(it) > 3 else None
        x_f32 = x.dtype == torch.float32
        B, T, D, xsb, xst = _as3d(x, "x", torch.float32 if x_f32 else bf16)
        if D0 is None:
            D0 = D
        elif D != D0:
            raise ValueError("all tensors of one launch must have the same width")
        if out is None:
            out = torch.empty(B, T, D, dtype=bf16, device=x.device)
        Bo, To, Do, ysb, yst = _as3d(out, "out")
        if (Bo, To, Do) != (B, T, D):
            raise ValueError("out shape differs from x")
        sh, st1 = _mod(shift, B, D, "shift")
        sc, st2 = _mod(scale, B, D, "scale")
        if sh is not None and sc is not None and st1 != st2:
            raise ValueError("shift and scale must share a batch stride")
        j = jobs[i]
        j.x, j.y, j.shift, j.scale = x.data_ptr(), out.data_ptr(), sh, sc
        j.x_sb, j.x_st, j.y_sb, j.y_st, j.mod_stride = xsb, xst, ysb, yst, (st1 or st2 or 0)
        j.batch, j.tokens, j.x_f32 = B, T, int(x_f32)
        if len(it) > 4 and it[4] is not None:
            dy, gate, x_out = it[4]
            if not x_f32:
                raise ValueError("a pending update needs the f32 stream")
            Bd, Td, Dd, dsb, dst = _as3d(dy, "delta y")
            g, gst = _mod(gate, B, D, "delta gate")
            if (Bd, Td, Dd) != (B, T, D):
                raise ValueError("delta y must have the shape of x")
            j.delta_y, j.delta_gate, j.d_sb, j.d_st, j.gate_stride = dy.data_ptr(), g, dsb, dst, gst
            if x_out is not None:
                Bx, Tx, Dx, xosb, xost = _as3d(x_out, "x_out", torch.float32)
                if (Bx, Tx, Dx) != (B, T, D):
                    raise ValueError("x_out must have the shape of x")
                j.x_out, j.xo_sb, j.xo_st = x_out.data_ptr(), xosb, xost
                nbytes += 4.0 * B * T * D
            nbytes += 2.0 * B * T * D
            keep.append((dy, gate, x_out))
        outs.append(out)
        keep.append((x, shift, scale, out))
        nbytes += (6.0 if x_f32 else 4.0) * B * T * D
    for w in (ln_weight, ln_bias):
        if w is not None:
            _need(w, bf16, "ln affine")
    check(
        _run("ln_modulate", nbytes,
             lambda: _lib.lib().hdit_layernorm_modulate_jobs(jobs, len(items), D0, _ptr(ln_weight), _ptr(ln_bias), eps,
                                                             _stream())),
        "hdit_layernorm_modulate_jobs",
    )
    return outs


def gate_residual(x, y, gate, out=None):
    B, T, D, xsb, xst = _as3d(x, "x")
    By, Ty, Dy, ysb, yst = _as3d(y, "y")
    if out is None:
        out = torch.empty(B, T, D, dtype=bf16, device=x.device)
    Bo, To, Do, osb, ost = _as3d(out, "out")
    if (By, Ty, Dy) != (B, T, D) or (Bo, To, Do) != (B, T, D):
        raise ValueError("gate_residual operand shapes differ")
    g, gs = _mod(gate, B, D, "gate")
    check(_run("gate_residual", 6.0 * B * T * D,
               lambda: _lib.lib().hdit_gate_residual(x.data_ptr(), y.data_ptr(), g, out.data_ptr(), B, T, D, xsb, xst, ysb,
                                                     yst, osb, ost, gs, _stream())),
          "hdit_gate_residual")
    return out


def adaln_gemv(temb: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """f32 [B, n] = w @ silu(temb) + bias."""
    _need(temb, bf16, "temb"), _need(w, bf16, "w")
    if not (temb.is_contiguous() and w.is_contiguous()):
        raise ValueError("adaln_gemv operands must be contiguous")
    B, k = temb.shape
    n = w.shape[0]
    if bias is not None:
        _need(bias, bf16, "bias")
    out = torch.empty(B, n, dtype=torch.float32, device=temb.device)
    check(_run("adaln_gemv", 2.0 * n * k,
               lambda: _lib.lib().hdit_adaln_gemv(temb.data_ptr(), w.data_ptr(), _ptr(bias), out.data_ptr(), B, n, k,
                                                  _stream())),
          "hdit_adaln_gemv")
    return out


ACT_GELU_ERF, ACT_GEGLU, ACT_SILU = 0, 1, 2


def ff_activation(x: torch.Tensor, kind: int, out=None) -> torch.Tensor:
    """The feed-forward activations without a fused GEMM epilogue, on the first projection's output ``x [..., n]``
    (bias already added): exact GELU and SiLU keep the width (and may run in place, ``out=x``), GEGLU halves it."""
    _need(x, bf16, "x")
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(1) != 1:
        raise ValueError("x needs a unit inner stride")
    dim = x2.shape[1] // 2 if kind == ACT_GEGLU else x2.shape[1]
    if kind == ACT_GEGLU and x2.shape[1] % 2:
        raise ValueError("GEGLU needs an even width")
    if out is None:
        out = torch.empty(*x.shape[:-1], dim, dtype=bf16, device=x.device)
    o2 = out.view(-1, dim)
    rows = x2.shape[0]
    check(_lib.lib().hdit_ff_activation(x2.data_ptr(), o2.data_ptr(), rows, dim, x2.stride(0) if rows > 1 else x2.shape[1],
                                        o2.stride(0) if rows > 1 else dim, kind, _stream()), "hdit_ff_activation")
    return out


def gelu_tanh(x: torch.Tensor, bias: Optional[torch.Tensor] = None, out=None) -> torch.Tensor:
    _need(x, bf16, "x")
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(1) != 1:
        raise ValueError("x needs a unit inner stride")
    if out is None:
        out = torch.empty(x.shape, dtype=bf16, device=x.device)
    o2 = out.view(-1, x.shape[-1])
    rows, dim = x2.shape
    check(_lib.lib().hdit_gelu_tanh(x2.data_ptr(), _ptr(bias), o2.data_ptr(), rows, dim,
                                    x2.stride(0) if rows > 1 else dim, o2.stride(0) if rows > 1 else dim, _stream()),
          "hdit_gelu_tanh")
    return out


def qk_norm_rope_job(x: torch.Tensor, norm_kind: int = 0, weight=None, bias=None, cos=None, sin=None,
                     rope_row0: int = 0) -> QkNormJob:
    """x: [B, S, H, d] bf16 view (unit stride on d), modified in place."""
    _need(x, bf16, "x")
    if x.dim() != 4 or x.stride(3) != 1:
        raise ValueError("x must be [B, S, H, d] with contiguous d")
    j = QkNormJob()
    j.x = x.data_ptr()
    j.stride_b, j.stride_s, j.stride_h = x.stride(0), x.stride(1), x.stride(2)
    j.seq = x.shape[1]
    j.norm_kind = norm_kind
    if weight is not None:
        _need(weight, bf16, "weight")
        j.weight = weight.data_ptr()
    if bias is not None:
        _need(bias, bf16, "bias")
        j.bias = bias.data_ptr()
    if cos is not None:
        _need(cos, torch.float32, "cos"), _need(sin, torch.float32, "sin")
        if cos.shape != sin.shape or cos.shape[1] != x.shape[3] or not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("cos/sin must be contiguous f32 [rows, head_dim]")
        if cos.shape[0] != x.shape[1] - rope_row0:
            # the reference's `x * cos` would fail to broadcast; a silent partial rotation must not happen
            raise ValueError(f"rotary table has {cos.shape[0]} rows for {x.shape[1] - rope_row0} rotated tokens "
                             f"(sequence {x.shape[1]}, first rotated row {rope_row0})")
        j.cos_table, j.sin_table = cos.data_ptr(), sin.data_ptr()
        j.rope_row0, j.rope_rows = rope_row0, cos.shape[0]
    j._keep = (x, weight, bias, cos, sin)
    return j


def qk_norm_rope(jobs: List[QkNormJob], batch: int, heads: int, head_dim: int, eps: float = 1e-6):
    arr = (QkNormJob * len(jobs))(*jobs)
    nbytes = sum(4.0 * batch * j.seq * heads * head_dim for j in jobs)
    check(_run("qk_norm_rope", nbytes,
               lambda: _lib.lib().hdit_qk_norm_rope(arr, len(jobs), batch, heads, head_dim, eps, _stream())),
          "hdit_qk_norm_rope")


def copy_rows(src: torch.Tensor, dst: torch.Tensor):
    """dst[b, t, :] = src[b, t, :] for [B, T, D] bf16 views with unit inner stride."""
    _need(src, bf16, "src"), _need(dst, bf16, "dst")
    if src.shape != dst.shape or src.dim() != 3 or src.stride(2) != 1 or dst.stride(2) != 1:
        raise ValueError("copy_rows needs equal-shape [B, T, D] views with unit inner stride")
    B, T, D = src.shape
    check(_lib.lib().hdit_copy_rows(src.data_ptr(), dst.data_ptr(), B, T, D, src.stride(0), src.stride(1), dst.stride(0),
                                    dst.stride(1), _stream()), "hdit_copy_rows")
    return dst


def patchify(latent: torch.Tensor, patch: int) -> torch.Tensor:
    """bf16 [B, C, H, W] -> [B, (H/p)(W/p), C p p]: rows for the patch-embedding GEMM."""
    _need(latent, bf16, "latent")
    if latent.dim() != 4 or not latent.is_contiguous():
        raise ValueError("latent must be a contiguous [B, C, H, W] tensor")
    B, Cc, H, W = latent.shape
    out = torch.empty(B, (H // patch) * (W // patch), Cc * patch * patch, dtype=bf16, device=latent.device)
    check(_lib.lib().hdit_patchify(latent.data_ptr(), out.data_ptr(), B, Cc, H, W, patch, _stream()), "hdit_patchify")
    return out


def unpatchify(x: torch.Tensor, channels: int, height: int, width: int, patch: int,
               channel_major: bool = False) -> torch.Tensor:
    """bf16 [B, (H/p)(W/p), p p C] -> [B, C, H, W]; token columns ordered (py, px, c), or (c, py, px) if
    ``channel_major``."""
    _need(x, bf16, "x")
    B = x.shape[0]
    if not x.is_contiguous() or tuple(x.shape) != (B, (height // patch) * (width // patch), patch * patch * channels):
        raise ValueError("unpatchify input shape does not match the latent geometry")
    out = torch.empty(B, channels, height, width, dtype=bf16, device=x.device)
    check(_lib.lib().hdit_unpatchify(x.data_ptr(), out.data_ptr(), B, channels, height, width, patch, int(channel_major),
                                     _stream()), "hdit_unpatchify")
    return out


def timestep_embedding(timesteps: torch.Tensor, dim: int, max_period: float = 10000.0) -> torch.Tensor:
    """f32 [B] -> bf16 [B, dim] = [cos | sin]."""
    _need(timesteps, torch.float32, "timesteps")
    t = timesteps.contiguous()
    out = torch.empty(t.shape[0], dim, dtype=bf16, device=t.device)
    check(_lib.lib().hdit_timestep_embedding(t.data_ptr(), out.data_ptr(), t.shape[0], dim, max_period, _stream()),
          "hdit_timestep_embedding")
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    _need(x, bf16, "x")
    if not x.is_contiguous():
        raise ValueError("silu input must be contiguous")
    y = torch.empty_like(x)
    check(_lib.lib().hdit_silu(x.data_ptr(), y.data_ptr(), x.numel(), _stream()), "hdit_silu")
    return y


def cfg_euler_step(noise_uncond, noise_cond, sample, guidance: float, sigma: float, sigma_next: float) -> torch.Tensor:
    """bf16: sample + d/dsigma step of the guided prediction (see include/hdit.h)."""
    for t, n in ((noise_uncond, "noise_uncond"), (noise_cond, "noise_cond"), (sample, "sample")):
        _need(t, bf16, n)
        if not t.is_contiguous() or t.shape != sample.shape:
            raise ValueError("cfg_euler_step operands must be contiguous and of one shape")
    out = torch.empty_like(sample)
    check(_lib.lib().hdit_cfg_euler_step(noise_uncond.data_ptr(), noise_cond.data_ptr(), sample.data_ptr(), out.data_ptr(),
                                         sample.numel(), guidance, sigma, sigma_next, _stream()), "hdit_cfg_euler_step")
    return out


def rope_table(positions: torch.Tensor, axes_dim, theta: float = 10000.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """f32 positions [S, len(axes_dim)] -> (cos, sin) f32 [S, sum(axes_dim)], the ``image_rotary_emb`` the blocks take."""
    _need(positions, torch.float32, "positions")
    axes = [int(a) for a in axes_dim]
    if positions.dim() != 2 or positions.shape[1] != len(axes) or not positions.is_contiguous():
        raise ValueError("positions must be a contiguous [tokens, axes] tensor with one column per rotary axis")
    rows = positions.shape[0]
    cos = torch.empty(rows, sum(axes), dtype=torch.float32, device=positions.device)
    sin = torch.empty_like(cos)
    arr = (C.c_int * len(axes))(*axes)
    check(_lib.lib().hdit_rope_table(positions.data_ptr(), rows, arr, len(axes), float(theta), cos.data_ptr(), sin.data_ptr(),
                                     _stream()), "hdit_rope_table")
    return cos, sin


PROBE_IDLE, PROBE_MFMA, PROBE_VALU, PROBE_INTERLEAVED = 0, 1, 2, 3


def probe_coissue(role_a: int, role_b: int, iters: int = 2000, workgroups: int = 16):
    """``hdit_probe_coissue``: waves 0-3 of every workgroup run ``role_a``, waves 4-7 (same SIMDs) ``role_b``.
    Returns ``(cycles_a, us_a, cycles_b, us_b)``: mean shader cycles and microseconds per wave of each group."""
    out = torch.zeros(workgroups * 16 + 1, dtype=torch.int64, device="cuda")
    check(_lib.lib().hdit_probe_coissue(role_a, role_b, iters, workgroups, out.data_ptr(), _stream()), "hdit_probe_coissue")
    torch.cuda.synchronize()
    t = out[: workgroups * 16].view(workgroups, 8, 2).double().cpu()
    a, b = t[:, :4].mean(dim=(0, 1)), t[:, 4:].mean(dim=(0, 1))
    return a[0].item(), a[1].item() / 100.0, b[0].item(), b[1].item() / 100.0


def clock_sample(slots: int = 1024) -> torch.Tensor:
    """int64 [slots, 4] on the device, filled on the current stream with (shader-clock counter, 100 MHz counter,
    XCD id, hardware id) of `slots` one-wave workgroups (enough of them to land on every CU)."""
    out = torch.zeros(slots, 4, dtype=torch.int64, device="cuda")
    check(_lib.lib().hdit_clock_sample(out.data_ptr(), slots, _stream()), "hdit_clock_sample")
    return out


def shader_clock_ghz(before: torch.Tensor, after: torch.Tensor) -> Optional[float]:
    """Average shader clock between two ``clock_sample`` results.  Every CU counts its own shader clock, so a
    sample is paired with the later sample of the same CU (XCD id + shader-engine / shader-array / CU fields of the
    hardware id); the median over the CUs is returned (None if no pair is usable)."""
    def cu_key(row):
        return (row[2], (row[3] >> 8) & 0xFF)

    first = {}
    for row in before.cpu().tolist():
        first.setdefault(cu_key(row), row)
    rates, seen = [], set()
    for row in after.cpu().tolist():
        k = cu_key(row)
        if k in first and k not in seen:
            seen.add(k)
            d_ticks, d_real = row[0] - first[k][0], row[1] - first[k][1]
            if d_ticks > 0 and d_real > 0:
                rates.append(d_ticks / d_real * 0.1)
    if not rates:
        return None
    rates.sort()
    return rates[len(rates) // 2]
