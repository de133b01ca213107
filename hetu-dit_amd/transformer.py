"""Block-loop callers: the part of the reference's transformer wrappers'
``forward`` that sits between the embedders and ``norm_out`` -- "for block in
blocks" with each model family's call convention and patch-mode rules.

* SD3 (``models/transformers/transformer_sd3.py:107-152``): in patch mode,
  patch 0 stores every block's *input* text states; later patches feed those
  back and drop the block's text output.
* Flux (``transformer_flux.py:133-201``): double blocks, then
  ``cat([text, image])``, single blocks on the joint sequence, split.
* CogVideoX (``cogvideox_transformer_3d.py:99-127``).
"""
import os
import warnings
from typing import List, Optional, Tuple

import torch
from torch import nn

from . import _lib, ops
from ._lib import eager_only
from .blocks import (CogVideoXBlock, FluxSingleTransformerBlock, FluxTransformerBlock, JointTransformerBlock,
                     StackModulation, use_fp32_residual_stream)
from .cache_manager import get_cache_manager
from .runtime_state import get_runtime_state


# Side streams are shared by every stack of the process and kept few: a process has GPU_MAX_HW_QUEUES (4 by
# default) hardware queues, streams beyond that share one, and two chains on one hardware queue run one after
# the other however many streams they were issued on.
_SIDE_STREAMS = {}  # device -> list of streams
MAX_SIDE_STREAMS = 3


def side_streams(device: torch.device, count: int) -> List["torch.cuda.Stream"]:
    device = torch.device(device)
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    have = _SIDE_STREAMS.setdefault(device, [])
    while len(have) < min(count, MAX_SIDE_STREAMS):
        have.append(torch.cuda.Stream(device=device))  # default priority, like the caller's stream
    return have[: min(count, MAX_SIDE_STREAMS)]


class _Chain:
    """What one chain of SD3 blocks (a full pass, one batch lane, one pipeline patch) carries from a block to the
    next besides the streams: the gated MLP residual the block did not add itself.  ``img`` / ``txt``: ``(y bf16
    [batch, rows, dim], address of the f32 gate, its batch stride)`` or None -- the stream a block hands over is
    then short of ``gate * y``, and the next block's first normalisation, which reads the stream anyway, adds it
    (``hdit_sd3_block_args.pending_*`` / ``defer_*``).  The GEMM that produced ``y`` is spared the
    read-modify-write of the f32 stream in its epilogue."""

    __slots__ = ("img", "txt")

    def __init__(self):
        self.img = None
        self.txt = None

    def take(self, left, skipped_text_output: bool):
        """``left``: what the block that just ran left owing, ``(img, txt_or_None)`` or None."""
        self.img = left[0] if left is not None else None
        if not skipped_text_output:  # a call that drops its text output leaves the text stream's state alone
            self.txt = left[1] if left is not None else None


class SD3TransformerBlocks(nn.Module):
    """The 24 joint blocks of the SD3 transformer with the reference's block loop.

    ``use_block_entry_points``: run every block through ``hdit_block_sd3`` (one foreign call per block, the
    same launches on the same operands as the Python block: results are bit for bit the same) instead of one
    foreign call per kernel.  An eager pass is then bound by the GPU and not by the interpreter, which is what
    lets independent work run side by side on several streams:

    * ``batch_streams``: a full-sequence pass of B >= 2 batch elements (the CFG pair) runs the elements as
      independent chains on that many side streams, blocks issued alternately -- one chain's launches fill the
      CUs another's partial last round of tiles leaves idle (about 5 % of the SD3 step at B = 2);
    * ``forward_patches``: the patches of a PipeFusion step, one block apart.

    Neither is recorded into a HIP graph: under capture, and whenever a per-launch timer is installed, the pass
    runs on the caller's stream alone."""

    def __init__(self, num_layers: int = 24, dim: int = 1536, num_attention_heads: int = 24,
                 attention_head_dim: int = 64):
        super().__init__()
        self.transformer_blocks = nn.ModuleList(
            [
                JointTransformerBlock(dim, num_attention_heads, attention_head_dim,
                                      context_pre_only=(i == num_layers - 1))
                for i in range(num_layers)
            ]
        )
        self.encoder_hidden_states_cache: List[Optional[torch.Tensor]] = [None] * num_layers
        self.modulation = StackModulation(self.transformer_blocks)
        use_fp32_residual_stream(self.transformer_blocks)
        self.use_block_entry_points = True
        self.batch_streams = 2
        self.reuse_text_kv = True  # patch mode: later patches take the text keys / values the first patch projected
        self.group_fronts = True   # forward_patches on one stream: one merged call per front of independent blocks
        # entry-point passes: a block leaves its MLP residual to the next block's norm1 (HDIT_DEFER_RESIDUALS=0: fused
        # into the GEMM epilogue as in a block called on its own)
        self.defer_residuals = os.environ.get("HDIT_DEFER_RESIDUALS", "1") != "0"
        # patch mode: the pending text update that goes with encoder_hidden_states_cache[i]
        self._text_pending: List[Optional[tuple]] = [None] * num_layers
        self._block_calls: Optional[List[ops.Sd3BlockCall]] = None
        # per block: (k|v buffer of the text stream, the text states and temb it was projected from, with their
        # in-place modification counters) -- patch mode
        self._text_kv: List[Optional[tuple]] = [None] * num_layers
        self._patch_events = {}  # (patch, block) -> "block done" event of forward_patches

    # -- launching one block ------------------------------------------------------------------------------
    def _entry_point_calls(self) -> Optional[List["ops.Sd3BlockCall"]]:
        """The prefilled whole-block calls, weight pointers (and the fp8 attention switch) re-read, or None where
        the per-kernel path has to run: switched off, or a per-launch timer installed."""
        if not self.use_block_entry_points or ops.timer_installed():
            return None
        if self._block_calls is None or len(self._block_calls) != len(self.transformer_blocks):
            unfit = [i for i, b in enumerate(self.transformer_blocks) if not ops.Sd3BlockCall.describes(b)]
            if unfit:
                # sub-modules replaced by something the entry point's weight table cannot describe
                warnings.warn(f"SD3TransformerBlocks: blocks {unfit} do not have the layout hdit_block_sd3 takes; "
                              "the stack runs kernel by kernel on one stream from now on", RuntimeWarning)
                self._block_calls = None
                self.use_block_entry_points = False
                return None
            self._block_calls = [ops.Sd3BlockCall(b) for b in self.transformer_blocks]
        else:
            for call in self._block_calls:
                call.refresh()
        return self._block_calls

    def _run_block(self, i: int, calls, mods, hidden, encoder, temb, skip_text_output: bool = False,
                   kv_buffer=None, kv_row0: int = 0, batch0: int = 0, hidden_out=None, patch: Optional[int] = None,
                   defer: Optional[list] = None, chain: Optional["_Chain"] = None):
        """Block i on the current stream: ``(encoder_out_or_None, hidden_out)``.  ``chain``: the gated residuals
        the previous block of this chain of blocks left to this one's first normalisation (``_Chain``); updated
        with what this block leaves to the next.  ``batch0``: index of the
        first batch element of ``hidden`` within the ``temb`` the modulation ``mods`` was computed for.
        ``defer``: a list -- the call is prepared and appended to it instead of launched (``_launch_front``).
        ``patch``: index of the pipeline patch in patch mode.  The later patches of a step are fed the text states
        the first one stored (``transformer_sd3.py:131-146``), so the text stream's keys and values are the same
        numbers for all of them: the first patch's call leaves them in a buffer and the later ones take them from
        there -- as long as they really come with the same text states and the same ``temb``."""
        block = self.transformer_blocks[i]
        # every block but the last leaves its MLP residuals to the next block's first normalisation
        leave = chain is not None and i + 1 < len(self.transformer_blocks) and block.stream_dtype == torch.float32
        if calls is None:
            if chain is None:
                return block(hidden_states=hidden, encoder_hidden_states=encoder, temb=temb,
                             skip_text_output=skip_text_output)
            out = block(hidden_states=hidden, encoder_hidden_states=encoder, temb=temb,
                        skip_text_output=skip_text_output, pending=(chain.img, chain.txt), defer=leave)
            chain.take(block.deferred, skip_text_output)
            return out
        text_kv, text_kv_mode = None, _lib.TEXT_KV_NONE
        if not self.reuse_text_kv:
            pass
        elif patch == 0:
            held = self._text_kv[i]
            shape = (encoder.shape[0], encoder.shape[1], 2 * encoder.shape[2])
            text_kv = held[0] if held is not None and tuple(held[0].shape) == shape and held[0].device == encoder.device \
                else torch.empty(shape, dtype=torch.bfloat16, device=encoder.device)
            self._text_kv[i] = (text_kv, encoder, encoder._version, temb, temb._version)
            text_kv_mode = _lib.TEXT_KV_STORE
        elif patch is not None and skip_text_output:
            held = self._text_kv[i]
            if held is not None and held[1] is encoder and held[2] == encoder._version and held[3] is temb \
                    and held[4] == temb._version:
                text_kv, text_kv_mode = held[0], _lib.TEXT_KV_REUSE
        flat, offsets = mods
        dim = hidden.shape[2]
        rows_txt = (2 if block.context_pre_only else 6) * dim
        base = flat.data_ptr()
        kwargs = dict(
            out_dtype=block.stream_dtype, skip_text_output=skip_text_output, kv_buffer=kv_buffer, kv_row0=kv_row0,
            modulation_img=base + 4 * (offsets[block.norm1] + batch0 * 6 * dim),
            modulation_txt=base + 4 * (offsets[block.norm1_context] + batch0 * rows_txt),
            hidden_out=hidden_out, text_kv=text_kv, text_kv_mode=text_kv_mode,
        )
        if chain is not None:
            kwargs.update(pending_img=chain.img, pending_txt=chain.txt, defer=leave, lazy=True)
        encoder_out, hidden_new, ws = calls[i].prepare(hidden, encoder, temb, **kwargs)
        if chain is not None:
            chain.take(calls[i].deferred, skip_text_output)
        if defer is None:
            calls[i].launch()
            del ws  # stream-ordered reuse: the workspace may be freed as soon as the launches are queued
        else:
            # the struct is filled, the launch is the caller's (merged with the other blocks of its front)
            defer.append((calls[i], ws))
        return encoder_out, hidden_new

    def _kv_buffer(self, i: int, hidden: torch.Tensor):
        """``(buffer, first row)``: the K|V buffer block i's image stream writes into, from the cache manager --
        a fresh full-length buffer with patch mode off, the persistent one and the current patch's rows in
        patch mode."""
        attn = self.transformer_blocks[i].attn
        buf, start, _ = get_cache_manager().kv_buffer(attn, hidden.shape[0], hidden.shape[1], hidden.shape[2], hidden.device)
        return buf, start

    def _persistent_buffers_contiguous(self) -> bool:
        """A full pass of the per-kernel path keeps q|k|v in one tensor and registers its k|v columns, a strided
        view, as the layer's buffer; the whole-block entry point wants a contiguous [B, rows, 2 dim] buffer.  A
        patch pass therefore stays on the path that filled the buffers."""
        cm = get_cache_manager()
        for block in self.transformer_blocks:
            buf = cm._entry(block.attn, "attn").tensors[0]
            if buf is None or not buf.is_contiguous():
                return False
        return True

    # -- the reference's block loop -----------------------------------------------------------------------
    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states, encoder_hidden_states, temb):
        rs = get_runtime_state()
        calls = self._entry_point_calls()
        if calls is not None and rs.patch_mode and not self._persistent_buffers_contiguous():
            calls = None
        if calls is None:
            self.modulation.precompute(temb)
            mods = None
        else:
            hidden_states, encoder_hidden_states = hidden_states.contiguous(), encoder_hidden_states.contiguous()
            temb = temb.contiguous()
            mods = self.modulation.precompute_by_module(temb)
            lanes = min(self.batch_streams, hidden_states.shape[0])
            if not rs.patch_mode and lanes > 1 and not torch.cuda.is_current_stream_capturing():
                return self._forward_batch_lanes(calls, mods, hidden_states, encoder_hidden_states, temb, lanes)
        chain = _Chain() if self.defer_residuals else None
        for i in range(len(self.transformer_blocks)):
            kv = self._kv_buffer(i, hidden_states) if calls is not None else (None, 0)
            if rs.patch_mode and rs.pipeline_patch_idx == 0:
                self.encoder_hidden_states_cache[i] = encoder_hidden_states
                self._text_pending[i] = chain.txt if chain is not None else None
                encoder_hidden_states, hidden_states = self._run_block(
                    i, calls, mods, hidden_states, encoder_hidden_states, temb, kv_buffer=kv[0], kv_row0=kv[1], patch=0,
                    chain=chain)
            elif rs.patch_mode:
                # the text output of these calls is dropped: the block does not compute it
                if chain is not None:
                    chain.txt = self._text_pending[i]
                _, hidden_states = self._run_block(
                    i, calls, mods, hidden_states, self.encoder_hidden_states_cache[i], temb, skip_text_output=True,
                    kv_buffer=kv[0], kv_row0=kv[1], patch=rs.pipeline_patch_idx, chain=chain)
            else:
                encoder_hidden_states, hidden_states = self._run_block(
                    i, calls, mods, hidden_states, encoder_hidden_states, temb, kv_buffer=kv[0], kv_row0=kv[1],
                    chain=chain)
        return hidden_states

    def _forward_batch_lanes(self, calls, mods, hidden_states, encoder_hidden_states, temb, lanes: int):
        """Full-sequence pass with the batch elements as ``lanes`` independent chains on side streams."""
        B = hidden_states.shape[0]
        L = len(self.transformer_blocks)
        main = torch.cuda.current_stream()
        streams = side_streams(hidden_states.device, lanes)
        lanes = len(streams)
        bounds = [B * k // lanes for k in range(lanes + 1)]
        kv = [self._kv_buffer(i, hidden_states)[0] for i in range(L)]  # fresh [B, N, 2D] buffers, one per layer
        out = torch.empty(hidden_states.shape, dtype=self.transformer_blocks[-1].stream_dtype, device=hidden_states.device)
        start = torch.cuda.Event()
        start.record(main)
        state = []
        for k, s in enumerate(streams):
            s.wait_event(start)
            b0, b1 = bounds[k], bounds[k + 1]
            # no residual chain here: with a second chain of blocks in flight the read-modify-write of a fused
            # gated epilogue runs under the other chain's MFMAs, and moving it into the normalisation kernels
            # only lengthens those (measured: 19.85 ms fused, 20.18 ms deferred for the SD3 step on two streams)
            state.append([hidden_states[b0:b1], encoder_hidden_states[b0:b1], temb[b0:b1], None])
        for i in range(L):
            for k, s in enumerate(streams):
                b0, b1 = bounds[k], bounds[k + 1]
                h, e, t, chain = state[k]
                with torch.cuda.stream(s):
                    e, h = self._run_block(i, calls, mods, h, e, t, kv_buffer=kv[i][b0:b1], batch0=b0,
                                           hidden_out=out[b0:b1] if i == L - 1 else None, chain=chain)
                state[k][0], state[k][1] = h, e
        for s in streams:
            done = torch.cuda.Event()
            done.record(s)
            main.wait_event(done)
        return out

    @torch.no_grad()
    @eager_only
    def forward_patches(self, hidden_states_patches: List[torch.Tensor], encoder_hidden_states: torch.Tensor,
                        temb: torch.Tensor, num_streams: int = 2) -> List[torch.Tensor]:
        """One PipeFusion step of this stage: every patch through every block, the same kernels on the same
        operands as ``forward`` called once per patch in patch order (the loop of
        ``pipelines/pipeline_stable_diffusion_3.py:1549-1644``), with the patches spread over ``num_streams``
        side streams so that the GPU works on neighbouring patches at once.

        A patch-sized launch leaves CUs idle (1024-token problems make 48-192 tiles for 256 CUs); a second
        patch's launches fill them.  Patch p runs block l once patch p-1 has finished block l: by then p-1 has
        written its fresh K/V rows of layer l (which p must see), has read p's still stale rows (which p is about
        to overwrite), and patch 0 has stored the text states p feeds to block l.  Every other pair of launches
        touches different layers' buffers.  The modulation of all blocks is computed once for the step.

        Expects patch mode with ``pipeline_patch_idx == 0`` and leaves it at 0, like one ``next_patch()`` per
        patch.  Not to be recorded into a HIP graph with more than one stream (refused)."""
        rs = get_runtime_state()
        P, L = len(hidden_states_patches), len(self.transformer_blocks)
        if not rs.patch_mode or rs.pipeline_patch_idx != 0 or P != rs.num_pipeline_patch:
            raise ValueError("forward_patches needs patch mode, pipeline_patch_idx 0 and one input per patch")
        if num_streams < 1:
            raise ValueError("num_streams must be at least 1")
        main = torch.cuda.current_stream()
        if num_streams > 1 and torch.cuda.is_current_stream_capturing():
            raise RuntimeError("forward_patches with several streams cannot be captured into a graph "
                               "(num_streams=1 can: its fronts are merged launches on the caller's stream)")
        calls = self._entry_point_calls()
        if calls is not None and not self._persistent_buffers_contiguous():
            calls = None
        hidden = list(hidden_states_patches)
        if calls is None:
            self.modulation.precompute(temb)
            mods = None
        else:
            hidden = [h.contiguous() for h in hidden]
            encoder_hidden_states, temb = encoder_hidden_states.contiguous(), temb.contiguous()
            mods = self.modulation.precompute_by_module(temb)
        device = hidden[0].device
        if num_streams == 1 and calls is not None and self.group_fronts:
            return self._forward_patches_grouped(calls, mods, hidden, encoder_hidden_states, temb)
        streams = [main] if num_streams == 1 else side_streams(device, min(num_streams, P))
        start = torch.cuda.Event()
        start.record(main)
        for s in streams:
            if s is not main:
                s.wait_event(start)
        events = self._patch_events
        cache = self.encoder_hidden_states_cache
        # residual chains only where the patches run one after the other (see _forward_batch_lanes)
        chains = [_Chain() for _ in range(P)] if self.defer_residuals and len(streams) == 1 else [None] * P
        try:
            for front in range(L + P - 1):  # launches are issued along the diagonal, the order they can start in
                for p in range(P):
                    i = front - p
                    if not 0 <= i < L:
                        continue
                    s = streams[p % len(streams)]
                    rs.pipeline_patch_idx = p
                    with torch.cuda.stream(s):
                        if p > 0 and streams[(p - 1) % len(streams)] is not s:
                            s.wait_event(events[(p - 1, i)])
                        kv = self._kv_buffer(i, hidden[p]) if calls is not None else (None, 0)
                        if p == 0:
                            cache[i] = encoder_hidden_states
                            self._text_pending[i] = chains[0].txt if chains[0] is not None else None
                            encoder_hidden_states, hidden[0] = self._run_block(
                                i, calls, mods, hidden[0], encoder_hidden_states, temb, kv_buffer=kv[0], kv_row0=kv[1],
                                patch=0, chain=chains[0])
                        else:
                            if chains[p] is not None:
                                chains[p].txt = self._text_pending[i]
                            _, hidden[p] = self._run_block(
                                i, calls, mods, hidden[p], cache[i], temb, skip_text_output=True,
                                kv_buffer=kv[0], kv_row0=kv[1], patch=p, chain=chains[p])
                        if P > 1 and len(streams) > 1:
                            done = events.get((p, i))
                            if done is None:
                                done = events[(p, i)] = torch.cuda.Event()
                            done.record(s)
        finally:
            rs.pipeline_patch_idx = 0
        for s in streams:
            if s is not main:
                joined = torch.cuda.Event()
                joined.record(s)
                main.wait_event(joined)
        for h in hidden:
            h.record_stream(main)  # allocated on a side stream, read by the caller on its own
        return hidden

    def _forward_patches_grouped(self, calls, mods, hidden, encoder_hidden_states, temb):
        """``forward_patches`` on ONE stream: the blocks (patch p, layer l) of a front p + l = const do not depend on
        each other, so every front is one ``hdit_block_sd3_multi`` call -- each stage of its up to four blocks
        one merged launch (one grouped q|k|v GEMM of 4 x 198 tiles, one attention grid of 4 x 192 workgroups, ...)
        instead of four patch-sized launches that each fill a fraction of the GPU.  No side stream, no event, every
        allocation on the caller's stream: the pass can be recorded into a HIP graph.  Same operands and kernels
        per block as the sequential pass, so the same bits."""
        rs = get_runtime_state()
        P, L = len(hidden), len(self.transformer_blocks)
        cache = self.encoder_hidden_states_cache
        chains = [_Chain() if self.defer_residuals else None for _ in range(P)]
        try:
            for front in range(L + P - 1):
                group = []
                for p in range(P):
                    i = front - p
                    if not 0 <= i < L:
                        continue
                    rs.pipeline_patch_idx = p
                    kv = self._kv_buffer(i, hidden[p])
                    if p == 0:
                        cache[i] = encoder_hidden_states
                        self._text_pending[i] = chains[0].txt if chains[0] is not None else None
                        encoder_hidden_states, hidden[0] = self._run_block(
                            i, calls, mods, hidden[0], encoder_hidden_states, temb, kv_buffer=kv[0], kv_row0=kv[1], patch=0,
                            defer=group, chain=chains[0])
                    else:
                        if chains[p] is not None:
                            chains[p].txt = self._text_pending[i]
                        _, hidden[p] = self._run_block(
                            i, calls, mods, hidden[p], cache[i], temb, skip_text_output=True, kv_buffer=kv[0],
                            kv_row0=kv[1], patch=p, defer=group, chain=chains[p])
                ops.sd3_blocks_launch([c for c, _ in group])
                del group  # the workspaces: stream-ordered reuse once the launches are queued
        finally:
            rs.pipeline_patch_idx = 0
        return hidden


def _modulation_address(mods, module) -> int:
    """Device address of ``module``'s [batch, rows] block inside the regrouped stack modulation."""
    flat, offsets = mods
    return flat.data_ptr() + 4 * offsets[module]


class FluxTransformerBlocks(nn.Module):
    """The double- and single-stream blocks of the Flux transformer with the reference's loop
    (``transformer_flux.py:133-201``).  ``use_block_entry_points``: every block is one call of
    ``hdit_block_flux_double`` / ``hdit_block_flux_single`` -- the launches of the Python blocks on the same
    operands, so the same bits -- fed from the stack's one adaLN GEMV, its image K|V written straight into the
    layer's buffer from the cache manager (a fresh one on a full pass, this patch's rows of the persistent one in
    patch mode).  With a per-launch timer installed, or an fp8 attention switch set on a block, the blocks run
    kernel by kernel."""

    def __init__(self, num_layers: int = 19, num_single_layers: int = 38, dim: int = 3072,
                 num_attention_heads: int = 24, attention_head_dim: int = 128):
        super().__init__()
        self.transformer_blocks = nn.ModuleList(
            [FluxTransformerBlock(dim, num_attention_heads, attention_head_dim) for _ in range(num_layers)]
        )
        self.single_transformer_blocks = nn.ModuleList(
            [FluxSingleTransformerBlock(dim, num_attention_heads, attention_head_dim) for _ in range(num_single_layers)]
        )
        self.modulation = StackModulation(list(self.transformer_blocks) + list(self.single_transformer_blocks))
        use_fp32_residual_stream(list(self.transformer_blocks) + list(self.single_transformer_blocks))
        self.use_block_entry_points = True

    def _entry_points_usable(self) -> bool:
        if not self.use_block_entry_points or ops.timer_installed():
            return False
        blocks = list(self.transformer_blocks) + list(self.single_transformer_blocks)
        return not any(getattr(b.attn, "fp8_attention", False) for b in blocks)

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb):
        if not self._entry_points_usable():
            return self._forward_per_kernel(hidden_states, encoder_hidden_states, temb, image_rotary_emb)
        temb = temb.contiguous()
        hidden_states, encoder_hidden_states = hidden_states.contiguous(), encoder_hidden_states.contiguous()
        mods = self.modulation.precompute_by_module(temb)
        cm = get_cache_manager()
        B, n_img, dim = hidden_states.shape
        n_txt = encoder_hidden_states.shape[1]
        dev = hidden_states.device
        for block in self.transformer_blocks:
            buf, start, _ = cm.kv_buffer(block.attn, B, n_img, dim, dev)
            encoder_hidden_states, hidden_states = ops.block_flux_double(
                block, hidden_states, encoder_hidden_states, temb, image_rotary_emb, out_dtype=block.stream_dtype,
                kv_buffer=buf, kv_row0=start, modulation_img=_modulation_address(mods, block.norm1),
                modulation_txt=_modulation_address(mods, block.norm1_context))
        hidden_states = torch.cat([encoder_hidden_states, hidden_states], dim=1)
        for block in self.single_transformer_blocks:
            buf, start, _ = cm.kv_buffer(block.attn, B, n_img, dim, dev)
            hidden_states = ops.block_flux_single(
                block, hidden_states, temb, image_rotary_emb, out_dtype=block.stream_dtype, kv_buffer=buf, kv_row0=start,
                n_txt=n_txt, modulation=_modulation_address(mods, block.norm))
        return hidden_states[:, n_txt:, ...], hidden_states[:, :n_txt, ...]

    def _forward_per_kernel(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb):
        self.modulation.precompute(temb)
        for block in self.transformer_blocks:
            encoder_hidden_states, hidden_states = block(
                hidden_states=hidden_states, encoder_hidden_states=encoder_hidden_states, temb=temb,
                image_rotary_emb=image_rotary_emb,
            )
        n_txt = encoder_hidden_states.shape[1]
        hidden_states = torch.cat([encoder_hidden_states, hidden_states], dim=1)
        for block in self.single_transformer_blocks:
            hidden_states = block(hidden_states=hidden_states, temb=temb, image_rotary_emb=image_rotary_emb)
        encoder_hidden_states = hidden_states[:, :n_txt, ...]
        hidden_states = hidden_states[:, n_txt:, ...]
        return hidden_states, encoder_hidden_states


class CogVideoXTransformerBlocks(nn.Module):
    """The blocks of the CogVideoX transformer (``cogvideox_transformer_3d.py:99-127``); with
    ``use_block_entry_points`` each block is one ``hdit_block_cogvideox`` call fed from the stack's adaLN GEMV
    (same launches, same bits as the Python block)."""

    def __init__(self, num_layers: int = 42, dim: int = 3072, num_attention_heads: int = 48,
                 attention_head_dim: int = 64, time_embed_dim: int = 512):
        super().__init__()
        self.transformer_blocks = nn.ModuleList(
            [CogVideoXBlock(dim, num_attention_heads, attention_head_dim, time_embed_dim) for _ in range(num_layers)]
        )
        self.modulation = StackModulation(self.transformer_blocks)
        use_fp32_residual_stream(self.transformer_blocks)
        self.use_block_entry_points = True

    @torch.no_grad()
    @eager_only
    def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None) -> Tuple[torch.Tensor, torch.Tensor]:
        if self.use_block_entry_points and not ops.timer_installed():
            temb = temb.contiguous()
            hidden_states, encoder_hidden_states = hidden_states.contiguous(), encoder_hidden_states.contiguous()
            mods = self.modulation.precompute_by_module(temb)
            for block in self.transformer_blocks:
                hidden_states, encoder_hidden_states = ops.block_cogvideox(
                    block, hidden_states, encoder_hidden_states, temb, image_rotary_emb, out_dtype=block.stream_dtype,
                    modulation1=_modulation_address(mods, block.norm1), modulation2=_modulation_address(mods, block.norm2))
            return hidden_states, encoder_hidden_states
        self.modulation.precompute(temb)
        for block in self.transformer_blocks:
            hidden_states, encoder_hidden_states = block(
                hidden_states=hidden_states, encoder_hidden_states=encoder_hidden_states, temb=temb,
                image_rotary_emb=image_rotary_emb,
            )
        return hidden_states, encoder_hidden_states
