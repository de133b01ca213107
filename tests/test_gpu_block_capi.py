"""``hdit_block_sd3`` -- a whole SD3 joint block as ONE call of the C ABI, what a host that is not Python would
bind -- against the Python block, which launches the same kernels one by one (bit-identical outputs), and
against the fp32 oracle."""
import ctypes as C

import pytest
import torch

import oracle
from tests.util import assert_parity, oracle_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def fresh_state():
    from hetu_dit_amd.cache_manager import reset_cache_manager
    from hetu_dit_amd.runtime_state import reset_runtime_state

    reset_runtime_state()
    reset_cache_manager()
    yield
    reset_cache_manager()
    reset_runtime_state()


def make_block(pre_only, seed, D=512, H=8):
    from hetu_dit_amd import blocks, synthetic

    blk = blocks.JointTransformerBlock(D, H, 64, context_pre_only=pre_only)
    synthetic.init_module_(blk, seed)
    return blk.to(DEV), oracle_params(blk)


@pytest.mark.parametrize("pre_only", [False, True])
@pytest.mark.parametrize("stream_f32", [False, True])
def test_block_sd3_one_call_matches_python_block(hdit, pre_only, stream_f32):
    from hetu_dit_amd import synthetic

    print(f"hdit_block_sd3 pre_only={pre_only} fp32 stream={stream_f32}", flush=True)
    B, N, Nt, D, H = 2, 700, 77, 512, 8
    blk, params = make_block(pre_only, 1, D, H)
    x, e, t = synthetic.randn_bf16((B, N, D), 2), synthetic.randn_bf16((B, Nt, D), 3), synthetic.randn_bf16((B, D), 4)
    xd, ed, td = x.to(DEV), e.to(DEV), t.to(DEV)
    if stream_f32:  # the residual stream of a stack: f32 in, f32 out
        xd, ed = xd.float() + 1e-3, ed.float() - 1e-3  # values bf16 cannot hold
        blk.stream_dtype = torch.float32
    enc_py, hid_py = blk(hidden_states=xd, encoder_hidden_states=ed, temb=td)
    enc_c, hid_c = hdit.ops.block_sd3(blk, xd, ed, td, out_dtype=torch.float32 if stream_f32 else torch.bfloat16)
    torch.cuda.synchronize()
    assert hid_c.dtype == hid_py.dtype and torch.equal(hid_c, hid_py)
    if pre_only:
        assert enc_c is None and enc_py is None
    else:
        assert torch.equal(enc_c, enc_py)
    o_enc, o_hid = oracle.sd3_joint_block(params, xd.float().cpu(), ed.float().cpu(), t.float(), H, context_pre_only=pre_only)
    assert_parity(hid_c, o_hid, what="hdit_block_sd3 hidden")
    if not pre_only:
        assert_parity(enc_c, o_enc, what="hdit_block_sd3 encoder")


def test_block_sd3_one_call_pipefusion_patch(hdit):
    """A patch over a stale K|V buffer, with and without the text output, against the Python block driven through
    the runtime state and cache manager."""
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, N, Nt, D, H, P = 2, 512, 77, 512, 8, 4
    starts = [N // P * i for i in range(P + 1)]
    blk, params = make_block(False, 11, D, H)
    x_prev, x_now = synthetic.randn_bf16((B, N, D), 12).to(DEV), synthetic.randn_bf16((B, N, D), 13).to(DEV)
    e, t = synthetic.randn_bf16((B, Nt, D), 14).to(DEV), synthetic.randn_bf16((B, D), 15).to(DEV)
    rs = get_runtime_state()
    rs.set_token_patches(starts)
    rs.set_patched_mode(False)
    blk(hidden_states=x_prev, encoder_hidden_states=e, temb=t)  # fills the layer's buffer
    torch.cuda.synchronize()
    entry = get_cache_manager()._entry(blk.attn, "attn")
    kv_c = entry.tensors[0].contiguous().clone()  # the C call's own copy of the stale buffer
    entry.tensors[0] = entry.tensors[0].contiguous().clone()
    rs.set_patched_mode(True)
    for p, skip in ((0, False), (1, True), (2, True), (3, False)):
        rs.pipeline_patch_idx = p
        xp = x_now[:, starts[p]:starts[p + 1]].contiguous()
        enc_py, hid_py = blk(hidden_states=xp, encoder_hidden_states=e, temb=t, skip_text_output=skip)
        enc_c, hid_c = hdit.ops.block_sd3(blk, xp, e, t, skip_text_output=skip, kv_buffer=kv_c, kv_row0=starts[p])
        torch.cuda.synchronize()
        assert torch.equal(hid_c, hid_py), f"patch {p}"
        assert (enc_c is None and enc_py is None) if skip else torch.equal(enc_c, enc_py)
        assert torch.equal(kv_c, entry.tensors[0]), f"stale buffer after patch {p}"


def test_block_sd3_text_keys_and_values_stored_once_per_step(hdit):
    """The first patch's call leaves the text stream's keys | values in a buffer (``HDIT_TEXT_KV_STORE``), the later
    patches of the step take them from there (``HDIT_TEXT_KV_REUSE``) instead of normalising and projecting the same
    text states again: same bits as the calls that project them every time, and as the Python block."""
    from hetu_dit_amd import _lib, ops, synthetic
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, N, Nt, D, H, P = 2, 512, 77, 512, 8, 4
    starts = [N // P * i for i in range(P + 1)]
    blk, params = make_block(False, 11, D, H)
    x_prev, x_now = synthetic.randn_bf16((B, N, D), 12).to(DEV), synthetic.randn_bf16((B, N, D), 13).to(DEV)
    e, t = synthetic.randn_bf16((B, Nt, D), 14).to(DEV), synthetic.randn_bf16((B, D), 15).to(DEV)
    rs = get_runtime_state()
    rs.set_token_patches(starts)
    rs.set_patched_mode(False)
    blk(hidden_states=x_prev, encoder_hidden_states=e, temb=t)  # fills the layer's buffer
    torch.cuda.synchronize()
    entry = get_cache_manager()._entry(blk.attn, "attn")
    kv_c = entry.tensors[0].contiguous().clone()
    entry.tensors[0] = entry.tensors[0].contiguous().clone()
    rs.set_patched_mode(True)
    call = ops.Sd3BlockCall(blk)
    text_kv = torch.full((B, Nt, 2 * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    for p in range(P):
        rs.pipeline_patch_idx = p
        xp = x_now[:, starts[p]:starts[p + 1]].contiguous()
        enc_py, hid_py = blk(hidden_states=xp, encoder_hidden_states=e, temb=t, skip_text_output=p > 0)
        enc_c, hid_c = call(xp, e, t, skip_text_output=p > 0, kv_buffer=kv_c, kv_row0=starts[p], text_kv=text_kv,
                            text_kv_mode=_lib.TEXT_KV_STORE if p == 0 else _lib.TEXT_KV_REUSE)
        torch.cuda.synchronize()
        assert torch.equal(hid_c, hid_py), f"patch {p}"
        assert torch.equal(enc_c, enc_py) if p == 0 else enc_c is None
        assert torch.equal(kv_c, entry.tensors[0]), f"stale buffer after patch {p}"
        assert torch.isfinite(text_kv.float()).all()
    # what cannot be meant is refused before anything is launched
    with pytest.raises(_lib.HditError):
        call(xp, e, t, skip_text_output=False, kv_buffer=kv_c, kv_row0=starts[1], text_kv=text_kv, text_kv_mode=_lib.TEXT_KV_REUSE)
    with pytest.raises(ValueError):
        call(xp, e, t, skip_text_output=True, kv_buffer=kv_c, kv_row0=starts[1], text_kv=text_kv[:, :10], text_kv_mode=_lib.TEXT_KV_REUSE)
    a = call.args
    a.text_kv, a.text_kv_mode = None, _lib.TEXT_KV_STORE
    assert _lib.lib().hdit_block_sd3_workspace_bytes(C.byref(a)) == -1


def test_block_sd3_one_call_with_fp8_attention(hdit):
    """``fp8_attention`` in the entry point's arguments: absmax scales, quantised K / V copy and the fp8 kernel from
    inside the one call, against the Python block with its attention on the same path (bit-identical) and the
    oracle at the fp8 tolerance."""
    from hetu_dit_amd import ops, synthetic

    B, N, Nt, D, H = 2, 700, 77, 512, 8
    blk, params = make_block(False, 41, D, H)
    blk.attn.fp8_attention = True
    x, e, t = synthetic.randn_bf16((B, N, D), 42), synthetic.randn_bf16((B, Nt, D), 43), synthetic.randn_bf16((B, D), 44)
    enc_py, hid_py = blk(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV))
    enc_c, hid_c = ops.Sd3BlockCall(blk)(x.to(DEV), e.to(DEV), t.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(hid_c, hid_py) and torch.equal(enc_c, enc_py)
    want_e, want_h = oracle.sd3_joint_block(params, x.float(), e.float(), t.float(), H)
    assert_parity(hid_c, want_h, rel=3e-2, cos=0.999, what="fp8 block hidden")
    assert_parity(enc_c, want_e, rel=3e-2, cos=0.999, what="fp8 block encoder")


def test_block_sd3_residuals_left_to_the_next_normalisation(hdit):
    """``lazy_residual`` / ``defer_*`` / ``pending_*``: a chain of three blocks (the last ``context_pre_only``)
    in which every gated residual of the f32 streams is added by the normalisation that reads the stream next
    returns the bits of the chain with the residuals fused into the GEMM epilogues; and what the entry point
    refuses."""
    from hetu_dit_amd import _lib, synthetic
    from hetu_dit_amd.blocks import StackModulation

    B, N, Nt, D, H = 2, 300, 45, 512, 8
    blks = [make_block(i == 2, 10 + i, D, H)[0] for i in range(3)]
    for b in blks[:2]:
        b.stream_dtype = torch.float32
    x, e, t = (synthetic.randn_bf16(s, k).to(DEV) for s, k in (((B, N, D), 5), ((B, Nt, D), 6), ((B, D), 7)))
    mods = StackModulation(torch.nn.ModuleList(blks)).precompute_by_module(t)
    flat, offsets = mods
    calls = [hdit.ops.Sd3BlockCall(b) for b in blks]

    def chain(lazy):
        h, enc, pend = x, e, (None, None)
        for i, (b, call) in enumerate(zip(blks, calls)):
            addr = lambda m: flat.data_ptr() + 4 * offsets[m]
            enc, h = call(h, enc, t, out_dtype=b.stream_dtype, modulation_img=addr(b.norm1),
                          modulation_txt=addr(b.norm1_context), pending_img=pend[0], pending_txt=pend[1],
                          defer=lazy and i < 2, lazy=lazy)
            pend = call.deferred if call.deferred is not None else (None, None)
            assert (call.deferred is not None) == (lazy and i < 2)
        return h

    fused, lazy = chain(False).clone(), chain(True).clone()
    torch.cuda.synchronize()
    assert fused.dtype == torch.bfloat16 and torch.equal(fused, lazy)
    # refusals: nothing may be left owing on a bf16 output, without the modulation, or owed to a bf16 stream
    lib = _lib.lib()
    call = calls[0]
    call.prepare(x.float(), e.float(), t, out_dtype=torch.float32, modulation_img=flat.data_ptr() + 4 * offsets[blks[0].norm1],
                 modulation_txt=flat.data_ptr() + 4 * offsets[blks[0].norm1_context], defer=True, lazy=True)
    a = call.args
    assert lib.hdit_block_sd3_workspace_bytes(C.byref(a)) > 0
    keep = a.modulation_img
    a.modulation_img = None
    assert lib.hdit_block_sd3_workspace_bytes(C.byref(a)) == -1
    a.modulation_img = keep
    a.out_f32 = 0
    assert lib.hdit_block_sd3_workspace_bytes(C.byref(a)) == -1
    a.out_f32 = 1
    a.pending_img, a.pending_img_gate, a.hidden_f32 = a.defer_img, a.modulation_img, 0
    assert lib.hdit_block_sd3_workspace_bytes(C.byref(a)) == -1
    a.hidden_f32 = 1
    a.pending_img_gate = None
    assert lib.hdit_block_sd3_workspace_bytes(C.byref(a)) == -1
    a.pending_img = None
    a.lazy_residual = 2
    assert lib.hdit_block_sd3_workspace_bytes(C.byref(a)) == -1
    with pytest.raises(ValueError):  # the binding refuses the same before the library sees it
        call.prepare(x.float(), e.float(), t, out_dtype=torch.bfloat16, modulation_img=keep, modulation_txt=keep, defer=True)


def test_block_sd3_refuses_bad_arguments(hdit):
    from hetu_dit_amd import _lib

    lib = _lib.lib()
    a = _lib.Sd3BlockArgs()
    assert lib.hdit_block_sd3_workspace_bytes(C.byref(a)) == -1
    assert lib.hdit_block_sd3(C.byref(a), None) == -1
    assert lib.hdit_block_sd3(None, None) == -1


@pytest.mark.parametrize("stream_f32", [False, True])
def test_block_flux_one_call_matches_python_blocks(hdit, stream_f32):
    """``hdit_block_flux_double`` and ``hdit_block_flux_single`` against the Python blocks (bit-identical) and the
    oracle."""
    from hetu_dit_amd import blocks, synthetic
    from hetu_dit_amd.runtime_state import get_runtime_state

    print(f"hdit_block_flux_* fp32 stream={stream_f32}", flush=True)
    B, Nt, gh, gw, D, H, hd = 2, 40, 12, 16, 512, 4, 128
    N = gh * gw
    cos, sin = synthetic.rope_table(synthetic.flux_ids(Nt, gh, gw), (16, 56, 56))
    rope = (cos.to(DEV), sin.to(DEV))
    dbl = synthetic.init_module_(blocks.FluxTransformerBlock(D, H, hd), 21)
    sgl = synthetic.init_module_(blocks.FluxSingleTransformerBlock(D, H, hd), 22)
    p_dbl, p_sgl = oracle_params(dbl), oracle_params(sgl)
    dbl, sgl = dbl.to(DEV), sgl.to(DEV)
    x, e, t = synthetic.randn_bf16((B, N, D), 23).to(DEV), synthetic.randn_bf16((B, Nt, D), 24).to(DEV), synthetic.randn_bf16((B, D), 25).to(DEV)
    dt = torch.bfloat16
    if stream_f32:
        x, e, dt = x.float() + 1e-3, e.float() - 1e-3, torch.float32
        dbl.stream_dtype = sgl.stream_dtype = torch.float32
    enc_py, hid_py = dbl(hidden_states=x, encoder_hidden_states=e, temb=t, image_rotary_emb=rope)
    enc_c, hid_c = hdit.ops.block_flux_double(dbl, x, e, t, rope, out_dtype=dt)
    torch.cuda.synchronize()
    assert torch.equal(hid_c, hid_py) and torch.equal(enc_c, enc_py)
    o_enc, o_hid = oracle.flux_double_block(p_dbl, x.float().cpu(), e.float().cpu(), t.float().cpu(), (cos, sin), H)
    assert_parity(hid_c, o_hid, what="hdit_block_flux_double hidden")
    assert_parity(enc_c, o_enc, what="hdit_block_flux_double encoder")
    get_runtime_state().max_condition_sequence_length = Nt
    joint = torch.cat([e, x], 1).contiguous()
    out_py = sgl(hidden_states=joint, temb=t, image_rotary_emb=rope)
    out_c = hdit.ops.block_flux_single(sgl, joint, t, rope, out_dtype=dt)
    torch.cuda.synchronize()
    assert torch.equal(out_c, out_py)
    assert_parity(out_c, oracle.flux_single_block(p_sgl, joint.float().cpu(), t.float().cpu(), (cos, sin), H, n_text=Nt),
                  what="hdit_block_flux_single")


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("stream_f32", [False, True])
def test_block_cogvideox_one_call_matches_python_block(hdit, stream_f32, fp8):
    from hetu_dit_amd import blocks, synthetic

    print(f"hdit_block_cogvideox fp32 stream={stream_f32} fp8 attention={fp8}", flush=True)
    B, Nt, grid, D, H, hd = 2, 26, (3, 6, 8), 256, 4, 64
    N = grid[0] * grid[1] * grid[2]
    cos, sin = synthetic.rope_table(synthetic.cogvideox_positions(*grid), (16, 24, 24))
    rope = (cos.to(DEV), sin.to(DEV))
    blk = synthetic.init_module_(blocks.CogVideoXBlock(D, H, hd, time_embed_dim=64), 31)
    params = oracle_params(blk)
    blk = blk.to(DEV)
    blk.attn1.fp8_attention = fp8
    x, e, t = synthetic.randn_bf16((B, N, D), 32).to(DEV), synthetic.randn_bf16((B, Nt, D), 33).to(DEV), synthetic.randn_bf16((B, 64), 34).to(DEV)
    dt = torch.bfloat16
    if stream_f32:
        x, e, dt = x.float() + 1e-3, e.float() - 1e-3, torch.float32
        blk.stream_dtype = torch.float32
    hid_py, enc_py = blk(hidden_states=x, encoder_hidden_states=e, temb=t, image_rotary_emb=rope)
    hid_c, enc_c = hdit.ops.block_cogvideox(blk, x, e, t, rope, out_dtype=dt)
    torch.cuda.synchronize()
    assert torch.equal(hid_c, hid_py) and torch.equal(enc_c, enc_py)
    o_hid, o_enc = oracle.cogvideox_block(params, x.float().cpu(), e.float().cpu(), t.float().cpu(), (cos, sin), H)
    tol = dict(rel=3e-2, cos=0.999) if fp8 else {}
    assert_parity(hid_c, o_hid, what="hdit_block_cogvideox hidden", **tol)
    assert_parity(enc_c, o_enc, what="hdit_block_cogvideox encoder", **tol)


def _flux_stack(seed, layers=2, single_layers=3, D=512, H=4, hd=128):
    from hetu_dit_amd import synthetic, transformer

    stack = transformer.FluxTransformerBlocks(layers, single_layers, D, H, hd)
    synthetic.init_module_(stack, seed)
    return stack.to(DEV)


@pytest.mark.parametrize("B", [1, 2])
def test_flux_stack_through_entry_points_full_and_patches(hdit, B):
    """``FluxTransformerBlocks`` with every block as one ``hdit_block_flux_double`` / ``_single`` call (modulation
    from the stack's one GEMV, image K|V written straight into the layers' buffers) against the same stack
    launched kernel by kernel: a full-sequence pass, then every pipeline patch over the stale buffers
    (reference layers/attention_processor.py:908-922), bit for bit, outputs and buffers."""
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state

    Nt, gh, gw, D, P = 24, 16, 8, 512, 4
    N = gh * gw
    starts = [gh // P * gw * i for i in range(P + 1)]
    cos, sin = synthetic.rope_table(synthetic.flux_ids(Nt, gh, gw), (16, 56, 56))
    stack = _flux_stack(71)
    x_prev, x_now = synthetic.randn_bf16((B, N, D), 72).to(DEV), synthetic.randn_bf16((B, N, D), 73).to(DEV)
    e, t = synthetic.randn_bf16((B, Nt, D), 74).to(DEV), synthetic.randn_bf16((B, D), 75).to(DEV)
    rs = get_runtime_state()
    rs.set_token_patches(starts)
    rs.max_condition_sequence_length = Nt
    cm = get_cache_manager()

    def buffers():
        return [entry.tensors[0] for entry in cm.cache.values() if entry.tensors[0] is not None]

    def run_step(entry_points: bool):
        stack.use_block_entry_points = entry_points
        outs = []
        rs.set_patched_mode(False)
        rope = (cos.to(DEV), sin.to(DEV))
        outs.append([o.clone() for o in stack(x_prev, e, t, rope)])
        rs.set_patched_mode(True)
        for p in range(P):
            rows = torch.cat([torch.arange(Nt), Nt + torch.arange(starts[p], starts[p + 1])])
            rope = (cos[rows].contiguous().to(DEV), sin[rows].contiguous().to(DEV))
            outs.append([o.clone() for o in stack(x_now[:, starts[p]:starts[p + 1]].contiguous(), e, t, rope)])
            rs.next_patch()
        rs.set_patched_mode(False)
        torch.cuda.synchronize()
        return outs, [b.clone() for b in buffers()]

    want, want_buf = run_step(False)
    got, got_buf = run_step(True)
    assert len(want_buf) == len(got_buf) == 5
    for i, (g, w) in enumerate(zip(got, want)):
        assert torch.equal(g[0], w[0]) and torch.equal(g[1], w[1]), f"pass {i}"
    # the per-kernel full pass registers strided views of its q|k|v tensors, the entry points contiguous buffers:
    # compare contents
    for g, w in zip(got_buf, want_buf):
        assert torch.equal(g, w)


def test_cogvideox_stack_through_entry_points(hdit):
    from hetu_dit_amd import synthetic, transformer

    B, Nt, grid, D, H, hd, L = 2, 26, (3, 6, 8), 256, 4, 64, 3
    N = grid[0] * grid[1] * grid[2]
    cos, sin = synthetic.rope_table(synthetic.cogvideox_positions(*grid), (16, 24, 24))
    stack = transformer.CogVideoXTransformerBlocks(L, D, H, hd, time_embed_dim=64)
    synthetic.init_module_(stack, 81)
    stack = stack.to(DEV)
    x, e, t = synthetic.randn_bf16((B, N, D), 82).to(DEV), synthetic.randn_bf16((B, Nt, D), 83).to(DEV), synthetic.randn_bf16((B, 64), 84).to(DEV)
    rope = (cos.to(DEV), sin.to(DEV))
    stack.use_block_entry_points = False
    want = [o.clone() for o in stack(x, e, t, rope)]
    stack.use_block_entry_points = True
    got = stack(x, e, t, rope)
    torch.cuda.synchronize()
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
