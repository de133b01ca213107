"""Block-level parity: each of the four block types, on the HIP path, against
the fp32 oracle fed the same bf16-rounded weights and inputs."""
import pytest
import torch

import oracle
from tests.util import assert_parity, oracle_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make(hdit, cls, seed, *args, **kw):
    from hetu_dit_amd import synthetic

    blk = cls(*args, **kw)
    synthetic.init_module_(blk, seed)
    params = oracle_params(blk)
    return blk.to(DEV), params


@pytest.fixture(autouse=True)
def fresh_state():
    from hetu_dit_amd.cache_manager import reset_cache_manager
    from hetu_dit_amd.runtime_state import reset_runtime_state

    reset_runtime_state()
    yield
    reset_cache_manager()
    reset_runtime_state()


@pytest.mark.parametrize("pre_only", [False, True])
def test_sd3_joint_block(hdit, pre_only):
    from hetu_dit_amd import blocks, synthetic

    B, N, Nt, D, H = 2, 320, 77, 256, 4
    blk, params = make(hdit, blocks.JointTransformerBlock, 1, D, H, 64, context_pre_only=pre_only)
    x, e, t = synthetic.randn_bf16((B, N, D), 2), synthetic.randn_bf16((B, Nt, D), 3), synthetic.randn_bf16((B, D), 4)
    enc, hid = blk(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV))
    torch.cuda.synchronize()
    o_enc, o_hid = oracle.sd3_joint_block(params, x.float(), e.float(), t.float(), H, context_pre_only=pre_only)
    assert_parity(hid, o_hid, what="sd3 hidden")
    if pre_only:
        assert enc is None and o_enc is None
    else:
        assert_parity(enc, o_enc, what="sd3 encoder")


def test_sd3_block_config0_shape(hdit):
    """BASELINE config[0]: B1, 1024 image + 333 text tokens, hidden 1536, 24 x 64 heads."""
    from hetu_dit_amd import blocks, synthetic

    B, N, Nt, D, H = 1, 1024, 333, 1536, 24
    blk, params = make(hdit, blocks.JointTransformerBlock, 11, D, H, 64)
    x, e, t = synthetic.randn_bf16((B, N, D), 12), synthetic.randn_bf16((B, Nt, D), 13), synthetic.randn_bf16((B, D), 14)
    enc, hid = blk(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV))
    torch.cuda.synchronize()
    o_enc, o_hid = oracle.sd3_joint_block(params, x.float(), e.float(), t.float(), H)
    assert_parity(hid, o_hid, what="cfg0 hidden")
    assert_parity(enc, o_enc, what="cfg0 encoder")


def test_sd3_attention_wrapper_reference_api(hdit):
    """hetuDiTAttentionWrapper.forward / hetuDiTFeedForwardWrapper.forward as the
    reference's blocks call them (no fused residual)."""
    from hetu_dit_amd import blocks, synthetic
    from oracle.blocks import feed_forward, sd3_joint_attention

    B, N, Nt, D, H = 1, 200, 50, 256, 4
    blk, params = make(hdit, blocks.JointTransformerBlock, 5, D, H, 64)
    x, e = synthetic.randn_bf16((B, N, D), 6), synthetic.randn_bf16((B, Nt, D), 7)
    a, ca = blk.attn(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV))
    f = blk.ff(x.to(DEV))
    torch.cuda.synchronize()
    oa, oca = sd3_joint_attention(params, x.float(), e.float(), H, False)
    assert_parity(a, oa, what="attn hidden")
    assert_parity(ca, oca, what="attn encoder")
    assert_parity(f, feed_forward(params, "ff", x.float()), what="ff")


def test_layer_wrappers_inside_a_compiled_caller(hdit):
    """A traced block of the caller's own (the reference compiles diffusers' block code around the wrapped layers,
    ``base_pipeline.py:274-279``) reaches the attention and feed-forward wrappers: Dynamo must break the graph at
    them, run them as written and resume -- same bits as the uncompiled caller."""
    from hetu_dit_amd import blocks, synthetic

    B, N, Nt, D, H = 1, 200, 50, 256, 4
    blk, _ = make(hdit, blocks.JointTransformerBlock, 5, D, H, 64)
    x, e = synthetic.randn_bf16((B, N, D), 6).to(DEV), synthetic.randn_bf16((B, Nt, D), 7).to(DEV)

    def caller(x, e):
        a, ca = blk.attn(hidden_states=x * 0.5, encoder_hidden_states=e)
        return x + a, e + ca, blk.ff(x) * 2.0

    want = caller(x, e)
    torch.cuda.synchronize()
    torch._dynamo.reset()
    got = torch.compile(caller, backend="eager")(x, e)
    torch.cuda.synchronize()
    for g_, w_ in zip(got, want):
        assert torch.equal(g_, w_)
    torch._dynamo.reset()


@pytest.mark.parametrize("activation_fn", ["gelu", "geglu", "linear-silu", "gelu-approximate"])
def test_feed_forward_wrapper_other_first_layers(hdit, activation_fn):
    """hetuDiTFeedForwardWrapper over the first-layer classes the reference's wrapper accepts
    (``layers/feedforward.py:25-57``): exact GELU, GEGLU, LinearActivation, beside the tanh GELU of the models."""
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.base_model import wrap_layer
    from hetu_dit_amd.layers.modules import FeedForward
    from oracle.blocks import feed_forward

    print(f"ff wrapper activation_fn={activation_fn}", flush=True)
    D, Fi = 256, 640
    ff = FeedForward(D, inner_dim=Fi, activation_fn=activation_fn)
    synthetic.init_module_(ff, 31, std=0.1)
    params = {"ff." + k: v.detach().float() for k, v in ff.state_dict().items()}
    wrapped = wrap_layer(ff).to(DEV)
    x = synthetic.randn_bf16((2, 333, D), 32)
    got = wrapped(x.to(DEV))
    torch.cuda.synchronize()
    assert got.shape == x.shape
    assert_parity(got, feed_forward(params, "ff", x.float(), activation_fn=activation_fn), what=f"ff {activation_fn}")
    if activation_fn != "gelu-approximate":
        with pytest.raises(TypeError):
            wrapped.in_problem(x.to(DEV).view(-1, D))


def test_ff_activation_entry_point_refusals(hdit):
    import ctypes as C

    lib = hdit._lib.lib()
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=DEV)
    y = torch.zeros(4, 32, dtype=torch.bfloat16, device=DEV)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ok = lib.hdit_ff_activation(x.data_ptr(), y.data_ptr(), 4, 32, 64, 32, hdit.ops.ACT_GEGLU, st)
    assert ok == 0
    assert lib.hdit_ff_activation(x.data_ptr(), x.data_ptr(), 4, 32, 64, 64, hdit.ops.ACT_GEGLU, st) != 0  # in place
    assert lib.hdit_ff_activation(x.data_ptr(), y.data_ptr(), 4, 32, 32, 32, hdit.ops.ACT_GEGLU, st) != 0  # no gate half
    assert lib.hdit_ff_activation(x.data_ptr(), y.data_ptr(), 4, 32, 64, 32, 7, st) != 0                  # unknown kind
    assert lib.hdit_ff_activation(x.data_ptr(), y.data_ptr(), 4, 30, 64, 32, hdit.ops.ACT_SILU, st) != 0    # width % 8
    assert lib.hdit_ff_activation(x.data_ptr(), x.data_ptr(), 4, 64, 64, 64, hdit.ops.ACT_SILU, st) == 0    # in place ok
    torch.cuda.synchronize()


def test_flux_double_and_single_blocks(hdit):
    from hetu_dit_amd import blocks, synthetic
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, Nt, gh, gw, D, H, hd = 1, 40, 12, 16, 512, 4, 128
    N = gh * gw
    ids = synthetic.flux_ids(Nt, gh, gw)
    cos, sin = synthetic.rope_table(ids, (16, 56, 56))
    ocos, osin = oracle.flux_rope_table(ids, (16, 56, 56))
    assert torch.equal(cos, ocos) and torch.equal(sin, osin)
    rope = (cos.to(DEV), sin.to(DEV))
    dbl, p_dbl = make(hdit, blocks.FluxTransformerBlock, 21, D, H, hd)
    sgl, p_sgl = make(hdit, blocks.FluxSingleTransformerBlock, 22, D, H, hd)
    x, e, t = synthetic.randn_bf16((B, N, D), 23), synthetic.randn_bf16((B, Nt, D), 24), synthetic.randn_bf16((B, D), 25)
    enc, hid = dbl(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV), image_rotary_emb=rope)
    torch.cuda.synchronize()
    o_enc, o_hid = oracle.flux_double_block(p_dbl, x.float(), e.float(), t.float(), (cos, sin), H)
    assert_parity(hid, o_hid, what="flux double hidden")
    assert_parity(enc, o_enc, what="flux double encoder")
    # single block on the joint [text, image] sequence
    get_runtime_state().max_condition_sequence_length = Nt
    joint = torch.cat([e, x], dim=1)
    out = sgl(hidden_states=joint.to(DEV), temb=t.to(DEV), image_rotary_emb=rope)
    torch.cuda.synchronize()
    o_out = oracle.flux_single_block(p_sgl, joint.float(), t.float(), (cos, sin), H, n_text=Nt)
    assert_parity(out, o_out, what="flux single")


def test_cogvideox_block(hdit):
    from hetu_dit_amd import blocks, synthetic

    B, Nt, grid, D, H, hd = 1, 26, (3, 6, 8), 256, 4, 64
    N = grid[0] * grid[1] * grid[2]
    pos = synthetic.cogvideox_positions(*grid)
    cos, sin = synthetic.rope_table(pos, (16, 24, 24))
    ocos, osin = oracle.cogvideox_rope_table(*grid, head_dim=64)
    torch.testing.assert_close(cos, ocos, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(sin, osin, rtol=1e-6, atol=1e-6)
    blk, params = make(hdit, blocks.CogVideoXBlock, 31, D, H, hd, time_embed_dim=64)
    x, e, t = synthetic.randn_bf16((B, N, D), 32), synthetic.randn_bf16((B, Nt, D), 33), synthetic.randn_bf16((B, 64), 34)
    hid, enc = blk(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV),
                   image_rotary_emb=(cos.to(DEV), sin.to(DEV)))
    torch.cuda.synchronize()
    o_hid, o_enc = oracle.cogvideox_block(params, x.float(), e.float(), t.float(), (cos, sin), H)
    assert_parity(hid, o_hid, what="cog hidden")
    assert_parity(enc, o_enc, what="cog encoder")
    # reference-shaped wrapper call: (hidden, encoder) after to_out, split from the joint tensor
    from oracle.blocks import cogvideox_attention

    a, ea = blk.attn1(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), image_rotary_emb=(cos.to(DEV), sin.to(DEV)))
    torch.cuda.synchronize()
    oa, oea = cogvideox_attention(params, x.float(), e.float(), (cos, sin), H)
    assert_parity(a, oa, what="cog attn hidden")
    assert_parity(ea, oea, what="cog attn encoder")


def test_sd3_pipefusion_patches_stale_kv(hdit):
    """PipeFusion shard: warm-up pass fills the K/V buffers, then each patch's
    query attends to the whole buffer whose other patches are stale; patch k
    sees patches < k refreshed in this step (in-place update)."""
    from hetu_dit_amd import synthetic, transformer
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, N, Nt, D, H, L, P = 2, 256, 40, 256, 4, 3, 4
    stack = transformer.SD3TransformerBlocks(L, D, H, 64)
    synthetic.init_module_(stack, 41)
    params = [oracle_params(b) for b in stack.transformer_blocks]
    stack = stack.to(DEV)
    rs = get_runtime_state()
    rs.set_token_patches([0, 64, 128, 192, 256])
    x_prev, x_now = synthetic.randn_bf16((B, N, D), 42), synthetic.randn_bf16((B, N, D), 43)
    e, t = synthetic.randn_bf16((B, Nt, D), 44), synthetic.randn_bf16((B, D), 45)

    # oracle: same sequence of calls with StaleKVBuffer per layer
    bufs = [oracle.StaleKVBuffer() for _ in range(L)]
    for kb in bufs:
        kb.set_patches([0, 64, 128, 192, 256])

    def oracle_stack(x, enc, enc_cache, patch_mode, patch_idx):
        for i in range(L):
            bufs[i].patch_mode, bufs[i].pipeline_patch_idx = patch_mode, patch_idx
            if patch_mode and patch_idx == 0:
                enc_cache[i] = enc
            enc_in = enc_cache[i] if (patch_mode and patch_idx > 0) else enc
            new_enc, x = oracle.sd3_joint_block(params[i], x, enc_in, t.float(), H, context_pre_only=(i == L - 1),
                                                kv=bufs[i])
            if not (patch_mode and patch_idx > 0):
                enc = new_enc
        return x

    # warm-up (previous step), whole sequence
    rs.set_patched_mode(False)
    got = stack(x_prev.to(DEV), e.to(DEV), t.to(DEV))
    want = oracle_stack(x_prev.float(), e.float(), [None] * L, False, 0)
    torch.cuda.synchronize()
    assert_parity(got, want, what="warm-up step")

    rs.set_patched_mode(True)
    enc_cache = [None] * L
    for p in range(P):
        assert rs.pipeline_patch_idx == p
        sl = slice(64 * p, 64 * (p + 1))
        got = stack(x_now[:, sl].to(DEV), e.to(DEV), t.to(DEV))
        want = oracle_stack(x_now[:, sl].float(), e.float(), enc_cache, True, p)
        torch.cuda.synchronize()
        assert_parity(got, want, what=f"patch {p}")
        rs.next_patch()
    assert rs.pipeline_patch_idx == 0


@pytest.mark.parametrize("family", ["sd3", "cogvideox"])
def test_block_with_fp8_attention(hdit, family):
    """The fp8-e4m3 attention path inside a block, against the fp32 oracle at the tolerance BASELINE.json
    states for it: relative L2 <= 3e-2 on the block outputs."""
    from hetu_dit_amd import blocks, synthetic

    if family == "sd3":
        B, N, Nt, D, H = 2, 320, 77, 256, 4
        blk, params = make(hdit, blocks.JointTransformerBlock, 51, D, H, 64)
        blk.attn.fp8_attention = True
        x, e, t = synthetic.randn_bf16((B, N, D), 52), synthetic.randn_bf16((B, Nt, D), 53), synthetic.randn_bf16((B, D), 54)
        enc, hid = blk(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV))
        torch.cuda.synchronize()
        o_enc, o_hid = oracle.sd3_joint_block(params, x.float(), e.float(), t.float(), H)
    else:
        B, Nt, grid, D, H, hd = 1, 26, (3, 6, 8), 256, 4, 64
        N = grid[0] * grid[1] * grid[2]
        cos, sin = synthetic.rope_table(synthetic.cogvideox_positions(*grid), (16, 24, 24))
        blk, params = make(hdit, blocks.CogVideoXBlock, 55, D, H, hd, time_embed_dim=64)
        blk.attn1.fp8_attention = True
        x, e, t = synthetic.randn_bf16((B, N, D), 56), synthetic.randn_bf16((B, Nt, D), 57), synthetic.randn_bf16((B, 64), 58)
        hid, enc = blk(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV),
                       image_rotary_emb=(cos.to(DEV), sin.to(DEV)))
        torch.cuda.synchronize()
        o_hid, o_enc = oracle.cogvideox_block(params, x.float(), e.float(), t.float(), (cos, sin), H)
    assert_parity(hid, o_hid, rel=3e-2, cos=0.999, what=f"{family} fp8 hidden")
    assert_parity(enc, o_enc, rel=3e-2, cos=0.999, what=f"{family} fp8 encoder")
