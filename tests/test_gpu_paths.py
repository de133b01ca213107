"""Product paths beside the fused block calls, on the HIP path against the oracle: Flux double and single
blocks in PipeFusion patch mode (stale K/V buffer, ``slice_dim=2`` in the reference), the reference-shaped
``CacheManager.update_and_get_kv_cache`` for both cache layouts, ``hetuDiTAttentionWrapper.forward`` for the
Flux branches, layers wrapped by ``wrap_layers`` + ``register_cache`` the way the reference's model wrappers
do it, and a block called on its own after a stack runner with a different ``temb``."""
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


def dev_randn(shape, seed, scale=1.0):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(shape, generator=gen, device=DEV) * scale).to(torch.bfloat16)


def make(cls, seed, *args, **kw):
    from hetu_dit_amd import synthetic

    blk = cls(*args, **kw)
    synthetic.init_module_(blk, seed)
    params = oracle_params(blk)
    return blk.to(DEV), params


@pytest.mark.parametrize("B", [1, 2])
def test_flux_blocks_pipefusion_patches_stale_kv(hdit, B):
    """A full-sequence pass fills the K/V buffers of a double and a single block, then every patch's rows run
    through both blocks against buffers whose other patches are stale.  The cached K rows are normalised and
    rotated before they are stored (attention_processor.py:903-922); the rotary table of a patch call covers
    that call's [text, patch] rows."""
    from hetu_dit_amd import blocks, synthetic
    from hetu_dit_amd.runtime_state import get_runtime_state

    Nt, gh, gw, D, H, hd, P = 24, 16, 8, 512, 4, 128, 4
    N = gh * gw
    rows_per_patch = gh // P
    starts = [rows_per_patch * gw * i for i in range(P + 1)]
    ids = synthetic.flux_ids(Nt, gh, gw)
    cos, sin = synthetic.rope_table(ids, (16, 56, 56))
    dbl, p_dbl = make(blocks.FluxTransformerBlock, 61, D, H, hd)
    sgl, p_sgl = make(blocks.FluxSingleTransformerBlock, 62, D, H, hd)
    x_prev, x_now = synthetic.randn_bf16((B, N, D), 63), synthetic.randn_bf16((B, N, D), 64)
    e, t = synthetic.randn_bf16((B, Nt, D), 65), synthetic.randn_bf16((B, D), 66)
    rs = get_runtime_state()
    rs.set_token_patches(starts)
    rs.max_condition_sequence_length = Nt
    kv_d, kv_s = oracle.StaleKVBuffer(), oracle.StaleKVBuffer()
    kv_d.set_patches(starts), kv_s.set_patches(starts)

    def run_pair(x, rope_rows, patch_mode, patch_idx):
        c, s = cos[rope_rows], sin[rope_rows]
        rope_dev = (c.contiguous().to(DEV), s.contiguous().to(DEV))
        enc, hid = dbl(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=t.to(DEV), image_rotary_emb=rope_dev)
        out = sgl(hidden_states=torch.cat([enc, hid], 1), temb=t.to(DEV), image_rotary_emb=rope_dev)
        torch.cuda.synchronize()
        for kb in (kv_d, kv_s):
            kb.patch_mode, kb.pipeline_patch_idx = patch_mode, patch_idx
        o_enc, o_hid = oracle.flux_double_block(p_dbl, x.float(), e.float(), t.float(), (c, s), H, kv=kv_d)
        o_out = oracle.flux_single_block(p_sgl, torch.cat([o_enc, o_hid], 1), t.float(), (c, s), H, n_text=Nt, kv=kv_s)
        return (enc, hid, out), (o_enc, o_hid, o_out)

    rs.set_patched_mode(False)
    got, want = run_pair(x_prev, torch.arange(Nt + N), False, 0)
    for g, w, name in zip(got, want, ("encoder", "hidden", "single")):
        assert_parity(g, w, what=f"full pass {name}")

    rs.set_patched_mode(True)
    for p in range(P):
        assert rs.pipeline_patch_idx == p
        rows = torch.cat([torch.arange(Nt), Nt + torch.arange(starts[p], starts[p + 1])])
        got, want = run_pair(x_now[:, starts[p]:starts[p + 1]], rows, True, p)
        for g, w, name in zip(got, want, ("encoder", "hidden", "single")):
            assert_parity(g, w, what=f"patch {p} {name}")
        rs.next_patch()
    # the stale buffers were really used: a patch pass on a fresh buffer gives something else
    fresh = oracle.flux_double_block(p_dbl, x_now[:, :starts[1]].float(), e.float(), t.float(),
                                     (cos[: Nt + starts[1]], sin[: Nt + starts[1]]), H)[1]
    kv_d.patch_mode, kv_d.pipeline_patch_idx = True, 0
    stale = oracle.flux_double_block(p_dbl, x_now[:, :starts[1]].float(), e.float(), t.float(),
                                     (cos[: Nt + starts[1]], sin[: Nt + starts[1]]), H, kv=kv_d)[1]
    assert (fresh - stale).norm() / stale.norm() > 1e-3


@pytest.mark.parametrize("slice_dim", [1, 2])
def test_update_and_get_kv_cache_reference_api(hdit, slice_dim):
    """``update_and_get_kv_cache(new_kv=[k, v], layer=, slice_dim=)`` as the reference's processors call it
    (SD3: [B, N, H*d], slice_dim 1; Flux: [B, H, N, d], slice_dim 2): the packed buffer replaces the entry when
    patch mode is off, the current patch's rows are overwritten in place in patch mode, and the two returned
    tensors are strided views of the packed buffer."""
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, H, N, d, P = 2, 3, 64, 64, 4
    starts = [N // P * i for i in range(P + 1)]
    shape = (B, N, H * d) if slice_dim == 1 else (B, H, N, d)
    gen = torch.Generator().manual_seed(7)
    k0, v0 = torch.randn(shape, generator=gen).bfloat16(), torch.randn(shape, generator=gen).bfloat16()
    layer = object()
    cm = get_cache_manager()
    cm.register_cache_entry(layer, "attn", "naive_cache")
    rs = get_runtime_state()
    rs.set_token_patches(starts)
    ref = oracle.StaleKVBuffer()
    ref.set_patches(starts)

    rs.set_patched_mode(False)
    k, v = cm.update_and_get_kv_cache(new_kv=[k0.to(DEV), v0.to(DEV)], layer=layer, slice_dim=slice_dim, layer_type="attn")
    torch.cuda.synchronize()
    rk, rv = ref.update_and_get(k0, v0, slice_dim)
    assert torch.equal(k.float().cpu(), rk) and torch.equal(v.float().cpu(), rv)
    packed = cm.cache["attn", layer].tensors[0]
    inner = shape[-1]
    assert packed.shape[-1] == 2 * inner
    assert k.data_ptr() == packed.data_ptr() and v.data_ptr() == packed.data_ptr() + inner * 2
    assert k.stride(-2) == 2 * inner and v.stride(-2) == 2 * inner  # views of the packed rows, not copies

    rs.set_patched_mode(True)
    ref.patch_mode = True
    for p in (0, 1, 3):  # patch 2 stays stale
        rs.pipeline_patch_idx = ref.pipeline_patch_idx = p
        sl = [slice(None)] * len(shape)
        sl[slice_dim] = slice(starts[p], starts[p + 1])
        kn = torch.randn(k0[tuple(sl)].shape, generator=gen).bfloat16()
        vn = torch.randn(kn.shape, generator=gen).bfloat16()
        k, v = cm.update_and_get_kv_cache(new_kv=[kn.to(DEV), vn.to(DEV)], layer=layer, slice_dim=slice_dim, layer_type="attn")
        torch.cuda.synchronize()
        rk, rv = ref.update_and_get(kn, vn, slice_dim)
        assert k.shape == k0.shape
        assert torch.equal(k.float().cpu(), rk) and torch.equal(v.float().cpu(), rv), f"patch {p}"
        assert cm.cache["attn", layer].tensors[0].data_ptr() == packed.data_ptr()  # updated in place
    sl = [slice(None)] * len(shape)
    sl[slice_dim] = slice(starts[2], starts[3])
    assert torch.equal(k[tuple(sl)].cpu(), k0[tuple(sl)])  # the patch never written kept the first pass's rows
    # a single tensor (already packed) is accepted and returned packed
    rs.set_patched_mode(False)
    whole = torch.randn(*shape[:-1], 2 * inner, generator=gen).bfloat16().to(DEV)
    assert cm.update_and_get_kv_cache(new_kv=whole, layer=layer, slice_dim=slice_dim) is whole
    with pytest.raises(KeyError):
        cm.update_and_get_kv_cache(new_kv=whole, layer=object(), slice_dim=slice_dim)


def test_flux_attention_wrapper_forward_branches(hdit):
    """``hetuDiTAttentionWrapper.forward`` as the diffusers Flux blocks call it: the double block's attention
    returns ``(hidden, encoder)`` after the out-projections (text projection without its bias, as the reference's
    Flux branch, attention_processor.py:284-305), the single block's returns the joint attention output with no
    projection (``:306-319``)."""
    from hetu_dit_amd import blocks, synthetic
    from hetu_dit_amd.runtime_state import get_runtime_state
    from oracle.blocks import flux_attention

    B, Nt, gh, gw, D, H, hd = 2, 20, 6, 8, 512, 4, 128
    N = gh * gw
    cos, sin = synthetic.rope_table(synthetic.flux_ids(Nt, gh, gw), (16, 56, 56))
    rope = (cos.to(DEV), sin.to(DEV))
    dbl, p_dbl = make(blocks.FluxTransformerBlock, 71, D, H, hd)
    sgl, p_sgl = make(blocks.FluxSingleTransformerBlock, 72, D, H, hd)
    x, e = synthetic.randn_bf16((B, N, D), 73), synthetic.randn_bf16((B, Nt, D), 74)
    a, ca = dbl.attn(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), image_rotary_emb=rope)
    torch.cuda.synchronize()
    oa, oca = flux_attention(p_dbl, x.float(), e.float(), (cos, sin), H)
    assert_parity(a, oa, what="flux double attn hidden")
    assert_parity(ca, oca, what="flux double attn encoder")
    get_runtime_state().max_condition_sequence_length = Nt
    joint = torch.cat([e, x], 1)
    o = sgl.attn(hidden_states=joint.to(DEV), image_rotary_emb=rope)
    torch.cuda.synchronize()
    assert o.shape == (B, Nt + N, D)
    assert_parity(o, flux_attention(p_sgl, joint.float(), None, (cos, sin), H, n_text_single=Nt), what="flux single attn")
    # a rotary table that does not cover this call's rows is refused instead of rotating only some of them
    with pytest.raises(ValueError, match="rows"):
        sgl.attn(hidden_states=joint.to(DEV), image_rotary_emb=(rope[0][:-3].contiguous(), rope[1][:-3].contiguous()))
    with pytest.raises(ValueError, match="rows"):
        dbl.attn(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV),
                 image_rotary_emb=(rope[0][:N].contiguous(), rope[1][:N].contiguous()))


def test_layers_wrapped_the_reference_way_run_the_processors(hdit):
    """Unwrapped Attention / FeedForward children wrapped by ``wrap_layers`` (by name / by class) and
    registered by ``register_cache`` -- the wrapper is the cache key -- then called through the wrappers'
    reference-shaped ``forward``, with and without patch mode."""
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.base_model import register_cache, wrap_layers
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.layers.modules import Attention, FeedForward, JointAttnProcessor2_0
    from hetu_dit_amd.runtime_state import get_runtime_state
    from oracle.blocks import feed_forward, sd3_joint_attention
    from torch import nn

    D, H = 256, 4

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = Attention(D, H, 64, added_kv_proj_dim=D, context_pre_only=False, bias=True,
                                  processor=JointAttnProcessor2_0())
            self.ff = FeedForward(D)

    blk = Block()
    wrapped = wrap_layers(blk, submodule_classes_to_wrap=[FeedForward], submodule_name_to_wrap=["attn"])
    register_cache(wrapped)
    synthetic.init_module_(blk, 81)
    params = oracle_params(blk)
    blk = blk.to(DEV)
    assert ("attn", blk.attn) in get_cache_manager().cache
    B, N, Nt = 2, 128, 30
    x, x2, e = synthetic.randn_bf16((B, N, D), 82), synthetic.randn_bf16((B, N, D), 83), synthetic.randn_bf16((B, Nt, D), 84)
    kv = oracle.StaleKVBuffer()
    kv.set_patches([0, 64, 128])
    rs = get_runtime_state()
    rs.set_token_patches([0, 64, 128])
    a, ca = blk.attn(hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV))
    f = blk.ff(x.to(DEV))
    torch.cuda.synchronize()
    oa, oca = sd3_joint_attention(params, x.float(), e.float(), H, False, kv=kv)
    assert_parity(a, oa, what="wrapped attn hidden")
    assert_parity(ca, oca, what="wrapped attn encoder")
    assert_parity(f, feed_forward(params, "ff", x.float()), what="wrapped ff")
    rs.set_patched_mode(True)
    kv.patch_mode = True
    rs.pipeline_patch_idx = kv.pipeline_patch_idx = 1
    a, ca = blk.attn(hidden_states=x2[:, 64:].to(DEV), encoder_hidden_states=e.to(DEV))
    torch.cuda.synchronize()
    oa, oca = sd3_joint_attention(params, x2[:, 64:].float(), e.float(), H, False, kv=kv)
    assert_parity(a, oa, what="wrapped attn hidden, patch 1 over a stale buffer")
    assert_parity(ca, oca, what="wrapped attn encoder, patch 1 over a stale buffer")


def test_block_called_alone_after_a_stack_run_uses_its_own_temb(hdit):
    """The stack runner computes every block's adaLN projection in one launch and hands it to the blocks; a
    block called on its own afterwards with another conditioning vector must not reuse that result, even when
    the allocator places the new ``temb`` where the old one lived."""
    from hetu_dit_amd import synthetic, transformer

    B, N, Nt, D, H, L = 2, 96, 20, 256, 4, 2
    stack = transformer.SD3TransformerBlocks(L, D, H, 64)
    synthetic.init_module_(stack, 91)
    params = oracle_params(stack.transformer_blocks[0])
    stack = stack.to(DEV)
    x, e = synthetic.randn_bf16((B, N, D), 92), synthetic.randn_bf16((B, Nt, D), 93)
    t1, t2 = synthetic.randn_bf16((B, D), 94), synthetic.randn_bf16((B, D), 95)
    temb = t1.to(DEV)
    addr = temb.data_ptr()
    stack(x.to(DEV), e.to(DEV), temb)
    torch.cuda.synchronize()
    del temb
    new = t2.to(DEV)  # same size: the caching allocator may return the block just freed
    same_address = new.data_ptr() == addr
    enc, hid = stack.transformer_blocks[0](hidden_states=x.to(DEV), encoder_hidden_states=e.to(DEV), temb=new)
    torch.cuda.synchronize()
    o_enc, o_hid = oracle.sd3_joint_block(params, x.float(), e.float(), t2.float(), H)
    assert_parity(hid, o_hid, what=f"block alone with a new temb (address reused: {same_address})")
    assert_parity(enc, o_enc, what="block alone with a new temb, encoder")


def test_sd3_patches_skip_the_dropped_text_stream_bit_exact(hdit):
    """For pipeline patches after the first the block loop drops every block's text output
    (transformer_sd3.py:131-146); the runner therefore asks the blocks not to compute it.  The image output of
    every patch must equal, bit for bit, what the same blocks return when they do compute the text stream."""
    from hetu_dit_amd import synthetic, transformer
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, N, Nt, D, H, L, P = 2, 1024, 333, 512, 8, 3, 4
    starts = [N // P * i for i in range(P + 1)]
    stack = transformer.SD3TransformerBlocks(L, D, H, 64)
    synthetic.init_module_(stack, 101)
    stack = stack.to(DEV)
    x_prev, x_now = synthetic.randn_bf16((B, N, D), 102).to(DEV), synthetic.randn_bf16((B, N, D), 103).to(DEV)
    e, t = synthetic.randn_bf16((B, Nt, D), 104).to(DEV), synthetic.randn_bf16((B, D), 105).to(DEV)
    rs = get_runtime_state()
    rs.set_token_patches(starts)
    rs.set_patched_mode(False)
    stack(x_prev, e, t)
    torch.cuda.synchronize()
    saved = {k: [None if b is None else b.clone() for b in v.tensors] for k, v in get_cache_manager().cache.items()}

    def full_text_pass(p):
        """the reference's loop: every block computes both streams, the text output is dropped for p > 0"""
        hid, enc = x_now[:, starts[p]:starts[p + 1]].contiguous(), e
        for i, blk in enumerate(stack.transformer_blocks):
            if p == 0:
                enc_cache[i] = enc
                enc, hid = blk(hidden_states=hid, encoder_hidden_states=enc, temb=t)
            else:
                _, hid = blk(hidden_states=hid, encoder_hidden_states=enc_cache[i], temb=t)
        return hid

    rs.set_patched_mode(True)
    enc_cache = [None] * L
    want = []
    for p in range(P):
        want.append(full_text_pass(p).clone())
        rs.next_patch()
    torch.cuda.synchronize()
    for k, v in get_cache_manager().cache.items():  # back to the buffers of the previous step
        for dst, src in zip(v.tensors, saved[k]):
            if dst is not None:
                dst.copy_(src)
    rs.set_patched_mode(True)
    for p in range(P):
        got = stack(x_now[:, starts[p]:starts[p + 1]].contiguous(), e, t)
        torch.cuda.synchronize()
        assert torch.equal(got, want[p]), f"patch {p}: skipping the text stream changed the image output"
        rs.next_patch()
    # and a block asked to skip it returns None for the text stream
    enc, hid = stack.transformer_blocks[0](hidden_states=x_now[:, :starts[1]].contiguous(), encoder_hidden_states=e, temb=t,
                                           skip_text_output=True)
    assert enc is None and hid.shape == (B, starts[1], D)


def test_sd3_attention_wrapper_takes_channel_major_4d_inputs(hdit):
    """``[B, C, H, W]`` inputs to the wrapper are token sequences in channel-major layout
    (attention_processor.py:672-683) and the outputs come back in that layout (:436-443): same numbers as the
    ``[B, T, C]`` call, which is checked against the oracle elsewhere."""
    from hetu_dit_amd import blocks, synthetic

    B, D, H, gh, gw, th, tw = 2, 256, 4, 6, 10, 3, 7
    blk, _ = make(blocks.JointTransformerBlock, 201, D, H, 64)
    wrapper = blk.attn
    x4 = synthetic.randn_bf16((B, D, gh, gw), 202).to(DEV)
    e4 = synthetic.randn_bf16((B, D, th, tw), 203).to(DEV)
    out4, enc4 = wrapper(x4, encoder_hidden_states=e4)
    x3, e3 = x4.flatten(2).transpose(1, 2).contiguous(), e4.flatten(2).transpose(1, 2).contiguous()
    out3, enc3 = wrapper(x3, encoder_hidden_states=e3)
    torch.cuda.synchronize()
    assert out4.shape == (B, D, gh, gw) and enc4.shape == (B, D, th, tw)
    assert torch.equal(out4.flatten(2).transpose(1, 2), out3) and torch.equal(enc4.flatten(2).transpose(1, 2), enc3)
