"""Head and tail of an SD3 denoise step on the HIP path against the oracle: patchify / unpatchify (bit-exact
data movement), timestep projection, SiLU, guidance + Euler update (bit-exact against the bf16 / fp32 tensor
expressions), the patch-embedding wrapper with and without pipeline patches, and the whole transformer
from latent to predicted noise."""
import pytest
import torch

from oracle import step as S
from tests.util import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def fresh_state():
    from hetu_dit_amd.cache_manager import reset_cache_manager
    from hetu_dit_amd.runtime_state import reset_runtime_state

    reset_runtime_state()
    yield
    reset_cache_manager()
    reset_runtime_state()


def step_params(model) -> dict:
    """fp32 parameters and buffers under the unwrapped names the oracle uses."""
    from tests.util import oracle_params

    out = {}
    for i, blk in enumerate(model.transformer_blocks):
        for k, v in oracle_params(blk).items():
            out[f"transformer_blocks.{i}.{k}"] = v
    for name, p in list(model.named_parameters()) + list(model.named_buffers()):
        if not name.startswith("transformer_blocks."):
            out[name.replace(".module.", ".")] = p.detach().float().cpu()
    return out


@pytest.mark.parametrize("B,C,H,W,p", [(2, 16, 32, 48, 2), (1, 3, 8, 16, 4), (3, 5, 6, 6, 1), (1, 16, 128, 128, 2)])
def test_patchify_unpatchify_exact(hdit, B, C, H, W, p):
    print(f"patchify {B} {C} {H} {W} {p}", flush=True)
    ops = hdit.ops
    torch.manual_seed(0)
    lat = torch.randn(B, C, H, W).bfloat16()
    got = ops.patchify(lat.to(DEV), p)
    want = lat.reshape(B, C, H // p, p, W // p, p).permute(0, 2, 4, 1, 3, 5).reshape(B, (H // p) * (W // p), C * p * p)
    assert torch.equal(got.cpu(), want)
    x = torch.randn(B, (H // p) * (W // p), p * p * C).bfloat16()
    got = ops.unpatchify(x.to(DEV), C, H, W, p)
    assert torch.equal(got.cpu(), S.unpatchify(x, C, H, W, p))


def test_patchify_refuses_ragged_grid(hdit):
    from hetu_dit_amd._lib import HditError

    with pytest.raises((HditError, ValueError)):
        hdit.ops.patchify(torch.zeros(1, 4, 7, 8, dtype=torch.bfloat16, device=DEV), 2)
    assert hdit.ops.patchify(torch.zeros(0, 4, 8, 8, dtype=torch.bfloat16, device=DEV), 2).shape == (0, 16, 16)


def test_timestep_embedding_and_silu(hdit):
    ops = hdit.ops
    t = torch.tensor([0.0, 1.0, 17.5, 500.0, 999.0, 1000.0])
    got = ops.timestep_embedding(t.to(DEV), 256).float().cpu()
    want = S.timestep_embedding(t, 256)
    # bf16 rounding of values in [-1, 1]: absolute error below 2^-9
    assert (got - want).abs().max() < 2.0 ** -8
    assert_parity(got, want, what="timestep embedding")
    assert torch.equal(got[0, :128], torch.ones(128)) and torch.equal(got[0, 128:], torch.zeros(128))
    x = (torch.randn(7, 1536) * 3).bfloat16()
    y = ops.silu(x.to(DEV))
    assert_parity(y, torch.nn.functional.silu(x.float()), rel=4e-3, what="silu")


@pytest.mark.parametrize("guidance,sigma,sigma_next", [(7.0, 1.0, 0.9644), (4.5, 0.3127, 0.25), (1.0, 0.0421, 0.0), (0.0, 0.5, 0.5)])
def test_cfg_euler_step_bit_exact(hdit, guidance, sigma, sigma_next):
    torch.manual_seed(3)
    u, c, x = (torch.randn(2, 16, 64, 64).bfloat16() for _ in range(3))
    got = hdit.ops.cfg_euler_step(u.to(DEV), c.to(DEV), x.to(DEV), guidance, sigma, sigma_next)
    want = S.cfg_euler_step(u, c, x, guidance, sigma, sigma_next)
    assert torch.equal(got.cpu(), want)


def test_patch_embed_wrapper_full_and_patches(hdit):
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.layers.embeddings import hetuDiTPatchEmbedWrapper
    from hetu_dit_amd.layers.modules import PatchEmbed
    from hetu_dit_amd.registry import hetuDiTLayerWrappersRegister
    from hetu_dit_amd.runtime_state import get_runtime_state

    pe = PatchEmbed(64, 64, 2, 16, 256, pos_embed_max_size=48)
    synthetic.init_module_(pe, 5)
    assert hetuDiTLayerWrappersRegister.get_wrapper(pe) is hetuDiTPatchEmbedWrapper
    wrap = hetuDiTPatchEmbedWrapper(pe).to(DEV)
    w, b = pe.proj.weight.detach().float().cpu(), pe.proj.bias.detach().float().cpu()
    table = pe.pos_embed[0].float().cpu()
    lat = synthetic.randn_bf16((2, 16, 48, 40), 6)  # 24 x 20 tokens, not the module's own 32 x 32
    want = S.patch_embed(lat.float(), w, b, S.cropped_pos_embed(table, 48, 24, 20))
    got = wrap(lat.to(DEV))
    assert_parity(got, want, what="patch embed (full image)")

    # pipeline patches: rows [0, 16), [16, 32), [32, 48) of the latent get rows of the whole image's table
    rs = get_runtime_state()
    rs.set_patches(48, 40, 2, 3)
    rs.set_patched_mode(True)
    for i in range(rs.num_pipeline_patch):
        r0, r1 = rs.pp_patches_start_idx_local[i], rs.pp_patches_start_idx_local[i + 1]
        t0, t1 = rs.pp_patches_token_start_end_idx_global[i]
        got = wrap(lat[:, :, r0:r1].contiguous().to(DEV))
        assert_parity(got, want[:, t0:t1], what=f"patch embed (pipeline patch {i})")
        rs.next_patch()
    rs.set_patched_mode(False)
    with pytest.raises(ValueError):
        wrap(torch.zeros(1, 16, 100, 40, dtype=torch.bfloat16, device=DEV))  # 50 token rows > max 48


def test_sd3_transformer_latent_to_noise(hdit):
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.transformer_sd3 import SD3Transformer2DModel

    L, heads = 3, 4
    model = SD3Transformer2DModel(sample_size=32, patch_size=2, in_channels=16, num_layers=L, attention_head_dim=64,
                                  num_attention_heads=heads, joint_attention_dim=128, caption_projection_dim=256,
                                  pooled_projection_dim=64, out_channels=16, pos_embed_max_size=24)
    synthetic.init_module_(model, 7)
    params = step_params(model)
    model = model.to(DEV)
    B = 2
    lat = synthetic.randn_bf16((B, 16, 32, 40), 8)
    enc = synthetic.randn_bf16((B, 77, 128), 9)
    pooled = synthetic.randn_bf16((B, 64), 10)
    t = torch.tensor([981.0, 981.0])
    got = model(lat.to(DEV), enc.to(DEV), pooled.to(DEV), t.to(DEV))
    torch.cuda.synchronize()
    want = S.sd3_transformer(params, lat.float(), enc.float(), pooled.float(), t, heads, L, 2, 24)
    assert got.shape == lat.shape
    assert_parity(got, want, what="sd3 transformer")

    # conditioning vector on its own
    temb = model.conditioning(t.to(DEV), pooled.to(DEV))
    assert_parity(temb, S.combined_timestep_text_embed(params, "time_text_embed.", t, pooled.float()), what="temb")

    # one guided step: [uncond, cond] batch, guidance and Euler update against the oracle's expressions
    lat1 = lat[:1]
    new = model.denoise_step(lat1.to(DEV), enc.to(DEV), pooled.to(DEV), t[:1].to(DEV), 7.0, 0.981, 0.95)
    noise = S.sd3_transformer(params, torch.cat([lat1, lat1]).float(), enc.float(), pooled.float(), t, heads, L, 2, 24)
    want = S.cfg_euler_step(noise[:1], noise[1:], lat1, 7.0, 0.981, 0.95)
    assert_parity(new, want.float(), what="denoise step")


@pytest.mark.parametrize("backend", ["eager", "inductor"])
def test_sd3_transformer_forward_under_torch_compile(hdit, backend):
    """The reference compiles ``transformer.forward`` when ``use_torch_compile`` is set (``base_pipeline.py:274-279``).
    The modules here are marked opaque to Dynamo (they reach the C ABI through ctypes), so the compiled callable must
    run them as written and return the eager result bit for bit, call after call."""
    import os

    from hetu_dit_amd import synthetic
    from hetu_dit_amd.transformer_sd3 import SD3Transformer2DModel

    os.environ.setdefault("TORCHINDUCTOR_COMPILE_THREADS", "1")
    L, heads = 2, 4
    model = SD3Transformer2DModel(sample_size=32, patch_size=2, in_channels=16, num_layers=L, attention_head_dim=64,
                                  num_attention_heads=heads, joint_attention_dim=128, caption_projection_dim=256,
                                  pooled_projection_dim=64, out_channels=16, pos_embed_max_size=24)
    synthetic.init_module_(model, 7)
    model = model.to(DEV)
    lat = synthetic.randn_bf16((2, 16, 32, 40), 8).to(DEV)
    enc = synthetic.randn_bf16((2, 77, 128), 9).to(DEV)
    pooled = synthetic.randn_bf16((2, 64), 10).to(DEV)
    t = torch.tensor([981.0, 981.0]).to(DEV)
    want = model(lat, enc, pooled, t)
    torch.cuda.synchronize()
    torch._dynamo.reset()
    compiled = torch.compile(model.forward, backend=backend)
    for _ in range(2):
        got = compiled(lat, enc, pooled, t)
        torch.cuda.synchronize()
        assert torch.equal(got, want)

    # a compiled caller that does tensor work of its own around the transformer: traced up to the call, resumed after
    def guided(lat, enc, pooled, t, scale):
        noise = model(lat, enc, pooled, t)
        u, c = noise.float().chunk(2)
        return u + scale * (c - u)

    want2 = guided(lat, enc, pooled, t, 7.0)
    got2 = torch.compile(guided, backend=backend)(lat, enc, pooled, t, 7.0)
    torch.cuda.synchronize()
    assert torch.allclose(got2, want2, rtol=1e-5, atol=1e-5)
    torch._dynamo.reset()


def test_conv2d_wrapper_patch_convolution(hdit):
    """``hetuDiTConv2dWrapper`` (reference layers/conv.py:19-113) on one GPU: the p x p stride-p convolution
    against ``F.conv2d`` in fp32; other geometries are refused."""
    from torch import nn

    from hetu_dit_amd import synthetic
    from hetu_dit_amd.layers.conv import hetuDiTConv2dWrapper

    for (cin, cout, p, H, W, bias) in [(16, 256, 2, 32, 48, True), (4, 64, 4, 16, 16, False), (64, 128, 1, 6, 10, True)]:
        print(f"conv wrapper {cin} {cout} {p} {H} {W} {bias}", flush=True)
        conv = nn.Conv2d(cin, cout, p, stride=p, bias=bias)
        synthetic.init_module_(conv, 21)
        w = conv.weight.detach().float()
        b = conv.bias.detach().float() if bias else None
        wrap = hetuDiTConv2dWrapper(conv, is_first_layer=True).to(DEV)
        x = synthetic.randn_bf16((2, cin, H, W), 22)
        got = wrap(x.to(DEV))
        want = torch.nn.functional.conv2d(x.float(), w, b, stride=p)
        assert got.shape == want.shape
        assert_parity(got, want, what="conv2d wrapper")
    bad = hetuDiTConv2dWrapper(nn.Conv2d(4, 8, 3, padding=1)).to(DEV).to(torch.bfloat16)
    with pytest.raises(NotImplementedError):
        bad(torch.zeros(1, 4, 8, 8, dtype=torch.bfloat16, device=DEV))


def test_sd3_transformer_wrapped_with_the_reference_class_list(hdit):
    """The transformer after ``wrap_layers(model, [FeedForward, nn.Conv2d, PatchEmbed], ["attn"])`` -- the call
    of the reference's SD3 wrapper (transformer_sd3.py:36) -- computes what it did before: the patch embedding
    reads its weights through the Conv2d wrapper."""
    from torch import nn

    from hetu_dit_amd import synthetic
    from hetu_dit_amd.base_model import wrap_layers
    from hetu_dit_amd.layers.conv import hetuDiTConv2dWrapper
    from hetu_dit_amd.layers.modules import FeedForward, PatchEmbed
    from hetu_dit_amd.transformer_sd3 import SD3Transformer2DModel

    L, heads = 2, 4
    model = SD3Transformer2DModel(sample_size=32, patch_size=2, in_channels=16, num_layers=L, attention_head_dim=64,
                                  num_attention_heads=heads, joint_attention_dim=128, caption_projection_dim=256,
                                  pooled_projection_dim=64, out_channels=16, pos_embed_max_size=24)
    synthetic.init_module_(model, 7)
    model = model.to(DEV)
    lat = synthetic.randn_bf16((2, 16, 32, 40), 8).to(DEV)
    enc = synthetic.randn_bf16((2, 77, 128), 9).to(DEV)
    pooled = synthetic.randn_bf16((2, 64), 10).to(DEV)
    t = torch.tensor([981.0, 981.0], device=DEV)
    before = model(lat, enc, pooled, t).clone()
    wrapped = wrap_layers(model, [FeedForward, nn.Conv2d, PatchEmbed], ["attn"])
    assert len(wrapped) == 1 and isinstance(model.pos_embed.module.proj, hetuDiTConv2dWrapper)
    params = step_params(model)
    assert "pos_embed.proj.weight" in params
    after = model(lat, enc, pooled, t)
    torch.cuda.synchronize()
    assert torch.equal(before, after)
    want = S.sd3_transformer(params, lat.float().cpu(), enc.float().cpu(), pooled.float().cpu(), t.cpu(), heads, L, 2, 24)
    assert_parity(after, want, what="sd3 transformer through the Conv2d wrapper")


def test_rope_table_kernel(hdit):
    from hetu_dit_amd import synthetic
    from oracle import ops as O

    ids = synthetic.flux_ids(37, 12, 20)
    cos, sin = hdit.ops.rope_table(ids.float().to(DEV), (16, 56, 56))
    ocos, osin = O.flux_rope_table(ids, (16, 56, 56))
    assert cos.shape == ocos.shape == (37 + 240, 128)
    assert (cos.cpu() - ocos).abs().max() < 2e-6 and (sin.cpu() - osin).abs().max() < 2e-6
    assert torch.equal(cos[:37].cpu(), torch.ones(37, 128)) and torch.equal(sin[:37].cpu(), torch.zeros(37, 128))
    # CogVideoX: (frame, row, col) positions over axes (16, 24, 24)
    pos = synthetic.cogvideox_positions(3, 6, 10)
    cos, sin = hdit.ops.rope_table(pos.float().to(DEV), (16, 24, 24))
    ocos, osin = O.cogvideox_rope_table(3, 6, 10, 64)
    assert (cos.cpu() - ocos).abs().max() < 2e-6 and (sin.cpu() - osin).abs().max() < 2e-6
    with pytest.raises(Exception):
        hdit.ops.rope_table(pos.float().to(DEV), (16, 24, 23))


def test_flux_transformer_packed_latent_to_noise(hdit):
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.transformer_flux import FluxTransformer2DModel

    heads, L, Ls, gh, gw, Nt = 2, 2, 2, 12, 16, 64
    model = FluxTransformer2DModel(num_layers=L, num_single_layers=Ls, attention_head_dim=128, num_attention_heads=heads,
                                   joint_attention_dim=192, pooled_projection_dim=64)
    synthetic.init_module_(model, 21)
    params = step_params(model)
    for i, blk in enumerate(model.single_transformer_blocks):
        from tests.util import oracle_params

        for k, v in oracle_params(blk).items():
            params[f"single_transformer_blocks.{i}.{k}"] = v
    model = model.to(DEV)
    B = 1
    lat = synthetic.randn_bf16((B, gh * gw, 64), 22)
    enc = synthetic.randn_bf16((B, Nt, 192), 23)
    pooled = synthetic.randn_bf16((B, 64), 24)
    t, g = torch.tensor([0.7071]), torch.tensor([3.5])
    ids = synthetic.flux_ids(Nt, gh, gw)
    txt_ids, img_ids = ids[:Nt], ids[Nt:]
    got = model(lat.to(DEV), enc.to(DEV), pooled.to(DEV), t.to(DEV), img_ids.to(DEV), txt_ids.to(DEV), g.to(DEV))
    torch.cuda.synchronize()
    want = S.flux_transformer(params, lat.float(), enc.float(), pooled.float(), t, img_ids, txt_ids, g, heads, L, Ls)
    assert got.shape == lat.shape
    assert_parity(got, want, what="flux transformer")
    temb = model.conditioning(t.to(DEV), pooled.to(DEV), g.to(DEV))
    assert_parity(temb, S.flux_conditioning(params, "time_text_embed.", t, pooled.float(), g), what="flux temb")
    with pytest.raises(ValueError):
        model.conditioning(t.to(DEV), pooled.to(DEV), None)


def test_scheduler_steps_match_oracle_expressions(hdit):
    from hetu_dit_amd.runtime_state import get_runtime_state
    from hetu_dit_amd.schedulers import FlowMatchEulerDiscreteScheduler

    torch.manual_seed(5)
    sch = FlowMatchEulerDiscreteScheduler(shift=3.0)
    sch.set_timesteps(6, device=DEV)
    sig = S.flow_match_sigmas(6)
    x = torch.randn(1, 16, 32, 32).bfloat16()
    ref = x.clone()
    cur = x.to(DEV)
    for i, t in enumerate(sch.timesteps):
        u, c = torch.randn_like(x), torch.randn_like(x)
        if i % 2 == 0:  # guidance fused with the update
            cur = sch.step_with_guidance(u.to(DEV), c.to(DEV), 5.0, t, cur)
            ref = S.cfg_euler_step(u, c, ref, 5.0, float(sig[i]), float(sig[i + 1]))
        else:           # the reference's two-call form: guidance by tensor expressions, then scheduler.step
            noise = u + 5.0 * (c - u)
            cur = sch.step(noise.to(DEV), t, cur, return_dict=False)[0]
            ref = S.cfg_euler_step(noise, noise, ref, 0.0, float(sig[i]), float(sig[i + 1]))
        assert sch.step_index == i + 1
        assert torch.equal(cur.cpu(), ref), f"step {i}"
    # patch mode: the index moves after the last patch only
    rs = get_runtime_state()
    sch.set_timesteps(4, device=DEV)
    rs.set_patches(32, 32, 2, 2)
    rs.set_patched_mode(True)
    t0 = sch.timesteps[0]
    for patch, expect in ((0, 0), (1, 1)):
        sch.step(x[:, :, :16].contiguous().to(DEV), t0, x[:, :, :16].contiguous().to(DEV))
        assert sch.step_index == expect
        rs.next_patch()


def test_clock_sample_counts_forward(hdit):
    a = hdit.ops.clock_sample()
    x = torch.randn(4096, 4096, device=DEV)
    for _ in range(5):
        x = x @ x * 1e-3
    b = hdit.ops.clock_sample()
    torch.cuda.synchronize()
    assert a.shape == (1024, 4)
    xcds = sorted(set(a[:, 2].tolist()))
    print("XCDs sampled:", xcds, flush=True)
    assert len(xcds) >= 1 and all(0 <= x < 16 for x in xcds)
    assert bool((b[:, 1] > a[:, 1]).all())  # the 100 MHz counter is global
    ghz = hdit.ops.shader_clock_ghz(a, b)
    assert ghz is not None and 0.05 < ghz < 3.5, ghz  # a plausible shader clock


def test_unpatchify_channel_major_exact(hdit):
    torch.manual_seed(1)
    B, Fr, C, H, W, p = 1, 3, 16, 12, 20, 2
    x = torch.randn(B, Fr * (H // p) * (W // p), C * p * p).bfloat16()
    got = hdit.ops.unpatchify(x.view(B * Fr, -1, C * p * p).to(DEV), C, H, W, p, channel_major=True)
    assert torch.equal(got.cpu().view(B, Fr, C, H, W), S.unpatchify_channel_major(x, Fr, C, H, W, p))


def test_cogvideox_transformer_video_to_noise(hdit):
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.layers.embeddings import hetuDiTCogVideoXPatchEmbedWrapper
    from hetu_dit_amd.layers.modules import CogVideoXPatchEmbed
    from hetu_dit_amd.registry import hetuDiTLayerWrappersRegister
    from hetu_dit_amd.transformer_cogvideox import CogVideoXTransformer3DModel
    from oracle import ops as O

    heads, L, Fr, H, W, Nt = 4, 2, 3, 12, 20, 34
    model = CogVideoXTransformer3DModel(num_attention_heads=heads, attention_head_dim=64, num_layers=L, text_embed_dim=128,
                                        time_embed_dim=64)
    synthetic.init_module_(model, 31)
    assert hetuDiTLayerWrappersRegister.get_wrapper(model.patch_embed.module) is hetuDiTCogVideoXPatchEmbedWrapper
    assert isinstance(model.patch_embed.module, CogVideoXPatchEmbed)
    params = step_params(model)
    model = model.to(DEV)
    B = 1
    video = synthetic.randn_bf16((B, Fr, 16, H, W), 32)
    text = synthetic.randn_bf16((B, Nt, 128), 33)
    t = torch.tensor([731.0])
    pos = synthetic.cogvideox_positions(Fr, H // 2, W // 2)
    cos, sin = hdit.ops.rope_table(pos.float().to(DEV), (16, 24, 24))
    got = model(video.to(DEV), text.to(DEV), t.to(DEV), (cos, sin))
    torch.cuda.synchronize()
    rope = O.cogvideox_rope_table(Fr, H // 2, W // 2, 64)
    want = S.cogvideox_transformer(params, video.float(), text.float(), t, rope, heads, L, 2)
    assert got.shape == video.shape
    assert_parity(got, want, what="cogvideox transformer")
    joint = model.patch_embed(text.to(DEV), video.to(DEV))
    assert_parity(joint, S.cogvideox_patch_embed(params, "patch_embed.", text.float(), video.float()), what="cogvideox patch embed")
