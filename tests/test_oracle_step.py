"""Pins for the oracle of the step's head and tail (``oracle/step.py``) by library routines and closed forms,
and host-side checks of the product's position table and crop (CPU only)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import step as S


def test_patch_embed_is_a_strided_convolution():
    torch.manual_seed(0)
    lat, w, b = torch.randn(2, 5, 12, 8), torch.randn(24, 5, 2, 2), torch.randn(24)
    want = F.conv2d(lat, w, b, stride=2).flatten(2).transpose(1, 2)  # diffusers PatchEmbed: conv, flatten(2), transpose
    got = S.patch_embed(lat, w, b, None)
    assert torch.allclose(got, want, atol=1e-5)
    pos = torch.randn(24, 24)
    assert torch.allclose(S.patch_embed(lat, w, b, pos), want + pos[None], atol=1e-5)
    # rectangular, p = 4: a transposed patch layout would fail here
    lat, w = torch.randn(1, 3, 8, 16), torch.randn(7, 3, 4, 4)
    want = F.conv2d(lat, w, None, stride=4).flatten(2).transpose(1, 2)
    assert torch.allclose(S.patch_embed(lat, w, torch.zeros(7), None), want, atol=1e-5)


def test_unpatchify_inverts_patch_major_layout():
    # element (n, hy, wx, py, px, c) must land at out[n, c, hy*p+py, wx*p+px]
    n, h, w, p, c = 2, 3, 5, 2, 4
    x = torch.arange(n * h * w * p * p * c, dtype=torch.float32).reshape(n, h * w, p * p * c)
    out = S.unpatchify(x, c, h * p, w * p, p)
    assert out.shape == (n, c, h * p, w * p)
    for (b, hy, wx, py, px, ch) in [(0, 0, 0, 0, 0, 0), (1, 2, 4, 1, 0, 3), (0, 1, 3, 0, 1, 2), (1, 0, 2, 1, 1, 1)]:
        assert out[b, ch, hy * p + py, wx * p + px] == x[b, hy * w + wx, (py * p + px) * c + ch]
    # F.fold of channel-major columns is the same permutation up to the (c, py, px) -> (py, px, c) order
    cols = x.reshape(n, h * w, p, p, c).permute(0, 4, 2, 3, 1).reshape(n, c * p * p, h * w)
    assert torch.equal(F.fold(cols, (h * p, w * p), kernel_size=p, stride=p), out)


def test_timestep_embedding_closed_form():
    t = torch.tensor([0.0, 1.0, 500.0, 999.0])
    e = S.timestep_embedding(t, 256)
    assert e.shape == (4, 256)
    assert torch.equal(e[0, :128], torch.ones(128)) and torch.equal(e[0, 128:], torch.zeros(128))  # cos first
    assert abs(e[1, 0] - math.cos(1.0)) < 1e-6 and abs(e[1, 128] - math.sin(1.0)) < 1e-6  # first frequency is 1
    k = 37
    f = 10000.0 ** (-k / 128)
    assert abs(e[2, k] - math.cos(500.0 * f)) < 1e-4 and abs(e[2, 128 + k] - math.sin(500.0 * f)) < 1e-4
    assert torch.allclose(e[:, :128] ** 2 + e[:, 128:] ** 2, torch.ones(4, 128), atol=1e-5)
    # last frequency: 10000^(-(half-1)/half), not 10000^-1 (downscale_freq_shift = 0)
    f_last = 10000.0 ** (-127 / 128)
    assert abs(e[3, 127] - math.cos(999.0 * f_last)) < 1e-5


def test_sincos_table_closed_form_and_crop():
    D, G, base = 32, 12, 8
    tab = S.sincos_pos_embed_2d(D, G, base)
    assert tab.shape == (G * G, D)
    scale = base / G
    q = D // 4
    for (r, c) in [(0, 0), (3, 7), (11, 2)]:
        row = tab[r * G + c]
        for i in (0, 1, q - 1):
            om = 10000.0 ** (-i / q)
            assert abs(row[i] - math.sin(c * scale * om)) < 1e-6
            assert abs(row[q + i] - math.cos(c * scale * om)) < 1e-6
            assert abs(row[2 * q + i] - math.sin(r * scale * om)) < 1e-6
            assert abs(row[3 * q + i] - math.cos(r * scale * om)) < 1e-6
    crop = S.cropped_pos_embed(tab, G, 4, 6)
    top, left = (G - 4) // 2, (G - 6) // 2
    assert torch.equal(crop[0], tab[top * G + left]) and torch.equal(crop[-1], tab[(top + 3) * G + left + 5])
    assert torch.equal(crop[6], tab[(top + 1) * G + left])


def test_product_position_table_matches_oracle():
    from hetu_dit_amd.layers.modules import PatchEmbed, sincos_pos_embed_2d

    assert torch.allclose(sincos_pos_embed_2d(64, 24, 16), S.sincos_pos_embed_2d(64, 24, 16), atol=1e-6)
    pe = PatchEmbed(32, 32, 2, 4, 64, pos_embed_max_size=24)
    assert pe.pos_embed.shape == (1, 576, 64)
    assert torch.equal(pe.cropped_pos_embed(20, 28)[0], S.cropped_pos_embed(pe.pos_embed[0], 24, 10, 14))
    with pytest.raises(ValueError):
        pe.cropped_pos_embed(50, 8)


def test_cfg_and_euler_identities():
    torch.manual_seed(1)
    u, c, x = (torch.randn(1000).bfloat16() for _ in range(3))
    # guidance 1 returns the conditional prediction up to one bf16 rounding of (c - u); guidance 0 the unconditional
    x0 = S.cfg_euler_step(u, c, x, 0.0, 0.7, 0.7)
    assert torch.equal(x0, x)  # dt = 0: the sample does not move
    # exact arithmetic: prev = x + (sigma_next - sigma) * noise; check against fp64 within bf16 rounding
    got = S.cfg_euler_step(u, c, x, 4.5, 0.8, 0.6).double()
    want = x.double() + (0.6 - 0.8) * (u.double() + 4.5 * (c.double() - u.double()))
    assert ((got - want).norm() / want.norm()) < 6e-3
    # sigma_next = 0 lands on the denoised sample x - sigma * noise
    got = S.cfg_euler_step(u, u, x, 7.0, 0.5, 0.0).double()
    assert ((got - (x.double() - 0.5 * u.double())).norm() / got.norm()) < 6e-3


def test_combined_embedding_and_norm_out_against_torch_modules():
    torch.manual_seed(2)
    D, Pd = 48, 20
    t1, t2, p1, p2 = torch.nn.Linear(256, D), torch.nn.Linear(D, D), torch.nn.Linear(Pd, D), torch.nn.Linear(D, D)
    p = {}
    for name, lin in (("timestep_embedder.linear_1", t1), ("timestep_embedder.linear_2", t2),
                      ("text_embedder.linear_1", p1), ("text_embedder.linear_2", p2)):
        p["tte." + name + ".weight"], p["tte." + name + ".bias"] = lin.weight.detach(), lin.bias.detach()
    t, pooled = torch.tensor([3.0, 700.0]), torch.randn(2, Pd)
    want = t2(F.silu(t1(S.timestep_embedding(t, 256)))) + p2(F.silu(p1(pooled)))
    assert torch.allclose(S.combined_timestep_text_embed(p, "tte.", t, pooled), want, atol=1e-5)
    lin, proj = torch.nn.Linear(D, 2 * D), torch.nn.Linear(D, 16)
    q = {"norm_out.linear.weight": lin.weight.detach(), "norm_out.linear.bias": lin.bias.detach(),
         "proj_out.weight": proj.weight.detach(), "proj_out.bias": proj.bias.detach()}
    hidden, temb = torch.randn(2, 9, D), torch.randn(2, D)
    scale, shift = lin(F.silu(temb)).chunk(2, dim=1)
    want = proj(F.layer_norm(hidden, (D,), eps=1e-6) * (1 + scale[:, None]) + shift[:, None])
    assert torch.allclose(S.norm_out_proj(q, hidden, temb), want, atol=1e-5)


def test_flow_match_sigmas_closed_form_and_scheduler_host_logic():
    from hetu_dit_amd.runtime_state import get_runtime_state, reset_runtime_state
    from hetu_dit_amd.schedulers import FlowMatchEulerDiscreteScheduler

    sig = S.flow_match_sigmas(28)
    assert sig.shape == (29,) and sig[0] == 1.0 and sig[-1] == 0.0
    assert torch.all(sig[1:] < sig[:-1])
    # published SD3 schedule (shift 3, 28 steps): second sigma 0.9874, last non-zero 3 s / (1 + 2 s) at s = sigma_min
    assert abs(float(sig[1]) - 0.9874) < 1e-4
    s_min = 3 * 0.001 / 1.002
    assert abs(float(sig[-2]) - 3 * s_min / (1 + 2 * s_min)) < 1e-6
    # un-shifting gives back evenly spaced points
    un = sig[:-1].double() / (3 - 2 * sig[:-1].double())
    assert torch.allclose(un[1:] - un[:-1], (un[-1] - un[0]) / 27 * torch.ones(27, dtype=torch.float64), atol=1e-6)

    sch = FlowMatchEulerDiscreteScheduler(shift=3.0)
    sch.set_timesteps(28)
    assert torch.allclose(sch.sigmas, sig, atol=1e-7)
    assert torch.allclose(sch.timesteps, sig[:-1] * 1000, atol=1e-4)
    assert sch.step_index is None and sch.index_for_timestep(sch.timesteps[3]) == 3
    with pytest.raises(ValueError):
        sch._sigma_pair(3)
    with pytest.raises(ValueError):
        sch.index_for_timestep(123.456)
    # the step index advances once per step: after every call outside patch mode, after the last patch inside
    reset_runtime_state()
    rs = get_runtime_state()
    assert sch._sigma_pair(sch.timesteps[0]) == (float(sig[0]), float(sig[1]))
    sch._advance()
    assert sch.step_index == 1
    rs.set_token_patches([0, 4, 8, 12])
    rs.set_patched_mode(True)
    for expect in (1, 1, 2):
        sch._advance()
        assert sch.step_index == expect
        rs.next_patch()
    reset_runtime_state()


def test_flux_conditioning_against_torch_modules():
    torch.manual_seed(4)
    D, Pd = 32, 24
    lins = {n: (torch.nn.Linear(256 if n != "text_embedder" else Pd, D), torch.nn.Linear(D, D))
            for n in ("timestep_embedder", "guidance_embedder", "text_embedder")}
    p = {}
    for n, (l1, l2) in lins.items():
        p[f"e.{n}.linear_1.weight"], p[f"e.{n}.linear_1.bias"] = l1.weight.detach(), l1.bias.detach()
        p[f"e.{n}.linear_2.weight"], p[f"e.{n}.linear_2.bias"] = l2.weight.detach(), l2.bias.detach()
    t, g, pooled = torch.tensor([0.7071, 0.25]), torch.tensor([3.5, 3.5]), torch.randn(2, Pd)

    def emb(n, x):
        return lins[n][1](F.silu(lins[n][0](x)))

    tb = (t.bfloat16() * 1000).float()  # 0.7071 -> bf16 0.70703125 -> 707.03125 -> bf16 708
    assert tb[0] == 708.0
    want = emb("timestep_embedder", S.timestep_embedding(tb, 256)) + emb("guidance_embedder", S.timestep_embedding(
        torch.tensor([3504.0, 3504.0]), 256)) + emb("text_embedder", pooled)  # 3500 rounds to 3504 in bf16
    assert torch.allclose(S.flux_conditioning(p, "e.", t, pooled, g), want, atol=1e-5)
    want = emb("timestep_embedder", S.timestep_embedding(tb, 256)) + emb("text_embedder", pooled)
    assert torch.allclose(S.flux_conditioning(p, "e.", t, pooled, None), want, atol=1e-5)


def test_cogvideox_head_tail_against_torch():
    torch.manual_seed(6)
    B, Fr, C, H, W, D, E, Nt, p = 2, 3, 4, 6, 8, 24, 10, 5, 2
    conv, tproj = torch.nn.Conv2d(C, D, p, stride=p), torch.nn.Linear(E, D)
    prm = {"pe.proj.weight": conv.weight.detach(), "pe.proj.bias": conv.bias.detach(),
           "pe.text_proj.weight": tproj.weight.detach(), "pe.text_proj.bias": tproj.bias.detach()}
    text, video = torch.randn(B, Nt, E), torch.randn(B, Fr, C, H, W)
    # the wrapper's own expressions: conv per frame, flatten(3).transpose(2, 3), flatten(1, 2), cat [text, video]
    img = conv(video.reshape(-1, C, H, W)).view(B, Fr, D, H // p, W // p).flatten(3).transpose(2, 3).flatten(1, 2)
    want = torch.cat([tproj(text), img], dim=1)
    assert torch.allclose(S.cogvideox_patch_embed(prm, "pe.", text, video), want, atol=1e-5)

    # AdaLayerNorm (shift first, affine LayerNorm)
    lin, ln = torch.nn.Linear(7, 2 * D), torch.nn.LayerNorm(D, eps=1e-5)
    with torch.no_grad():
        ln.weight.normal_(1, 0.1), ln.bias.normal_(0, 0.1)
    q = {"n.linear.weight": lin.weight.detach(), "n.linear.bias": lin.bias.detach(), "n.norm.weight": ln.weight.detach(),
         "n.norm.bias": ln.bias.detach()}
    x, temb = torch.randn(B, 9, D), torch.randn(B, 7)
    shift, scale = lin(F.silu(temb)).chunk(2, dim=1)
    want = ln(x) * (1 + scale[:, None]) + shift[:, None]
    assert torch.allclose(S.ada_layer_norm(q, "n.", x, temb), want, atol=1e-5)

    # channel-major unpatchify: token (f, hy, wx), column (c, py, px) -> out[b, f, c, hy p + py, wx p + px]
    h, w = H // p, W // p
    tok = torch.arange(B * Fr * h * w * C * p * p, dtype=torch.float32).reshape(B, Fr * h * w, C * p * p)
    out = S.unpatchify_channel_major(tok, Fr, C, H, W, p)
    assert out.shape == (B, Fr, C, H, W)
    for (b, f, c, hy, py, wx, px) in [(0, 0, 0, 0, 0, 0, 0), (1, 2, 3, 2, 1, 3, 0), (0, 1, 2, 1, 0, 2, 1)]:
        assert out[b, f, c, hy * p + py, wx * p + px] == tok[b, (f * h + hy) * w + wx, (c * p + py) * p + px]
    # F.fold takes exactly channel-major columns
    cols = tok.reshape(B * Fr, h * w, C * p * p).transpose(1, 2)
    assert torch.equal(F.fold(cols, (H, W), kernel_size=p, stride=p).view(B, Fr, C, H, W), out)
