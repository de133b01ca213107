"""Pins every primitive of the oracle against a PyTorch library routine, a
numpy brute force or a mathematical invariant chosen so that a dropped term,
a wrong sign or a transposed operand fails."""
import math

import numpy as np
import torch
import torch.nn.functional as F

import oracle
from oracle import ops

torch.manual_seed(0)


def close(a, b, tol=1e-5):
    torch.testing.assert_close(a, b, rtol=tol, atol=tol)


def test_linear_matches_library_and_kats():
    x = torch.randn(3, 5, 7)
    w = torch.randn(11, 7)
    b = torch.randn(11)
    close(ops.linear(x, w, b), F.linear(x, w, b))
    # identity weight: y = x + b;  one-hot row picks a column of x
    close(ops.linear(x, torch.eye(7), torch.zeros(7)), x)
    onehot = torch.zeros(1, 7)
    onehot[0, 3] = 1.0
    close(ops.linear(x, onehot)[..., 0], x[..., 3])


def test_layer_norm_matches_library_and_invariants():
    x = torch.randn(2, 9, 48) * 3 + 1.5
    w, b = torch.randn(48), torch.randn(48)
    for eps in (1e-6, 1e-5):
        close(ops.layer_norm(x, eps), F.layer_norm(x, (48,), eps=eps))
        close(ops.layer_norm(x, eps, w, b), F.layer_norm(x, (48,), w, b, eps=eps))
    y = ops.layer_norm(x, 1e-12)
    close(y.mean(-1), torch.zeros(2, 9), 1e-5)
    close((y * y).mean(-1), torch.ones(2, 9), 1e-4)
    # shift invariance, scale invariance
    close(ops.layer_norm(x + 7.0, 1e-6), ops.layer_norm(x, 1e-6), 1e-4)


def test_rms_norm_matches_library():
    x = torch.randn(2, 4, 6, 128)
    w = torch.randn(128)
    close(ops.rms_norm(x, 1e-6, w), F.rms_norm(x, (128,), w, eps=1e-6))
    close(ops.rms_norm(x * 5.0, 0.0), ops.rms_norm(x, 0.0), 1e-5)


def test_gelu_erf_pinned_by_library_erf_and_symmetry():
    import math

    x = torch.linspace(-6, 6, 101)
    close(ops.gelu_erf(x), F.gelu(x), 1e-6)
    for v in (-3.0, -1.0, -0.25, 0.0, 0.5, 1.0, 2.5):
        want = 0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0)))
        assert abs(ops.gelu_erf(torch.tensor([v])).item() - want) < 1e-6
    close(ops.gelu_erf(x) - ops.gelu_erf(-x), x, 1e-5)  # x Phi(x) + x Phi(-x) = x
    # it is not the tanh form: the two differ by up to 2e-4 around |x| = 2
    assert (ops.gelu_erf(x) - ops.gelu_tanh(x)).abs().max().item() > 1e-4


def test_gelu_tanh_and_silu():
    x = torch.linspace(-6, 6, 101)
    close(ops.gelu_tanh(x), F.gelu(x, approximate="tanh"), 1e-6)
    close(ops.silu(x), F.silu(x), 1e-6)
    assert ops.gelu_tanh(torch.tensor([0.0])).item() == 0.0
    assert abs(ops.gelu_tanh(torch.tensor([1.0])).item() - 0.841192) < 1e-5
    assert abs(ops.gelu_tanh(torch.tensor([-1.0])).item() + 0.158808) < 1e-5
    assert abs(ops.gelu_tanh(torch.tensor([10.0])).item() - 10.0) < 1e-5
    assert abs(ops.gelu_tanh(torch.tensor([-10.0])).item()) < 1e-5


def _brute_attention(q, k, v):
    q, k, v = (t.double().numpy() for t in (q, k, v))
    B, H, Sq, d = q.shape
    out = np.zeros((B, H, Sq, v.shape[-1]))
    for b in range(B):
        for h in range(H):
            for i in range(Sq):
                s = np.array([np.dot(q[b, h, i], k[b, h, j]) / math.sqrt(d) for j in range(k.shape[2])])
                p = np.exp(s - s.max())
                p /= p.sum()
                out[b, h, i] = (p[:, None] * v[b, h]).sum(0)
    return torch.from_numpy(out).float()


def test_attention_matches_sdpa_and_brute_force():
    q = torch.randn(2, 3, 17, 16)
    k = torch.randn(2, 3, 29, 16)
    v = torch.randn(2, 3, 29, 16)
    o = ops.attention(q, k, v)
    close(o, F.scaled_dot_product_attention(q, k, v), 1e-5)
    close(o, _brute_attention(q, k, v), 1e-5)


def test_attention_invariants():
    q = torch.randn(1, 2, 8, 16)
    k = torch.randn(1, 2, 12, 16)
    v = torch.randn(1, 2, 12, 16)
    o = ops.attention(q, k, v)
    # constant V -> output is that constant (rows of P sum to one)
    vc = torch.ones_like(v) * 3.25
    close(ops.attention(q, k, vc), torch.full_like(o, 3.25), 1e-5)
    # permutation invariance over the KV order ([img, txt] vs [txt, img])
    perm = torch.randperm(12)
    close(ops.attention(q, k[:, :, perm], v[:, :, perm]), o, 1e-5)
    # query-row independence (a query patch equals the same rows of the full result)
    close(ops.attention(q[:, :, 2:5], k, v), o[:, :, 2:5], 1e-6)
    # large logits do not overflow
    assert torch.isfinite(ops.attention(q * 1e3, k, v)).all()


def test_rope_against_complex_form_and_invariants():
    S, d = 10, 16
    ang = torch.rand(S, d // 2) * 6.28
    cos = torch.cos(ang).repeat_interleave(2, dim=1)
    sin = torch.sin(ang).repeat_interleave(2, dim=1)
    x = torch.randn(2, 3, S, d)
    y = ops.apply_rotary_emb(x, cos, sin)
    # complex multiplication (x0 + i x1) * e^{i ang}
    xc = torch.view_as_complex(x.reshape(2, 3, S, d // 2, 2).contiguous())
    yc = xc * torch.polar(torch.ones_like(ang), ang)[None, None]
    close(y, torch.view_as_real(yc).reshape(2, 3, S, d), 1e-5)
    # pairwise norm preserved
    close(y.reshape(2, 3, S, d // 2, 2).norm(dim=-1), x.reshape(2, 3, S, d // 2, 2).norm(dim=-1), 1e-5)
    # zero angle is the identity
    close(ops.apply_rotary_emb(x, torch.ones(S, d), torch.zeros(S, d)), x, 0)


def test_rope_relative_position_property():
    d = 16
    ids = torch.zeros(32, 3)
    ids[:, 1] = torch.arange(32)
    cos, sin = ops.flux_rope_table(ids, axes_dim=(4, 8, 4))
    q = torch.randn(1, 1, 1, d).expand(1, 1, 32, d)
    k = torch.randn(1, 1, 1, d).expand(1, 1, 32, d)
    rq = ops.apply_rotary_emb(q, cos, sin)[0, 0]
    rk = ops.apply_rotary_emb(k, cos, sin)[0, 0]
    dots = rq @ rk.T
    # <rope(q, m), rope(k, n)> depends only on m - n
    for delta in (0, 3, 7):
        diag = torch.diagonal(dots, offset=delta)
        close(diag, diag[0].expand_as(diag), 1e-4)


def test_flux_rope_table_closed_form():
    ids = torch.tensor([[0, 0, 0], [0, 5, 9], [0, 63, 1]], dtype=torch.float32)
    cos, sin = ops.flux_rope_table(ids)
    assert cos.shape == (3, 128) and sin.shape == (3, 128)
    # text row (all ids zero): identity rotation
    close(cos[0], torch.ones(128), 0)
    close(sin[0], torch.zeros(128), 0)
    # axis 1 (dims 16..71), pair i: angle = row * 10000^(-2i/56)
    for i in (0, 3, 27):
        a = 5.0 * 10000.0 ** (-2.0 * i / 56.0)
        assert abs(cos[1, 16 + 2 * i].item() - math.cos(a)) < 1e-6
        assert abs(cos[1, 16 + 2 * i + 1].item() - math.cos(a)) < 1e-6
        assert abs(sin[1, 16 + 2 * i].item() - math.sin(a)) < 1e-6
    # axis 2 (dims 72..127)
    a = 9.0 * 10000.0 ** (-2.0 * 4 / 56.0)
    assert abs(sin[1, 72 + 8].item() - math.sin(a)) < 1e-6


def test_cogvideox_rope_table_closed_form():
    T, H, W = 3, 4, 5
    cos, sin = ops.cogvideox_rope_table(T, H, W, head_dim=64)
    assert cos.shape == (T * H * W, 64)
    tok = (2 * H + 3) * W + 4  # t=2, h=3, w=4
    a_t = 2.0 * 10000.0 ** (-2.0 * 1 / 16.0)
    a_h = 3.0 * 10000.0 ** (-2.0 * 2 / 24.0)
    a_w = 4.0 * 10000.0 ** (-2.0 * 5 / 24.0)
    assert abs(cos[tok, 2].item() - math.cos(a_t)) < 1e-5
    assert abs(sin[tok, 16 + 4].item() - math.sin(a_h)) < 1e-5
    assert abs(sin[tok, 40 + 10].item() - math.sin(a_w)) < 1e-5
    close(cos[0], torch.ones(64), 0)


def test_adaln_modulation_and_modulate():
    temb = torch.randn(2, 8)
    w, b = torch.randn(24, 8), torch.randn(24)
    parts = ops.adaln_modulation(temb, w, b, 6)
    full = F.linear(F.silu(temb), w, b)
    assert len(parts) == 6
    close(torch.cat(parts, dim=1), full)
    x = torch.randn(2, 5, 4)
    close(ops.modulate(x, torch.zeros(2, 4), torch.zeros(2, 4)), x, 0)
    close(ops.modulate(x, parts[0], parts[1]), x * (1 + full[:, None, 4:8]) + full[:, None, 0:4])


def test_stale_kv_buffer_brute_force():
    B, N, D = 2, 8, 6
    buf = oracle.StaleKVBuffer()
    k0, v0 = torch.randn(B, N, D), torch.randn(B, N, D)
    k, v = buf.update_and_get(k0, v0, slice_dim=1)  # warm-up: whole sequence
    close(k, k0, 0)
    buf.set_patches([0, 2, 4, 6, 8])
    buf.patch_mode = True
    fresh_k, fresh_v = [], []
    for patch in range(4):
        buf.pipeline_patch_idx = patch
        nk, nv = torch.randn(B, 2, D), torch.randn(B, 2, D)
        fresh_k.append(nk)
        fresh_v.append(nv)
        k, v = buf.update_and_get(nk, nv, slice_dim=1)
        # patches <= patch are fresh, > patch are stale
        want_k = torch.cat(fresh_k + [k0[:, 2 * (patch + 1):]], dim=1)
        want_v = torch.cat(fresh_v + [v0[:, 2 * (patch + 1):]], dim=1)
        close(k, want_k, 0)
        close(v, want_v, 0)
