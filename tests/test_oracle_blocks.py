"""Pins on the oracle's block wiring that do not need the reference: adaLN-"Zero" identity, call-site
conventions the reference fixes (joint order, return order, split points), reduction of the stale-KV
patch path to the full-sequence path, and cross-checks between block families."""
import pytest
import torch

import oracle
from oracle import blocks as OB
from oracle import ops as O


def _params(names_shapes, seed=0, std=0.05):
    g = torch.Generator().manual_seed(seed)
    return {n: torch.randn(*s, generator=g) * std for n, s in names_shapes.items()}


def sd3_params(D, pre_only=False, seed=0):
    F = 4 * D
    shapes = {"norm1.linear.weight": (6 * D, D), "norm1.linear.bias": (6 * D,),
              "norm1_context.linear.weight": ((2 if pre_only else 6) * D, D),
              "norm1_context.linear.bias": ((2 if pre_only else 6) * D,)}
    for n in ("to_q", "to_k", "to_v", "add_q_proj", "add_k_proj", "add_v_proj", "to_out.0"):
        shapes[f"attn.{n}.weight"] = (D, D)
        shapes[f"attn.{n}.bias"] = (D,)
    if not pre_only:
        shapes["attn.to_add_out.weight"], shapes["attn.to_add_out.bias"] = (D, D), (D,)
    for ff in ("ff",) + (() if pre_only else ("ff_context",)):
        shapes[f"{ff}.net.0.proj.weight"], shapes[f"{ff}.net.0.proj.bias"] = (F, D), (F,)
        shapes[f"{ff}.net.2.weight"], shapes[f"{ff}.net.2.bias"] = (D, F), (D,)
    return _params(shapes, seed)


def test_sd3_zero_modulation_is_identity():
    """adaLN-Zero: with the modulation projections at zero every gate is zero, so both residual streams
    pass through unchanged whatever the other weights are."""
    D, H = 32, 2
    p = sd3_params(D)
    for k in list(p):
        if k.startswith("norm1"):
            p[k] = torch.zeros_like(p[k])
    x, e, t = torch.randn(2, 10, D), torch.randn(2, 4, D), torch.randn(2, D)
    enc, hid = oracle.sd3_joint_block(p, x, e, t, H)
    torch.testing.assert_close(hid, x)
    torch.testing.assert_close(enc, e)


def test_sd3_return_order_and_pre_only():
    D, H = 32, 2
    x, e, t = torch.randn(1, 10, D), torch.randn(1, 4, D), torch.randn(1, D)
    enc, hid = oracle.sd3_joint_block(sd3_params(D), x, e, t, H)
    assert enc.shape == e.shape and hid.shape == x.shape  # (encoder_hidden_states, hidden_states)
    enc, hid = oracle.sd3_joint_block(sd3_params(D, pre_only=True), x, e, t, H, context_pre_only=True)
    assert enc is None and hid.shape == x.shape


def test_sd3_gate_only_attention_term():
    """With the MLP gate chunk zeroed, hidden = x + gate_msa * attn(...) exactly; checks the chunk order
    (shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp) against a hand assembly."""
    D, H = 32, 2
    p = sd3_params(D, seed=3)
    p["norm1.linear.weight"][5 * D:] = 0
    p["norm1.linear.bias"][5 * D:] = 0
    x, e, t = torch.randn(1, 6, D), torch.randn(1, 3, D), torch.randn(1, D)
    _, hid = oracle.sd3_joint_block(p, x, e, t, H)
    emb = torch.nn.functional.linear(torch.nn.functional.silu(t), p["norm1.linear.weight"], p["norm1.linear.bias"])
    cemb = torch.nn.functional.linear(torch.nn.functional.silu(t), p["norm1_context.linear.weight"],
                                      p["norm1_context.linear.bias"])
    n = torch.nn.functional.layer_norm(x, (D,), eps=1e-6) * (1 + emb[:, None, D:2 * D]) + emb[:, None, :D]
    nc = torch.nn.functional.layer_norm(e, (D,), eps=1e-6) * (1 + cemb[:, None, D:2 * D]) + cemb[:, None, :D]
    a, _ = OB.sd3_joint_attention(p, n, nc, H, False)
    torch.testing.assert_close(hid, x + emb[:, None, 2 * D:3 * D] * a, rtol=1e-5, atol=1e-5)


def test_sd3_joint_attention_against_library_sdpa():
    D, H = 32, 2
    p = sd3_params(D, seed=5)
    x, e = torch.randn(2, 9, D), torch.randn(2, 5, D)
    F = torch.nn.functional
    q = torch.cat([F.linear(x, p["attn.to_q.weight"], p["attn.to_q.bias"]),
                   F.linear(e, p["attn.add_q_proj.weight"], p["attn.add_q_proj.bias"])], 1)
    k = torch.cat([F.linear(x, p["attn.to_k.weight"], p["attn.to_k.bias"]),
                   F.linear(e, p["attn.add_k_proj.weight"], p["attn.add_k_proj.bias"])], 1)
    v = torch.cat([F.linear(x, p["attn.to_v.weight"], p["attn.to_v.bias"]),
                   F.linear(e, p["attn.add_v_proj.weight"], p["attn.add_v_proj.bias"])], 1)
    sp = lambda z: z.view(2, -1, H, D // H).transpose(1, 2)
    o = F.scaled_dot_product_attention(sp(q), sp(k), sp(v)).transpose(1, 2).reshape(2, -1, D)
    want_img = F.linear(o[:, :9], p["attn.to_out.0.weight"], p["attn.to_out.0.bias"])
    want_txt = F.linear(o[:, 9:], p["attn.to_add_out.weight"], p["attn.to_add_out.bias"])
    a, ca = OB.sd3_joint_attention(p, x, e, H, False)
    torch.testing.assert_close(a, want_img, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ca, want_txt, rtol=1e-5, atol=1e-5)


def test_patch_mode_with_fresh_buffer_equals_rows_of_full_pass():
    """Query-row independence reduces the stale-KV case to the full case: if the buffer holds exactly
    this step's K/V, a patch's image output equals the same rows of the full-sequence output."""
    D, H, N = 32, 2, 16
    p = sd3_params(D, seed=7)
    x, e, t = torch.randn(1, N, D), torch.randn(1, 5, D), torch.randn(1, D)
    buf = oracle.StaleKVBuffer()
    _, full = oracle.sd3_joint_block(p, x, e, t, H, kv=buf)  # whole sequence: fills the buffer
    buf.set_patches([0, 4, 8, 12, 16])
    buf.patch_mode = True
    for patch in range(4):
        buf.pipeline_patch_idx = patch
        sl = slice(4 * patch, 4 * patch + 4)
        _, part = oracle.sd3_joint_block(p, x[:, sl], e, t, H, kv=buf)
        torch.testing.assert_close(part, full[:, sl], rtol=1e-5, atol=1e-5)


def test_flux_joint_order_and_dropped_text_bias():
    D, H, hd = 64, 2, 32
    shapes = {}
    for n in ("to_q", "to_k", "to_v", "add_q_proj", "add_k_proj", "add_v_proj", "to_out.0", "to_add_out"):
        shapes[f"attn.{n}.weight"], shapes[f"attn.{n}.bias"] = (D, D), (D,)
    for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"):
        shapes[f"attn.{n}.weight"] = (hd,)
    p = _params(shapes, seed=9, std=0.2)
    x, e = torch.randn(1, 6, D), torch.randn(1, 3, D)
    ids = torch.zeros(9, 3)
    ids[3:, 1] = torch.arange(6)
    cos, sin = O.flux_rope_table(ids, (8, 12, 12))
    a, ca = OB.flux_attention(p, x, e, (cos, sin), H)
    assert a.shape == x.shape and ca.shape == e.shape
    # the text out-projection bias must not matter (the reference's Flux branch drops it)
    p2 = dict(p)
    p2["attn.to_add_out.bias"] = p["attn.to_add_out.bias"] + 100.0
    _, ca2 = OB.flux_attention(p2, x, e, (cos, sin), H)
    torch.testing.assert_close(ca, ca2)
    # text ids are zero -> identity rotation on text rows: perturbing the table's text rows to identity is a no-op
    assert torch.all(cos[:3] == 1) and torch.all(sin[:3] == 0)


def test_cogvideox_return_order_and_shared_weights():
    D, H, hd, Tt = 64, 2, 32, 16
    shapes = {"norm1.linear.weight": (6 * D, Tt), "norm1.linear.bias": (6 * D,), "norm1.norm.weight": (D,),
              "norm1.norm.bias": (D,), "norm2.linear.weight": (6 * D, Tt), "norm2.linear.bias": (6 * D,),
              "norm2.norm.weight": (D,), "norm2.norm.bias": (D,),
              "ff.net.0.proj.weight": (4 * D, D), "ff.net.0.proj.bias": (4 * D,), "ff.net.2.weight": (D, 4 * D),
              "ff.net.2.bias": (D,)}
    for n in ("to_q", "to_k", "to_v", "to_out.0"):
        shapes[f"attn1.{n}.weight"], shapes[f"attn1.{n}.bias"] = (D, D), (D,)
    for n in ("norm_q", "norm_k"):
        shapes[f"attn1.{n}.weight"], shapes[f"attn1.{n}.bias"] = (hd,), (hd,)
    p = _params(shapes, seed=11, std=0.1)
    x, e, t = torch.randn(1, 8, D), torch.randn(1, 3, D), torch.randn(1, Tt)
    hid, enc = oracle.cogvideox_block(p, x, e, t, None, H)
    assert hid.shape == x.shape and enc.shape == e.shape  # (hidden_states, encoder_hidden_states)
    # zero modulation -> identity on both streams
    pz = dict(p)
    for k in list(pz):
        if ".linear." in k:
            pz[k] = torch.zeros_like(pz[k])
    hid, enc = oracle.cogvideox_block(pz, x, e, t, None, H)
    torch.testing.assert_close(hid, x)
    torch.testing.assert_close(enc, e)


def test_feed_forward_against_library():
    D = 16
    p = _params({"ff.net.0.proj.weight": (4 * D, D), "ff.net.0.proj.bias": (4 * D,), "ff.net.2.weight": (D, 4 * D),
                 "ff.net.2.bias": (D,)}, seed=13, std=0.3)
    x = torch.randn(2, 5, D)
    F = torch.nn.functional
    want = F.linear(F.gelu(F.linear(x, p["ff.net.0.proj.weight"], p["ff.net.0.proj.bias"]), approximate="tanh"),
                    p["ff.net.2.weight"], p["ff.net.2.bias"])
    torch.testing.assert_close(oracle.feed_forward(p, "ff", x), want, rtol=1e-5, atol=1e-5)


def test_feed_forward_other_first_layers_against_library():
    """The first-layer classes the reference's wrapper accepts besides the tanh GELU (``layers/feedforward.py:25-57``),
    each against a chain of library calls, and each mutation of that chain (tanh for erf, halves swapped, gate not
    activated) must break the agreement."""
    D, Fi = 16, 48
    F = torch.nn.functional
    x = torch.randn(2, 5, D)
    for name, width in (("gelu", Fi), ("geglu", 2 * Fi), ("linear-silu", Fi)):
        p = _params({"ff.net.0.proj.weight": (width, D), "ff.net.0.proj.bias": (width,), "ff.net.2.weight": (D, Fi),
                     "ff.net.2.bias": (D,)}, seed=17, std=0.5)
        h = F.linear(x, p["ff.net.0.proj.weight"], p["ff.net.0.proj.bias"])
        if name == "gelu":
            good, bad = F.gelu(h), [F.gelu(h, approximate="tanh"), F.silu(h)]
        elif name == "geglu":
            a, g = h.chunk(2, dim=-1)
            good, bad = a * F.gelu(g), [g * F.gelu(a), a * g, a * F.gelu(g, approximate="tanh"), F.gelu(a) * g]
        else:
            good, bad = F.silu(h), [F.gelu(h), h]
        out = lambda hh: F.linear(hh, p["ff.net.2.weight"], p["ff.net.2.bias"])  # noqa: E731
        got = oracle.feed_forward(p, "ff", x, activation_fn=name)
        torch.testing.assert_close(got, out(good), rtol=1e-5, atol=1e-5)
        for b in bad:
            assert (got - out(b)).abs().max().item() > 1e-4, name
    with pytest.raises(ValueError):
        oracle.feed_forward(p, "ff", x, activation_fn="swiglu")
