"""Pins of the oracle's block wiring by independent assemblies.

Every block the oracle restates (``sd3_joint_block`` with and without ``context_pre_only``, ``flux_double_block``,
``flux_single_block``, ``cogvideox_block``) is built here a second time, from PyTorch's own library modules
(``nn.LayerNorm``, ``nn.Linear``, ``F.silu``, ``F.gelu(approximate="tanh")``, ``F.rms_norm``,
``F.scaled_dot_product_attention``, complex multiplication for the rotary embedding) in the order of the published
diffusers ``forward`` of each block (diffusers 0.31 / 0.32: ``JointTransformerBlock``, ``FluxTransformerBlock``,
``FluxSingleTransformerBlock``, ``CogVideoXBlock``, ``AdaLayerNormZero``, ``AdaLayerNormZeroSingle``,
``AdaLayerNormContinuous``, ``CogVideoXLayerNormZero``, ``FeedForward``) and of the reference's attention
processors (``layers/attention_processor.py:657-793,:824-987,:1022-1158``).  The two must agree to fp32
round-off.  So that agreement means something, every assembly takes a *mutation* -- a plausible wiring mistake
(shift and scale swapped, gate chunks swapped, eps 1e-5 <-> 1e-6, scale-first <-> shift-first, affine dropped,
joint order flipped, text bias kept, ...) -- and each mutation must break the agreement.

None of this imports diffusers or the reference; the assemblies share no code with ``oracle/``.
"""
import pytest
import torch
import torch.nn.functional as F
from torch import nn

import oracle
from oracle import ops as O

torch.manual_seed(0)


# ---------------------------------------------------------------------------
# building blocks from the library
# ---------------------------------------------------------------------------

def lin(p, name, bias=True):
    w = p[name + ".weight"]
    m = nn.Linear(w.shape[1], w.shape[0], bias=bias and (name + ".bias") in p)
    with torch.no_grad():
        m.weight.copy_(w)
        if m.bias is not None:
            m.bias.copy_(p[name + ".bias"])
    return m


def ada_chunks(p, name, temb, n):
    return lin(p, name + ".linear")(F.silu(temb)).chunk(n, dim=1)


def layer_norm_noaffine(D, eps):
    return nn.LayerNorm(D, elementwise_affine=False, eps=eps)


def feed_forward(p, prefix, x):
    h = F.gelu(lin(p, prefix + ".net.0.proj")(x), approximate="tanh")
    return lin(p, prefix + ".net.2")(h)


def rope_complex(x, cos, sin):
    """x [B, H, S, d]; rotate pairs (x[2i], x[2i+1]) by the angle whose cos / sin sit at columns 2i, 2i+1 --
    as a complex multiplication, which shares nothing with the oracle's even/odd formula."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2).contiguous())
    rot = torch.complex(cos[:, 0::2].double(), sin[:, 0::2].double()).to(torch.complex64)
    return torch.view_as_real(xc * rot[None, None]).flatten(3)


def split_heads(x, H):
    B, S, I = x.shape
    return x.view(B, S, H, I // H).transpose(1, 2)


def merge_heads(x):
    B, H, S, d = x.shape
    return x.transpose(1, 2).reshape(B, S, H * d)


# ---------------------------------------------------------------------------
# SD3 JointTransformerBlock
# ---------------------------------------------------------------------------

def nn_sd3_block(p, x, e, t, H, pre_only, mut=None):
    D = x.shape[-1]
    eps = 1e-5 if mut == "eps" else 1e-6
    c = list(ada_chunks(p, "norm1", t, 6))  # shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp
    if mut == "swap_shift_scale":
        c[0], c[1] = c[1], c[0]
    if mut == "swap_gates":
        c[2], c[5] = c[5], c[2]
    if mut == "swap_mlp_shift_scale":
        c[3], c[4] = c[4], c[3]
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = c
    n = layer_norm_noaffine(D, eps)(x) * (1 + scale_msa[:, None]) + shift_msa[:, None]
    if pre_only:
        scale, shift = ada_chunks(p, "norm1_context", t, 2)  # AdaLayerNormContinuous: scale first
        if mut == "continuous_shift_first":
            scale, shift = shift, scale
        nc = layer_norm_noaffine(D, eps)(e) * (1 + scale)[:, None, :] + shift[:, None, :]
    else:
        cc = list(ada_chunks(p, "norm1_context", t, 6))
        if mut == "swap_context_gates":
            cc[2], cc[5] = cc[5], cc[2]
        if mut == "swap_context_shift_scale":
            cc[0], cc[1] = cc[1], cc[0]
        c_shift_msa, c_scale_msa, c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp = cc
        nc = layer_norm_noaffine(D, eps)(e) * (1 + c_scale_msa[:, None]) + c_shift_msa[:, None]
    # joint attention, reference processor order [image, text], no QK norm
    q = torch.cat([lin(p, "attn.to_q")(n), lin(p, "attn.add_q_proj")(nc)], 1)
    k = torch.cat([lin(p, "attn.to_k")(n), lin(p, "attn.add_k_proj")(nc)], 1)
    v = torch.cat([lin(p, "attn.to_v")(n), lin(p, "attn.add_v_proj")(nc)], 1)
    o = merge_heads(F.scaled_dot_product_attention(split_heads(q, H), split_heads(k, H), split_heads(v, H)))
    Ni = x.shape[1]
    a = lin(p, "attn.to_out.0")(o[:, :Ni])
    x = x + gate_msa.unsqueeze(1) * a
    n2 = layer_norm_noaffine(D, eps)(x) * (1 + scale_mlp[:, None]) + shift_mlp[:, None]
    x = x + gate_mlp.unsqueeze(1) * feed_forward(p, "ff", n2)
    if pre_only:
        return None, x
    ca = lin(p, "attn.to_add_out")(o[:, Ni:])
    e = e + c_gate_msa.unsqueeze(1) * ca
    nc2 = layer_norm_noaffine(D, eps)(e) * (1 + c_scale_mlp[:, None]) + c_shift_mlp[:, None]
    if mut == "context_uses_image_ff":
        e = e + c_gate_mlp.unsqueeze(1) * feed_forward(p, "ff", nc2)
    else:
        e = e + c_gate_mlp.unsqueeze(1) * feed_forward(p, "ff_context", nc2)
    return e, x


# ---------------------------------------------------------------------------
# Flux
# ---------------------------------------------------------------------------

def nn_flux_attention(p, n, nc, rope, H, n_txt_single=0, mut=None):
    hd = p["attn.to_q.weight"].shape[0] // H
    rms = lambda z, name: F.rms_norm(z, (hd,), p[f"attn.{name}.weight"], eps=1e-5 if mut == "qk_eps" else 1e-6)
    q = rms(split_heads(lin(p, "attn.to_q")(n), H), "norm_q")
    k = rms(split_heads(lin(p, "attn.to_k")(n), H), "norm_k")
    v = split_heads(lin(p, "attn.to_v")(n), H)
    if nc is not None:
        eq = rms(split_heads(lin(p, "attn.add_q_proj")(nc), H), "norm_added_q")
        ek = rms(split_heads(lin(p, "attn.add_k_proj")(nc), H), "norm_k" if mut == "text_k_uses_image_norm" else "norm_added_k")
        ev = split_heads(lin(p, "attn.add_v_proj")(nc), H)
        if mut == "image_first":
            q, k, v = torch.cat([q, eq], 2), torch.cat([k, ek], 2), torch.cat([v, ev], 2)
        else:
            q, k, v = torch.cat([eq, q], 2), torch.cat([ek, k], 2), torch.cat([ev, v], 2)  # [text, image]
    cos, sin = rope
    q = rope_complex(q, cos, sin)
    if mut != "no_rope_on_k":
        k = rope_complex(k, cos, sin)
    o = merge_heads(F.scaled_dot_product_attention(q, k, v))
    if nc is None:
        return o
    nt = nc.shape[1]
    if mut == "image_first":
        o_img, o_txt = o[:, : n.shape[1]], o[:, n.shape[1]:]
    else:
        o_txt, o_img = o[:, :nt], o[:, nt:]
    # the reference's wrapper detaches to_add_out.bias and its Flux branch never adds it back
    return lin(p, "attn.to_out.0")(o_img), lin(p, "attn.to_add_out", bias=(mut == "keep_text_bias"))(o_txt)


def nn_flux_double(p, x, e, t, rope, H, mut=None):
    D = x.shape[-1]
    eps = 1e-5 if mut == "eps" else 1e-6
    c = list(ada_chunks(p, "norm1", t, 6))
    cc = list(ada_chunks(p, "norm1_context", t, 6))
    if mut == "swap_shift_scale":
        c[0], c[1] = c[1], c[0]
    if mut == "swap_gates":
        c[2], c[5] = c[5], c[2]
    if mut == "swap_context_gates":
        cc[2], cc[5] = cc[5], cc[2]
    if mut == "context_mod_from_image":
        cc = c
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = c
    c_shift_msa, c_scale_msa, c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp = cc
    n = layer_norm_noaffine(D, eps)(x) * (1 + scale_msa[:, None]) + shift_msa[:, None]
    nc = layer_norm_noaffine(D, eps)(e) * (1 + c_scale_msa[:, None]) + c_shift_msa[:, None]
    a, ca = nn_flux_attention(p, n, nc, rope, H, mut=mut)
    x = x + gate_msa.unsqueeze(1) * a
    n2 = layer_norm_noaffine(D, eps)(x) * (1 + scale_mlp[:, None]) + shift_mlp[:, None]
    x = x + gate_mlp.unsqueeze(1) * feed_forward(p, "ff", n2)
    e = e + c_gate_msa.unsqueeze(1) * ca
    nc2 = layer_norm_noaffine(D, eps)(e) * (1 + c_scale_mlp[:, None]) + c_shift_mlp[:, None]
    e = e + c_gate_mlp.unsqueeze(1) * feed_forward(p, "ff_context", nc2)
    return e, x


def nn_flux_single(p, x, t, rope, H, mut=None):
    D = x.shape[-1]
    c = list(ada_chunks(p, "norm", t, 3))  # shift, scale, gate
    if mut == "swap_shift_scale":
        c[0], c[1] = c[1], c[0]
    if mut == "gate_is_scale":
        c[1], c[2] = c[2], c[1]
    shift, scale, gate = c
    n = layer_norm_noaffine(D, 1e-5 if mut == "eps" else 1e-6)(x) * (1 + scale[:, None]) + shift[:, None]
    m = F.gelu(lin(p, "proj_mlp")(n), approximate="tanh")
    a = nn_flux_attention(p, n, None, rope, H, mut=mut)
    cat = torch.cat([m, a], 2) if mut == "cat_mlp_first" else torch.cat([a, m], 2)
    return x + gate.unsqueeze(1) * lin(p, "proj_out")(cat)


# ---------------------------------------------------------------------------
# CogVideoX
# ---------------------------------------------------------------------------

def nn_cog_norm_zero(p, name, x, e, t, mut=None):
    D = x.shape[-1]
    c = list(ada_chunks(p, name, t, 6))  # shift, scale, gate, enc_shift, enc_scale, enc_gate
    if mut == "swap_shift_scale":
        c[0], c[1] = c[1], c[0]
    if mut == "swap_stream_chunks":
        c = c[3:] + c[:3]
    if mut == "enc_gate_is_gate":
        c[5] = c[2]
    shift, scale, gate, enc_shift, enc_scale, enc_gate = c
    norm = nn.LayerNorm(D, eps=1e-6 if mut == "eps" else 1e-5, elementwise_affine=True)
    with torch.no_grad():
        if mut != "no_affine":
            norm.weight.copy_(p[name + ".norm.weight"])
            norm.bias.copy_(p[name + ".norm.bias"])
    xn = norm(x) * (1 + scale)[:, None, :] + shift[:, None, :]
    en = norm(e) * (1 + enc_scale)[:, None, :] + enc_shift[:, None, :]
    return xn, en, gate[:, None, :], enc_gate[:, None, :]


def nn_cog_block(p, x, e, t, rope, H, mut=None):
    nt = e.shape[1]
    hd = p["attn1.to_q.weight"].shape[0] // H
    xn, en, gate, enc_gate = nn_cog_norm_zero(p, "norm1", x, e, t, mut)
    joint = torch.cat([en, xn], 1)  # [text, video]
    qn = nn.LayerNorm(hd, eps=1e-5 if mut == "qk_eps" else 1e-6)
    kn = nn.LayerNorm(hd, eps=1e-5 if mut == "qk_eps" else 1e-6)
    with torch.no_grad():
        qn.weight.copy_(p["attn1.norm_q.weight"]), qn.bias.copy_(p["attn1.norm_q.bias"])
        kn.weight.copy_(p["attn1.norm_k.weight"]), kn.bias.copy_(p["attn1.norm_k.bias"])
    q = qn(split_heads(lin(p, "attn1.to_q")(joint), H))
    k = kn(split_heads(lin(p, "attn1.to_k")(joint), H))
    v = split_heads(lin(p, "attn1.to_v")(joint), H)
    cos, sin = rope
    if mut == "rope_on_all_rows":
        full_cos = torch.cat([cos[:nt], cos], 0)
        full_sin = torch.cat([sin[:nt], sin], 0)
        q, k = rope_complex(q, full_cos, full_sin), rope_complex(k, full_cos, full_sin)
    else:
        q = torch.cat([q[:, :, :nt], rope_complex(q[:, :, nt:], cos, sin)], 2)
        k = torch.cat([k[:, :, :nt], rope_complex(k[:, :, nt:], cos, sin)], 2)
    o = lin(p, "attn1.to_out.0")(merge_heads(F.scaled_dot_product_attention(q, k, v)))
    a_e, a_x = o[:, :nt], o[:, nt:]
    x = x + gate * a_x
    e = e + enc_gate * a_e
    xn, en, gate_ff, enc_gate_ff = nn_cog_norm_zero(p, "norm1" if mut == "norm2_is_norm1" else "norm2", x, e, t, mut)
    f = feed_forward(p, "ff", torch.cat([en, xn], 1))
    x = x + gate_ff * f[:, nt:]
    e = e + enc_gate_ff * f[:, :nt]
    return x, e


# ---------------------------------------------------------------------------
# parameters and inputs
# ---------------------------------------------------------------------------

def randp(shapes, seed, std=0.15):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for n, s in shapes.items():
        v = torch.randn(*s, generator=g) * std
        if n.endswith("norm_q.weight") or n.endswith("norm_k.weight") or n.endswith("norm.weight"):
            v = 1.0 + v  # norm weights around one
        out[n] = v
    return out


def sd3_shapes(D, pre_only):
    Fd = 4 * D
    s = {"norm1.linear.weight": (6 * D, D), "norm1.linear.bias": (6 * D,),
         "norm1_context.linear.weight": ((2 if pre_only else 6) * D, D),
         "norm1_context.linear.bias": ((2 if pre_only else 6) * D,)}
    for n in ("to_q", "to_k", "to_v", "add_q_proj", "add_k_proj", "add_v_proj", "to_out.0"):
        s[f"attn.{n}.weight"], s[f"attn.{n}.bias"] = (D, D), (D,)
    if not pre_only:
        s["attn.to_add_out.weight"], s["attn.to_add_out.bias"] = (D, D), (D,)
    for ff in ("ff",) + (() if pre_only else ("ff_context",)):
        s[f"{ff}.net.0.proj.weight"], s[f"{ff}.net.0.proj.bias"] = (Fd, D), (Fd,)
        s[f"{ff}.net.2.weight"], s[f"{ff}.net.2.bias"] = (D, Fd), (D,)
    return s


def flux_double_shapes(D, hd):
    s = sd3_shapes(D, False)
    for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"):
        s[f"attn.{n}.weight"] = (hd,)
    return s


def flux_single_shapes(D, hd):
    s = {"norm.linear.weight": (3 * D, D), "norm.linear.bias": (3 * D,), "proj_mlp.weight": (4 * D, D),
         "proj_mlp.bias": (4 * D,), "proj_out.weight": (D, 5 * D), "proj_out.bias": (D,)}
    for n in ("to_q", "to_k", "to_v"):
        s[f"attn.{n}.weight"], s[f"attn.{n}.bias"] = (D, D), (D,)
    for n in ("norm_q", "norm_k"):
        s[f"attn.{n}.weight"] = (hd,)
    return s


def cog_shapes(D, hd, Tt):
    s = {}
    for nm in ("norm1", "norm2"):
        s[f"{nm}.linear.weight"], s[f"{nm}.linear.bias"] = (6 * D, Tt), (6 * D,)
        s[f"{nm}.norm.weight"], s[f"{nm}.norm.bias"] = (D,), (D,)
    s.update({"ff.net.0.proj.weight": (4 * D, D), "ff.net.0.proj.bias": (4 * D,), "ff.net.2.weight": (D, 4 * D),
              "ff.net.2.bias": (D,)})
    for n in ("to_q", "to_k", "to_v", "to_out.0"):
        s[f"attn1.{n}.weight"], s[f"attn1.{n}.bias"] = (D, D), (D,)
    for n in ("norm_q", "norm_k"):
        s[f"attn1.{n}.weight"], s[f"attn1.{n}.bias"] = (hd,), (hd,)
    return s


def inputs(B, Ni, Nt, D, Tt, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    # a non-zero mean and a small spread (with `scale` < 1) make eps and the affine terms visible
    return (torch.randn(B, Ni, D, generator=g) * scale + 0.3 * scale, torch.randn(B, Nt, D, generator=g) * scale,
            torch.randn(B, Tt, generator=g))


def rel(a, b):
    return float((a - b).norm() / b.norm())


def agree(got, want, what):
    assert got.shape == want.shape, what
    assert rel(got, want) < 2e-5, f"{what}: oracle and library assembly differ by {rel(got, want):.2e}"


def differ(got, want, what):
    assert rel(got, want) > 1e-3, f"{what}: this wiring mistake goes unnoticed ({rel(got, want):.2e})"


# ---------------------------------------------------------------------------
# tests
# ---------------------------------------------------------------------------

SD3_MUTATIONS = ["swap_shift_scale", "swap_gates", "swap_mlp_shift_scale", "swap_context_gates",
                 "swap_context_shift_scale", "context_uses_image_ff", "eps"]


@torch.no_grad()
def test_sd3_joint_block_against_library_assembly():
    D, H = 64, 2
    p = randp(sd3_shapes(D, False), 1)
    for scale in (1.0, 2e-3):  # the small-spread inputs are where eps matters
        x, e, t = inputs(2, 10, 4, D, D, 2, scale)
        enc, hid = oracle.sd3_joint_block(p, x, e, t, H)
        n_enc, n_hid = nn_sd3_block(p, x, e, t, H, False)
        agree(hid, n_hid, "sd3 hidden")
        agree(enc, n_enc, "sd3 encoder")


@pytest.mark.parametrize("mut", SD3_MUTATIONS)
@torch.no_grad()
def test_sd3_joint_block_mutations_are_caught(mut):
    D, H = 64, 2
    p = randp(sd3_shapes(D, False), 1)
    x, e, t = inputs(2, 10, 4, D, D, 2, 2e-3 if mut == "eps" else 1.0)
    enc, hid = oracle.sd3_joint_block(p, x, e, t, H)
    m_enc, m_hid = nn_sd3_block(p, x, e, t, H, False, mut=mut)
    differ(torch.cat([m_hid, m_enc], 1), torch.cat([hid, enc], 1), f"sd3 {mut}")


@torch.no_grad()
def test_sd3_context_pre_only_block_against_library_assembly():
    """Last SD3 block: the text stream is normalised by AdaLayerNormContinuous (chunk order scale, shift), has
    no out-projection, no MLP, and returns None."""
    D, H = 64, 2
    p = randp(sd3_shapes(D, True), 3)
    x, e, t = inputs(2, 10, 4, D, D, 4)
    enc, hid = oracle.sd3_joint_block(p, x, e, t, H, context_pre_only=True)
    n_enc, n_hid = nn_sd3_block(p, x, e, t, H, True)
    assert enc is None and n_enc is None
    agree(hid, n_hid, "sd3 pre-only hidden")
    for mut in ("continuous_shift_first", "swap_gates", "swap_mlp_shift_scale"):
        _, m_hid = nn_sd3_block(p, x, e, t, H, True, mut=mut)
        differ(m_hid, hid, f"sd3 pre-only {mut}")


def flux_rope(n_txt, gh, gw, axes):
    ids = torch.zeros(n_txt + gh * gw, 3)
    ids[n_txt:, 1] = torch.arange(gh).repeat_interleave(gw)
    ids[n_txt:, 2] = torch.arange(gw).repeat(gh)
    # table from the textbook formula, not from the oracle: angle = pos * theta^(-2i/dim), repeated per pair
    cos, sin = [], []
    for a, dim in enumerate(axes):
        freq = 1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
        ang = ids[:, a].double()[:, None] * freq[None]
        cos.append(torch.cos(ang).repeat_interleave(2, 1))
        sin.append(torch.sin(ang).repeat_interleave(2, 1))
    return torch.cat(cos, 1).float(), torch.cat(sin, 1).float()


FLUX_DOUBLE_MUTATIONS = ["swap_shift_scale", "swap_gates", "swap_context_gates", "context_mod_from_image", "eps",
                         "qk_eps", "text_k_uses_image_norm", "image_first", "no_rope_on_k", "keep_text_bias"]


@torch.no_grad()
def test_flux_double_block_against_library_assembly():
    D, H, hd = 64, 2, 32
    p = randp(flux_double_shapes(D, hd), 5)
    rope = flux_rope(4, 3, 4, (8, 12, 12))
    for scale in (1.0, 2e-3):
        x, e, t = inputs(2, 12, 4, D, D, 6, scale)
        enc, hid = oracle.flux_double_block(p, x, e, t, rope, H)
        n_enc, n_hid = nn_flux_double(p, x, e, t, rope, H)
        agree(hid, n_hid, "flux double hidden")
        agree(enc, n_enc, "flux double encoder")


@pytest.mark.parametrize("mut", FLUX_DOUBLE_MUTATIONS)
@torch.no_grad()
def test_flux_double_block_mutations_are_caught(mut):
    D, H, hd = 64, 2, 32
    p = randp(flux_double_shapes(D, hd), 5)
    if mut == "keep_text_bias":
        p["attn.to_add_out.bias"] = p["attn.to_add_out.bias"] + 1.0
    rope = flux_rope(4, 3, 4, (8, 12, 12))
    small = mut in ("eps", "qk_eps")
    x, e, t = inputs(2, 12, 4, D, D, 6, 2e-3 if mut == "eps" else 1.0)
    if small and mut == "qk_eps":
        # q and k must be small before their RMSNorm for its eps to matter
        for n in ("to_q", "to_k", "add_q_proj", "add_k_proj"):
            p[f"attn.{n}.weight"] = p[f"attn.{n}.weight"] * 1e-3
            p[f"attn.{n}.bias"] = p[f"attn.{n}.bias"] * 1e-3
    enc, hid = oracle.flux_double_block(p, x, e, t, rope, H)
    if mut == "qk_eps":  # the unmutated assembly still agrees on these parameters
        n_enc, n_hid = nn_flux_double(p, x, e, t, rope, H)
        agree(n_hid, hid, "flux double hidden (small q, k)")
    m_enc, m_hid = nn_flux_double(p, x, e, t, rope, H, mut=mut)
    differ(torch.cat([m_hid, m_enc], 1), torch.cat([hid, enc], 1), f"flux double {mut}")


# (erf- against tanh-GELU differs by < 1e-4 of a block output: that choice is pinned on the primitive, in
# tests/test_oracle_ops.py, not here)
FLUX_SINGLE_MUTATIONS = ["swap_shift_scale", "gate_is_scale", "eps", "cat_mlp_first", "no_rope_on_k"]


@torch.no_grad()
def test_flux_single_block_against_library_assembly():
    D, H, hd, nt = 64, 2, 32, 4
    p = randp(flux_single_shapes(D, hd), 7)
    rope = flux_rope(nt, 3, 4, (8, 12, 12))
    for scale in (1.0, 2e-3):
        x, _, t = inputs(2, nt + 12, 1, D, D, 8, scale)
        got = oracle.flux_single_block(p, x, t, rope, H, n_text=nt)
        agree(got, nn_flux_single(p, x, t, rope, H), "flux single")


@pytest.mark.parametrize("mut", FLUX_SINGLE_MUTATIONS)
@torch.no_grad()
def test_flux_single_block_mutations_are_caught(mut):
    D, H, hd, nt = 64, 2, 32, 4
    p = randp(flux_single_shapes(D, hd), 7)
    rope = flux_rope(nt, 3, 4, (8, 12, 12))
    x, _, t = inputs(2, nt + 12, 1, D, D, 8, 2e-3 if mut == "eps" else 1.0)
    got = oracle.flux_single_block(p, x, t, rope, H, n_text=nt)
    differ(nn_flux_single(p, x, t, rope, H, mut=mut), got, f"flux single {mut}")


def cog_rope(grid, hd):
    f, h, w = grid
    dims = (hd // 4, hd // 8 * 3, hd // 8 * 3)
    pos = torch.stack(torch.meshgrid(torch.arange(f), torch.arange(h), torch.arange(w), indexing="ij"), -1).reshape(-1, 3)
    cos, sin = [], []
    for a, dim in enumerate(dims):
        freq = 1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
        ang = pos[:, a].double()[:, None] * freq[None]
        cos.append(torch.cos(ang).repeat_interleave(2, 1))
        sin.append(torch.sin(ang).repeat_interleave(2, 1))
    return torch.cat(cos, 1).float(), torch.cat(sin, 1).float()


COG_MUTATIONS = ["swap_shift_scale", "swap_stream_chunks", "enc_gate_is_gate", "eps", "no_affine", "qk_eps",
                 "rope_on_all_rows", "norm2_is_norm1"]
# (joining [video, text] instead of [text, video] with the rotation kept on the video rows is not a mistake a
# test can see: full attention is permutation-equivariant and everything else is row-wise)


@torch.no_grad()
def test_cogvideox_block_against_library_assembly():
    D, H, hd, Tt = 64, 2, 32, 16
    p = randp(cog_shapes(D, hd, Tt), 9)
    rope = cog_rope((2, 2, 3), hd)
    for scale in (1.0, 5e-3):
        x, e, t = inputs(2, 12, 5, D, Tt, 10, scale)
        hid, enc = oracle.cogvideox_block(p, x, e, t, rope, H)
        n_hid, n_enc = nn_cog_block(p, x, e, t, rope, H)
        agree(hid, n_hid, "cogvideox hidden")
        agree(enc, n_enc, "cogvideox encoder")
    # the oracle's own 3-D table is the same table
    ocos, osin = O.cogvideox_rope_table(2, 2, 3, head_dim=hd)
    torch.testing.assert_close(ocos, rope[0], rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(osin, rope[1], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("mut", COG_MUTATIONS)
@torch.no_grad()
def test_cogvideox_block_mutations_are_caught(mut):
    D, H, hd, Tt = 64, 2, 32, 16
    p = randp(cog_shapes(D, hd, Tt), 9)
    rope = cog_rope((2, 2, 3), hd)
    x, e, t = inputs(2, 12, 5, D, Tt, 10, 5e-3 if mut == "eps" else 1.0)
    if mut == "qk_eps":
        for n in ("to_q", "to_k"):
            p[f"attn1.{n}.weight"] = p[f"attn1.{n}.weight"] * 1e-3
            p[f"attn1.{n}.bias"] = p[f"attn1.{n}.bias"] * 1e-3
    hid, enc = oracle.cogvideox_block(p, x, e, t, rope, H)
    if mut == "qk_eps":
        n_hid, _ = nn_cog_block(p, x, e, t, rope, H)
        agree(n_hid, hid, "cogvideox hidden (small q, k)")
    m_hid, m_enc = nn_cog_block(p, x, e, t, rope, H, mut=mut)
    differ(torch.cat([m_hid, m_enc], 1), torch.cat([hid, enc], 1), f"cogvideox {mut}")


@torch.no_grad()
def test_flux_rope_table_against_textbook_formula():
    ids = torch.zeros(4 + 12, 3)
    ids[4:, 1] = torch.arange(3).repeat_interleave(4)
    ids[4:, 2] = torch.arange(4).repeat(3)
    ocos, osin = O.flux_rope_table(ids, (8, 12, 12))
    cos, sin = flux_rope(4, 3, 4, (8, 12, 12))
    torch.testing.assert_close(ocos, cos, rtol=0, atol=1e-7)
    torch.testing.assert_close(osin, sin, rtol=0, atol=1e-7)
