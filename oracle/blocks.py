"""fp32 restatement of the four transformer blocks on the hot path (test
infrastructure, never shipped).

Parameters are passed as a flat ``dict`` keyed by the parameter paths of the
*unwrapped* diffusers block (``"attn.to_q.weight"``, ``"ff.net.0.proj.bias"``,
``"norm1.linear.weight"`` ...), i.e. the paths the reference's weight hot-swap
addresses (``hetu_dit/utils.py:561-582``) without the ``.module.`` hop its layer
wrappers insert.

The attention part of each block follows the reference's processors
(``layers/attention_processor.py``); the rest follows the published diffusers
blocks the reference calls (see the package docstring for what is unpinned).
An optional ``kv`` argument (a ``StaleKVBuffer``) reproduces the KV-cache call
the processors make for the image stream.
"""

from typing import Dict, Optional, Tuple

import torch

from .ops import (
    adaln_modulation,
    apply_rotary_emb,
    attention,
    gelu_erf,
    gelu_tanh,
    layer_norm,
    linear,
    modulate,
    rms_norm,
    silu,
)

P = Dict[str, torch.Tensor]


def _lin(p: P, name: str, x: torch.Tensor) -> torch.Tensor:
    return linear(x, p[name + ".weight"], p.get(name + ".bias"))


def _heads(x: torch.Tensor, heads: int) -> torch.Tensor:
    """[B, S, H*d] -> [B, H, S, d]"""
    b, s, inner = x.shape
    return x.reshape(b, s, heads, inner // heads).transpose(1, 2)


def _unheads(x: torch.Tensor) -> torch.Tensor:
    """[B, H, S, d] -> [B, S, H*d]"""
    b, h, s, d = x.shape
    return x.transpose(1, 2).reshape(b, s, h * d)


def feed_forward(p: P, prefix: str, x: torch.Tensor, activation_fn: str = "gelu-approximate") -> torch.Tensor:
    """``net = [activation(proj), Dropout, Linear]`` -- the module ``hetuDiTFeedForwardWrapper`` wraps
    (``layers/feedforward.py:17-78``); at one GPU the detached output bias is simply added back (``:75-77``).
    ``activation_fn`` as diffusers names the first-layer classes the wrapper accepts (``:25-57``): tanh GELU (every
    model on this path), exact GELU, GEGLU (value half times exact GELU of the gate half), LinearActivation (SiLU)."""
    h = _lin(p, prefix + ".net.0.proj", x)
    if activation_fn == "gelu-approximate":
        h = gelu_tanh(h)
    elif activation_fn == "gelu":
        h = gelu_erf(h)
    elif activation_fn == "geglu":
        value, gate_half = h.chunk(2, dim=-1)
        h = value * gelu_erf(gate_half)
    elif activation_fn == "linear-silu":
        h = silu(h)
    else:
        raise ValueError(activation_fn)
    return _lin(p, prefix + ".net.2", h)


# --------------------------------------------------------------------------
# SD3 joint block
# --------------------------------------------------------------------------

def sd3_joint_attention(
    p: P,
    hidden: torch.Tensor,
    encoder: torch.Tensor,
    heads: int,
    context_pre_only: bool,
    kv=None,
    prefix: str = "attn",
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``hetuDiTJointAttnProcessor2_0.__call__`` (``attention_processor.py:657-793``)
    followed by the out-projections of ``hetuDiTAttentionWrapper.forward``
    (``:404-449``).  Joint order is [image, text]; no QK-norm is applied; the
    softmax scale is 1/sqrt(d).  Only the image K/V go through the KV cache
    (``:701-707``), so in patch mode the query is the patch (plus text) and the
    keys are the whole buffer (plus text)."""
    q = _lin(p, prefix + ".to_q", hidden)
    k = _lin(p, prefix + ".to_k", hidden)
    v = _lin(p, prefix + ".to_v", hidden)
    eq = _lin(p, prefix + ".add_q_proj", encoder)
    ek = _lin(p, prefix + ".add_k_proj", encoder)
    ev = _lin(p, prefix + ".add_v_proj", encoder)
    if kv is not None:
        k, v = kv.update_and_get(k, v, slice_dim=1)
    n_img = hidden.shape[1]
    q = torch.cat([q, eq], dim=1)
    k = torch.cat([k, ek], dim=1)
    v = torch.cat([v, ev], dim=1)
    o = _unheads(attention(_heads(q, heads), _heads(k, heads), _heads(v, heads)))
    o_img, o_txt = o[:, :n_img], o[:, n_img:]
    o_img = _lin(p, prefix + ".to_out.0", o_img)
    if not context_pre_only:
        o_txt = _lin(p, prefix + ".to_add_out", o_txt)
    return o_img, o_txt


def sd3_joint_block(
    p: P,
    hidden: torch.Tensor,
    encoder: torch.Tensor,
    temb: torch.Tensor,
    heads: int,
    context_pre_only: bool = False,
    kv=None,
) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
    """diffusers ``JointTransformerBlock.forward`` as called at
    ``models/transformers/transformer_sd3.py:136-152``.

    Returns ``(encoder_hidden_states, hidden_states)``; the text output is
    ``None`` for the last block (``context_pre_only``), whose text stream uses
    AdaLayerNormContinuous (chunk order **scale, shift**)."""
    eps = 1e-6
    sh_a, sc_a, g_a, sh_m, sc_m, g_m = adaln_modulation(temb, p["norm1.linear.weight"], p["norm1.linear.bias"], 6)
    n = modulate(layer_norm(hidden, eps), sh_a, sc_a)
    if context_pre_only:
        c_sc, c_sh = adaln_modulation(temb, p["norm1_context.linear.weight"], p["norm1_context.linear.bias"], 2)
        nc = modulate(layer_norm(encoder, eps), c_sh, c_sc)
    else:
        c_sh_a, c_sc_a, c_g_a, c_sh_m, c_sc_m, c_g_m = adaln_modulation(
            temb, p["norm1_context.linear.weight"], p["norm1_context.linear.bias"], 6
        )
        nc = modulate(layer_norm(encoder, eps), c_sh_a, c_sc_a)

    a, ca = sd3_joint_attention(p, n, nc, heads, context_pre_only, kv=kv)

    hidden = hidden.float() + g_a[:, None] * a
    n2 = modulate(layer_norm(hidden, eps), sh_m, sc_m)
    hidden = hidden + g_m[:, None] * feed_forward(p, "ff", n2)

    if context_pre_only:
        return None, hidden
    encoder = encoder.float() + c_g_a[:, None] * ca
    nc2 = modulate(layer_norm(encoder, eps), c_sh_m, c_sc_m)
    encoder = encoder + c_g_m[:, None] * feed_forward(p, "ff_context", nc2)
    return encoder, hidden


# --------------------------------------------------------------------------
# Flux double- and single-stream blocks
# --------------------------------------------------------------------------

def flux_attention(
    p: P,
    hidden: torch.Tensor,
    encoder: Optional[torch.Tensor],
    rope: Optional[Tuple[torch.Tensor, torch.Tensor]],
    heads: int,
    n_text_single: int = 0,
    kv=None,
    prefix: str = "attn",
):
    """``hetuDiTFluxAttnProcessor2_0.__call__`` (``attention_processor.py:824-987``)
    plus the wrapper's Flux branch (``:284-319``).

    RMSNorm (eps 1e-6) on q, k per head; joint order [text, image]; RoPE over
    all joint tokens for q and k; the image part of K/V goes through the KV
    cache (``slice_dim=2``).  With ``encoder is None`` (single-stream block)
    the text/image split point of the joint input is ``n_text_single``
    (``get_runtime_state().max_condition_sequence_length``, ``:897-901``) and
    the joint attention output is returned without an out-projection."""
    eps = 1e-6
    q = _heads(_lin(p, prefix + ".to_q", hidden), heads)
    k = _heads(_lin(p, prefix + ".to_k", hidden), heads)
    v = _heads(_lin(p, prefix + ".to_v", hidden), heads)
    q = rms_norm(q, eps, p.get(prefix + ".norm_q.weight"))
    k = rms_norm(k, eps, p.get(prefix + ".norm_k.weight"))
    if encoder is not None:
        eq = _heads(_lin(p, prefix + ".add_q_proj", encoder), heads)
        ek = _heads(_lin(p, prefix + ".add_k_proj", encoder), heads)
        ev = _heads(_lin(p, prefix + ".add_v_proj", encoder), heads)
        eq = rms_norm(eq, eps, p.get(prefix + ".norm_added_q.weight"))
        ek = rms_norm(ek, eps, p.get(prefix + ".norm_added_k.weight"))
        n_txt = eq.shape[2]
        q = torch.cat([eq, q], dim=2)
        k = torch.cat([ek, k], dim=2)
        v = torch.cat([ev, v], dim=2)
    else:
        n_txt = n_text_single
    if rope is not None:
        q = apply_rotary_emb(q, rope[0], rope[1])
        k = apply_rotary_emb(k, rope[0], rope[1])
    if kv is not None:
        k_txt, k_img = k[:, :, :n_txt], k[:, :, n_txt:]
        v_txt, v_img = v[:, :, :n_txt], v[:, :, n_txt:]
        k_img, v_img = kv.update_and_get(k_img, v_img, slice_dim=2)
        k = torch.cat([k_txt, k_img], dim=2)
        v = torch.cat([v_txt, v_img], dim=2)
    o = _unheads(attention(q, k, v))
    if encoder is None:
        return o
    o_txt, o_img = o[:, :n_txt], o[:, n_txt:]
    o_img = _lin(p, prefix + ".to_out.0", o_img)
    # The wrapper moves to_add_out.bias into `encoder_output_bias`
    # (attention_processor.py:176-192) and its Flux branch never adds it back
    # (:284-305): the reference computes the text out-projection WITHOUT bias.
    o_txt = linear(o_txt, p[prefix + ".to_add_out.weight"], None)
    return o_img, o_txt


def flux_double_block(
    p: P,
    hidden: torch.Tensor,
    encoder: torch.Tensor,
    temb: torch.Tensor,
    rope: Tuple[torch.Tensor, torch.Tensor],
    heads: int,
    kv=None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """diffusers ``FluxTransformerBlock.forward`` as called at
    ``models/transformers/transformer_flux.py:160-165``; returns
    ``(encoder_hidden_states, hidden_states)``."""
    eps = 1e-6
    sh_a, sc_a, g_a, sh_m, sc_m, g_m = adaln_modulation(temb, p["norm1.linear.weight"], p["norm1.linear.bias"], 6)
    c_sh_a, c_sc_a, c_g_a, c_sh_m, c_sc_m, c_g_m = adaln_modulation(
        temb, p["norm1_context.linear.weight"], p["norm1_context.linear.bias"], 6
    )
    n = modulate(layer_norm(hidden, eps), sh_a, sc_a)
    nc = modulate(layer_norm(encoder, eps), c_sh_a, c_sc_a)
    a, ca = flux_attention(p, n, nc, rope, heads, kv=kv)
    hidden = hidden.float() + g_a[:, None] * a
    n2 = modulate(layer_norm(hidden, eps), sh_m, sc_m)
    hidden = hidden + g_m[:, None] * feed_forward(p, "ff", n2)
    encoder = encoder.float() + c_g_a[:, None] * ca
    nc2 = modulate(layer_norm(encoder, eps), c_sh_m, c_sc_m)
    encoder = encoder + c_g_m[:, None] * feed_forward(p, "ff_context", nc2)
    return encoder, hidden


def flux_single_block(
    p: P,
    hidden: torch.Tensor,
    temb: torch.Tensor,
    rope: Tuple[torch.Tensor, torch.Tensor],
    heads: int,
    n_text: int,
    kv=None,
) -> torch.Tensor:
    """diffusers ``FluxSingleTransformerBlock.forward`` as called at
    ``models/transformers/transformer_flux.py:194-198`` on the joint
    ``[text, image]`` sequence: adaLN-ZeroSingle (shift, scale, gate), MLP-in
    in parallel with attention, ``proj_out`` over ``cat([attn, mlp], 2)``."""
    eps = 1e-6
    sh, sc, g = adaln_modulation(temb, p["norm.linear.weight"], p["norm.linear.bias"], 3)
    n = modulate(layer_norm(hidden, eps), sh, sc)
    m = gelu_tanh(_lin(p, "proj_mlp", n))
    a = flux_attention(p, n, None, rope, heads, n_text_single=n_text, kv=kv)
    y = _lin(p, "proj_out", torch.cat([a, m], dim=2))
    return hidden.float() + g[:, None] * y


# --------------------------------------------------------------------------
# CogVideoX block
# --------------------------------------------------------------------------

def cogvideox_attention(
    p: P,
    hidden: torch.Tensor,
    encoder: torch.Tensor,
    rope: Optional[Tuple[torch.Tensor, torch.Tensor]],
    heads: int,
    prefix: str = "attn1",
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``hetuDiTCogVideoXAttnProcessor2_0.__call__``
    (``attention_processor.py:1022-1158``) plus the wrapper's CogVideoX branch
    (``:253-283``): cat [text, video] *before* one set of projections,
    LayerNorm (eps 1e-6, affine) on q, k per head, RoPE on the video rows only,
    attention, ``to_out`` on the joint tensor, split; no KV-cache call."""
    n_txt = encoder.shape[1]
    x = torch.cat([encoder, hidden], dim=1)
    q = _heads(_lin(p, prefix + ".to_q", x), heads)
    k = _heads(_lin(p, prefix + ".to_k", x), heads)
    v = _heads(_lin(p, prefix + ".to_v", x), heads)
    q = layer_norm(q, 1e-6, p.get(prefix + ".norm_q.weight"), p.get(prefix + ".norm_q.bias"))
    k = layer_norm(k, 1e-6, p.get(prefix + ".norm_k.weight"), p.get(prefix + ".norm_k.bias"))
    if rope is not None:
        q = torch.cat([q[:, :, :n_txt], apply_rotary_emb(q[:, :, n_txt:], rope[0], rope[1])], dim=2)
        k = torch.cat([k[:, :, :n_txt], apply_rotary_emb(k[:, :, n_txt:], rope[0], rope[1])], dim=2)
    o = _unheads(attention(q, k, v))
    o = _lin(p, prefix + ".to_out.0", o)
    return o[:, n_txt:], o[:, :n_txt]


def _cog_norm_zero(p: P, prefix: str, hidden, encoder, temb):
    """diffusers ``CogVideoXLayerNormZero``: chunk order shift, scale, gate,
    enc_shift, enc_scale, enc_gate; one affine LayerNorm (eps 1e-5) shared by
    both streams."""
    sh, sc, g, e_sh, e_sc, e_g = adaln_modulation(temb, p[prefix + ".linear.weight"], p[prefix + ".linear.bias"], 6)
    w, b = p[prefix + ".norm.weight"], p[prefix + ".norm.bias"]
    n = modulate(layer_norm(hidden, 1e-5, w, b), sh, sc)
    ne = modulate(layer_norm(encoder, 1e-5, w, b), e_sh, e_sc)
    return n, ne, g, e_g


def cogvideox_block(
    p: P,
    hidden: torch.Tensor,
    encoder: torch.Tensor,
    temb: torch.Tensor,
    rope: Optional[Tuple[torch.Tensor, torch.Tensor]],
    heads: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """diffusers ``CogVideoXBlock.forward`` as called at
    ``models/transformers/cogvideox_transformer_3d.py:122-127``; returns
    ``(hidden_states, encoder_hidden_states)`` -- the opposite order to the
    SD3 / Flux blocks."""
    n_txt = encoder.shape[1]
    n, ne, g, e_g = _cog_norm_zero(p, "norm1", hidden, encoder, temb)
    a, ea = cogvideox_attention(p, n, ne, rope, heads)
    hidden = hidden.float() + g[:, None] * a
    encoder = encoder.float() + e_g[:, None] * ea
    n, ne, g, e_g = _cog_norm_zero(p, "norm2", hidden, encoder, temb)
    f = feed_forward(p, "ff", torch.cat([ne, n], dim=1))
    hidden = hidden + g[:, None] * f[:, n_txt:]
    encoder = encoder + e_g[:, None] * f[:, :n_txt]
    return hidden, encoder
