"""CPU oracle (test infrastructure only) for the head and tail of an SD3 denoise step around the block
stack: patch embedding with the cropped sin-cos position table, the timestep / pooled-text conditioning
embedding, the context projection, ``norm_out`` + ``proj_out`` + unpatchify, classifier-free guidance and the
flow-match Euler update.

What the reference owns: the order of these calls (``hetu_dit/model_executor/diffusion_executor/models/
transformers/transformer_sd3.py:92-185``), the patch-embedding wrapper (``.../layers/embeddings.py:32-112``),
the guidance expression (``hetu_dit/model_executor/pipelines/pipeline_stable_diffusion_3.py:1703-1713``) and the
scheduler step (``.../schedulers/scheduling_flow_match_euler_discrete.py:74-118``).  The modules it wraps
(``PatchEmbed``, ``get_2d_sincos_pos_embed``, ``CombinedTimestepTextProjEmbeddings``, ``AdaLayerNormContinuous``)
live in diffusers, which is absent: their published formulas are restated here.

Pinning: ``patch_embed`` against ``F.conv2d``; ``unpatchify`` against the reference's reshape/einsum
expression; ``timestep_embedding`` against the closed form (t = 0 gives [1.., 0..], first frequency is 1);
``cfg_euler_step`` IS the reference's tensor expression sequence in bf16 / fp32 torch arithmetic.
``sincos_pos_embed_2d`` (which axis comes first, the base_size scaling, the centre crop), the order of the
[cos | sin] halves of the timestep projection and ``flow_match_sigmas`` (diffusers' schedule, checked only
against its closed form and the published SD3 28-step values 1.0, 0.9874, ...) are **parity unpinned**: only an
import of diffusers could confirm them.  ``flux_conditioning`` / ``flux_transformer`` compose functions pinned
elsewhere in the order of ``transformer_flux.py:101-207``.  ``cogvideox_patch_embed`` is pinned by ``F.conv2d`` and the
wrapper's own flatten/transpose/cat expressions, ``ada_layer_norm`` by ``torch.nn`` modules (its shift-first chunk order
is diffusers' and unpinned), ``unpatchify_channel_major`` by ``F.fold``.
"""
import math
from typing import Dict, Optional, Tuple

import torch

from . import ops as O

P = Dict[str, torch.Tensor]


def patch_embed(latent: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, pos_embed: Optional[torch.Tensor]) -> torch.Tensor:
    """latent [B, C, H, W], conv weight [D, C, p, p] (stride p) -> tokens [B, (H/p)(W/p), D] (+ pos_embed [T, D])."""
    B, C, H, W = latent.shape
    D, _, p, _ = weight.shape
    x = latent.float().reshape(B, C, H // p, p, W // p, p).permute(0, 2, 4, 1, 3, 5).reshape(B, (H // p) * (W // p), C * p * p)
    tok = O.linear(x, weight.float().reshape(D, C * p * p), bias)
    if pos_embed is not None:
        tok = tok + pos_embed.float()[None]
    return tok


def _sincos_1d(embed_dim: int, pos: torch.Tensor) -> torch.Tensor:
    omega = torch.arange(embed_dim // 2, dtype=torch.float64) / (embed_dim / 2.0)
    omega = 1.0 / 10000.0 ** omega
    out = pos.reshape(-1).double()[:, None] * omega[None]
    return torch.cat([out.sin(), out.cos()], dim=1)


def sincos_pos_embed_2d(embed_dim: int, grid_size: int, base_size: int, interpolation_scale: float = 1.0) -> torch.Tensor:
    """[grid_size^2, embed_dim] fp32 table; positions scaled by base_size / grid_size."""
    coord = torch.arange(grid_size, dtype=torch.float64) / (grid_size / base_size) / interpolation_scale
    gw, gh = torch.meshgrid(coord, coord, indexing="xy")  # gw varies along the row (w first)
    emb_a = _sincos_1d(embed_dim // 2, gw)
    emb_b = _sincos_1d(embed_dim // 2, gh)
    return torch.cat([emb_a, emb_b], dim=1).float()


def cropped_pos_embed(table: torch.Tensor, max_size: int, height: int, width: int) -> torch.Tensor:
    """Centre crop of the [max_size^2, D] table to [height*width, D]."""
    top, left = (max_size - height) // 2, (max_size - width) // 2
    t = table.reshape(max_size, max_size, -1)[top : top + height, left : left + width]
    return t.reshape(height * width, -1)


def timestep_embedding(t: torch.Tensor, dim: int, max_period: float = 10000.0) -> torch.Tensor:
    half = dim // 2
    freq = torch.exp(-math.log(max_period) * torch.arange(half, dtype=torch.float32) / half)
    arg = t.float()[:, None] * freq[None]
    return torch.cat([arg.cos(), arg.sin()], dim=1)


def combined_timestep_text_embed(p: P, prefix: str, timestep: torch.Tensor, pooled: torch.Tensor, freq_dim: int = 256) -> torch.Tensor:
    """temb = linear_2(silu(linear_1(sincos(t)))) + linear_2(silu(linear_1(pooled)))."""
    tp = timestep_embedding(timestep, freq_dim)
    te = O.linear(O.silu(O.linear(tp, p[prefix + "timestep_embedder.linear_1.weight"], p[prefix + "timestep_embedder.linear_1.bias"])),
                  p[prefix + "timestep_embedder.linear_2.weight"], p[prefix + "timestep_embedder.linear_2.bias"])
    pe = O.linear(O.silu(O.linear(pooled.float(), p[prefix + "text_embedder.linear_1.weight"], p[prefix + "text_embedder.linear_1.bias"])),
                  p[prefix + "text_embedder.linear_2.weight"], p[prefix + "text_embedder.linear_2.bias"])
    return te + pe


def norm_out_proj(p: P, hidden: torch.Tensor, temb: torch.Tensor) -> torch.Tensor:
    """AdaLayerNormContinuous (scale first) then proj_out."""
    scale, shift = O.adaln_modulation(temb, p["norm_out.linear.weight"], p["norm_out.linear.bias"], 2)
    x = O.modulate(O.layer_norm(hidden, 1e-6), shift, scale)
    return O.linear(x, p["proj_out.weight"], p["proj_out.bias"])


def unpatchify(x: torch.Tensor, channels: int, height: int, width: int, patch: int) -> torch.Tensor:
    """transformer_sd3.py:160-182: [B, h*w, p*p*C] -> [B, C, h*p, w*p]."""
    B = x.shape[0]
    h, w = height // patch, width // patch
    x = x.reshape(B, h, w, patch, patch, channels)
    x = torch.einsum("nhwpqc->nchpwq", x)
    return x.reshape(B, channels, h * patch, w * patch)


def cfg_euler_step(noise_uncond: torch.Tensor, noise_cond: torch.Tensor, sample: torch.Tensor, guidance: float,
                   sigma: float, sigma_next: float) -> torch.Tensor:
    """The reference's expressions on bf16 tensors (each tensor operation rounds to bf16; the scheduler works
    in fp32 with 0-dim fp32 sigmas)."""
    u, c, x = noise_uncond.bfloat16(), noise_cond.bfloat16(), sample.bfloat16()
    noise = u + guidance * (c - u)
    sig, sig_next = torch.tensor(sigma, dtype=torch.float32), torch.tensor(sigma_next, dtype=torch.float32)
    x32 = x.to(torch.float32)
    denoised = x32 - noise * sig
    derivative = (x32 - denoised) / sig
    prev = x32 + derivative * (sig_next - sig)
    return prev.to(torch.bfloat16)


def sd3_transformer(p: P, latent: torch.Tensor, encoder: torch.Tensor, pooled: torch.Tensor, timestep: torch.Tensor,
                    heads: int, layers: int, patch: int, pos_embed_max_size: int) -> torch.Tensor:
    """transformer_sd3.py:92-185 outside patch mode: latent [B, C, H, W] -> predicted noise [B, C_out, H, W].
    ``p`` uses the unwrapped parameter names (``pos_embed.proj.weight``, ``pos_embed.pos_embed`` [1, max^2, D],
    ``time_text_embed.*``, ``context_embedder.*``, ``transformer_blocks.N.*``, ``norm_out.linear.*``, ``proj_out.*``)."""
    from . import blocks as BL

    B, _, H, W = latent.shape
    pos = cropped_pos_embed(p["pos_embed.pos_embed"][0], pos_embed_max_size, H // patch, W // patch)
    hidden = patch_embed(latent, p["pos_embed.proj.weight"], p["pos_embed.proj.bias"], pos)
    temb = combined_timestep_text_embed(p, "time_text_embed.", timestep, pooled)
    enc = O.linear(encoder.float(), p["context_embedder.weight"], p["context_embedder.bias"])
    for i in range(layers):
        pre = f"transformer_blocks.{i}."
        bp = {k[len(pre):]: v for k, v in p.items() if k.startswith(pre)}
        enc, hidden = BL.sd3_joint_block(bp, hidden, enc, temb, heads, context_pre_only=(i == layers - 1))
    out = norm_out_proj(p, hidden, temb)
    channels = p["proj_out.weight"].shape[0] // (patch * patch)
    return unpatchify(out, channels, H, W, patch)


def flux_conditioning(p: P, prefix: str, timestep: torch.Tensor, pooled: torch.Tensor, guidance: Optional[torch.Tensor],
                      freq_dim: int = 256) -> torch.Tensor:
    """transformer_flux.py:104-112: the timestep (and guidance) is scaled by 1000 in the model's dtype (bf16)
    before the sinusoidal projection; the embedders' outputs are summed."""
    def embed(name, x):
        return O.linear(O.silu(O.linear(x, p[f"{prefix}{name}.linear_1.weight"], p[f"{prefix}{name}.linear_1.bias"])),
                        p[f"{prefix}{name}.linear_2.weight"], p[f"{prefix}{name}.linear_2.bias"])

    t = (timestep.to(torch.bfloat16) * 1000).float()
    out = embed("timestep_embedder", timestep_embedding(t, freq_dim))
    if guidance is not None:
        g = (guidance.to(torch.bfloat16) * 1000).float()
        out = out + embed("guidance_embedder", timestep_embedding(g, freq_dim))
    return out + embed("text_embedder", pooled.float())


def flux_transformer(p: P, hidden: torch.Tensor, encoder: torch.Tensor, pooled: torch.Tensor, timestep: torch.Tensor,
                     img_ids: torch.Tensor, txt_ids: torch.Tensor, guidance: Optional[torch.Tensor], heads: int, layers: int,
                     single_layers: int, axes_dim=(16, 56, 56)) -> torch.Tensor:
    """transformer_flux.py:101-207 on one stage: packed latent [B, N_img, C] -> [B, N_img, C]."""
    from . import blocks as BL

    def sub(prefix):
        return {k[len(prefix):]: v for k, v in p.items() if k.startswith(prefix)}

    x = O.linear(hidden.float(), p["x_embedder.weight"], p["x_embedder.bias"])
    temb = flux_conditioning(p, "time_text_embed.", timestep, pooled, guidance)
    enc = O.linear(encoder.float(), p["context_embedder.weight"], p["context_embedder.bias"])
    rope = O.flux_rope_table(torch.cat([txt_ids, img_ids], 0), axes_dim)
    for i in range(layers):
        enc, x = BL.flux_double_block(sub(f"transformer_blocks.{i}."), x, enc, temb, rope, heads)
    n_txt = enc.shape[1]
    joint = torch.cat([enc, x], dim=1)
    for i in range(single_layers):
        joint = BL.flux_single_block(sub(f"single_transformer_blocks.{i}."), joint, temb, rope, heads, n_text=n_txt)
    return norm_out_proj(p, joint[:, n_txt:], temb)


def flow_match_sigmas(num_inference_steps: int, shift: float = 3.0, num_train_timesteps: int = 1000) -> torch.Tensor:
    """diffusers ``FlowMatchEulerDiscreteScheduler.set_timesteps`` (static shift): t evenly spaced from sigma_max
    to sigma_min of the shifted training schedule, shifted again, with a final 0.  fp32 [steps + 1]."""
    def sh(s):
        return shift * s / (1 + (shift - 1) * s)

    s_max, s_min = sh(1.0), float(torch.tensor(sh(1.0 / num_train_timesteps), dtype=torch.float32))
    t = torch.linspace(s_max, s_min, num_inference_steps, dtype=torch.float64)
    return torch.cat([sh(t).float(), torch.zeros(1)])


def cogvideox_patch_embed(p: P, prefix: str, text: torch.Tensor, video: torch.Tensor) -> torch.Tensor:
    """layers/embeddings.py:126-165 (2-D patches, no position table): text [B, N_t, E], video [B, F, C, H, W] ->
    [B, N_t + F (H/p)(W/p), D], text rows first."""
    B, F, C, H, W = video.shape
    w, b = p[prefix + "proj.weight"], p[prefix + "proj.bias"]
    img = patch_embed(video.reshape(B * F, C, H, W), w, b, None)          # [B F, h w, D]
    img = img.reshape(B, F * img.shape[1], -1)
    txt = O.linear(text.float(), p[prefix + "text_proj.weight"], p[prefix + "text_proj.bias"])
    return torch.cat([txt, img], dim=1)


def ada_layer_norm(p: P, prefix: str, x: torch.Tensor, temb: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """diffusers ``AdaLayerNorm`` with ``chunk_dim=1``: (shift, scale) = linear(silu(temb)).chunk(2); affine
    LayerNorm, then * (1 + scale) + shift."""
    shift, scale = O.adaln_modulation(temb, p[prefix + "linear.weight"], p[prefix + "linear.bias"], 2)
    n = O.layer_norm(x, eps, p[prefix + "norm.weight"], p[prefix + "norm.bias"])
    return O.modulate(n, shift, scale)


def unpatchify_channel_major(x: torch.Tensor, frames: int, channels: int, height: int, width: int, patch: int) -> torch.Tensor:
    """cogvideox_transformer_3d.py:143-146: [B, F h w, C p p] -> [B, F, C, H, W]."""
    B = x.shape[0]
    out = x.reshape(B, frames, height // patch, width // patch, channels, patch, patch)
    return out.permute(0, 1, 4, 2, 5, 3, 6).flatten(5, 6).flatten(3, 4)


def cogvideox_transformer(p: P, video: torch.Tensor, text: torch.Tensor, timestep: torch.Tensor, rope, heads: int,
                          layers: int, patch: int) -> torch.Tensor:
    """cogvideox_transformer_3d.py:72-160 for the rotary-embedding model: [B, F, C, H, W] -> [B, F, C_out, H, W]."""
    from . import blocks as BL

    B, F, _, H, W = video.shape
    D = p["patch_embed.proj.weight"].shape[0]
    t_emb = timestep_embedding(timestep, D)
    emb = O.linear(O.silu(O.linear(t_emb, p["time_embedding.linear_1.weight"], p["time_embedding.linear_1.bias"])),
                   p["time_embedding.linear_2.weight"], p["time_embedding.linear_2.bias"])
    joint = cogvideox_patch_embed(p, "patch_embed.", text, video)
    n_txt = text.shape[1]
    enc, hid = joint[:, :n_txt], joint[:, n_txt:]
    for i in range(layers):
        pre = f"transformer_blocks.{i}."
        bp = {k[len(pre):]: v for k, v in p.items() if k.startswith(pre)}
        hid, enc = BL.cogvideox_block(bp, hid, enc, emb, rope, heads)
    joint = O.layer_norm(torch.cat([enc, hid], dim=1), 1e-5, p["norm_final.weight"], p["norm_final.bias"])
    hid = ada_layer_norm(p, "norm_out.", joint[:, n_txt:], emb)
    out = O.linear(hid, p["proj_out.weight"], p["proj_out.bias"])
    channels = p["proj_out.weight"].shape[0] // (patch * patch)
    return unpatchify_channel_major(out, F, channels, H, W, patch)
