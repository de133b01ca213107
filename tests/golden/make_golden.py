"""Writes the golden vectors under tests/golden/: tiny instances of the four block types, inputs and fp32
oracle outputs, as .npz (plain arrays, loadable with numpy's default allow_pickle=False).

The reference holds no tests or fixtures of its own and cannot be imported (its third-party dependencies
are absent), so these vectors are produced by THIS repository's oracle from seeded inputs; they freeze the
oracle (a later edit that changes its arithmetic fails tests/test_golden.py on the CPU) and give the GPU
path a second, file-based target.  Weights are not stored: they are re-derived from the seed with
hetu_dit_amd.synthetic.init_module_, and a checksum of them is stored instead.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from hetu_dit_amd import blocks, synthetic  # noqa: E402
from hetu_dit_amd.cache_manager import reset_cache_manager  # noqa: E402
from tests.util import oracle_params  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    "sd3_joint": dict(cls="JointTransformerBlock", args=(128, 2, 64), kw={}, seed=101, B=2, N=48, Nt=13),
    "sd3_joint_pre_only": dict(cls="JointTransformerBlock", args=(128, 2, 64), kw={"context_pre_only": True}, seed=102,
                               B=1, N=40, Nt=9),
    "flux_double": dict(cls="FluxTransformerBlock", args=(256, 2, 128), kw={}, seed=103, B=1, grid=(5, 8), Nt=7),
    "flux_single": dict(cls="FluxSingleTransformerBlock", args=(256, 2, 128), kw={}, seed=104, B=1, grid=(5, 8), Nt=7),
    "cogvideox": dict(cls="CogVideoXBlock", args=(128, 2, 64), kw={"time_embed_dim": 32}, seed=105, B=1,
                      grid=(2, 3, 4), Nt=6),
}


def build(name):
    reset_cache_manager()  # drop entries of earlier blocks; the new block registers its own below
    c = CASES[name]
    blk = getattr(blocks, c["cls"])(*c["args"], **c["kw"])
    synthetic.init_module_(blk, c["seed"])
    params = oracle_params(blk)
    checksum = float(sum(v.double().abs().sum() for v in params.values()))
    D, H = c["args"][0], c["args"][1]
    s = c["seed"] * 10
    out = {"weights_abs_sum": np.float64(checksum)}
    if name.startswith("sd3"):
        x = synthetic.randn_bf16((c["B"], c["N"], D), s + 1).float()
        e = synthetic.randn_bf16((c["B"], c["Nt"], D), s + 2).float()
        t = synthetic.randn_bf16((c["B"], D), s + 3).float()
        enc, hid = oracle.sd3_joint_block(params, x, e, t, H, context_pre_only=c["kw"].get("context_pre_only", False))
        out.update(hidden_states=x, encoder_hidden_states=e, temb=t, out_hidden=hid)
        if enc is not None:
            out["out_encoder"] = enc
    elif name.startswith("flux"):
        gh, gw = c["grid"]
        N = gh * gw
        cos, sin = synthetic.rope_table(synthetic.flux_ids(c["Nt"], gh, gw), (16, 56, 56))
        x = synthetic.randn_bf16((c["B"], N, D), s + 1).float()
        e = synthetic.randn_bf16((c["B"], c["Nt"], D), s + 2).float()
        t = synthetic.randn_bf16((c["B"], D), s + 3).float()
        out.update(cos=cos, sin=sin, temb=t)
        if name == "flux_double":
            enc, hid = oracle.flux_double_block(params, x, e, t, (cos, sin), H)
            out.update(hidden_states=x, encoder_hidden_states=e, out_hidden=hid, out_encoder=enc)
        else:
            joint = torch.cat([e, x], dim=1)
            out.update(hidden_states=joint, n_text=np.int64(c["Nt"]),
                       out_hidden=oracle.flux_single_block(params, joint, t, (cos, sin), H, n_text=c["Nt"]))
    else:
        N = c["grid"][0] * c["grid"][1] * c["grid"][2]
        cos, sin = synthetic.rope_table(synthetic.cogvideox_positions(*c["grid"]), (16, 24, 24))
        x = synthetic.randn_bf16((c["B"], N, D), s + 1).float()
        e = synthetic.randn_bf16((c["B"], c["Nt"], D), s + 2).float()
        t = synthetic.randn_bf16((c["B"], c["kw"]["time_embed_dim"]), s + 3).float()
        hid, enc = oracle.cogvideox_block(params, x, e, t, (cos, sin), H)
        out.update(cos=cos, sin=sin, hidden_states=x, encoder_hidden_states=e, temb=t, out_hidden=hid, out_encoder=enc)
    return blk, params, {k: (v.numpy() if isinstance(v, torch.Tensor) else v) for k, v in out.items()}


STEP_CFG = dict(sample_size=16, patch_size=2, in_channels=16, num_layers=2, attention_head_dim=64, num_attention_heads=2,
                joint_attention_dim=64, caption_projection_dim=128, pooled_projection_dim=64, out_channels=16,
                pos_embed_max_size=12)


def step_params(model):
    """fp32 parameters and buffers of a whole-transformer model under the unwrapped names the oracle uses."""
    out = {}
    for stack in ("transformer_blocks", "single_transformer_blocks"):
        for i, blk in enumerate(getattr(model, stack, [])):
            for k, v in oracle_params(blk).items():
                out[f"{stack}.{i}.{k}"] = v
    for name, p in list(model.named_parameters()) + list(model.named_buffers()):
        if "transformer_blocks." not in name:
            out[name.replace(".module.", ".")] = p.detach().float().cpu()
    return out


def build_step():
    """A tiny SD3 transformer from latent to predicted noise, the guided Euler update and the sigma schedule."""
    from hetu_dit_amd.transformer_sd3 import SD3Transformer2DModel
    from oracle import step as S

    reset_cache_manager()
    model = SD3Transformer2DModel(**STEP_CFG)
    synthetic.init_module_(model, 201)
    params = step_params(model)
    checksum = float(sum(v.double().abs().sum() for k, v in params.items() if not k.endswith("pos_embed.pos_embed")))
    lat = synthetic.randn_bf16((2, 16, 16, 24), 2011).float()
    enc = synthetic.randn_bf16((2, 11, 64), 2012).float()
    pooled = synthetic.randn_bf16((2, 64), 2013).float()
    t = torch.tensor([640.0, 640.0])
    noise = S.sd3_transformer(params, lat, enc, pooled, t, STEP_CFG["num_attention_heads"], STEP_CFG["num_layers"],
                              STEP_CFG["patch_size"], STEP_CFG["pos_embed_max_size"])
    new = S.cfg_euler_step(noise[:1], noise[1:], lat[:1], 7.0, 0.9, 0.8)
    out = dict(weights_abs_sum=np.float64(checksum), latent=lat, encoder_hidden_states=enc, pooled=pooled, timestep=t,
               noise=noise, guided_step=new.float(), sigmas_10=S.flow_match_sigmas(10))
    return model, params, {k: (v.numpy() if isinstance(v, torch.Tensor) else v) for k, v in out.items()}


def main():
    for name in CASES:
        _, _, arrays = build(name)
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **arrays)
        print(f"{path}: {os.path.getsize(path) / 1024:.1f} KiB")
    _, _, arrays = build_step()
    path = os.path.join(HERE, "sd3_step.npz")
    np.savez_compressed(path, **arrays)
    print(f"{path}: {os.path.getsize(path) / 1024:.1f} KiB")


if __name__ == "__main__":
    main()
