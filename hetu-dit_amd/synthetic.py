"""Seeded synthetic weights and inputs for the benchmark configurations:
every Linear weight and bias ~ N(0, 0.02) (adaLN included, so the gates are
live), norm weights 1 + N(0, 0.02) and norm biases N(0, 0.02), activations and
conditioning ~ N(0, 1).  Values are drawn in fp32 on the CPU from a
``torch.Generator`` and rounded to bf16, so an fp32 checker that upcasts the
same tensors sees exactly the inputs the kernels see."""
import math
from typing import Dict, Tuple

import torch
from torch import nn


def init_module_(module: nn.Module, seed: int, std: float = 0.02) -> nn.Module:
    gen = torch.Generator().manual_seed(seed)
    for name, p in sorted(module.named_parameters(), key=lambda kv: kv[0]):
        if name.endswith("norm_q.weight") or name.endswith("norm_k.weight") or name.endswith("norm.weight") or \
                name.endswith("norm_added_q.weight") or name.endswith("norm_added_k.weight"):
            v = 1.0 + torch.randn(p.shape, generator=gen) * std
        else:
            v = torch.randn(p.shape, generator=gen) * std
        p.data = v.to(torch.bfloat16).to(p.device)
        p.requires_grad_(False)
    return module


def randn_bf16(shape, seed: int, device="cpu") -> torch.Tensor:
    gen = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=gen).to(torch.bfloat16).to(device)


def flux_ids(n_txt: int, height: int, width: int) -> torch.Tensor:
    """[n_txt + height*width, 3] position ids: text rows zero, image (0, row, col)."""
    img = torch.zeros(height, width, 3)
    img[..., 1] = torch.arange(height)[:, None]
    img[..., 2] = torch.arange(width)[None, :]
    return torch.cat([torch.zeros(n_txt, 3), img.reshape(-1, 3)], dim=0)


def rope_table(pos: torch.Tensor, axes_dim, theta: float = 10000.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin f32 [S, sum(axes_dim)] from integer positions [S, len(axes_dim)]:
    per axis angle[p, i] = pos * theta^(-2i/dim) (float64), each repeated for its
    rotation pair, axes concatenated.  This is the table the pipeline hands the
    blocks as ``image_rotary_emb`` (Flux: ``transformer_flux.py:130-131``;
    CogVideoX: ``pipeline_cogvideox.py:303-309``)."""
    cos, sin = [], []
    for a, dim in enumerate(axes_dim):
        i = torch.arange(0, dim, 2, dtype=torch.float64)[: dim // 2]
        ang = pos[:, a].to(torch.float64)[:, None] / (theta ** (i / dim))[None, :]
        cos.append(torch.cos(ang).repeat_interleave(2, dim=1))
        sin.append(torch.sin(ang).repeat_interleave(2, dim=1))
    return torch.cat(cos, dim=-1).float().contiguous(), torch.cat(sin, dim=-1).float().contiguous()


def cogvideox_positions(frames: int, height: int, width: int) -> torch.Tensor:
    t, h, w = torch.meshgrid(torch.arange(frames), torch.arange(height), torch.arange(width), indexing="ij")
    return torch.stack([t, h, w], dim=-1).reshape(-1, 3)


# name -> shape parameters of BASELINE.json's configs
CONFIGS: Dict[str, dict] = {
    "sd3_512": dict(family="sd3", batch=1, n_img=1024, n_txt=333, dim=1536, heads=24, head_dim=64),
    "sd3_1024": dict(family="sd3", batch=2, n_img=4096, n_txt=333, dim=1536, heads=24, head_dim=64, layers=24),
    "flux_1024": dict(family="flux", batch=1, n_img=4096, n_txt=512, dim=3072, heads=24, head_dim=128, grid=(64, 64)),
    "sd3_pipefusion": dict(family="sd3", batch=2, n_img=4096, n_txt=333, dim=1536, heads=24, head_dim=64, layers=24,
                           patches=4),
    "sd3_pipefusion_b1": dict(family="sd3", batch=1, n_img=4096, n_txt=333, dim=1536, heads=24, head_dim=64, layers=24,
                              patches=4),
    "cogvideox_5b": dict(family="cogvideox", batch=1, n_img=17550, n_txt=226, dim=3072, heads=48, head_dim=64,
                         grid=(13, 30, 45), temb_dim=512),
}
