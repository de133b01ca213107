"""``torch.ops.hdit.*``: the C-ABI kernels registered with ``torch.library`` (with fake/meta kernels),
for callers that trace or compile the transformer -- the reference optionally wraps
``transformer.forward`` in ``torch.compile`` (``model_executor/pipelines/base_pipeline.py:274-279``).
Each op forwards to the function of the same name in ``ops.py``; there is no other implementation."""
from typing import List, Optional

import torch

from . import ops

_lib_def = torch.library.Library("hdit", "DEF")
_lib_def.define("linear(Tensor x, Tensor weight, Tensor? bias=None, bool gelu=False) -> Tensor")
_lib_def.define("layernorm_modulate(Tensor x, Tensor? shift=None, Tensor? scale=None, float eps=1e-6, "
                "Tensor? ln_weight=None, Tensor? ln_bias=None) -> Tensor")
_lib_def.define("gate_residual(Tensor x, Tensor y, Tensor gate) -> Tensor")
_lib_def.define("adaln_gemv(Tensor temb, Tensor weight, Tensor? bias=None) -> Tensor")
_lib_def.define("gelu_tanh(Tensor x, Tensor? bias=None) -> Tensor")
_lib_def.define("attention(Tensor[] q, Tensor[] k, Tensor[] v, float scale=0.0, bool fp8=False) -> Tensor[]")
_lib_def.define("patchify(Tensor latent, int patch) -> Tensor")
_lib_def.define("unpatchify(Tensor x, int channels, int height, int width, int patch, bool channel_major=False) -> Tensor")
_lib_def.define("timestep_embedding(Tensor timesteps, int dim, float max_period=10000.0) -> Tensor")
_lib_def.define("silu(Tensor x) -> Tensor")
_lib_def.define("rope_table(Tensor positions, int[] axes_dim, float theta=10000.0) -> (Tensor, Tensor)")
_lib_def.define("cfg_euler_step(Tensor noise_uncond, Tensor noise_cond, Tensor sample, float guidance, float sigma, "
                "float sigma_next) -> Tensor")


def _linear(x, weight, bias=None, gelu=False):
    return ops.linear(x, weight, bias, gelu=gelu)


def _layernorm_modulate(x, shift=None, scale=None, eps=1e-6, ln_weight=None, ln_bias=None):
    return ops.layernorm_modulate(x, shift, scale, eps, ln_weight, ln_bias)


def _attention(q, k, v, scale=0.0, fp8=False):
    return ops.attention(list(q), list(k), list(v), scale=scale, fp8=fp8)


_impl = torch.library.Library("hdit", "IMPL", "CUDA")
_impl.impl("linear", _linear)
_impl.impl("layernorm_modulate", _layernorm_modulate)
_impl.impl("gate_residual", lambda x, y, gate: ops.gate_residual(x, y, gate))
_impl.impl("adaln_gemv", lambda temb, weight, bias=None: ops.adaln_gemv(temb, weight, bias))
_impl.impl("gelu_tanh", lambda x, bias=None: ops.gelu_tanh(x, bias))
_impl.impl("attention", _attention)
_impl.impl("patchify", lambda latent, patch: ops.patchify(latent, patch))
_impl.impl("unpatchify", lambda x, channels, height, width, patch, channel_major=False: ops.unpatchify(
    x, channels, height, width, patch, channel_major))
_impl.impl("timestep_embedding", lambda t, dim, max_period=10000.0: ops.timestep_embedding(t, dim, max_period))
_impl.impl("silu", lambda x: ops.silu(x))
_impl.impl("rope_table", lambda positions, axes_dim, theta=10000.0: ops.rope_table(positions, list(axes_dim), theta))
_impl.impl("cfg_euler_step", lambda u, c, x, guidance, sigma, sigma_next: ops.cfg_euler_step(u, c, x, guidance, sigma,
                                                                                          sigma_next))


@torch.library.register_fake("hdit::linear")
def _(x, weight, bias=None, gelu=False):
    return x.new_empty(*x.shape[:-1], weight.shape[0])


@torch.library.register_fake("hdit::layernorm_modulate")
def _(x, shift=None, scale=None, eps=1e-6, ln_weight=None, ln_bias=None):
    return x.new_empty(x.shape)


@torch.library.register_fake("hdit::gate_residual")
def _(x, y, gate):
    return x.new_empty(x.shape)


@torch.library.register_fake("hdit::adaln_gemv")
def _(temb, weight, bias=None):
    return temb.new_empty(temb.shape[0], weight.shape[0], dtype=torch.float32)


@torch.library.register_fake("hdit::gelu_tanh")
def _(x, bias=None):
    return x.new_empty(x.shape)


@torch.library.register_fake("hdit::attention")
def _(q, k, v, scale=0.0, fp8=False):
    return [t.new_empty(t.shape) for t in q]


@torch.library.register_fake("hdit::patchify")
def _(latent, patch):
    B, C, H, W = latent.shape
    return latent.new_empty(B, (H // patch) * (W // patch), C * patch * patch)


@torch.library.register_fake("hdit::unpatchify")
def _(x, channels, height, width, patch, channel_major=False):
    return x.new_empty(x.shape[0], channels, height, width)


@torch.library.register_fake("hdit::timestep_embedding")
def _(timesteps, dim, max_period=10000.0):
    return timesteps.new_empty(timesteps.shape[0], dim, dtype=torch.bfloat16)


@torch.library.register_fake("hdit::silu")
def _(x):
    return x.new_empty(x.shape)


@torch.library.register_fake("hdit::rope_table")
def _(positions, axes_dim, theta=10000.0):
    width = sum(axes_dim)
    return positions.new_empty(positions.shape[0], width), positions.new_empty(positions.shape[0], width)


@torch.library.register_fake("hdit::cfg_euler_step")
def _(noise_uncond, noise_cond, sample, guidance, sigma, sigma_next):
    return sample.new_empty(sample.shape)
