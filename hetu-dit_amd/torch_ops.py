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
