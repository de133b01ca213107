"""Wrapping of a model's layers and registration of their K/V cache entries, with the rules of the
reference's ``hetuDiTBaseWrapper._wrap_layers`` / ``_register_cache``
(``model_executor/diffusion_executor/models/base_model.py:59-112,:162-178``): every child whose *name* is in
``submodule_name_to_wrap`` or whose *class* is in ``submodule_classes_to_wrap`` is replaced by
``hetuDiTLayerWrappersRegister.get_wrapper(child)(child, **submodule_addition_args.get(name, {}))``.  A wrapper
itself is skipped by the walk, but the module it wraps is not: the walk goes on into ``wrapper.module`` and wraps
what matches there too (with the reference's SD3 class list ``[FeedForward, nn.Conv2d, PatchEmbed]`` that is how
``pos_embed.module.proj`` becomes a ``hetuDiTConv2dWrapper``).  Every attention wrapper gets a cache entry
**keyed by the wrapper object** -- the object the attention processors later pass as ``layer=attn``
(``layers/attention_processor.py:702-707``)."""
from typing import Dict, List, Optional, Sequence, Type

from torch import nn

from .cache_manager import get_cache_manager
from .layers import conv as _conv  # noqa: F401  (registers the nn.Conv2d wrapper)
from .layers.base_layer import hetuDiTDiffusionLayerBaseWrapper
from .parallel_state import get_sequence_parallel_world_size
from .registry import hetuDiTLayerWrappersRegister


def wrap_layers(model: nn.Module, submodule_classes_to_wrap: Sequence[Type] = (),
                submodule_name_to_wrap: Sequence[str] = (),
                submodule_addition_args: Optional[Dict[str, Dict]] = None) -> List[nn.Module]:
    """Replace the matching children of ``model`` in place; returns the wrappers (the reference's
    ``self.wrapped_layers``).  A child that already is a wrapper is left as it is."""
    submodule_addition_args = submodule_addition_args or {}
    wrapped = []
    for _, module in list(model.named_modules()):
        if isinstance(module, hetuDiTDiffusionLayerBaseWrapper):
            continue
        for subname, submodule in list(module.named_children()):
            if isinstance(submodule, hetuDiTDiffusionLayerBaseWrapper):
                continue
            need_wrap = subname in submodule_name_to_wrap or any(
                isinstance(submodule, c) for c in submodule_classes_to_wrap)
            if need_wrap:
                wrapper_cls = hetuDiTLayerWrappersRegister.get_wrapper(submodule)
                setattr(module, subname, wrapper_cls(submodule, **submodule_addition_args.get(subname, {})))
                wrapped.append(getattr(module, subname))
    return wrapped


def register_cache(wrapped_layers: Sequence[nn.Module]) -> None:
    """One ``"attn"`` entry per attention wrapper, keyed by the wrapper (``base_model.py:162-178``)."""
    from .layers.attention_processor import hetuDiTAttentionWrapper

    for layer in wrapped_layers:
        if isinstance(layer, hetuDiTAttentionWrapper):
            naive = get_sequence_parallel_world_size() == 1 or not getattr(
                layer.processor, "use_long_ctx_attn_kvcache", False)
            get_cache_manager().register_cache_entry(
                layer, layer_type="attn", cache_type="naive_cache" if naive else "sequence_parallel_attn_cache")


def wrap_layer(layer: nn.Module, **additional_args) -> nn.Module:
    """Both steps for one layer: what a block built already wrapped does for each of its sub-layers."""
    wrapper = hetuDiTLayerWrappersRegister.get_wrapper(layer)(layer, **additional_args)
    register_cache([wrapper])
    return wrapper
