"""Decorator registries mapping an original layer / attention-processor /
transformer class to its hetuDiT replacement, with the lookup rules of
``hetu_dit/model_executor/utils/register_warpper.py:10-112``: the most specific
registered base class wins for layers and transformers; processors are matched
by ``isinstance`` and must subclass the class they replace; an unknown class
raises ``ValueError``."""
from typing import Dict, Type

import torch.nn as nn


class hetuDiTLayerWrappersRegister:
    _HETUDIT_LAYER_MAPPING: Dict = {}

    @classmethod
    def register(cls, origin_layer_class: Type[nn.Module]):
        def decorator(wrapper_class):
            cls._HETUDIT_LAYER_MAPPING[origin_layer_class] = wrapper_class
            return wrapper_class

        return decorator

    @classmethod
    def get_wrapper(cls, layer: nn.Module):
        best, best_origin = None, None
        for origin, wrapper in cls._HETUDIT_LAYER_MAPPING.items():
            if isinstance(layer, origin):
                if best is None or origin == layer.__class__ or issubclass(origin, best_origin):
                    best, best_origin = wrapper, origin
        if best is None:
            raise ValueError(f"Layer class {layer.__class__.__name__} is not supported by hetuDiT")
        return best


class hetuDiTAttentionProcessorRegister:
    _HETUDIT_ATTENTION_PROCESSOR_MAPPING: Dict = {}

    @classmethod
    def register(cls, origin_processor_class):
        def decorator(processor_class):
            if not issubclass(processor_class, origin_processor_class):
                raise ValueError(
                    f"{processor_class.__name__} is not a subclass of origin class {origin_processor_class.__name__}"
                )
            cls._HETUDIT_ATTENTION_PROCESSOR_MAPPING[origin_processor_class] = processor_class
            return processor_class

        return decorator

    @classmethod
    def get_processor(cls, processor):
        for origin, replacement in cls._HETUDIT_ATTENTION_PROCESSOR_MAPPING.items():
            if isinstance(processor, origin):
                return replacement
        raise ValueError(f"Attention Processor class {processor.__class__.__name__} is not supported by hetuDiT")


class hetuDiTTransformerWrappersRegister:
    _HETUDIT_TRANSFORMER_MAPPING: Dict = {}

    @classmethod
    def register(cls, origin_transformer_class: Type[nn.Module]):
        def decorator(wrapper_class: Type[nn.Module]):
            cls._HETUDIT_TRANSFORMER_MAPPING[origin_transformer_class] = wrapper_class
            return wrapper_class

        return decorator

    @classmethod
    def get_wrapper(cls, transformer: nn.Module):
        best, best_origin = None, None
        for origin, wrapper in cls._HETUDIT_TRANSFORMER_MAPPING.items():
            if isinstance(transformer, origin):
                if best is None or origin == transformer.__class__ or issubclass(origin, best_origin):
                    best, best_origin = wrapper, origin
        if best is None:
            raise ValueError(f"Transformer class {transformer.__class__.__name__} is not supported by hetuDiT")
        return best
