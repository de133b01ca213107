"""Layer-wrapper base: holds the original layer as ``self.module`` (so parameter
paths gain a ``.module.`` hop), an ``activation_cache`` slot, and falls through
to the wrapped module for unknown attributes -- the contract of
``layers/base_layer.py:10-40`` in the reference."""
from abc import ABCMeta, abstractmethod

import torch.nn as nn

from .._lib import eager_only


class hetuDiTDiffusionLayerBaseWrapper(nn.Module, metaclass=ABCMeta):
    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        if "forward" in cls.__dict__ and not getattr(cls.__dict__["forward"], "__isabstractmethod__", False):
            cls.forward = eager_only(cls.__dict__["forward"])  # the wrappers launch kernels through ctypes

    def __init__(self, module: nn.Module):
        super().__init__()
        self.module = module
        self.activation_cache = None

    def __getattr__(self, name: str):
        d = self.__dict__
        for store in ("_parameters", "_buffers", "_modules"):
            if store in d and name in d[store]:
                return d[store][name]
        try:
            return getattr(d["_modules"]["module"], name)
        except (KeyError, RecursionError):
            raise AttributeError(f"{type(self).__name__} has no attribute {name}")

    @abstractmethod
    def forward(self, *args, **kwargs):
        pass
