"""Conv2d wrapper with the interface of the reference's ``layers/conv.py:19-113`` (``hetuDiTConv2dWrapper``):
registered for ``nn.Conv2d``, keyword ``is_first_layer``, ``naive_forward`` on one GPU.  The reference's model
wrappers list ``nn.Conv2d`` among the classes to wrap (``models/transformers/transformer_sd3.py:36``), and the
walk reaches the patch embedding's ``proj`` through the already wrapped ``PatchEmbed``
(``models/base_model.py:72-104``), so this wrapper has to exist for that class list to be usable unchanged.

The only convolution on the denoise path is the patch embedding's p x p, stride-p, unpadded one.  It is run as
im2col rows (``hdit_patchify``) times the flattened weight through the grouped GEMM, bias in the epilogue; the
result is returned as a ``[B, C_out, H/p, W/p]`` view of the token-major GEMM output.  Any other geometry raises
``NotImplementedError``: no library convolution stands behind this wrapper.  The sliced (multi-GPU patch) path of
the reference (``conv.py:39-66,:79-110``) is only reached with pipeline or sequence parallelism above one and
raises as the reference's own ``else`` branch does."""
import torch
from torch import nn

from .. import ops
from ..parallel_state import get_pipeline_parallel_world_size, get_sequence_parallel_world_size
from ..registry import hetuDiTLayerWrappersRegister
from .base_layer import hetuDiTDiffusionLayerBaseWrapper


def _pair(v):
    return tuple(v) if isinstance(v, (tuple, list)) else (v, v)


@hetuDiTLayerWrappersRegister.register(nn.Conv2d)
class hetuDiTConv2dWrapper(hetuDiTDiffusionLayerBaseWrapper):
    def __init__(self, conv2d: nn.Conv2d, *, is_first_layer: bool = True):
        super().__init__(module=conv2d)
        self.is_first_layer = is_first_layer

    def _patch_size(self) -> int:
        m = self.module
        k, s, p, d = _pair(m.kernel_size), _pair(m.stride), _pair(m.padding), _pair(m.dilation)
        if k[0] != k[1] or k != s or p != (0, 0) or d != (1, 1) or m.groups != 1 or isinstance(m.padding, str):
            raise NotImplementedError(
                "hetuDiTConv2dWrapper runs square kernel = stride, unpadded, ungrouped convolutions (the patch "
                f"embedding); got kernel {k}, stride {s}, padding {m.padding}, dilation {d}, groups {m.groups}")
        return k[0]

    @torch.no_grad()
    def naive_forward(self, x: torch.Tensor) -> torch.Tensor:
        """x bf16 [B, C, H, W] -> bf16 [B, C_out, H/p, W/p] (a view of the token-major GEMM result)."""
        m = self.module
        p = self._patch_size()
        B, C, H, W = x.shape
        if H % p or W % p:
            raise ValueError(f"input {H}x{W} is not a multiple of the kernel size {p}")
        D = m.weight.shape[0]
        if (C * p * p) % 64 or D % 8:
            raise NotImplementedError(f"the GEMM behind this wrapper needs in_channels * p * p ({C * p * p}) to be a "
                                      f"multiple of 64 and out_channels ({D}) a multiple of 8")
        rows = ops.patchify(x.contiguous(), p)  # [B, T, C p p]
        out = torch.empty(B, rows.shape[1], D, dtype=torch.bfloat16, device=x.device)
        bias = m.bias.data if m.bias is not None else None
        ops.gemm_launch([ops.gemm_problem(rows.view(-1, C * p * p), m.weight.data.reshape(D, C * p * p),
                                          out.view(-1, D), bias)])
        return out.view(B, H // p, W // p, D).permute(0, 3, 1, 2)

    def sliced_forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError("the sliced patch convolution needs pipeline or sequence parallelism above one")

    def forward(self, x: torch.Tensor, *args, **kwargs) -> torch.Tensor:
        one_gpu = get_pipeline_parallel_world_size() == 1 and get_sequence_parallel_world_size() == 1
        if one_gpu or _pair(self.module.kernel_size) == (1, 1):
            return self.naive_forward(x)
        if not self.is_first_layer:
            raise NotImplementedError
        return self.sliced_forward(x)
