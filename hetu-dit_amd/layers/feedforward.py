"""FeedForward wrapper with the interface of the reference's
``layers/feedforward.py:17-78``: wraps ``net = [activation(proj), Dropout, Linear]``,
slices ``net[0].proj`` rows / ``net[2]`` columns by tensor-parallel rank (the two
halves of a GEGLU projection separately, ``:34-46``), moves ``net[2].bias`` to
``self.output_bias`` (added after the reduce).  With the tanh GELU every model here
uses, ``forward`` is two GEMM launches: bias + GELU-tanh fused into the first
epilogue, the output bias (and optionally the block's gated residual) into the
second.  The other first layers the reference accepts (exact GELU, GEGLU,
LinearActivation) take a bias-only first GEMM and one elementwise launch."""
import torch
from torch import nn

from .. import ops
from ..parallel_state import get_tensor_model_parallel_rank, get_tensor_model_parallel_world_size, get_tp_group
from ..registry import hetuDiTLayerWrappersRegister
from .base_layer import hetuDiTDiffusionLayerBaseWrapper
from .modules import GEGLU, GELU, FeedForward, LinearActivation


@hetuDiTLayerWrappersRegister.register(FeedForward)
class hetuDiTFeedForwardWrapper(hetuDiTDiffusionLayerBaseWrapper):
    def __init__(self, feedforward: FeedForward):
        super().__init__(module=feedforward)
        tp_degree = get_tensor_model_parallel_world_size()
        tp_rank = get_tensor_model_parallel_rank()
        act = self.module.net[0]
        # The first layer is recognised by class or, for diffusers' own instances, by class name: what is used of
        # it is ``proj`` and, for GELU, ``approximate`` (diffusers' default there is "none").
        name = type(act).__name__
        is_gelu = isinstance(act, GELU) or name == "GELU"
        is_geglu = isinstance(act, GEGLU) or name == "GEGLU"
        is_linear_act = isinstance(act, LinearActivation) or name == "LinearActivation"
        if is_gelu or is_linear_act:
            act.proj.weight.data = act.proj.weight.data.chunk(tp_degree, dim=0)[tp_rank]
            if act.proj.bias is not None:
                act.proj.bias.data = act.proj.bias.data.chunk(tp_degree, dim=0)[tp_rank]
        elif is_geglu:
            # value half and gate half are sliced separately and joined again
            act.proj.weight.data = torch.cat([h.chunk(tp_degree, dim=0)[tp_rank] for h in act.proj.weight.data.chunk(2, dim=0)], dim=0)
            if act.proj.bias is not None:
                act.proj.bias.data = torch.cat([h.chunk(tp_degree, dim=0)[tp_rank] for h in act.proj.bias.data.chunk(2, dim=0)], dim=0)
        else:
            raise TypeError(f"activation_fn {type(act)} not supported")
        approximate = getattr(act, "approximate", "none") if is_gelu else None
        if is_gelu and approximate not in ("tanh", "none"):
            raise TypeError(f"GELU(approximate={approximate!r}) is not built")
        if is_linear_act:
            fn = getattr(act, "activation", "silu")
            if not (fn == "silu" or isinstance(fn, nn.SiLU)):
                raise TypeError(f"LinearActivation({fn!r}): only SiLU is built")
        # the activation that follows the first projection: None = tanh GELU, fused into that GEMM's epilogue
        self.activation_kind = (None if approximate == "tanh" else ops.ACT_GELU_ERF if is_gelu else
                                ops.ACT_GEGLU if is_geglu else ops.ACT_SILU)
        self.module.net[2].weight.data = self.module.net[2].weight.chunk(tp_degree, dim=1)[tp_rank]
        self.has_output_bias = False
        if self.module.net[2].bias is not None:
            self.register_parameter("output_bias", nn.Parameter(self.module.net[2].bias.data.clone(), requires_grad=False))
            self.module.net[2].bias = None
            self.has_output_bias = True

    # -- problems, so that both streams of a joint block share launches ---------
    def in_problem(self, x2: torch.Tensor):
        """x2 [rows, D] -> (problem, h [rows, F]) with bias + GELU-tanh epilogue."""
        if self.activation_kind is not None:
            raise TypeError("the blocks fuse the tanh GELU into the first GEMM; other activations go through forward()")
        proj = self.module.net[0].proj
        h = torch.empty(x2.shape[0], proj.weight.shape[0], dtype=torch.bfloat16, device=x2.device)
        bias = proj.bias.data if proj.bias is not None else None
        return ops.gemm_problem(x2, proj.weight.data, h, bias, ops.EPI_BIAS_GELU), h

    def out_problem(self, h: torch.Tensor, out2: torch.Tensor, resid2=None, gate=None, rows_per_batch: int = 0):
        w = self.module.net[2].weight.data
        bias = self.output_bias.data if self.has_output_bias else None
        if resid2 is None:
            return ops.gemm_problem(h, w, out2, bias)
        return ops.gemm_problem(h, w, out2, bias, ops.EPI_GATE_RESIDUAL, resid=resid2, gate=gate,
                                rows_per_batch=rows_per_batch)

    def forward(self, hidden_states: torch.Tensor, *args, **kwargs) -> torch.Tensor:
        x = hidden_states if hidden_states.is_contiguous() else hidden_states.contiguous()
        x2 = x.view(-1, x.shape[-1])
        if self.activation_kind is None:
            p1, h = self.in_problem(x2)
            ops.gemm_launch([p1])
        else:
            proj = self.module.net[0].proj
            h = torch.empty(x2.shape[0], proj.weight.shape[0], dtype=torch.bfloat16, device=x2.device)
            ops.gemm_launch([ops.gemm_problem(x2, proj.weight.data, h, proj.bias.data if proj.bias is not None else None)])
            # exact GELU and SiLU in place; GEGLU into a buffer of half the width
            h = ops.ff_activation(h, self.activation_kind, out=None if self.activation_kind == ops.ACT_GEGLU else h)
        out = torch.empty(*x.shape[:-1], self.module.net[2].weight.shape[0], dtype=torch.bfloat16, device=x.device)
        ops.gemm_launch([self.out_problem(h, out.view(-1, out.shape[-1]))])
        get_tp_group().all_reduce(out)
        return out
