"""Patch-embedding wrapper with the interface of the reference's ``layers/embeddings.py:20-112``
(``hetuDiTPatchEmbedWrapper``): projects the latent, adds the (cropped) position table, and in patch mode
adds only the rows of the table that belong to the current pipeline patch.

The p x p, stride-p convolution is a GEMM over the im2col rows (``hdit_patchify``); the position rows ride
the GEMM's residual epilogue, so tokens leave the matrix core already position-encoded."""
import torch

from .. import ops
from ..registry import hetuDiTLayerWrappersRegister
from ..runtime_state import get_runtime_state
from .base_layer import hetuDiTDiffusionLayerBaseWrapper
from .modules import PatchEmbed


@hetuDiTLayerWrappersRegister.register(PatchEmbed)
class hetuDiTPatchEmbedWrapper(hetuDiTDiffusionLayerBaseWrapper):
    def __init__(self, patch_embedding: PatchEmbed):
        super().__init__(module=patch_embedding)
        self._pos_cache = {}
        self._ones = None

    def _pos_rows(self, height: int, width: int, start: int, end: int, device) -> torch.Tensor:
        """bf16 rows [start, end) of the table cropped for a latent of height x width pixels."""
        key = (height, width, start, end, self.module.pos_embed.data_ptr())
        rows = self._pos_cache.get(key)
        if rows is None:
            table = self.module.cropped_pos_embed(height, width)[0]
            if end > table.shape[0]:
                raise ValueError(f"pipeline patch ends at token {end} but the position table has {table.shape[0]} rows")
            rows = table[start:end].to(device=device, dtype=torch.bfloat16).contiguous()
            if len(self._pos_cache) >= 16:
                self._pos_cache.clear()
            self._pos_cache[key] = rows
        return rows

    @torch.no_grad()
    def forward(self, latent: torch.Tensor) -> torch.Tensor:
        m = self.module
        rs = get_runtime_state()
        p = m.patch_size
        B, C, H, W = latent.shape
        D = m.proj.weight.shape[0]
        x = ops.patchify(latent.contiguous(), p)  # [B, T, C p p]
        T = x.shape[1]
        w2 = m.proj.weight.data.reshape(D, C * p * p)
        bias = m.proj.bias.data if m.proj.bias is not None else None
        out = torch.empty(B, T, D, dtype=torch.bfloat16, device=latent.device)
        if m.pos_embed is None:
            ops.gemm_launch([ops.gemm_problem(x.view(-1, C * p * p), w2, out.view(-1, D), bias)])
            return out
        if rs.patch_mode:
            # the latent holds the rows of the current pipeline patch; the table is that of the whole image
            height = rs.whole_image_latent_rows()
            if not height:
                raise ValueError("patch mode needs the height of the whole image: input_config.height and "
                                 "vae_scale_factor on the runtime state (set_input_parameters), or set_patches")
            start, end = rs.pp_patches_token_start_end_idx_global[rs.pipeline_patch_idx]
        else:
            height, start, end = H, 0, T
        if end - start != T:
            raise ValueError(f"latent has {T} tokens but the pipeline patch covers {end - start}")
        pos = self._pos_rows(height, W, start, end, latent.device)
        if self._ones is None or self._ones.device != latent.device or self._ones.shape[1] != D:
            self._ones = torch.ones(1, D, dtype=torch.float32, device=latent.device)
        problems = [
            ops.gemm_problem(x[b], w2, out[b], bias, ops.EPI_GATE_RESIDUAL, resid=pos, gate=self._ones, rows_per_batch=T)
            for b in range(B)
        ]
        ops.gemm_launch(problems)
        return out


def project(x2: torch.Tensor, lin, **epilogue) -> torch.Tensor:
    """bf16 [m, k] -> [m, n] through one launch of the grouped GEMM (bias in the epilogue)."""
    out = torch.empty(x2.shape[0], lin.weight.shape[0], dtype=torch.bfloat16, device=x2.device)
    ops.gemm_launch([ops.gemm_problem(x2, lin.weight.data, out, lin.bias.data, **epilogue)])
    return out


def conditioning_embedding(tte, timestep: torch.Tensor, pooled_projection: torch.Tensor, guidance=None) -> torch.Tensor:
    """bf16 [B, D] conditioning vector of ``CombinedTimestepTextProjEmbeddings`` /
    ``CombinedTimestepGuidanceTextProjEmbeddings`` (called at ``transformer_sd3.py:101`` and
    ``transformer_flux.py:108-112``): each embedder is linear -> SiLU -> linear; the sum of the embedders
    rides the residual epilogue of the second linears."""
    B = timestep.shape[0]
    D = tte.timestep_embedder.linear_2.weight.shape[0]
    ones = getattr(tte, "_unit_gate", None)
    if ones is None or ones.device != timestep.device:
        ones = torch.ones(1, D, dtype=torch.float32, device=timestep.device)
        object.__setattr__(tte, "_unit_gate", ones)
    acc = None

    def add(embedder_in: torch.Tensor, lin1, lin2):
        nonlocal acc
        h = ops.silu(project(embedder_in, lin1))
        if acc is None:
            acc = project(h, lin2)
        else:
            acc = project(h, lin2, epilogue=ops.EPI_GATE_RESIDUAL, resid=acc, gate=ones, rows_per_batch=B)

    add(ops.timestep_embedding(timestep.to(torch.float32), tte.frequency_dim), tte.timestep_embedder.linear_1,
        tte.timestep_embedder.linear_2)
    if guidance is not None:
        add(ops.timestep_embedding(guidance.to(torch.float32), tte.frequency_dim), tte.guidance_embedder.linear_1,
            tte.guidance_embedder.linear_2)
    add(pooled_projection.contiguous(), tte.text_embedder.linear_1, tte.text_embedder.linear_2)
    return acc


def norm_out_project(norm_out, proj_out, hidden_states: torch.Tensor, temb: torch.Tensor) -> torch.Tensor:
    """``proj_out(norm_out(hidden_states, temb))`` (``transformer_sd3.py:156-157``, ``transformer_flux.py:203-205``):
    AdaLayerNormContinuous (chunk order scale, shift) fused into one normalise-and-modulate pass, then a GEMM."""
    from ..blocks import _adaln

    scale, shift = _adaln(norm_out, temb)
    x = ops.layernorm_modulate(hidden_states, shift, scale, norm_out.norm.eps)
    B, T, D = x.shape
    return project(x.view(-1, D), proj_out).view(B, T, -1)


from .modules import CogVideoXPatchEmbed  # noqa: E402


@hetuDiTLayerWrappersRegister.register(CogVideoXPatchEmbed)
class hetuDiTCogVideoXPatchEmbedWrapper(hetuDiTDiffusionLayerBaseWrapper):
    """``layers/embeddings.py:115-232`` of the reference for the rotary-embedding models (CogVideoX-5B): text
    projection and per-frame patch convolution written side by side into one joint [text, video] sequence --
    all projections of all batch elements in one grouped-GEMM launch, no ``cat``."""

    def __init__(self, patch_embedding: CogVideoXPatchEmbed):
        super().__init__(module=patch_embedding)

    @torch.no_grad()
    def forward(self, text_embeds: torch.Tensor, image_embeds: torch.Tensor) -> torch.Tensor:
        m = self.module
        if m.patch_size_t is not None or m.use_positional_embeddings or m.use_learned_positional_embeddings:
            raise NotImplementedError("only the CogVideoX-5B patch embedding (2-D patches, rotary positions) is built")
        B, F, C, H, W = image_embeds.shape
        p = m.patch_size
        D = m.proj.weight.shape[0]
        n_txt = text_embeds.shape[1]
        x = ops.patchify(image_embeds.contiguous().view(B * F, C, H, W), p)  # [B F, h w, C p p]
        n_img = F * x.shape[1]
        x = x.view(B, n_img, C * p * p)
        w2 = m.proj.weight.data.reshape(D, C * p * p)
        bias = m.proj.bias.data if m.proj.bias is not None else None
        text = text_embeds.contiguous()
        out = torch.empty(B, n_txt + n_img, D, dtype=torch.bfloat16, device=image_embeds.device)
        problems = []
        for b in range(B):
            problems.append(ops.gemm_problem(text[b], m.text_proj.weight.data, out[b, :n_txt], m.text_proj.bias.data))
            problems.append(ops.gemm_problem(x[b], w2, out[b, n_txt:], bias))
        ops.gemm_launch(problems)
        return out
