"""Patch state the hot path consults: the fields of the reference's
``DiTRuntimeState`` (``hetu_dit/core/distributed/runtime_state.py:97-111``)
that attention processors, the KV cache and the transformer block loop read,
with the same names, plus the patch-metadata arithmetic of
``_calc_patches_metadata`` (``:333-446``) for one sequence-parallel rank."""
from typing import List, Optional


class InputConfig:
    """The request geometry the reference keeps on its runtime state
    (``runtime_state.py:50-58,:305-321``): image height / width in pixels (0 = not set)."""

    def __init__(self):
        self.height: int = 0
        self.width: int = 0
        self.batch_size: int = 1
        self.num_frames: int = 0


class DiTRuntimeState:
    def __init__(self):
        # pixels; latent rows of the whole image = input_config.height // vae_scale_factor
        # (runtime_state.py:340-342, read by the patch-embedding wrapper at layers/embeddings.py:33-36)
        self.input_config = InputConfig()
        self.vae_scale_factor: int = 8
        self.patch_mode: bool = False
        self.pipeline_patch_idx: int = 0
        self.num_pipeline_patch: int = 1
        self.pp_patches_height: List[int] = []
        self.pp_patches_start_idx_local: List[int] = [0]
        self.pp_patches_token_start_idx_local: List[int] = [0]
        self.pp_patches_token_num: List[int] = []
        # [start, end) token range of every pipeline patch within the whole image (runtime_state.py:106); with one
        # sequence-parallel rank the global ranges are the local ones
        self.pp_patches_token_start_end_idx_global: List[List[int]] = []
        # latent rows of the whole image when no pixel geometry was given (set_patches / set_token_patches); 0 = unknown
        self.latents_height: int = 0
        self.max_condition_sequence_length: int = 0
        # forced False by the reference (runtime_state.py:188,:225)
        self.split_text_embed_in_sp: bool = False

    def set_input_parameters(self, height: Optional[int] = None, width: Optional[int] = None,
                             batch_size: Optional[int] = None, vae_scale_factor: Optional[int] = None):
        """Pixel geometry of the request (``runtime_state.py:296-309``)."""
        self.input_config.height = height or self.input_config.height
        self.input_config.width = width or self.input_config.width
        self.input_config.batch_size = batch_size or self.input_config.batch_size
        if vae_scale_factor:
            self.vae_scale_factor = vae_scale_factor

    def whole_image_latent_rows(self) -> int:
        """Latent rows of the whole image: ``input_config.height // vae_scale_factor`` as the reference's
        patch-embedding wrapper computes it, else what ``set_patches`` recorded; 0 if neither is known."""
        if self.input_config.height:
            return self.input_config.height // self.vae_scale_factor
        return self.latents_height

    # -- runtime_state.py:254-264 -------------------------------------------
    def set_patched_mode(self, patch_mode: bool):
        self.patch_mode = patch_mode
        self.pipeline_patch_idx = 0

    def next_patch(self):
        if self.patch_mode:
            self.pipeline_patch_idx += 1
            if self.pipeline_patch_idx == self.num_pipeline_patch:
                self.pipeline_patch_idx = 0
        else:
            self.pipeline_patch_idx = 0

    # -- runtime_state.py:333-446 at sequence-parallel degree 1 ---------------
    def set_patches(self, latents_height: int, latents_width: int, patch_size: int, num_pipeline_patch: int):
        """Split the latent rows into pipeline patches the way the reference
        does: equal heights rounded up to a multiple of ``patch_size``, the
        last patch takes the remainder; token ranges follow from the width."""
        want = num_pipeline_patch
        h = (latents_height + want - 1) // want
        h = (h + patch_size - 1) // patch_size * patch_size
        n = (latents_height + h - 1) // h
        heights = [h] * (n - 1)
        last = latents_height - h * (n - 1)
        if last % patch_size != 0:
            raise ValueError(
                f"The height of the last pipeline patch is {last}, which is not a multiple of patch_size {patch_size}"
            )
        heights.append(last)
        starts = [0]
        for x in heights:
            starts.append(starts[-1] + x)
        per_row = latents_width // patch_size
        tok = [per_row * (s // patch_size) for s in starts]
        self.num_pipeline_patch = n
        self.pp_patches_height = heights
        self.pp_patches_start_idx_local = starts
        self.pp_patches_token_start_idx_local = tok
        self.pp_patches_token_num = [tok[i + 1] - tok[i] for i in range(n)]
        self.pp_patches_token_start_end_idx_global = [[tok[i], tok[i + 1]] for i in range(n)]
        self.latents_height = latents_height
        self.pipeline_patch_idx = 0

    def set_token_patches(self, token_starts: List[int]):
        """Set the token ranges directly (a shard benchmark has no latent grid)."""
        self.num_pipeline_patch = len(token_starts) - 1
        self.pp_patches_token_start_idx_local = list(token_starts)
        self.pp_patches_token_num = [token_starts[i + 1] - token_starts[i] for i in range(self.num_pipeline_patch)]
        self.pp_patches_token_start_end_idx_global = [
            [token_starts[i], token_starts[i + 1]] for i in range(self.num_pipeline_patch)
        ]
        self.latents_height = 0
        self.pipeline_patch_idx = 0


_RUNTIME: Optional[DiTRuntimeState] = DiTRuntimeState()


def get_runtime_state() -> DiTRuntimeState:
    assert _RUNTIME is not None, "Runtime state has not been initialized."
    return _RUNTIME


def runtime_state_is_initialized() -> bool:
    return _RUNTIME is not None


def reset_runtime_state() -> DiTRuntimeState:
    global _RUNTIME
    _RUNTIME = DiTRuntimeState()
    return _RUNTIME
