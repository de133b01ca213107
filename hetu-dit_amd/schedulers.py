"""Flow-match Euler scheduler with the interface the reference's pipelines use
(``schedulers/scheduling_flow_match_euler_discrete.py:23-129`` over diffusers'
``FlowMatchEulerDiscreteScheduler``): ``set_timesteps``, ``timesteps``, ``sigmas``, ``step_index``, ``step``.
The update itself is one kernel (``hdit_cfg_euler_step``), optionally fused with classifier-free guidance; the
step index only advances after the last pipeline patch of a step, as in the reference."""
from typing import Optional, Tuple, Union

import numpy as np
import torch

from . import ops
from .runtime_state import get_runtime_state


class FlowMatchEulerDiscreteScheduler:
    order = 1

    def __init__(self, num_train_timesteps: int = 1000, shift: float = 3.0):
        self.num_train_timesteps, self.shift = num_train_timesteps, shift
        t = np.linspace(1, num_train_timesteps, num_train_timesteps, dtype=np.float32)[::-1].copy()
        sigmas = self._shifted(t / num_train_timesteps)
        self.timesteps = torch.from_numpy(sigmas * num_train_timesteps)
        self.sigmas = torch.from_numpy(sigmas)
        self.sigma_min, self.sigma_max = float(sigmas[-1]), float(sigmas[0])
        self._step_index: Optional[int] = None
        self._sigmas_host = [float(s) for s in sigmas]

    def _shifted(self, sigmas: np.ndarray) -> np.ndarray:
        return (self.shift * sigmas / (1 + (self.shift - 1) * sigmas)).astype(np.float32)

    @property
    def step_index(self) -> Optional[int]:
        return self._step_index

    def set_timesteps(self, num_inference_steps: int, device: Union[str, torch.device, None] = None):
        """Evenly spaced in t between sigma_max and sigma_min, then the time shift; a final sigma of 0 is appended."""
        t = np.linspace(self.sigma_max * self.num_train_timesteps, self.sigma_min * self.num_train_timesteps,
                        num_inference_steps)
        sigmas = self._shifted(t / self.num_train_timesteps)
        self.num_inference_steps = num_inference_steps
        self.timesteps = torch.from_numpy(sigmas * self.num_train_timesteps).to(device=device)
        self.sigmas = torch.cat([torch.from_numpy(sigmas), torch.zeros(1)]).to(device=device)
        # host copy of the fp32 sigmas: kernel arguments, no device read-back inside the step
        self._sigmas_host = [float(s) for s in sigmas] + [0.0]
        self._step_index = None

    def index_for_timestep(self, timestep) -> int:
        t = float(timestep)
        hits = [i for i, v in enumerate(self.timesteps.tolist()) if v == t]
        if not hits:
            raise ValueError(f"timestep {t} is not one of scheduler.timesteps")
        # the second match when a timestep repeats, so that a start in the middle of the schedule skips no sigma
        return hits[1] if len(hits) > 1 else hits[0]

    def _sigma_pair(self, timestep) -> Tuple[float, float]:
        if isinstance(timestep, int) or (isinstance(timestep, torch.Tensor) and not timestep.is_floating_point()):
            raise ValueError("pass one of scheduler.timesteps, not an integer index, to step()")
        if self._step_index is None:
            self._step_index = self.index_for_timestep(timestep)
        i = self._step_index
        return self._sigmas_host[i], self._sigmas_host[i + 1]

    def _advance(self):
        rs = get_runtime_state()
        if not rs.patch_mode or rs.pipeline_patch_idx == rs.num_pipeline_patch - 1:
            self._step_index += 1

    def step(self, model_output: torch.Tensor, timestep, sample: torch.Tensor, return_dict: bool = False):
        """prev_sample = sample + (sigma_next - sigma) * model_output in the reference's rounding sequence."""
        sigma, sigma_next = self._sigma_pair(timestep)
        out = ops.cfg_euler_step(model_output.contiguous(), model_output.contiguous(), sample.contiguous(), 0.0, sigma,
                                 sigma_next)
        self._advance()
        return (out,)

    def step_with_guidance(self, noise_uncond: torch.Tensor, noise_cond: torch.Tensor, guidance_scale: float, timestep,
                           sample: torch.Tensor) -> torch.Tensor:
        """Guidance (``pipeline_stable_diffusion_3.py:1703-1713``) and ``step`` in one pass over the latent."""
        sigma, sigma_next = self._sigma_pair(timestep)
        out = ops.cfg_euler_step(noise_uncond.contiguous(), noise_cond.contiguous(), sample.contiguous(), guidance_scale,
                                 sigma, sigma_next)
        self._advance()
        return out
