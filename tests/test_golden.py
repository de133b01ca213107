"""Golden vectors (tests/golden/*.npz): the CPU leg checks that the oracle still reproduces them bit for
bit up to fp32 round-off; the GPU leg checks the HIP blocks against the same files."""
import os

import numpy as np
import pytest
import torch

from tests.golden.make_golden import CASES, HERE, build, build_step
from tests.util import assert_parity


def load(name):
    with np.load(os.path.join(HERE, name + ".npz")) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_golden(name):
    gold = load(name)
    _, _, now = build(name)
    assert sorted(gold) == sorted(now)
    assert abs(float(gold["weights_abs_sum"]) - float(now["weights_abs_sum"])) < 1e-6 * float(gold["weights_abs_sum"])
    for k in gold:
        np.testing.assert_allclose(now[k], gold[k], rtol=1e-5, atol=1e-6, err_msg=f"{name}:{k}")


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_hip_blocks_match_golden(name, hdit):
    from hetu_dit_amd.cache_manager import reset_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state, reset_runtime_state

    reset_runtime_state()
    gold = load(name)
    blk, _, _ = build(name)
    blk = blk.to("cuda:0")
    dev = lambda k: torch.from_numpy(gold[k]).to(torch.bfloat16).to("cuda:0")
    if name.startswith("sd3"):
        enc, hid = blk(hidden_states=dev("hidden_states"), encoder_hidden_states=dev("encoder_hidden_states"), temb=dev("temb"))
    elif name == "flux_double":
        rope = (torch.from_numpy(gold["cos"]).cuda(), torch.from_numpy(gold["sin"]).cuda())
        enc, hid = blk(hidden_states=dev("hidden_states"), encoder_hidden_states=dev("encoder_hidden_states"), temb=dev("temb"),
                       image_rotary_emb=rope)
    elif name == "flux_single":
        get_runtime_state().max_condition_sequence_length = int(gold["n_text"])
        rope = (torch.from_numpy(gold["cos"]).cuda(), torch.from_numpy(gold["sin"]).cuda())
        hid, enc = blk(hidden_states=dev("hidden_states"), temb=dev("temb"), image_rotary_emb=rope), None
    else:
        rope = (torch.from_numpy(gold["cos"]).cuda(), torch.from_numpy(gold["sin"]).cuda())
        hid, enc = blk(hidden_states=dev("hidden_states"), encoder_hidden_states=dev("encoder_hidden_states"), temb=dev("temb"),
                       image_rotary_emb=rope)
    torch.cuda.synchronize()
    assert_parity(hid, torch.from_numpy(gold["out_hidden"]), what=f"{name} hidden")
    if "out_encoder" in gold:
        assert_parity(enc, torch.from_numpy(gold["out_encoder"]), what=f"{name} encoder")
    else:
        assert enc is None
    reset_cache_manager()
    reset_runtime_state()


def test_oracle_reproduces_golden_step():
    gold = load("sd3_step")
    _, _, now = build_step()
    assert sorted(gold) == sorted(now)
    assert abs(float(gold["weights_abs_sum"]) - float(now["weights_abs_sum"])) < 1e-6 * float(gold["weights_abs_sum"])
    for k in gold:
        np.testing.assert_allclose(now[k], gold[k], rtol=1e-5, atol=2e-6, err_msg=f"sd3_step:{k}")


@pytest.mark.gpu
def test_hip_transformer_matches_golden_step(hdit):
    from hetu_dit_amd.cache_manager import reset_cache_manager
    from hetu_dit_amd.runtime_state import reset_runtime_state

    reset_runtime_state()
    gold = load("sd3_step")
    model, _, _ = build_step()
    model = model.to("cuda:0")
    dev = lambda k: torch.from_numpy(gold[k]).to(torch.bfloat16).to("cuda:0")
    t = torch.from_numpy(gold["timestep"]).to("cuda:0")
    noise = model(dev("latent"), dev("encoder_hidden_states"), dev("pooled"), t)
    torch.cuda.synchronize()
    assert_parity(noise, torch.from_numpy(gold["noise"]), what="sd3_step noise")
    new = hdit.ops.cfg_euler_step(noise[:1].contiguous(), noise[1:].contiguous(), dev("latent")[:1].contiguous(), 7.0, 0.9, 0.8)
    assert_parity(new, torch.from_numpy(gold["guided_step"]), what="sd3_step guided Euler update")
    reset_cache_manager()
    reset_runtime_state()
