"""The SD3 block stack's launch forms, all of which must give the same bits: blocks through the whole-block entry
point (``hdit_block_sd3``, one foreign call per block) against blocks launched kernel by kernel; the batch elements
of a full pass as independent chains on side streams against one chain on the caller's stream; the patches of a
PipeFusion step one block apart on side streams (``forward_patches``) against one ``forward`` per patch in patch
order (reference ``pipeline_stable_diffusion_3.py:1549-1644``)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def fresh_state():
    from hetu_dit_amd.cache_manager import reset_cache_manager
    from hetu_dit_amd.runtime_state import reset_runtime_state

    reset_runtime_state()
    reset_cache_manager()
    yield
    reset_cache_manager()
    reset_runtime_state()


def dev_randn(shape, seed, scale=1.0):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(shape, generator=gen, device=DEV) * scale).to(torch.bfloat16)


def make_stack(L, D, H, seed):
    from hetu_dit_amd import synthetic, transformer

    with torch.device(DEV):
        stack = transformer.SD3TransformerBlocks(L, D, H, 64)
    synthetic.init_module_(stack, seed)
    return stack


def buffers():
    from hetu_dit_amd.cache_manager import get_cache_manager

    return [b for entry in get_cache_manager().cache.values() for b in entry.tensors if b is not None]


def run_step_sequence(stack, B, Ni, Nt, D, P, entry_points, batch_streams, patch_streams):
    """A full pass, then two PipeFusion steps of P patches; returns every output and the buffers after each."""
    from hetu_dit_amd.runtime_state import get_runtime_state

    stack.use_block_entry_points = entry_points
    stack.batch_streams = batch_streams
    rs = get_runtime_state()
    rs.set_token_patches([Ni // P * i for i in range(P + 1)])
    rs.set_patched_mode(False)
    e, t = dev_randn((B, Nt, D), 32), dev_randn((B, D), 33)
    seen = [stack(dev_randn((B, Ni, D), 34), e, t).clone()]
    torch.cuda.synchronize()
    seen += [b.clone() for b in buffers()]
    rs.set_patched_mode(True)
    for k in range(2):
        xs = [dev_randn((B, Ni // P, D), 40 + 10 * k + p) for p in range(P)]
        if patch_streams == 0:
            for p in range(P):
                seen.append(stack(xs[p], e, t).clone())
                rs.next_patch()
        else:
            stack.group_fronts = patch_streams > 0  # -1: one stream, one call per block
            seen += [o.clone() for o in stack.forward_patches(xs, e, t, num_streams=abs(patch_streams))]
            stack.group_fronts = True
        assert rs.pipeline_patch_idx == 0
        torch.cuda.synchronize()
        seen += [b.clone() for b in buffers()]
    return seen


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("B", [1, 2, 3])
def test_entry_point_blocks_lanes_and_overlapped_patches_give_the_same_bits(hdit, B, fp8):
    from hetu_dit_amd.runtime_state import reset_runtime_state

    Ni, Nt, D, H, P, L = 1024, 77, 256, 4, 4, 5
    stack = make_stack(L, D, H, 31)
    for block in stack.transformer_blocks:
        block.attn.fp8_attention = fp8  # the attention of every form on the fp8-e4m3 path
    want = run_step_sequence(stack, B, Ni, Nt, D, P, entry_points=False, batch_streams=1, patch_streams=0)
    # on one stream the entry-point passes leave every gated residual to the normalisation that reads the stream next
    # (stack.defer_residuals); batch lanes and patches on several streams keep them in the GEMM epilogues
    forms = [
        ("entry points, one stream", True, 1, 0),
        ("entry points, one stream, residuals fused into the GEMM epilogues", True, 1, 0, False),
        ("entry points, merged fronts, residuals fused into the GEMM epilogues", True, 1, 1, False),
        ("entry points, batch lanes", True, 2, 0),
        ("entry points, three batch lanes, patches on one stream through forward_patches (merged fronts)", True, 3, 1),
        ("entry points, patches on one stream through forward_patches, fronts not merged", True, 1, -1),
        ("entry points, batch lanes, patches on two streams", True, 2, 2),
        ("entry points, patches on three streams", True, 1, 3),
        ("kernel by kernel, patches on two streams", False, 1, 2),
    ]
    for name, entry_points, batch_streams, patch_streams, *rest in forms:
        reset_runtime_state()  # the full pass of every form replaces the K/V buffers of the one before
        stack.defer_residuals = rest[0] if rest else True
        got = run_step_sequence(stack, B, Ni, Nt, D, P, entry_points, batch_streams, patch_streams)
        stack.defer_residuals = True
        assert len(got) == len(want)
        for i, (a, b) in enumerate(zip(got, want)):
            assert a.shape == b.shape and torch.equal(a, b), f"{name}: item {i} differs"


def test_forward_patches_refuses_what_it_cannot_run(hdit):
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, Ni, Nt, D, H, P = 1, 512, 77, 256, 4, 2
    stack = make_stack(2, D, H, 5)
    rs = get_runtime_state()
    rs.set_token_patches([Ni // P * i for i in range(P + 1)])
    e, t = dev_randn((B, Nt, D), 1), dev_randn((B, D), 2)
    xs = [dev_randn((B, Ni // P, D), 3 + p) for p in range(P)]
    with pytest.raises(ValueError):  # patch mode is off
        stack.forward_patches(xs, e, t)
    rs.set_patched_mode(False)
    stack(dev_randn((B, Ni, D), 9), e, t)
    rs.set_patched_mode(True)
    with pytest.raises(ValueError):  # one input per patch
        stack.forward_patches(xs[:1], e, t)
    with pytest.raises(ValueError):
        stack.forward_patches(xs, e, t, num_streams=0)
    assert len(stack.forward_patches(xs, e, t)) == P


def test_stack_takes_changing_batch_and_sequence_sizes(hdit):
    """One stack, passes of different batch sizes, token counts and stream element types one after the other: the
    prefilled whole-block calls, the modulation regrouping and the side streams hold nothing that is tied to the
    first shape they saw.  Every pass is compared with the kernel-by-kernel pass on one stream."""
    D, H, L = 256, 4, 3
    stack = make_stack(L, D, H, 77)
    for k, (B, Ni, Nt, f32) in enumerate([(2, 512, 77, False), (1, 300, 40, False), (3, 1024, 8, True), (2, 512, 77, False)]):
        x, e, t = dev_randn((B, Ni, D), 100 + k), dev_randn((B, Nt, D), 200 + k), dev_randn((B, D), 300 + k)
        if f32:
            x, e = x.float(), e.float()
        stack.use_block_entry_points, stack.batch_streams = False, 1
        want = stack(x, e, t).clone()
        torch.cuda.synchronize()
        stack.use_block_entry_points, stack.batch_streams = True, 2
        got = stack(x, e, t)
        torch.cuda.synchronize()
        assert got.dtype == want.dtype and torch.equal(got, want), f"pass {k}: B {B}, {Ni}+{Nt} tokens"
