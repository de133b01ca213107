"""HIP-graph replay of the block stack and of the whole SD3 step: every replay, with eager work and
synchronisations of the same program in between, must reproduce the eager result bit for bit (the benchmark
times graph replays)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def fresh_state():
    from hetu_dit_amd.cache_manager import reset_cache_manager
    from hetu_dit_amd.runtime_state import reset_runtime_state

    reset_runtime_state()
    yield
    reset_cache_manager()
    reset_runtime_state()


def dev_randn(shape, seed, scale=1.0):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(shape, generator=gen, device=DEV) * scale).to(torch.bfloat16)


def replay_and_compare(step, eager_between, replays=4):
    for _ in range(2):
        step()  # warm-up: packed weights, cached tables
    torch.cuda.synchronize()
    want = step().clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for i in range(replays):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i} differs from the eager result"
        eager_between()  # the program's own eager launches between replays
        torch.cuda.synchronize()


def test_sd3_stack_graph_replay(hdit):
    from hetu_dit_amd import synthetic, transformer

    B, Ni, Nt, D, H = 2, 512, 77, 256, 4
    with torch.device(DEV):
        stack = transformer.SD3TransformerBlocks(3, D, H, 64)
    synthetic.init_module_(stack, 1)
    x, e, t = dev_randn((B, Ni, D), 2), dev_randn((B, Nt, D), 3), dev_randn((B, D), 4)
    x2 = dev_randn((B, Ni, D), 5)
    replay_and_compare(lambda: stack(x, e, t), lambda: stack(x2, e, t))


def test_sd3_denoise_step_graph_replay(hdit):
    from hetu_dit_amd import synthetic
    from hetu_dit_amd.transformer_sd3 import SD3Transformer2DModel

    with torch.device(DEV):
        model = SD3Transformer2DModel(sample_size=32, num_layers=2, attention_head_dim=64, num_attention_heads=4,
                                      joint_attention_dim=128, caption_projection_dim=256, pooled_projection_dim=64,
                                      pos_embed_max_size=24)
    synthetic.init_module_(model, 6)
    lat, enc, pooled = dev_randn((1, 16, 32, 40), 7), dev_randn((2, 77, 128), 8), dev_randn((2, 64), 9)
    ts = torch.full((1,), 500.0, device=DEV)
    other = dev_randn((1, 16, 32, 40), 10)
    replay_and_compare(lambda: model.denoise_step(lat, enc, pooled, ts, 7.0, 0.9, 0.8),
                       lambda: model.denoise_step(other, enc, pooled, ts, 3.0, 0.5, 0.4))


def test_pipefusion_patch_graph_replay_from_restored_buffers(hdit):
    """A patch pass reads and updates the stale K/V buffers, so a replay only reproduces the eager pass from the
    same buffer state: the buffers are restored before every replay."""
    from hetu_dit_amd import synthetic, transformer
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, Ni, Nt, D, H, P = 2, 512, 77, 256, 4, 2
    with torch.device(DEV):
        stack = transformer.SD3TransformerBlocks(2, D, H, 64)
    synthetic.init_module_(stack, 11)
    e, t = dev_randn((B, Nt, D), 12), dev_randn((B, D), 13)
    rs = get_runtime_state()
    rs.set_token_patches([Ni // P * i for i in range(P + 1)])
    rs.set_patched_mode(False)
    stack(dev_randn((B, Ni, D), 14), e, t)  # fills the K/V buffers
    rs.set_patched_mode(True)
    xs = [dev_randn((B, Ni // P, D), 15 + p) for p in range(P)]

    def step():
        out = None
        for p in range(P):
            out = stack(xs[p], e, t)
            rs.next_patch()
        return out

    def buffers():
        return [b for entry in get_cache_manager().cache.values() for b in entry.tensors if b is not None]

    step()
    torch.cuda.synchronize()
    saved = [b.clone() for b in buffers()]

    def restore():
        for b, s0 in zip(buffers(), saved):
            b.copy_(s0)

    want = step().clone()
    restore()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for i in range(3):
        restore()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i} differs from the eager result"
        step()  # eager passes in between move the buffers on
        torch.cuda.synchronize()


def test_pipefusion_grouped_fronts_graph_replay(hdit):
    """``forward_patches(num_streams=1)``: every front of independent (patch, layer) blocks is one merged
    ``hdit_block_sd3_multi`` call on the caller's stream, so the whole PipeFusion step can be recorded into a graph.
    Replays (from restored K/V buffers, with eager passes in between) reproduce the eager sequential pass."""
    from hetu_dit_amd import synthetic, transformer
    from hetu_dit_amd.cache_manager import get_cache_manager
    from hetu_dit_amd.runtime_state import get_runtime_state

    B, Ni, Nt, D, H, P, L = 2, 1024, 77, 256, 4, 4, 6
    with torch.device(DEV):
        stack = transformer.SD3TransformerBlocks(L, D, H, 64)
    synthetic.init_module_(stack, 21)
    e, t = dev_randn((B, Nt, D), 22), dev_randn((B, D), 23)
    rs = get_runtime_state()
    rs.set_token_patches([Ni // P * i for i in range(P + 1)])
    rs.set_patched_mode(False)
    stack(dev_randn((B, Ni, D), 24), e, t)  # fills the K/V buffers
    rs.set_patched_mode(True)
    xs = [dev_randn((B, Ni // P, D), 25 + p) for p in range(P)]

    def sequential():
        outs = []
        for p in range(P):
            outs.append(stack(xs[p], e, t))
            rs.next_patch()
        return outs

    def grouped():
        return stack.forward_patches(xs, e, t, num_streams=1)

    def buffers():
        return [b for entry in get_cache_manager().cache.values() for b in entry.tensors if b is not None]

    grouped()
    torch.cuda.synchronize()
    saved = [b.clone() for b in buffers()]

    def restore():
        for b, s0 in zip(buffers(), saved):
            b.copy_(s0)

    want = [o.clone() for o in sequential()]
    want_buf = [b.clone() for b in buffers()]
    restore()
    got = grouped()
    torch.cuda.synchronize()
    for p in range(P):
        assert torch.equal(got[p], want[p]), f"eager grouped pass, patch {p}"
    assert all(torch.equal(a, b) for a, b in zip(buffers(), want_buf))
    restore()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = grouped()
    for i in range(3):
        restore()
        graph.replay()
        torch.cuda.synchronize()
        for p in range(P):
            assert torch.equal(outs[p], want[p]), f"replay {i}, patch {p}"
        assert all(torch.equal(a, b) for a, b in zip(buffers(), want_buf)), f"replay {i}: K/V buffers"
        sequential()  # eager passes in between move the buffers on
        torch.cuda.synchronize()
