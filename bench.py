"""Benchmark of the one-GPU DiT denoise-step hot path.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` times K passes of the
24-block SD3-shape MMDiT stack (BASELINE.json configs[1]: bf16, batch 2 = CFG
pair, 4096 image + 333 text tokens, hidden 1536, 24 x 64 heads, last block
context_pre_only) on synthetic inputs already resident in HBM, and prints one
JSON line.  ``roofline`` describes the dominant kernel (the grouped MFMA GEMM):
algorithmic flops per launch / average launch time, measured with HIP events
on the launch stream in a separate instrumented pass.  ``cpu_baseline`` is the
fp32 oracle of one joint block at the same shape, timed on this host's cores
for a bounded sample (one warm-up and three blocks) and scaled to 24 blocks.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0
PEAK_HBM_GBS = 8000.0


def profiled_traffic():
    """HBM-side bytes per launch of the grouped GEMM and of the attention kernel in the headline workload, as
    summarised in profiles/sd3_1024_step_hbm_traffic.txt from two `rocprofv3 --pmc` passes (FETCH_SIZE, WRITE_SIZE;
    hardware counters cannot be read from inside this process).  (None, None) when the summary is absent."""
    path = os.path.join(ROOT, "profiles", "sd3_1024_step_hbm_traffic.txt")
    gemm = attn = None
    try:
        for line in open(path):
            if line.startswith("# bench.py reads:"):
                for item in line.split(":", 1)[1].split():
                    key, _, val = item.partition("=")
                    if key == "gemm_bytes_per_call":
                        gemm = float(val)
                    elif key == "attn_bytes_per_launch":
                        attn = float(val)
    except OSError:
        pass
    return gemm, attn


def build_stack(cfg, device, seed=0):
    import torch

    from hetu_dit_amd import transformer

    with torch.device(device):
        stack = transformer.SD3TransformerBlocks(cfg["layers"], cfg["dim"], cfg["heads"], cfg["head_dim"])
    return randomize_(stack, device, seed)


def algorithmic_flops(cfg):
    B, Ni, Nt, D = cfg["batch"], cfg["n_img"], cfg["n_txt"], cfg["dim"]
    S = Ni + Nt
    gemm = 24.0 * S * D * D * B * cfg["layers"] - 18.0 * Nt * D * D * B  # last block: text stream stops after q|k|v
    attn = 4.0 * S * S * D * B * cfg["layers"]
    return gemm, attn


def randomize_(module, device, seed=0):
    import torch

    gen = torch.Generator(device=device).manual_seed(seed)
    for _, p in sorted(module.named_parameters(), key=lambda kv: kv[0]):
        p.data = (torch.randn(p.shape, generator=gen, device=device) * 0.02).to(torch.bfloat16)
        p.requires_grad_(False)
    return module


WORKLOADS = ("sd3_1024", "sd3_1024_transformer", "sd3_pipefusion", "sd3_pipefusion_b1", "flux_1024", "cogvideox_5b", "sd3_1024_fp8",
             "cogvideox_5b_fp8", "flux_1024_step", "cogvideox_5b_step")


def make_workload(name, dev):
    """(step callable, description, gemm flops, attention flops, blocks per step, attention kernel name) of one of
    BASELINE.json's configs.  sd3_1024 (configs[1]) is the headline workload; the others are the shapes of
    configs[3], [2] and [4], selectable for profiling."""
    import torch

    from hetu_dit_amd import synthetic, transformer
    from hetu_dit_amd.runtime_state import get_runtime_state, reset_runtime_state

    reset_runtime_state()
    gen = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *shape: torch.randn(*shape, generator=gen, device=dev).to(torch.bfloat16)
    if name.endswith("_fp8"):
        # the same blocks with the attention on the fp8-e4m3 path (per-(batch, head) absmax scales)
        from hetu_dit_amd.layers.attention_processor import hetuDiTAttentionWrapper

        step, desc, gemm, attn, blocks, kernel = make_workload(name[:-4], dev)
        for obj in (c.cell_contents for c in step.__closure__):
            if isinstance(obj, torch.nn.Module):
                for m in obj.modules():
                    if isinstance(m, hetuDiTAttentionWrapper):
                        m.fp8_attention = True
        return step, desc + "; attention on the fp8-e4m3 path", gemm, attn, blocks, kernel.replace("attn_fwd_kernel", "attn_fp8_kernel")
    if name == "sd3_1024_transformer":
        # the same 24 blocks inside the whole transformer: latent in, guided and Euler-updated latent out
        from hetu_dit_amd.transformer_sd3 import SD3Transformer2DModel

        cfg = synthetic.CONFIGS["sd3_1024"]
        with torch.device(dev):
            model = SD3Transformer2DModel()  # SD3-medium geometry: 128 x 128 x 16 latent, patch 2, text 4096 -> 1536
        randomize_(model, dev)
        lat, enc, pooled = rnd(1, 16, 128, 128), rnd(2, cfg["n_txt"], 4096), rnd(2, 2048)
        ts = torch.full((1,), 981.0, device=dev)
        gemm, attn = algorithmic_flops(cfg)
        D, T, Nt = cfg["dim"], cfg["n_img"], cfg["n_txt"]
        gemm += 2.0 * 2 * (T * 64 * D * 2 + Nt * 4096 * D + 256 * D + D * D + 2048 * D + D * D)
        desc = ("configs[1] inside the whole SD3 transformer: patch embedding + position table, timestep/text conditioning, "
                "context projection, 24 joint blocks, norm_out + proj_out + unpatchify, guidance 7.0 and the Euler update")

        def step():
            return model.denoise_step(lat, enc, pooled, ts, 7.0, 0.981, 0.95)

        step.multi_stream = "eager, the two batch elements as independent block chains on two streams"
        step.set_single_stream = lambda on: setattr(model._runner, "batch_streams", 1 if on else 2)
        return step, desc, gemm, attn, cfg["layers"], "attn_fwd_kernel<64>"
    if name in ("flux_1024_step", "cogvideox_5b_step"):
        # the whole block stacks of the two models at the shapes of configs[2] / configs[4]: 19 double + 38 single
        # Flux blocks (the 1024^2 step BASELINE.md quotes 0.84 s for on the reference's hardware), 42 CogVideoX-5B
        # blocks; every block one call of its whole-block entry point
        cfg = synthetic.CONFIGS[name[:-5]]
        B, Ni, Nt, D = cfg["batch"], cfg["n_img"], cfg["n_txt"], cfg["dim"]
        S = Ni + Nt
        x, e = rnd(B, Ni, D), rnd(B, Nt, D)
        if name == "flux_1024_step":
            L2, L1 = 19, 38
            with torch.device(dev):
                stack = transformer.FluxTransformerBlocks(L2, L1, D, cfg["heads"], cfg["head_dim"])
            randomize_(stack, dev)
            get_runtime_state().max_condition_sequence_length = Nt
            cos, sin = synthetic.rope_table(synthetic.flux_ids(Nt, *cfg["grid"]), (16, 56, 56))
            rope, t = (cos.to(dev), sin.to(dev)), rnd(B, D)
            gemm = 24.0 * S * D * D * B * (L2 + L1)
            attn = 4.0 * S * S * D * B * (L2 + L1)
            desc = ("configs[2] as a whole step: Flux-shape, 19 double-stream + 38 single-stream blocks, B1, 4096 image + 512 "
                    "text tokens, D3072, 24x128 heads")
            return (lambda: stack(x, e, t, rope)[0]), desc, gemm, attn, L2 + L1, "attn_fwd_pipe_kernel<128>"
        L = 42
        with torch.device(dev):
            stack = transformer.CogVideoXTransformerBlocks(L, D, cfg["heads"], cfg["head_dim"], cfg["temb_dim"])
        randomize_(stack, dev)
        cos, sin = synthetic.rope_table(synthetic.cogvideox_positions(*cfg["grid"]), (16, 24, 24))
        rope, t = (cos.to(dev), sin.to(dev)), rnd(B, cfg["temb_dim"])
        desc = "configs[4] as a whole step: CogVideoX-5B-shape, 42 blocks, B1, 226 text + 17550 video tokens, D3072, 48x64 heads"
        return (lambda: stack(x, e, t, rope)[0]), desc, 24.0 * S * D * D * B * L, 4.0 * S * S * D * B * L, L, "attn_fwd_kernel<64>"
    cfg = synthetic.CONFIGS[name]
    B, Ni, Nt, D = cfg["batch"], cfg["n_img"], cfg["n_txt"], cfg["dim"]
    S = Ni + Nt
    if name in ("sd3_1024", "sd3_pipefusion", "sd3_pipefusion_b1"):
        stack = build_stack(cfg, dev)
        e, t = rnd(B, Nt, D), rnd(B, D)
        if name == "sd3_1024":
            x = rnd(B, Ni, D)
            gemm, attn = algorithmic_flops(cfg)
            desc = ("configs[1]: SD3-shape denoise step, 24 joint blocks, B2 (CFG pair), 4096 image + 333 text "
                    "tokens, D1536, 24x64 heads, last block context_pre_only")
            def step():
                return stack(x, e, t)

            # launched eagerly the stack runs the two batch elements as independent chains on two streams
            step.multi_stream = "eager, the two batch elements as independent block chains on two streams"
            step.set_single_stream = lambda on: setattr(stack, "batch_streams", 1 if on else 2)
            return step, desc, gemm, attn, cfg["layers"], "attn_fwd_kernel<64>"
        # PipeFusion shard: a full-sequence pass fills the K/V buffers ("previous step"), then one step is
        # four patch passes of 1024 image tokens each against the stale full-length buffers
        P = cfg["patches"]
        rs = get_runtime_state()
        rs.set_token_patches([Ni // P * i for i in range(P + 1)])
        rs.set_patched_mode(False)
        stack(rnd(B, Ni, D), e, t)
        rs.set_patched_mode(True)
        xs = [rnd(B, Ni // P, D) for _ in range(P)]

        single = [False]

        def step():
            # one stream: every front of independent (patch, layer) blocks one merged call (capturable);
            # HDIT_BENCH_UNGROUPED=1: one call per block, patch after patch
            if not single[0]:
                return stack.forward_patches(xs, e, t, num_streams=2)[-1]
            if os.environ.get("HDIT_BENCH_UNGROUPED") != "1":
                return stack.forward_patches(xs, e, t, num_streams=1)[-1]
            out = None
            for p in range(P):
                out = stack(xs[p], e, t)
                rs.next_patch()
            return out

        # Default form: one stream, every front one merged call, replayed as a HIP graph (faster than two streams:
        # 22.4 against 24.5 ms).  HDIT_BENCH_TWO_STREAMS=1 times the two-stream form beside its one-stream eager form.
        if os.environ.get("HDIT_BENCH_TWO_STREAMS") == "1":
            step.multi_stream = "eager, patch p one block behind patch p-1 on two streams"
            step.set_single_stream = lambda on: single.__setitem__(0, bool(on))
        else:
            single[0] = True

        L = cfg["layers"]
        Np = Ni // P
        Sq = Np + Nt
        # patch 0 runs both streams; the block loop drops the text output of patches 1..P-1, for which the text
        # stream only supplies keys and values (k|v projection, no query rows, no out-projection, no MLP)
        gemm = (24.0 * Sq * D * D * B * L - 18.0 * Nt * D * D * B) + (P - 1) * (24.0 * Np + 4.0 * Nt) * D * D * B * L
        attn = 4.0 * Sq * S * D * B * L + (P - 1) * 4.0 * Np * S * D * B * L
        desc = (f"configs[3]: SD3 PipeFusion shard, 24 joint blocks x 4 patches, B{B}, query 1024 image + 333 text tokens "
                "against the 4096 + 333 stale K/V buffer")
        return step, desc, gemm, attn, L * P, "attn_fwd_kernel<64>"
    if name == "flux_1024":
        with torch.device(dev):
            stack = transformer.FluxTransformerBlocks(1, 1, D, cfg["heads"], cfg["head_dim"])
        randomize_(stack, dev)
        get_runtime_state().max_condition_sequence_length = Nt
        cos, sin = synthetic.rope_table(synthetic.flux_ids(Nt, *cfg["grid"]), (16, 56, 56))
        rope = (cos.to(dev), sin.to(dev))
        x, e, t = rnd(B, Ni, D), rnd(B, Nt, D), rnd(B, D)
        gemm = 24.0 * S * D * D * B * 2
        attn = 4.0 * S * S * D * B * 2
        desc = "configs[2]: Flux-shape, one double-stream + one single-stream block, B1, 4096 image + 512 text tokens, D3072, 24x128 heads"
        return (lambda: stack(x, e, t, rope)[0]), desc, gemm, attn, 2, "attn_fwd_pipe_kernel<128>"
    with torch.device(dev):
        stack = transformer.CogVideoXTransformerBlocks(1, D, cfg["heads"], cfg["head_dim"], cfg["temb_dim"])
    randomize_(stack, dev)
    cos, sin = synthetic.rope_table(synthetic.cogvideox_positions(*cfg["grid"]), (16, 24, 24))
    rope = (cos.to(dev), sin.to(dev))
    x, e, t = rnd(B, Ni, D), rnd(B, Nt, D), rnd(B, cfg["temb_dim"])
    gemm = 24.0 * S * D * D * B
    attn = 4.0 * S * S * D * B
    desc = "configs[4]: CogVideoX-5B-shape block, B1, 226 text + 17550 video tokens, D3072, 48x64 heads"
    return (lambda: stack(x, e, t, rope)[0]), desc, gemm, attn, 1, "attn_fwd_kernel<64>"


def cpu_baseline(runs=3):
    """fp32 oracle of one joint block on the host cores (a reported baseline, not a target): at the headline
    shape (configs[1]: B2, 4096 + 333 tokens; about 10 s of CPU work for a warm-up and `runs` timed blocks,
    scaled to the 24 blocks of a step) and at configs[0] (B1, 1024 + 333 tokens, the CPU-sized case)."""
    import torch

    import oracle
    from hetu_dit_amd import blocks, synthetic
    from tests.util import oracle_params

    torch.set_num_threads(os.cpu_count() or 1)

    def block_ms(cfg_name):
        cfg = synthetic.CONFIGS[cfg_name]
        blk = blocks.JointTransformerBlock(cfg["dim"], cfg["heads"], cfg["head_dim"])
        synthetic.init_module_(blk, 100)
        params = oracle_params(blk)
        x = synthetic.randn_bf16((cfg["batch"], cfg["n_img"], cfg["dim"]), 101).float()
        e = synthetic.randn_bf16((cfg["batch"], cfg["n_txt"], cfg["dim"]), 102).float()
        t = synthetic.randn_bf16((cfg["batch"], cfg["dim"]), 103).float()
        oracle.sd3_joint_block(params, x, e, t, cfg["heads"])  # warm-up
        times = []
        for _ in range(runs):
            t0 = time.perf_counter()
            oracle.sd3_joint_block(params, x, e, t, cfg["heads"])
            times.append((time.perf_counter() - t0) * 1e3)
        return statistics.median(times)

    ms_small = block_ms("sd3_512")
    ms_block = block_ms("sd3_1024")
    return {
        "value": round(ms_block * 24, 1),
        "unit": "ms",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"fp32 oracle, one SD3 joint block at the headline shape (configs[1]: B2, 4096+333 tokens, D1536): "
                  f"median of {runs} runs = {ms_block:.0f} ms/block, value = 24 x block (the step has 24 blocks; the "
                  f"last one's shorter text path is not discounted); configs[0] (B1, 1024+333 tokens): "
                  f"{ms_small:.1f} ms/block; os.cpu_count()={os.cpu_count()}",
    }


def probe_coissue():
    """Times an MFMA wave and a softmax-VALU wave alone on a SIMD, two of a kind together, one of each together, and
    both kinds interleaved in one wave; at 16 workgroups (no power limit) and at one per CU.  If the two units
    overlapped, 'mfma | valu' would take the longer of the two; it takes their sum."""
    import torch

    import hetu_dit_amd  # noqa: F401
    from hetu_dit_amd import ops

    torch.cuda.set_device(0)
    iters = 2000
    I, M, V, X = ops.PROBE_IDLE, ops.PROBE_MFMA, ops.PROBE_VALU, ops.PROBE_INTERLEAVED
    cases = [("mfma | idle", M, I), ("valu | idle", V, I), ("mfma | mfma", M, M), ("valu | valu", V, V), ("mfma | valu", M, V),
             ("valu | mfma", V, M), ("interleaved | idle", X, I)]
    result = {}
    for wgs in (16, 256):
        print(f"# {wgs} workgroups of 8 waves, {iters} iterations of 32 MFMAs / one 64-score softmax block; waves w and w+4 share a SIMD")
        print(f"# {'waves 0-3 | waves 4-7':22s} {'kcycles A':>10s} {'us A':>9s} {'kcycles B':>10s} {'us B':>9s} {'GHz':>6s}")
        for name, ra, rb in cases:
            ops.probe_coissue(ra, rb, 50, wgs)
            ca, ua, cb, ub = ops.probe_coissue(ra, rb, iters, wgs)
            ghz = ca / ua / 1e3 if ua > 0 else 0.0
            print(f"  {name:22s} {ca / 1e3:10.0f} {ua:9.1f} {cb / 1e3:10.0f} {ub:9.1f} {ghz:6.2f}")
            result[f"{name} @{wgs}"] = {"kcycles_a": round(ca / 1e3), "kcycles_b": round(cb / 1e3), "us_a": round(ua, 1), "us_b": round(ub, 1)}
    m, v, mv = result["mfma | idle @16"]["kcycles_a"], result["valu | idle @16"]["kcycles_a"], result["mfma | valu @16"]["kcycles_b"]
    print(json.dumps({"probe": "coissue", "mfma_alone_kcycles": m, "valu_alone_kcycles": v, "valu_next_to_mfma_kcycles": mv,
                      "overlap": round(1.0 - (mv - max(m, v)) / min(m, v), 3), "cases": result}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--single-stream", action="store_true",
                    help="sd3_1024: time the pass on one stream (a HIP-graph replay unless --no-graph) instead of the "
                         "eager form that runs the batch elements as independent chains on two streams")
    ap.add_argument("--workload", choices=WORKLOADS, default="sd3_1024",
                    help="sd3_1024 (BASELINE.json configs[1]) is the headline metric; the others are for profiling")
    ap.add_argument("--probe", choices=["coissue"], default=None,
                    help="instead of a workload, run a hardware probe and print its table: coissue = do the matrix "
                         "pipe and the vector ALU of a SIMD work side by side (hdit_probe_coissue)")
    args = ap.parse_args()
    if args.probe == "coissue":
        return probe_coissue()
    if args.gpus != 1:
        print("bench.py measures the one-GPU hot path only: run with --gpus 1 "
              "(the path is built and measured on a single GPU; nothing here launches collectives)", file=sys.stderr)
        sys.exit(2)

    import torch

    import hetu_dit_amd  # noqa: F401  (raises if libhdit.so is missing)
    from hetu_dit_amd import ops, synthetic
    from hetu_dit_amd.runtime_state import reset_runtime_state

    hetu_dit_amd._lib.lib()
    dev = "cuda:0"
    torch.cuda.set_device(0)
    step, workload_desc, gemm_fl, attn_fl, n_blocks, attn_kernel = make_workload(args.workload, dev)
    headline = args.workload == "sd3_1024"

    if hasattr(step, "set_single_stream"):
        step.set_single_stream(args.single_stream)
    for _ in range(max(args.warmup, 1)):
        out = step()
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()

    # persistent state a pass reads and mutates (the stale K/V buffers of the PipeFusion workload)
    from hetu_dit_amd.cache_manager import get_cache_manager

    def kv_buffers():
        return [t for entry in get_cache_manager().cache.values() for t in entry.tensors if t is not None]

    use_graph = not args.no_graph
    launch = None
    multi_stream = getattr(step, "multi_stream", None)
    if multi_stream is not None and not args.single_stream:
        # launched eagerly (a multi-stream pass is not recorded into a graph); from the same buffer state it must
        # reproduce the single-stream pass bit for bit
        saved = [t.clone() for t in kv_buffers()]
        step.set_single_stream(True)
        ref = step().clone()
        for t, s0 in zip(kv_buffers(), saved):
            t.copy_(s0)
        step.set_single_stream(False)
        got = step()
        torch.cuda.synchronize()
        same = torch.equal(got, ref)
        del saved, got, ref
        if same:
            use_graph = False
            run = step
            launch = multi_stream
        else:
            print("bench.py: the multi-stream pass does not reproduce the single-stream pass; timing the latter",
                  file=sys.stderr)
            step.set_single_stream(True)
    if launch is None and use_graph:
        saved = [t.clone() for t in kv_buffers()]
        ref = step().clone()
        for t, s0 in zip(kv_buffers(), saved):
            t.copy_(s0)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            g_out = step()
        for t, s0 in zip(kv_buffers(), saved):
            t.copy_(s0)
        graph.replay()
        torch.cuda.synchronize()
        # from the same buffer state a replay must reproduce the eager result bit for bit
        if not torch.equal(g_out, ref):
            use_graph = False
        del saved
        run = graph.replay if use_graph else step
    elif launch is None:
        run = step

    torch.cuda.synchronize()
    clk0 = ops.clock_sample()  # enqueued in front of the timed passes, on their stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    clk1 = ops.clock_sample()
    torch.cuda.synchronize()
    # average shader clock over the timed passes (counter pairs per CU, median)
    shader_clock_ghz = ops.shader_clock_ghz(clk0, clk1)

    # the same workload on one stream, beside the multi-stream figure: eager, then the same passes again, so that
    # both forms are timed on this box in this run (HIP-graph replay of the single-stream pass: --single-stream)
    single_stream = None
    if launch is not None:
        step.set_single_stream(True)
        for _ in range(2):
            step()
        torch.cuda.synchronize()
        n = min(args.steps, 10)
        t0 = time.perf_counter()
        for _ in range(n):
            step()
        torch.cuda.synchronize()
        single_stream = {"ms_per_step": round((time.perf_counter() - t0) * 1e3 / n, 3), "steps": n, "launch": "eager"}
        step.set_single_stream(False)

    # one plain device copy of known size (256 MiB read + 256 MiB written): the scale reference for the
    # FETCH_SIZE / WRITE_SIZE hardware counters when this command runs under `rocprofv3 --pmc`
    calib_src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    calib_dst = torch.empty_like(calib_src)
    calib_dst.copy_(calib_src)
    torch.cuda.synchronize()
    del calib_src, calib_dst

    # instrumented eager pass: HIP events around every launch on the launch stream
    if hasattr(step, "set_single_stream"):
        step.set_single_stream(True)  # one launch at a time, so that a launch's events time that launch alone
    timer = ops.KernelTimer()
    ops.set_timer(timer)
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    ops.set_timer(None)
    summ = timer.summary()

    def per_class(kind):
        n, ms, work = summ.get(kind, (0, 0.0, 0.0))
        return n, ms, work

    gemm_traffic, attn_traffic = profiled_traffic()
    n_g, ms_g, fl_g = per_class("gemm")
    fp8 = args.workload.endswith("_fp8")
    n_a, ms_a, fl_a = per_class("attn_fp8" if fp8 else "attn_bf16")
    attn_peak = PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS
    if fp8:  # the fp8 path's own passes count as attention time: absmax of q, k, v and the K / V quantisation
        ms_a += per_class("attn_absmax")[1]
    gemm_tflops = fl_g / ms_g / 1e9 if ms_g else 0.0
    attn_tflops = fl_a / ms_a / 1e9 if ms_a else 0.0
    glue = {}
    for kind in ("ln_modulate", "adaln_gemv", "gate_residual", "qk_norm_rope"):
        recs = [(w, e0.elapsed_time(e1)) for k, w, e0, e1 in timer.records if k == kind]
        if not recs:
            continue
        big = max(w for w, _ in recs)
        # the launches at the largest size of the class (image stream); the text-stream launches move
        # ~2 MB and are launch-latency bound.  Event-bracketed times of such short kernels include launch
        # gaps; the rocprofv3 durations under profiles/ are the per-kernel figures.
        sel = [(w, ms) for w, ms in recs if w == big]
        nbytes, ms = sum(w for w, _ in sel), sum(t for _, t in sel)
        glue[kind] = {"launches_per_step": len(recs) // 3, "largest_launch_bytes": big,
                      "largest_avg_us": round(ms / len(sel) * 1e3, 2), "achieved_GBps": round(nbytes / ms / 1e6, 1),
                      "frac_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
    result = {
        "metric": "ms per DiT denoise step (1 GPU)",
        "value": round(ms_step, 3),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 3),
        "ms_per_block": round(ms_step / n_blocks, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (seeded N(0,1) activations, N(0,0.02) random-init weights, resident in HBM)",
        "config": {"workload": workload_desc, "launch": launch or ("hip-graph replay" if use_graph else "eager")},
        "single_stream": single_stream,
        "step_tflops": round((gemm_fl + attn_fl) / ms_step / 1e9, 1),
        "shader_clock_ghz": round(shader_clock_ghz, 3) if shader_clock_ghz else None,
        "shader_clock_note": "average over the timed passes, from the shader-clock and 100 MHz counters sampled on the "
                             "launch stream before and after them; the published peaks are quoted at 2.4 GHz",
        "roofline": {
            "kernel": "gemm_kernel (grouped bf16 MFMA GEMM, all projection/MLP launches of the step)",
            "bound": "mfma", "achieved": round(gemm_tflops, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
            "frac": round(gemm_tflops / PEAK_BF16_TFLOPS, 4), "traffic": gemm_traffic if headline else None,
            "traffic_note": "from profiles/sd3_1024_step_hbm_traffic.txt: rocprofv3 FETCH_SIZE and WRITE_SIZE, each scaled "
                            "by what the counter reads for a 256 MiB copy, mean over the step's hdit_gemm_bf16 calls; "
                            "algorithmic operand + result bytes average 137.5 MB per call (activations of both streams, both weight sets; "
                            "on one stream the gated residuals of the fp32 stream are added by the normalisation kernels, "
                            "not by the GEMM epilogues)",
            "launches_per_step": n_g // 3, "avg_launch_us": round(ms_g / max(n_g, 1) * 1e3, 2),
            "flops_per_launch": round(fl_g / max(n_g, 1), 1),
            "measured_in": "three instrumented passes after the timed ones: kernel by kernel on one stream (the launches of "
                           "the single-stream form), HIP events around every launch (a launch alone on the GPU); the rocprofv3 trace of `bench.py --single-stream "
                           "--no-graph` is profiles/<workload>_kernel_stats.txt, that of this command "
                           "profiles/<workload>_two_streams_kernel_stats.txt",
        },
        "roofline_attention": {
            "kernel": attn_kernel + " (joint flash attention)", "bound": "mfma", "achieved": round(attn_tflops, 1),
            "peak": attn_peak, "unit": "TFLOP/s", "frac": round(attn_tflops / attn_peak, 4),
            "traffic": attn_traffic if headline else None, "launches_per_step": n_a // 3, "avg_launch_us": round(ms_a / max(n_a, 1) * 1e3, 2),
            "flops_per_launch": round(fl_a / max(n_a, 1), 1),
        },
        "roofline_glue": glue,
        "reference_prior": {"ms_per_step": 242.7, "note": "hetu_dit/model_profiler.py:116-121, SD3 1024^2 1 GPU, "
                                                            "hardware unlabelled (README testbed NVIDIA L20); not the same hardware"},
    }
    if not headline:
        result["metric"] = "ms per pass of the named workload (1 GPU)"
        result.pop("reference_prior")
    if not args.no_cpu_baseline and headline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
