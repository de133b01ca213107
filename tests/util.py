import torch


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().flatten(), b.double().flatten()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().flatten(), b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm()).clamp_min(1e-30))


def assert_parity(got: torch.Tensor, want: torch.Tensor, rel=1e-2, cos=0.9995, what=""):
    """The tolerance BASELINE.json states for bf16: cosine >= 0.9995 and
    relative L2 <= 1e-2 against the fp32 oracle (3e-2 for the fp8 path)."""
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    r, c = rel_l2(got, want), cosine(got, want)
    assert r <= rel and c >= cos, f"{what}: rel_l2={r:.3e} (<= {rel}) cosine={c:.6f} (>= {cos})"
    return r, c


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    """fp32 values that are exactly representable in bf16 (so the oracle and
    the kernels consume identical inputs)."""
    return x.to(torch.bfloat16).float()


def oracle_params(block) -> dict:
    """fp32 parameter dict in the unwrapped (diffusers) naming the oracle
    uses, from a product block whose layers carry the reference's wrappers:
    drop the ``.module`` hop and put the re-homed output biases back under the
    Linear they came from."""
    out = {}
    for name, p in block.named_parameters():
        key = name.replace(".module.", ".")
        if key.endswith(".encoder_output_bias"):
            key = key[: -len("encoder_output_bias")] + "to_add_out.bias"
        elif key.endswith(".output_bias"):
            base = key[: -len(".output_bias")]
            key = base + (".net.2.bias" if base.startswith("ff") else ".to_out.0.bias")
        out[key] = p.detach().float().cpu()
    return out
