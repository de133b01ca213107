"""The C-ABI library loads and exports every symbol include/hdit.h declares, and the Python binding
declares a signature for each of them (no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hdit.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hdit_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def library():
    import hetu_dit_amd

    if not os.path.exists(hetu_dit_amd.LIB_PATH):
        from hetu_dit_amd.build import build_library

        build_library()
    return ctypes.CDLL(hetu_dit_amd.LIB_PATH)


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for name in ("hdit_gemm_bf16", "hdit_attn_fwd_bf16", "hdit_attn_fwd_fp8", "hdit_attn_absmax",
                 "hdit_layernorm_modulate", "hdit_layernorm_modulate_jobs", "hdit_gate_residual", "hdit_adaln_gemv", "hdit_gelu_tanh", "hdit_ff_activation",
                 "hdit_qk_norm_rope", "hdit_copy_rows", "hdit_patchify", "hdit_unpatchify", "hdit_timestep_embedding",
                 "hdit_silu", "hdit_cfg_euler_step",
    "hdit_rope_table", "hdit_clock_sample", "hdit_gemm_force_config", "hdit_abi_version", "hdit_last_error"):
        assert name in syms


def test_library_exports_every_declared_symbol(library):
    missing = [s for s in declared_symbols() if not hasattr(library, s)]
    assert not missing, f"libhdit.so lacks {missing}"


def test_binding_covers_every_declared_symbol():
    from hetu_dit_amd import _lib

    assert sorted(_lib.SIGNATURES) == declared_symbols()
    lib = _lib.lib()
    assert lib.hdit_abi_version() == _lib.ABI_VERSION == 5
    assert lib.hdit_last_error() == b""


def test_struct_layouts_match_the_header(library):
    """sizeof of the three descriptor structs as the C compiler lays them out."""
    from hetu_dit_amd import _lib

    assert ctypes.sizeof(_lib.GemmProblem) == 6 * 8 + 4 * 8 + 6 * 4
    assert ctypes.sizeof(_lib.SeqSegment) == 8 + 3 * 8 + 2 * 4
    assert ctypes.sizeof(_lib.AttnArgs) == 8 * ctypes.sizeof(_lib.SeqSegment) + 4 * 4
    assert ctypes.sizeof(_lib.QkNormJob) == 8 + 3 * 8 + 4 * 8 + 4 * 4
    assert ctypes.sizeof(_lib.LnJob) == 4 * 8 + 5 * 8 + 4 * 4 + 3 * 8 + 5 * 8
    assert ctypes.sizeof(_lib.Sd3BlockArgs) == 20 * 8 + 9 * 8 + 8 + 14 * 4 + 8 + 2 * 4 + 8 * 8 + 2 * 4


def test_struct_layouts_against_the_c_compiler(tmp_path):
    """Every argument struct of include/hdit.h: sizeof and the offset of every field as gcc lays the header out,
    against the ctypes mirror -- a field added on one side only, or in another order, fails here and not as a
    misread pointer on the GPU."""
    import subprocess

    from hetu_dit_amd import _lib

    pairs = {
        "hdit_gemm_problem": _lib.GemmProblem, "hdit_seq_segment": _lib.SeqSegment, "hdit_attn_args": _lib.AttnArgs,
        "hdit_qknorm_job": _lib.QkNormJob, "hdit_ln_job": _lib.LnJob, "hdit_sd3_block_weights": _lib.Sd3BlockWeights,
        "hdit_sd3_block_args": _lib.Sd3BlockArgs, "hdit_flux_double_block_args": _lib.FluxDoubleBlockArgs,
        "hdit_flux_single_block_args": _lib.FluxSingleBlockArgs, "hdit_cogvideox_block_args": _lib.CogVideoXBlockArgs,
    }
    lines = ["#include <stdio.h>", "#include <stddef.h>", f'#include "{HEADER}"', "int main(void) {"]
    for cname, ct in pairs.items():
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, ftype in ct._fields_:
            if fname.endswith("_") or isinstance(ftype, type) and issubclass(ftype, ctypes.Array):
                continue
            lines.append(f'  printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", str(src), "-o", str(exe)], check=True)
    got = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, ct in pairs.items():
        assert int(got[cname]) == ctypes.sizeof(ct), cname
        for fname, ftype in ct._fields_:
            key = f"{cname}.{fname}"
            if key in got:
                assert int(got[key]) == getattr(ct, fname).offset, key


def test_entry_points_reject_bad_arguments_without_a_gpu(library):
    """Validation happens before any HIP call, so error codes can be checked on the CPU."""
    from hetu_dit_amd import _lib

    lib = _lib.lib()
    assert lib.hdit_gemm_bf16(None, 1, None) == -1
    p = _lib.GemmProblem()
    p.m, p.n, p.k = 16, 16, 48  # k not a multiple of 32
    p.a = p.b = p.c = 4096
    p.lda = p.ldb = p.ldc = 48
    arr = (_lib.GemmProblem * 1)(p)
    assert lib.hdit_gemm_bf16(arr, 1, None) == -2
    p.k = 64
    p.a = 4100  # misaligned
    arr = (_lib.GemmProblem * 1)(p)
    assert lib.hdit_gemm_bf16(arr, 1, None) == -1
    a = _lib.AttnArgs()
    a.batch, a.heads, a.head_dim = 1, 1, 96
    assert lib.hdit_attn_fwd_bf16(ctypes.byref(a), None) == -2
    p.a = 4096
    p.epilogue = _lib.EPI_BIAS | _lib.EPI_OUT_F32  # the fp32 stream flags belong to the gated-residual epilogue only
    arr = (_lib.GemmProblem * 1)(p)
    assert lib.hdit_gemm_bf16(arr, 1, None) == -1
    assert lib.hdit_layernorm_modulate(None, None, None, None, None, None, 1, 1, 64, 64, 64, 64, 64, 0, 1e-6, None) == -1
    assert lib.hdit_layernorm_modulate_jobs(None, 1, 64, None, None, 1e-6, None) == -1
    assert lib.hdit_adaln_gemv(4096, 4096, None, 4096, 9, 16, 64, None) == -2
    assert lib.hdit_qk_norm_rope(None, 1, 1, 1, 64, 1e-6, None) == -1


def test_library_exports_nothing_the_header_does_not_declare(library):
    import shutil
    import subprocess

    import hetu_dit_amd

    nm = shutil.which("nm")
    if nm is None:
        pytest.skip("nm not available")
    out = subprocess.run([nm, "-D", "--defined-only", hetu_dit_amd.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted({line.split()[-1] for line in out.splitlines() if " T " in line and line.split()[-1].startswith("hdit_")})
    assert exported == declared_symbols()
