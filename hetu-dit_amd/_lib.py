"""ctypes binding of ``libhdit.so`` (the C ABI declared in ``include/hdit.h``).

There is no fallback: if the library has not been built the first call raises.
"""
import ctypes as C
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
# HDIT_LIBRARY selects another build of the same ABI (kernel experiments); default: the in-tree library
LIB_PATH = os.environ.get("HDIT_LIBRARY") or os.path.join(HERE, "libhdit.so")

HDIT_GEMM_MAX_PROBLEMS = 16
HDIT_BLOCK_MAX_MULTI = 4
HDIT_ATTN_MAX_MULTI = 4
EPI_BIAS, EPI_BIAS_GELU, EPI_GATE_RESIDUAL = 0, 1, 2
EPI_RESID_F32, EPI_OUT_F32 = 0x10, 0x20
ABI_VERSION = 5


class GemmProblem(C.Structure):
    _fields_ = [
        ("a", C.c_void_p),
        ("b", C.c_void_p),
        ("c", C.c_void_p),
        ("bias", C.c_void_p),
        ("resid", C.c_void_p),
        ("gate", C.c_void_p),
        ("lda", C.c_int64),
        ("ldb", C.c_int64),
        ("ldc", C.c_int64),
        ("ldr", C.c_int64),
        ("m", C.c_int32),
        ("n", C.c_int32),
        ("k", C.c_int32),
        ("epilogue", C.c_int32),
        ("rows_per_batch", C.c_int32),
        ("gate_stride", C.c_int32),
    ]


class SeqSegment(C.Structure):
    _fields_ = [
        ("ptr", C.c_void_p),
        ("stride_b", C.c_int64),
        ("stride_s", C.c_int64),
        ("stride_h", C.c_int64),
        ("len", C.c_int32),
        ("pad_", C.c_int32),
    ]


class AttnArgs(C.Structure):
    _fields_ = [
        ("q", SeqSegment * 2),
        ("k", SeqSegment * 2),
        ("v", SeqSegment * 2),
        ("o", SeqSegment * 2),
        ("batch", C.c_int32),
        ("heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("scale", C.c_float),
    ]


class QkNormJob(C.Structure):
    _fields_ = [
        ("x", C.c_void_p),
        ("stride_b", C.c_int64),
        ("stride_s", C.c_int64),
        ("stride_h", C.c_int64),
        ("weight", C.c_void_p),
        ("bias", C.c_void_p),
        ("cos_table", C.c_void_p),
        ("sin_table", C.c_void_p),
        ("seq", C.c_int32),
        ("rope_row0", C.c_int32),
        ("rope_rows", C.c_int32),
        ("norm_kind", C.c_int32),
    ]


class LnJob(C.Structure):
    _fields_ = [
        ("x", C.c_void_p),
        ("y", C.c_void_p),
        ("shift", C.c_void_p),
        ("scale", C.c_void_p),
        ("x_sb", C.c_int64),
        ("x_st", C.c_int64),
        ("y_sb", C.c_int64),
        ("y_st", C.c_int64),
        ("mod_stride", C.c_int64),
        ("batch", C.c_int32),
        ("tokens", C.c_int32),
        ("x_f32", C.c_int32),
        ("pad_", C.c_int32),
        ("delta_y", C.c_void_p),
        ("delta_gate", C.c_void_p),
        ("x_out", C.c_void_p),
        ("d_sb", C.c_int64),
        ("d_st", C.c_int64),
        ("gate_stride", C.c_int64),
        ("xo_sb", C.c_int64),
        ("xo_st", C.c_int64),
    ]


class Sd3BlockWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "norm1_w", "norm1_b", "norm1_context_w", "norm1_context_b", "qkv_w", "qkv_b", "add_qkv_w", "add_qkv_b",
        "to_out_w", "to_out_b", "to_add_out_w", "to_add_out_b", "ff_in_w", "ff_in_b", "ff_out_w", "ff_out_b",
        "ff_context_in_w", "ff_context_in_b", "ff_context_out_w", "ff_context_out_b")]


class Sd3BlockArgs(C.Structure):
    _fields_ = [
        ("w", Sd3BlockWeights),
        ("hidden", C.c_void_p),
        ("encoder", C.c_void_p),
        ("temb", C.c_void_p),
        ("hidden_out", C.c_void_p),
        ("encoder_out", C.c_void_p),
        ("modulation_img", C.c_void_p),
        ("modulation_txt", C.c_void_p),
        ("kv_buffer", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_int64),
    ] + [(n, C.c_int32) for n in (
        "batch", "n_img", "n_txt", "dim", "heads", "ff_dim", "temb_dim", "kv_rows", "kv_row0", "hidden_f32",
        "encoder_f32", "out_f32", "context_pre_only", "skip_text_output")] + [
        ("text_kv", C.c_void_p), ("text_kv_mode", C.c_int32), ("fp8_attention", C.c_int32),
        ("pending_img", C.c_void_p), ("pending_img_gate", C.c_void_p), ("pending_txt", C.c_void_p),
        ("pending_txt_gate", C.c_void_p), ("pending_img_gate_stride", C.c_int64), ("pending_txt_gate_stride", C.c_int64),
        ("defer_img", C.c_void_p), ("defer_txt", C.c_void_p), ("lazy_residual", C.c_int32), ("pad_", C.c_int32)]


TEXT_KV_NONE, TEXT_KV_STORE, TEXT_KV_REUSE = 0, 1, 2


def _ptrs(*names):
    return [(n, C.c_void_p) for n in names]


def _ints(*names):
    return [(n, C.c_int32) for n in names]


class FluxDoubleBlockArgs(C.Structure):
    _fields_ = ([("w", Sd3BlockWeights)] + _ptrs("norm_q_w", "norm_k_w", "norm_added_q_w", "norm_added_k_w", "hidden", "encoder",
                                                  "temb", "rope_cos", "rope_sin", "hidden_out", "encoder_out", "workspace")
                + [("workspace_bytes", C.c_int64), ("qk_norm_eps", C.c_float)]
                + _ints("qk_norm_kind", "batch", "n_img", "n_txt", "dim", "heads", "ff_dim", "temb_dim", "hidden_f32",
                        "encoder_f32", "out_f32", "kv_rows", "kv_row0")
                + _ptrs("modulation_img", "modulation_txt", "kv_buffer"))


class FluxSingleBlockArgs(C.Structure):
    _fields_ = (_ptrs("norm_w", "norm_b", "qkv_w", "qkv_b", "proj_mlp_w", "proj_mlp_b", "proj_out_w", "proj_out_b", "norm_q_w",
                      "norm_k_w", "hidden", "temb", "rope_cos", "rope_sin", "hidden_out", "workspace")
                + [("workspace_bytes", C.c_int64), ("qk_norm_eps", C.c_float)]
                + _ints("qk_norm_kind", "batch", "seq", "dim", "heads", "ff_dim", "temb_dim", "hidden_f32", "out_f32",
                        "n_txt", "kv_rows", "kv_row0", "pad_")
                + _ptrs("modulation", "kv_buffer"))


class CogVideoXBlockArgs(C.Structure):
    _fields_ = (_ptrs("norm1_w", "norm1_b", "norm1_ln_w", "norm1_ln_b", "norm2_w", "norm2_b", "norm2_ln_w", "norm2_ln_b",
                      "qkv_w", "qkv_b", "to_out_w", "to_out_b", "norm_q_w", "norm_q_b", "norm_k_w", "norm_k_b",
                      "ff_in_w", "ff_in_b", "ff_out_w", "ff_out_b", "hidden", "encoder", "temb", "rope_cos", "rope_sin",
                      "hidden_out", "encoder_out", "workspace")
                + [("workspace_bytes", C.c_int64), ("norm_eps", C.c_float), ("qk_norm_eps", C.c_float)]
                + _ints("qk_norm_kind", "batch", "n_img", "n_txt", "dim", "heads", "ff_dim", "temb_dim", "hidden_f32",
                        "encoder_f32", "out_f32", "fp8_attention")
                + _ptrs("modulation1", "modulation2"))


# name -> (restype, argtypes); every symbol include/hdit.h declares
SIGNATURES = {
    "hdit_abi_version": (C.c_int, []),
    "hdit_last_error": (C.c_char_p, []),
    "hdit_gemm_bf16": (C.c_int, [C.POINTER(GemmProblem), C.c_int, C.c_void_p]),
    "hdit_attn_fwd_bf16": (C.c_int, [C.POINTER(AttnArgs), C.c_void_p]),
    "hdit_attn_fwd_bf16_multi": (C.c_int, [C.POINTER(AttnArgs), C.c_int, C.c_void_p]),
    "hdit_block_sd3_multi": (C.c_int, [C.POINTER(Sd3BlockArgs), C.c_int, C.c_void_p]),
    "hdit_attn_absmax": (C.c_int, [C.POINTER(AttnArgs), C.c_void_p, C.c_void_p]),
    "hdit_attn_fp8_workspace_bytes": (C.c_int64, [C.POINTER(AttnArgs)]),
    "hdit_attn_fwd_fp8": (C.c_int, [C.POINTER(AttnArgs), C.c_void_p, C.c_void_p, C.c_void_p]),
    "hdit_attn_fwd_fp8_static": (C.c_int, [C.POINTER(AttnArgs), C.c_void_p, C.c_void_p]),
    "hdit_block_sd3_workspace_bytes": (C.c_int64, [C.POINTER(Sd3BlockArgs)]),
    "hdit_block_sd3": (C.c_int, [C.POINTER(Sd3BlockArgs), C.c_void_p]),
    "hdit_block_flux_double_workspace_bytes": (C.c_int64, [C.POINTER(FluxDoubleBlockArgs)]),
    "hdit_block_flux_double": (C.c_int, [C.POINTER(FluxDoubleBlockArgs), C.c_void_p]),
    "hdit_block_flux_single_workspace_bytes": (C.c_int64, [C.POINTER(FluxSingleBlockArgs)]),
    "hdit_block_flux_single": (C.c_int, [C.POINTER(FluxSingleBlockArgs), C.c_void_p]),
    "hdit_block_cogvideox_workspace_bytes": (C.c_int64, [C.POINTER(CogVideoXBlockArgs)]),
    "hdit_block_cogvideox": (C.c_int, [C.POINTER(CogVideoXBlockArgs), C.c_void_p]),
    "hdit_layernorm_modulate": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
         C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_float, C.c_void_p],
    ),
    "hdit_layernorm_modulate_jobs": (
        C.c_int,
        [C.POINTER(LnJob), C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p],
    ),
    "hdit_gate_residual": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64,
         C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_void_p],
    ),
    "hdit_adaln_gemv": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "hdit_gelu_tanh": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_void_p]),
    "hdit_ff_activation": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_void_p]),
    "hdit_qk_norm_rope": (C.c_int, [C.POINTER(QkNormJob), C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p]),
    "hdit_patchify": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "hdit_unpatchify": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                  C.c_void_p]),
    "hdit_timestep_embedding": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p]),
    "hdit_silu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "hdit_cfg_euler_step": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_float, C.c_float, C.c_float, C.c_void_p],
    ),
    "hdit_clock_sample": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "hdit_probe_coissue": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "hdit_gemm_force_config": (None, [C.c_int]),
    "hdit_rope_table": (
        C.c_int,
        [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int, C.c_double, C.c_void_p, C.c_void_p, C.c_void_p],
    ),
    "hdit_copy_rows": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_void_p],
    ),
}

_lock = threading.Lock()
_lib = None


def lib():
    """Load (once) and return the bound library; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"{LIB_PATH} is missing: the HIP kernels are not built. Run "
                    "`python -c 'import __graft_entry__ as g; g.build()'` (or hetu_dit_amd.build.build_library())."
                )
            handle = C.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(handle, name)  # AttributeError if the library lacks a declared symbol
                fn.restype = res
                fn.argtypes = args
            if handle.hdit_abi_version() != ABI_VERSION:
                raise RuntimeError(f"{LIB_PATH} has ABI version {handle.hdit_abi_version()}, this binding needs "
                                   f"{ABI_VERSION}: rebuild the library")
            _lib = handle
    return _lib


class HditError(RuntimeError):
    pass


_CODES = {-1: "HDIT_EINVAL", -2: "HDIT_EUNSUPPORTED", -3: "HDIT_ELAUNCH", -4: "HDIT_ETOOLARGE"}


def check(rc: int, what: str):
    if rc != 0:
        detail = ""
        if rc in (-3, -4):
            detail = ": " + lib().hdit_last_error().decode()
        raise HditError(f"{what} failed with {_CODES.get(rc, rc)}{detail}")


def eager_only(fn):
    """Mark ``fn`` as opaque to ``torch.compile``: it reaches the C ABI through ``ctypes`` (raw pointers, the current
    stream's handle), which Dynamo cannot trace.  A compiled caller -- the reference compiles ``transformer.forward``
    when ``use_torch_compile`` is set (``base_pipeline.py:274-279``) -- breaks the graph here and runs ``fn`` as
    written; everything else it traces is unaffected.  The disabled function sits behind a plain forwarding function:
    ``torch.compile`` of a bound method whose function is itself the disabled wrapper loses ``self``."""
    import functools

    import torch

    opaque = torch.compiler.disable(fn)

    @functools.wraps(fn)
    def call(*args, **kwargs):
        return opaque(*args, **kwargs)

    return call
