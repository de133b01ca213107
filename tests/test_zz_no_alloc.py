"""The fp8 attention entry point that allocates nothing (``hdit_attn_fwd_fp8_static``: the quantised K / V
copy lives in a fixed array inside the library) against ``hdit_attn_fwd_fp8`` with a caller workspace, through
the C ABI: bit-identical outputs on two calls in a row, the second with a smaller input, then a larger head
size, and a clear error beyond the array's size."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev_randn(shape, seed):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randn(shape, generator=gen, device=DEV).to(torch.bfloat16)


def both_paths(hdit, B, H, sq, skv, hd, seed, two_segments=False):
    from hetu_dit_amd import _lib

    ops = hdit.ops
    q, k, v = dev_randn((B, sq, H, hd), seed), dev_randn((B, skv, H, hd), seed + 1), dev_randn((B, skv, H, hd), seed + 2)
    if two_segments:  # a joint [image, text] sequence living in two buffers
        cut = skv // 3
        ks, vs = [k[:, :cut], k[:, cut:]], [v[:, :cut], v[:, cut:]]
    else:
        ks, vs = [k], [v]
    want, got = torch.zeros_like(q), torch.zeros_like(q)
    a_ref = ops.attention_args([q], ks, vs, [want])
    absmax = ops.attention_fp8_absmax(a_ref)
    lib = _lib.lib()
    ws = torch.empty(lib.hdit_attn_fp8_workspace_bytes(C.byref(a_ref)), dtype=torch.uint8, device=DEV)
    _lib.check(lib.hdit_attn_fwd_fp8(C.byref(a_ref), absmax.data_ptr(), ws.data_ptr(),
                                     torch.cuda.current_stream().cuda_stream), "hdit_attn_fwd_fp8")
    a_new = ops.attention_args([q], ks, vs, [got])
    ops.attention_fp8_static(a_new, absmax)
    torch.cuda.synchronize()
    assert torch.isfinite(want.float()).all() and want.float().abs().max() > 0
    assert torch.equal(got, want), f"B{B} H{H} {sq}x{skv} d{hd}: static-scratch path differs from the workspace path"


def test_fp8_attention_static_scratch_matches_workspace_path(hdit):
    print("no-alloc fp8 attention: first call 2x4x700x1000 d64", flush=True)
    both_paths(hdit, 2, 4, 700, 1000, 64, 1, two_segments=True)
    print("no-alloc fp8 attention: second, smaller call 1x2x300x333 d64", flush=True)
    both_paths(hdit, 1, 2, 300, 333, 64, 11)
    print("no-alloc fp8 attention: d128 1x3x520x777", flush=True)
    both_paths(hdit, 1, 3, 520, 777, 128, 21, two_segments=True)
    print("no-alloc fp8 attention: full SD3 shape 2x24x4429x4429 d64 (27.5 MB of the 32 MiB array)", flush=True)
    both_paths(hdit, 2, 24, 4429, 4429, 64, 31, two_segments=True)


def test_fp8_attention_static_scratch_refuses_what_does_not_fit(hdit):
    from hetu_dit_amd import _lib

    ops = hdit.ops
    B, H, S, hd = 2, 24, 8192, 128  # 2 * B * H * S * hd = 96 MiB of fp8 K / V
    q = dev_randn((B, 64, H, hd), 41)
    k = dev_randn((B, S, H, hd), 42)
    o = torch.empty_like(q)
    args = ops.attention_args([q], [k], [k], [o])
    assert _lib.lib().hdit_attn_fp8_workspace_bytes(C.byref(args)) > (32 << 20)
    absmax = ops.attention_fp8_absmax(args)
    rc = _lib.lib().hdit_attn_fwd_fp8_static(C.byref(args), absmax.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == -4
    assert b"HDIT_ATTN_FP8_STATIC_MAX_BYTES" in _lib.lib().hdit_last_error()
    with pytest.raises(hdit.HditError, match="HDIT_ETOOLARGE"):
        ops.attention_fp8_static(args, absmax)
    torch.cuda.synchronize()
