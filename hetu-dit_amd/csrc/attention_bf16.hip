// Joint (image + text) flash attention forward for gfx950, bf16 in/out: the C entry point and the head-dim-64
// kernels (device code and its description: attention_bf16_kernels.h).
#include "attention_bf16_kernels.h"

namespace {

bool seg_ok(const hdit_seq_segment& s, bool need_ptr) {
  if (s.len < 0) return false;
  if (s.len == 0) return true;
  if (need_ptr && !s.ptr) return false;
  if (((uintptr_t)s.ptr) & 15) return false;
  if (s.stride_b % 8 || s.stride_s % 8 || s.stride_h % 8) return false;
  return true;
}

Seg2 make_seg(const hdit_seq_segment* s) {
  Seg2 r;
  r.p0 = (const __bf16*)s[0].ptr;
  r.sb0 = s[0].stride_b;
  r.ss0 = s[0].stride_s;
  r.sh0 = s[0].stride_h;
  r.len0 = s[0].len;
  r.p1 = (const __bf16*)s[1].ptr;
  r.sb1 = s[1].stride_b;
  r.ss1 = s[1].stride_s;
  r.sh1 = s[1].stride_h;
  r.len1 = s[1].len;
  return r;
}

}  // namespace

namespace hdit_attn {
int launch_d64(const AttnParams& P, int q_tiles, unsigned grid, bool pipelined, hipStream_t stream) {
  if (pipelined) {
    static std::atomic<bool> attr{false};  // setting the attribute twice from two threads is harmless
    if (!attr.load(std::memory_order_acquire)) {
      if (hipFuncSetAttribute((const void*)attn_fwd_pipe_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              PipeLds<64>::TOTAL) != hipSuccess)
        return HDIT_ELAUNCH;
      attr.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(attn_fwd_pipe_kernel<64>, dim3(grid), dim3(256), PipeLds<64>::TOTAL, stream, P, q_tiles);
  } else {
    hipLaunchKernelGGL(attn_fwd_kernel<64>, dim3(grid), dim3(256), Lds<64>::TOTAL, stream, P, q_tiles);
  }
  return HDIT_OK;
}

int launch_multi_d64(const AttnParams* P, const int* q_tiles, const int* nblocks, int count, bool pipelined, hipStream_t stream) {
  AttnMulti M;
  const int grid = fill_multi(M, P, q_tiles, nblocks, count);
  static std::atomic<bool> attr{false};  // setting the attributes twice from two threads is harmless
  if (!attr.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)attn_fwd_pipe_multi_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            PipeLds<64>::TOTAL) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_fwd_multi_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            Lds<64>::TOTAL) != hipSuccess)
      return HDIT_ELAUNCH;
    attr.store(true, std::memory_order_release);
  }
  if (pipelined)
    hipLaunchKernelGGL(attn_fwd_pipe_multi_kernel<64>, dim3((unsigned)grid), dim3(256), PipeLds<64>::TOTAL, stream, M);
  else
    hipLaunchKernelGGL(attn_fwd_multi_kernel<64>, dim3((unsigned)grid), dim3(256), Lds<64>::TOTAL, stream, M);
  return HDIT_OK;
}
}  // namespace hdit_attn

namespace hdit_host {
int attn_validate(const hdit_attn_args* a) {
  if (!a) return HDIT_EINVAL;
  if (a->batch <= 0 || a->heads <= 0) return HDIT_EINVAL;
  if (a->head_dim != 64 && a->head_dim != 128) return HDIT_EUNSUPPORTED;
  for (int i = 0; i < 2; i++)
    if (!seg_ok(a->q[i], true) || !seg_ok(a->k[i], true) || !seg_ok(a->v[i], true) || !seg_ok(a->o[i], true))
      return HDIT_EINVAL;
  if (a->k[0].len != a->v[0].len || a->k[1].len != a->v[1].len) return HDIT_EINVAL;
  if (a->q[0].len != a->o[0].len || a->q[1].len != a->o[1].len) return HDIT_EINVAL;
  if (a->q[0].len + a->q[1].len > 0 && a->k[0].len + a->k[1].len == 0) return HDIT_EINVAL;
  return HDIT_OK;
}
}  // namespace hdit_host

namespace {
// validated arguments -> kernel parameters; false: no query rows, nothing to do
bool to_params(const hdit_attn_args* a, AttnParams& P, int& q_tiles, unsigned& grid) {
  P.q = make_seg(a->q);
  P.k = make_seg(a->k);
  P.v = make_seg(a->v);
  P.o = make_seg(a->o);
  P.heads = a->heads;
  P.sq = a->q[0].len + a->q[1].len;
  P.skv = a->k[0].len + a->k[1].len;
  if (P.sq == 0) return false;
  const float scale = a->scale > 0.f ? a->scale : 1.0f / sqrtf((float)a->head_dim);
  P.scale_log2 = scale * 1.4426950408889634f;
  q_tiles = (P.sq + BQ - 1) / BQ;
  grid = (unsigned)(q_tiles * a->batch * a->heads);
  return true;
}
}  // namespace

namespace {
// Which kernel serves a problem: decided from the problem alone, so that it gets the same kernel -- and the same
// bits -- launched on its own or merged with others.
// d = 64: one wave per SIMD (the pipelined kernel) pays off while every workgroup has a CU to itself and some to
// spare (measured: 68 against 81 us for 144 workgroups); from about 5/8 of the CUs upwards, and for grids of
// several rounds, two workgroups per CU hiding each other's stalls serve better (SD3 step shape, 864
// workgroups: 288 against 273 us), and a merged launch of such problems wants the two-per-CU kernel anyway.
// d = 128: the tracked kernel runs one wave per SIMD as well, so the pipelined one serves every grid.
// HDIT_ATTN_PIPE=0 keeps every launch on the tracked-reference kernels, =1 puts every eligible launch on the
// pipelined ones (for A/B timing).
bool wants_pipelined(const hdit_attn_args* a, const AttnParams& P, unsigned grid) {
  static const char* pipe_env = getenv("HDIT_ATTN_PIPE");
  const bool pipe_off = pipe_env && pipe_env[0] == '0', pipe_force = pipe_env && pipe_env[0] == '1';
  const bool strides_ok = a->k[0].stride_s < (1 << 22) && a->k[1].stride_s < (1 << 22) && a->v[0].stride_s < (1 << 22) &&
                          a->v[1].stride_s < (1 << 22);  // a tile step (64 rows, in bytes) fits 32 bits
  if (pipe_off || !strides_ok || (P.skv + BKV - 1) / BKV < PIPE_MIN_TILES) return false;
  if (a->head_dim == 128 || pipe_force) return true;
  return (int)grid * 8 <= hdit_host::num_cus() * 5;
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_bf16(const hdit_attn_args* a, void* stream) {
  int rc = hdit_host::attn_validate(a);
  if (rc != HDIT_OK) return rc;
  AttnParams P;
  int q_tiles;
  unsigned grid;
  if (!to_params(a, P, q_tiles, grid)) return HDIT_OK;
  hipStream_t s = (hipStream_t)stream;
  const bool pipelined = wants_pipelined(a, P, grid);
  rc = a->head_dim == 64 ? hdit_attn::launch_d64(P, q_tiles, grid, pipelined, s) : hdit_attn::launch_d128(P, q_tiles, grid, pipelined, s);
  if (rc != HDIT_OK) return rc;
  return hdit_host::check_launch("hdit_attn_fwd_bf16");
}

extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_bf16_multi(const hdit_attn_args* args, int count, void* stream) {
  if (!args || count <= 0 || count > HDIT_ATTN_MAX_MULTI) return HDIT_EINVAL;
  if (count == 1) return hdit_attn_fwd_bf16(args, stream);
  for (int i = 0; i < count; i++) {
    const int rc = hdit_host::attn_validate(&args[i]);
    if (rc != HDIT_OK) return rc;
    if (args[i].head_dim != args[0].head_dim) return HDIT_EINVAL;
  }
  // one merged launch per kind of kernel the problems want
  for (int kind = 0; kind < 2; kind++) {
    AttnParams P[HDIT_ATTN_MAX_MULTI];
    int q_tiles[HDIT_ATTN_MAX_MULTI], nblocks[HDIT_ATTN_MAX_MULTI], n = 0;
    for (int i = 0; i < count; i++) {
      unsigned grid;
      if (!to_params(&args[i], P[n], q_tiles[n], grid)) continue;
      if ((int)wants_pipelined(&args[i], P[n], grid) != kind) continue;
      nblocks[n++] = (int)grid;
    }
    if (n == 0) continue;
    hipStream_t s = (hipStream_t)stream;
    int rc;
    if (n == 1)
      rc = args[0].head_dim == 64 ? hdit_attn::launch_d64(P[0], q_tiles[0], (unsigned)nblocks[0], kind != 0, s)
                                  : hdit_attn::launch_d128(P[0], q_tiles[0], (unsigned)nblocks[0], kind != 0, s);
    else
      rc = args[0].head_dim == 64 ? hdit_attn::launch_multi_d64(P, q_tiles, nblocks, n, kind != 0, s)
                                  : hdit_attn::launch_multi_d128(P, q_tiles, nblocks, n, kind != 0, s);
    if (rc != HDIT_OK) return rc;
    if ((rc = hdit_host::check_launch("hdit_attn_fwd_bf16_multi")) != HDIT_OK) return rc;
  }
  return HDIT_OK;
}
