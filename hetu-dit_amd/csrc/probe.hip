// Measurement aid: do the matrix pipe and the vector ALU of a SIMD work side by side?
//
// One 512-thread workgroup per CU; waves w and w + 4 of a workgroup share a SIMD.  Waves 0-3 ("A") and waves 4-7
// ("B") each run one of: nothing; a loop of independent v_mfma_f32_32x32x16_bf16 (32 per iteration: the matrix
// work of one 64 x 64 x 64 attention tile); the VALU work of that tile's softmax (64 exponentials, 32 bf16 packs,
// 32 pair sums, 32 three-way maxima, 64 subtractions per iteration); or both interleaved in one instruction
// stream.  Every wave reports the shader cycles and the 100 MHz ticks it took.  If the two units overlapped, an
// MFMA wave and a VALU wave on one SIMD would finish in the time of the longer one; on gfx950 they take the sum.
#include "hdit_common.h"

namespace {

__device__ __forceinline__ void mfma_work(int iters, int tid, float& sink) {
  f32x16 acc[4];
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
#pragma unroll
    for (int v = 0; v < 16; v++) acc[i][v] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      a[i][e] = (__bf16)((float)((tid * 7 + i * 3 + e) % 13 - 6) * 0.01f);
      b[i][e] = (__bf16)((float)((tid * 5 + i + e * 3) % 11 - 5) * 0.01f);
    }
  }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int r = 0; r < 8; r++)
#pragma unroll
      for (int i = 0; i < 4; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + r) & 3], b[i], acc[i], 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int v = 0; v < 16; v++) sink += acc[i][v];
}

template <bool WITH_MFMA>
__device__ __forceinline__ void valu_work(int iters, int tid, float& sink) {
  f32x16 acc[4];
  bf16x8 a[4], b[4];
  if (WITH_MFMA) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][v] = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        a[i][e] = (__bf16)((float)((tid * 7 + i * 3 + e) % 13 - 6) * 0.01f);
        b[i][e] = (__bf16)((float)((tid * 5 + i + e * 3) % 11 - 5) * 0.01f);
      }
    }
  }
  float x[64];
#pragma unroll
  for (int i = 0; i < 64; i++) x[i] = -0.001f * (float)((tid + i * 17) % 97);
  float rs = 0.f;
  const bf16x2 ones2 = {(__bf16)1.0f, (__bf16)1.0f};
  for (int it = 0; it < iters; it++) {
    float mx = x[0];
#pragma unroll
    for (int i = 1; i < 64; i += 2) mx = fmaxf(fmaxf(mx, x[i]), x[(i + 1) & 63]);
#pragma unroll
    for (int i = 0; i < 64; i += 2) {
      if (WITH_MFMA)
        acc[(i / 2) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i / 2 + i / 8) & 3], b[(i / 2) & 3], acc[(i / 2) & 3], 0, 0, 0);
      const float p0 = __builtin_amdgcn_exp2f(x[i]), p1 = __builtin_amdgcn_exp2f(x[i + 1]);
      const uint32_t pp = hdit::pack2(p0, p1);
      rs = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pp), ones2, rs, false);
      x[i] = x[i] - 1e-7f * mx;  // keeps the chain alive without moving the magnitudes
      x[i + 1] = x[i + 1] - 1e-7f * mx;
    }
    if (WITH_MFMA) {
      // one MFMA, then seven VALU instructions, 32 times: the densest interleave one wave can offer
#pragma unroll
      for (int g = 0; g < 32; g++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
      }
    }
  }
  sink += rs + x[5];
  if (WITH_MFMA) {
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int v = 0; v < 16; v++) sink += acc[i][v];
  }
}

__global__ void __launch_bounds__(512, 1) coissue_probe_kernel(int role_a, int role_b, int iters, unsigned long long* out, float* sink_out) {
  const int tid = threadIdx.x, wave = tid >> 6;
  const int role = wave < 4 ? role_a : role_b;
  float sink = 0.f;
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  if (role == HDIT_PROBE_MFMA) mfma_work(iters, tid, sink);
  else if (role == HDIT_PROBE_VALU) valu_work<false>(iters, tid, sink);
  else if (role == HDIT_PROBE_INTERLEAVED) valu_work<true>(iters, tid, sink);
  const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if ((tid & 63) == 0) {
    out[((size_t)blockIdx.x * 8 + wave) * 2] = c1 - c0;
    out[((size_t)blockIdx.x * 8 + wave) * 2 + 1] = r1 - r0;
  }
  if (sink == 12345.678f) sink_out[0] = sink;  // keeps the work alive; never true in practice
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_probe_coissue(int role_a, int role_b, int iters, int workgroups,
                                                                         void* out, void* stream) {
  auto ok = [](int r) { return r >= HDIT_PROBE_IDLE && r <= HDIT_PROBE_INTERLEAVED; };
  if (!ok(role_a) || !ok(role_b) || iters <= 0 || iters > (1 << 20) || workgroups <= 0 || workgroups > 1024) return HDIT_EINVAL;
  if (!out || (((uintptr_t)out) & 7)) return HDIT_EINVAL;
  // the last 8 bytes of `out` double as the never-written sink
  float* sink = (float*)((unsigned long long*)out + (size_t)workgroups * 16);
  hipLaunchKernelGGL(coissue_probe_kernel, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream, role_a, role_b, iters,
                     (unsigned long long*)out, sink);
  return hdit_host::check_launch("hdit_probe_coissue");
}
