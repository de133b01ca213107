// Shared device helpers for the gfx950 (CDNA4, wave64) kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hdit.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;

#define HDIT_WAVE 64

namespace hdit {

__device__ __forceinline__ float bf16_to_f32(__bf16 x) { return (float)x; }

// 8 bf16 held in an int4 <-> 8 floats
__device__ __forceinline__ void unpack8(const i32x4& raw, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    uint32_t u = (uint32_t)raw[i];
    f[2 * i] = __uint_as_float(u << 16);
    f[2 * i + 1] = __uint_as_float(u & 0xffff0000u);
  }
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 b = __builtin_convertvector(v, bf16x2);  // v_cvt_pk_bf16_f32, round-nearest-even
  return __builtin_bit_cast(uint32_t, b);
}

__device__ __forceinline__ i32x4 pack8(const float (&f)[8]) {
  i32x4 r;
#pragma unroll
  for (int i = 0; i < 4; i++) r[i] = (int)pack2(f[2 * i], f[2 * i + 1]);
  return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float gelu_tanh_f(float x) {
  // 0.5 x (1 + tanh(u)), u = sqrt(2/pi) (x + 0.044715 x^3), equals x * sigmoid(2u) = x / (1 + 2^(-2u log2 e)).
  // Written on v_exp_f32 / v_rcp_f32 directly: five full-rate VALU ops and two transcendentals per value.
  const float k = 2.0f * 0.7978845608028654f * 1.4426950408889634f;  // 2 sqrt(2/pi) log2(e)
  const float t = x * x;
  const float p = __builtin_fmaf(t, 0.044715f * k, k);
  const float e = __builtin_amdgcn_exp2f(-(x * p));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ float silu_f(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

}  // namespace hdit

// Host-side error plumbing shared by the C-ABI entry points.
namespace hdit_host {
void set_error(const char* msg);
int check_launch(const char* what);
int num_cus();
}  // namespace hdit_host
