// Bandwidth-bound glue kernels for gfx950: every tensor is touched once, with
// 16-byte accesses laid out so that a wave reads/writes contiguous 1 KiB runs,
// statistics in fp32, wave64 cross-lane reductions.
#include <cstring>

#include "hdit_common.h"

namespace {

using hdit::pack8;
using hdit::unpack8;
using hdit::wave_sum;

// ---------------------------------------------------------------------------
// LayerNorm (optional affine) + adaLN modulate.  One wave per row; the row
// stays in registers between the statistics and the write.
// ---------------------------------------------------------------------------
struct LnJobs {
  int count;
  int block_start[HDIT_LN_MAX_JOBS + 1];  // first workgroup of each job
  hdit_ln_job j[HDIT_LN_MAX_JOBS];
};

// NCH = 16-byte input chunks per lane.  A chunk is 8 elements of a bf16 row or (XF32: the fp32 residual stream of
// a block stack) 4 elements of an f32 row; the output is bf16 either way, so a lane stores 16 or 8 bytes per
// chunk and a wave-wide access is contiguous in both cases.
//
// A workgroup is four waves on four consecutive rows of ONE batch element.  Its modulation vectors go through
// LDS (one read of scale | shift per workgroup instead of one per wave: they are as many bytes as a row), and
// they are requested BEFORE the rows: loads return in order, so the wait that precedes the LDS writes leaves
// the row loads in flight.  One row per wave, not two in a software pipeline: with operands that do not sit
// in the last-level cache (buffers rotated over 650 MB) the launch of the step's shape, 8858 rows of 1536 fp32,
// takes 16.6 us this way against 18.5 us, the time of a plain copy of the same bytes.
// Rows of up to 64 floats per lane are held to 128 registers (four waves per SIMD): left alone, the compiler hoists
// every LDS read of the modulation above the reductions and the wide kernels drop to three waves per SIMD.
//
// DELTA (fp32 stream only): a job may carry a pending update of the stream, x' = x + gate[b, :] * delta_y (the gated
// residual of the projection that ran before this normalisation, whose GEMM wrote only delta_y = bf16(A.W^T + bias)).
// It is applied here, in the registers the row is read into anyway, and x' is written back as the new stream: the
// GEMM's epilogue then has no read-modify-write of the fp32 stream, which four waves per CU cannot keep HBM busy with.
template <int NCH, bool XF32, bool DELTA>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NCH * (XF32 ? 4 : 8) <= 64 ? 4 : 2)))
ln_modulate_kernel(const LnJobs jobs, const __bf16* __restrict__ lw, const __bf16* __restrict__ lb, int dim, float eps) {
  static_assert(XF32 || !DELTA, "the pending update exists for the fp32 stream only");
  extern __shared__ __attribute__((aligned(16))) float lmod[];  // scale[dim] | shift[dim] (| gate[dim]) of this batch element
  // which job this workgroup belongs to (a launch normalises up to HDIT_LN_MAX_JOBS tensors, e.g. the
  // image and the text stream of a joint block)
  int ji = 0;
#pragma unroll 1
  while (ji + 1 < jobs.count && (int)blockIdx.x >= jobs.block_start[ji + 1]) ji++;
  const hdit_ln_job& job = jobs.j[ji];
  constexpr int EPC = XF32 ? 4 : 8;  // elements per chunk
  constexpr int XB = XF32 ? 4 : 2;   // bytes per input element
  const int lane = threadIdx.x & 63;
  const int local = (int)blockIdx.x - jobs.block_start[ji];
  const int per_batch = (job.tokens + 3) >> 2;  // workgroups per batch element
  const int b = local / per_batch;
  const int t = (local - b * per_batch) * 4 + (int)(threadIdx.x >> 6);
  const bool live = t < job.tokens;
  const float* __restrict__ shift = job.shift ? job.shift + (int64_t)b * job.mod_stride : nullptr;
  const float* __restrict__ scale = job.scale ? job.scale + (int64_t)b * job.mod_stride : nullptr;
  const bool has_delta = DELTA && job.delta_y != nullptr;
  const float* __restrict__ dgate = has_delta ? job.delta_gate + (int64_t)b * job.gate_stride : nullptr;
  const int nchunks = dim / EPC;
  const int nvec = dim >> 2;  // f32x4 pieces of a modulation vector
  constexpr int MV = (NCH * 64 * (EPC / 4) + 255) / 256;
  f32x4 mreg[DELTA ? 3 : 2][MV];
#pragma unroll
  for (int k = 0; k < MV; k++) {
    const int i = (int)threadIdx.x + k * 256;
    if (i < nvec) {
      if (scale) mreg[0][k] = *(const f32x4*)(scale + i * 4);
      if (shift) mreg[1][k] = *(const f32x4*)(shift + i * 4);
      if constexpr (DELTA) {
        if (has_delta) mreg[2][k] = *(const f32x4*)(dgate + i * 4);
      }
    }
  }
  i32x4 raw[NCH];
  i32x2 draw[DELTA ? NCH : 1];
  if (live) {
    const unsigned char* xr = (const unsigned char*)job.x + ((int64_t)b * job.x_sb + (int64_t)t * job.x_st) * XB;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      const int c = lane + i * 64;
      if (c < nchunks) raw[i] = *(const i32x4*)(xr + c * 16);
    }
    if constexpr (DELTA) {
      if (has_delta) {
        const __bf16* dr = (const __bf16*)job.delta_y + (int64_t)b * job.d_sb + (int64_t)t * job.d_st;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
          const int c = lane + i * 64;
          if (c < nchunks) draw[i] = *(const i32x2*)(dr + c * 4);
        }
      }
    }
  }
#pragma unroll
  for (int k = 0; k < MV; k++) {
    const int i = (int)threadIdx.x + k * 256;
    if (i < nvec) {
      if (scale) *(f32x4*)(lmod + i * 4) = mreg[0][k];
      if (shift) *(f32x4*)(lmod + dim + i * 4) = mreg[1][k];
      if constexpr (DELTA) {
        if (has_delta) *(f32x4*)(lmod + 2 * dim + i * 4) = mreg[2][k];
      }
    }
  }
  __syncthreads();
  if (!live) return;
  if constexpr (DELTA) {
    if (has_delta) {
      // x' = fma(gate, delta, x), the operation of the GEMM's gated-residual epilogue, bit for bit
      float* xo = job.x_out ? (float*)job.x_out + (int64_t)b * job.xo_sb + (int64_t)t * job.xo_st : nullptr;
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        const int c = lane + i * 64;
        if (c < nchunks) {
          const f32x4 g = *(const f32x4*)(lmod + 2 * dim + c * 4);
          const float d[4] = {__uint_as_float((uint32_t)draw[i][0] << 16), __uint_as_float((uint32_t)draw[i][0] & 0xffff0000u),
                              __uint_as_float((uint32_t)draw[i][1] << 16), __uint_as_float((uint32_t)draw[i][1] & 0xffff0000u)};
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = __builtin_fmaf(g[e], d[e], __int_as_float(raw[i][e]));
#pragma unroll
          for (int e = 0; e < 4; e++) raw[i][e] = __float_as_int(v[e]);
          if (xo) *(f32x4*)(xo + c * 4) = v;
        }
      }
    }
  }
  // EPC bf16 values (an affine weight or bias) at element offset c * EPC
  auto load_bf16 = [&](const __bf16* p, int c, float (&w)[EPC]) {
    if constexpr (XF32) {
      const i32x2 r = *(const i32x2*)(p + c * 4);
#pragma unroll
      for (int e = 0; e < 2; e++) {
        w[2 * e] = __uint_as_float((uint32_t)r[e] << 16);
        w[2 * e + 1] = __uint_as_float((uint32_t)r[e] & 0xffff0000u);
      }
    } else {
      unpack8(*(const i32x4*)(p + c * 8), w);
    }
  };
  auto load_lds = [&](const float* p, int c, float (&w)[EPC]) {
#pragma unroll
    for (int h = 0; h < EPC / 4; h++) {
      const f32x4 v = *(const f32x4*)(p + c * EPC + h * 4);
#pragma unroll
      for (int e = 0; e < 4; e++) w[h * 4 + e] = v[e];
    }
  };
  const float inv_d = 1.0f / (float)dim;
  float s = 0.f;
  float f[NCH][EPC];
#pragma unroll
  for (int i = 0; i < NCH; i++) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      if constexpr (XF32) {
#pragma unroll
        for (int e = 0; e < 4; e++) f[i][e] = __int_as_float(raw[i][e]);
      } else {
        unpack8(raw[i], f[i]);
      }
#pragma unroll
      for (int e = 0; e < EPC; e++) s += f[i][e];
    }
  }
  const float mean = wave_sum(s) * inv_d;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; i++) {
    const int c = lane + i * 64;
    if (c < nchunks) {
#pragma unroll
      for (int e = 0; e < EPC; e++) {
        f[i][e] -= mean;
        q += f[i][e] * f[i][e];
      }
    }
  }
  const float rstd = rsqrtf(wave_sum(q) * inv_d + eps);
  __bf16* yr = (__bf16*)job.y + (int64_t)b * job.y_sb + (int64_t)t * job.y_st;
#pragma unroll
  for (int i = 0; i < NCH; i++) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      float o[EPC], w[EPC];
#pragma unroll
      for (int e = 0; e < EPC; e++) o[e] = f[i][e] * rstd;
      if (lw) {
        load_bf16(lw, c, w);
#pragma unroll
        for (int e = 0; e < EPC; e++) o[e] *= w[e];
      }
      if (lb) {
        load_bf16(lb, c, w);
#pragma unroll
        for (int e = 0; e < EPC; e++) o[e] += w[e];
      }
      if (scale) {
        load_lds(lmod, c, w);
#pragma unroll
        for (int e = 0; e < EPC; e++) o[e] *= 1.0f + w[e];
      }
      if (shift) {
        load_lds(lmod + dim, c, w);
#pragma unroll
        for (int e = 0; e < EPC; e++) o[e] += w[e];
      }
      if constexpr (XF32) {
        i32x2 pk = {(int)hdit::pack2(o[0], o[1]), (int)hdit::pack2(o[2], o[3])};
        *(i32x2*)(yr + c * 4) = pk;
      } else {
        *(i32x4*)(yr + c * 8) = pack8(o);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// out = x + gate[b] * y
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) gate_residual_kernel(const __bf16* __restrict__ x, const __bf16* __restrict__ y,
                                                            const float* __restrict__ gate, __bf16* __restrict__ out,
                                                            int64_t total_chunks, int tokens, int chunks_per_row,
                                                            int64_t x_sb, int64_t x_st, int64_t y_sb, int64_t y_st,
                                                            int64_t o_sb, int64_t o_st, int64_t gate_stride) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total_chunks) return;
  int64_t row = i / chunks_per_row;
  int c = (int)(i - row * chunks_per_row);
  int b = (int)(row / tokens);
  int64_t t = row - (int64_t)b * tokens;
  float fx[8], fy[8];
  unpack8(__builtin_nontemporal_load((const i32x4*)(x + b * x_sb + t * x_st + c * 8)), fx);
  unpack8(__builtin_nontemporal_load((const i32x4*)(y + b * y_sb + t * y_st + c * 8)), fy);
  const float* g = gate + (int64_t)b * gate_stride + c * 8;
  f32x4 g0 = *(const f32x4*)g, g1 = *(const f32x4*)(g + 4);
#pragma unroll
  for (int e = 0; e < 4; e++) {
    fx[e] += g0[e] * fy[e];
    fx[e + 4] += g1[e] * fy[e + 4];
  }
  __builtin_nontemporal_store(pack8(fx), (i32x4*)(out + b * o_sb + t * o_st + c * 8));
}

// ---------------------------------------------------------------------------
// y = gelu_tanh(x + bias)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) gelu_kernel(const __bf16* __restrict__ x, const __bf16* __restrict__ bias,
                                                   __bf16* __restrict__ y, int64_t total_chunks, int chunks_per_row,
                                                   int64_t ldx, int64_t ldy) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total_chunks) return;
  int64_t row = i / chunks_per_row;
  int c = (int)(i - row * chunks_per_row);
  float f[8];
  unpack8(__builtin_nontemporal_load((const i32x4*)(x + row * ldx + c * 8)), f);
  if (bias) {
    float w[8];
    unpack8(*(const i32x4*)(bias + c * 8), w);
#pragma unroll
    for (int e = 0; e < 8; e++) f[e] += w[e];
  }
#pragma unroll
  for (int e = 0; e < 8; e++) f[e] = hdit::gelu_tanh_f(f[e]);
  __builtin_nontemporal_store(pack8(f), (i32x4*)(y + row * ldy + c * 8));
}

// ---------------------------------------------------------------------------
// The feed-forward activations that are not fused into a GEMM epilogue, applied to the first projection's output
// (bias already added): exact GELU, GEGLU (value half times exact GELU of the gate half), SiLU.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float gelu_erf_f(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f)); }

template <int KIND>
__global__ void __launch_bounds__(256) ff_activation_kernel(const __bf16* __restrict__ x, __bf16* __restrict__ y,
                                                            int64_t total_chunks, int chunks_per_row, int64_t ldx,
                                                            int64_t ldy) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total_chunks) return;
  int64_t row = i / chunks_per_row;
  int c = (int)(i - row * chunks_per_row);
  float f[8];
  unpack8(*(const i32x4*)(x + row * ldx + c * 8), f);
  if constexpr (KIND == HDIT_ACT_GEGLU) {
    float gte[8];
    unpack8(*(const i32x4*)(x + row * ldx + (int64_t)(chunks_per_row + c) * 8), gte);
#pragma unroll
    for (int e = 0; e < 8; e++) f[e] *= gelu_erf_f(gte[e]);
  } else if constexpr (KIND == HDIT_ACT_GELU_ERF) {
#pragma unroll
    for (int e = 0; e < 8; e++) f[e] = gelu_erf_f(f[e]);
  } else {
#pragma unroll
    for (int e = 0; e < 8; e++) f[e] = hdit::silu_f(f[e]);
  }
  *(i32x4*)(y + row * ldy + c * 8) = pack8(f);
}

// ---------------------------------------------------------------------------
// adaLN projection: out[b, n] = W[n, :] . silu(temb[b, :]) + bias[n]
// One wave per output row; the weight row is streamed once for all batches.
// ---------------------------------------------------------------------------
template <int MAXB, int NCH>
__global__ void __launch_bounds__(256) adaln_gemv_kernel(const __bf16* __restrict__ temb, const __bf16* __restrict__ w,
                                                         const __bf16* __restrict__ bias, float* __restrict__ out,
                                                         int batch, int n, int k) {
  // A wave produces RW consecutive output rows: all of their weight chunks are requested before any is
  // consumed (RW * NCH 16-byte loads in flight per lane), and the silu(temb) chunks are reused across rows.
  constexpr int RW = 4;
  const int lane = threadIdx.x & 63;
  const int row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * RW;
  if (row0 >= n) return;
  const int nchunks = k >> 3;
  i32x4 wraw[RW][NCH];
#pragma unroll
  for (int r = 0; r < RW; r++)
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      const int c = lane + i * 64;
      const int row = min(row0 + r, n - 1);
      if (c < nchunks) wraw[r][i] = __builtin_nontemporal_load((const i32x4*)(w + (int64_t)row * k + c * 8));
    }
  float acc[RW][MAXB];
#pragma unroll
  for (int r = 0; r < RW; r++)
#pragma unroll
    for (int b = 0; b < MAXB; b++) acc[r][b] = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; i++) {
    const int c = lane + i * 64;
    if (c < nchunks) {
#pragma unroll
      for (int b = 0; b < MAXB; b++) {
        if (b < batch) {
          float ft[8];
          unpack8(*(const i32x4*)(temb + (int64_t)b * k + c * 8), ft);
#pragma unroll
          for (int e = 0; e < 8; e++) ft[e] = hdit::silu_f(ft[e]);
#pragma unroll
          for (int r = 0; r < RW; r++) {
            float fw[8];
            unpack8(wraw[r][i], fw);
#pragma unroll
            for (int e = 0; e < 8; e++) acc[r][b] += fw[e] * ft[e];
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RW; r++) {
    const int row = row0 + r;
    if (row >= n) break;
    const float bv = bias ? (float)bias[row] : 0.f;
#pragma unroll
    for (int b = 0; b < MAXB; b++) {
      if (b < batch) {
        float v = wave_sum(acc[r][b]);
        if (lane == 0) out[(int64_t)b * n + row] = v + bv;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Per-head QK norm (RMS / LayerNorm) + rotate-pairs RoPE, in place.
// A head vector of HD elements is held by HD/8 adjacent lanes (8 elements each).
// ---------------------------------------------------------------------------
struct QkJobs {
  int count;
  hdit_qknorm_job j[4];
};

// A thread works on chunk c of NH heads of one row (heads h, h + heads/NH, ...): the cos / sin values of the chunk,
// which are the same for every head of a row and four times the bytes of the chunk itself, are fetched once per
// NH head vectors, and NH loads are in flight per lane.
template <int HD, int NH>
__global__ void __launch_bounds__(256) qk_norm_rope_kernel(const QkJobs jobs, int batch, int heads, float eps) {
  constexpr int LPH = HD / 8;  // lanes per head vector
  const hdit_qknorm_job& job = jobs.j[blockIdx.y];
  const int hs = heads / NH;   // heads per pass over a row
  const int per_row = hs * LPH;
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = tid / per_row;
  if (row >= (int64_t)batch * job.seq) return;
  const int rem = (int)(tid - row * per_row);
  const int h0 = rem / LPH;
  const int c = rem % LPH;  // = threadIdx.x % LPH (per_row and 256 are multiples of LPH): a head's lanes sit side by side in one wave
  const int s = (int)(row % job.seq);
  const int b = (int)(row / job.seq);
  __bf16* p = (__bf16*)job.x + b * job.stride_b + s * job.stride_s + h0 * job.stride_h + c * 8;
  const int64_t hstep = (int64_t)hs * job.stride_h;
  i32x4 raw[NH];
#pragma unroll
  for (int n = 0; n < NH; n++) raw[n] = *(const i32x4*)(p + n * hstep);
  const int rr = s - job.rope_row0;
  const bool rope = job.cos_table && rr >= 0 && rr < job.rope_rows;
  float cs[8], sn[8];
  if (rope) {
    const float* cp = job.cos_table + (int64_t)rr * HD + c * 8;
    const float* sp = job.sin_table + (int64_t)rr * HD + c * 8;
    const f32x4 c0 = *(const f32x4*)cp, c1 = *(const f32x4*)(cp + 4);
    const f32x4 s0 = *(const f32x4*)sp, s1 = *(const f32x4*)(sp + 4);
#pragma unroll
    for (int e = 0; e < 4; e++) cs[e] = c0[e], cs[e + 4] = c1[e], sn[e] = s0[e], sn[e + 4] = s1[e];
  }
  float w[8], wb[8];
  if (job.norm_kind != 0 && job.weight) unpack8(*(const i32x4*)((const __bf16*)job.weight + c * 8), w);
  if (job.norm_kind != 0 && job.bias) unpack8(*(const i32x4*)((const __bf16*)job.bias + c * 8), wb);
#pragma unroll
  for (int n = 0; n < NH; n++) {
    float f[8];
    unpack8(raw[n], f);
    if (job.norm_kind == 1) {
      float q = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) q += f[e] * f[e];
#pragma unroll
      for (int off = LPH / 2; off > 0; off >>= 1) q += __shfl_xor(q, off, 64);
      float r = rsqrtf(q * (1.0f / HD) + eps);
#pragma unroll
      for (int e = 0; e < 8; e++) f[e] *= r;
    } else if (job.norm_kind == 2) {
      float sm = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) sm += f[e];
#pragma unroll
      for (int off = LPH / 2; off > 0; off >>= 1) sm += __shfl_xor(sm, off, 64);
      float mean = sm * (1.0f / HD);
      float q = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        f[e] -= mean;
        q += f[e] * f[e];
      }
#pragma unroll
      for (int off = LPH / 2; off > 0; off >>= 1) q += __shfl_xor(q, off, 64);
      float r = rsqrtf(q * (1.0f / HD) + eps);
#pragma unroll
      for (int e = 0; e < 8; e++) f[e] *= r;
    }
    if (job.norm_kind != 0) {
      if (job.weight) {
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] *= w[e];
      }
      if (job.bias) {
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] += wb[e];
      }
    }
    if (rope) {
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        o[e] = f[e] * cs[e] - f[e + 1] * sn[e];
        o[e + 1] = f[e + 1] * cs[e + 1] + f[e] * sn[e + 1];
      }
#pragma unroll
      for (int e = 0; e < 8; e++) f[e] = o[e];
    }
    *(i32x4*)(p + n * hstep) = pack8(f);
  }
}

__global__ void __launch_bounds__(256) copy_rows_kernel(const __bf16* __restrict__ src, __bf16* __restrict__ dst,
                                                        int64_t total_chunks, int tokens, int chunks_per_row,
                                                        int64_t src_sb, int64_t src_st, int64_t dst_sb,
                                                        int64_t dst_st) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total_chunks) return;
  int64_t row = i / chunks_per_row;
  int c = (int)(i - row * chunks_per_row);
  int64_t b = row / tokens, t = row - b * tokens;
  i32x4 v = __builtin_nontemporal_load((const i32x4*)(src + b * src_sb + t * src_st + c * 8));
  __builtin_nontemporal_store(v, (i32x4*)(dst + b * dst_sb + t * dst_st + c * 8));
}

inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_layernorm_modulate_jobs(const hdit_ln_job* jobs, int count, int dim, const void* ln_weight,
                                            const void* ln_bias, float eps, void* stream) {
  if (!jobs || count <= 0 || count > HDIT_LN_MAX_JOBS || dim <= 0) return HDIT_EINVAL;
  if (dim % 8) return HDIT_EINVAL;
  if (dim > 8192) return HDIT_EUNSUPPORTED;
  if (!aligned16(ln_weight) || !aligned16(ln_bias)) return HDIT_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  // jobs that read a bf16 tensor and jobs that read the fp32 residual stream run as separate launches
  for (int f32 = 0; f32 < 2; f32++) {
    LnJobs tab;
    tab.count = 0;
    int64_t blocks = 0;
    bool any_delta = false;
    for (int i = 0; i < count; i++) {
      const hdit_ln_job& j = jobs[i];
      if (j.batch < 0 || j.tokens < 0) return HDIT_EINVAL;
      if ((j.x_f32 != 0) != (f32 != 0)) continue;
      const int64_t rows = (int64_t)j.batch * j.tokens;
      if (rows == 0) continue;  // an empty tensor may come with a null pointer
      if (!j.x || !j.y) return HDIT_EINVAL;
      if (j.x_sb % 8 || j.x_st % 8 || j.y_sb % 8 || j.y_st % 8 || j.mod_stride % 4) return HDIT_EINVAL;
      if (!aligned16(j.x) || !aligned16(j.y) || !aligned16(j.shift) || !aligned16(j.scale)) return HDIT_EINVAL;
      if (j.delta_y) {
        // a pending update of the fp32 stream: x' = x + gate * delta_y, optionally written back
        if (!f32 || !j.delta_gate) return HDIT_EINVAL;
        if (j.d_sb % 8 || j.d_st % 8 || j.gate_stride % 4 || j.xo_sb % 4 || j.xo_st % 4) return HDIT_EINVAL;
        if (!aligned16(j.delta_y) || !aligned16(j.delta_gate) || !aligned16(j.x_out)) return HDIT_EINVAL;
        any_delta = true;
      } else if (j.x_out || j.delta_gate) {
        return HDIT_EINVAL;
      }
      tab.block_start[tab.count] = (int)blocks;
      tab.j[tab.count++] = j;
      blocks += (int64_t)j.batch * ((j.tokens + 3) / 4);  // four rows of one batch element per workgroup
      if (blocks > 0x7fffffff) return HDIT_EUNSUPPORTED;
    }
    if (tab.count == 0) continue;
    for (int i = tab.count; i <= HDIT_LN_MAX_JOBS; i++) tab.block_start[i] = (int)blocks;
    dim3 grid((unsigned)blocks), block(256);
    if (f32 && dim > 4096) return HDIT_EUNSUPPORTED;  // a row of the fp32 stream is held in registers: 16 chunks per lane
    const int nch = (dim / (f32 ? 4 : 8) + 63) / 64;
    const size_t lds_bytes = (size_t)dim * (any_delta ? 12 : 8);  // scale | shift (| gate) of one batch element, fp32
#define LN_LAUNCH(N)                                                                                                  \
  do {                                                                                                                \
    if (f32 && any_delta)                                                                                             \
      hipLaunchKernelGGL((ln_modulate_kernel<N, true, true>), grid, block, lds_bytes, s, tab,                         \
                         (const __bf16*)ln_weight, (const __bf16*)ln_bias, dim, eps);                                 \
    else if (f32)                                                                                                     \
      hipLaunchKernelGGL((ln_modulate_kernel<N, true, false>), grid, block, lds_bytes, s, tab,                        \
                         (const __bf16*)ln_weight, (const __bf16*)ln_bias, dim, eps);                                 \
    else                                                                                                              \
      hipLaunchKernelGGL((ln_modulate_kernel<N, false, false>), grid, block, lds_bytes, s, tab,                       \
                         (const __bf16*)ln_weight, (const __bf16*)ln_bias, dim, eps);                                 \
  } while (0)
    if (nch <= 1) LN_LAUNCH(1);
    else if (nch <= 2) LN_LAUNCH(2);
    else if (nch <= 3) LN_LAUNCH(3);
    else if (nch <= 4) LN_LAUNCH(4);
    else if (nch <= 6) LN_LAUNCH(6);
    else if (nch <= 8) LN_LAUNCH(8);
    else if (nch <= 12) LN_LAUNCH(12);
    else LN_LAUNCH(16);
#undef LN_LAUNCH
    const int rc = hdit_host::check_launch("hdit_layernorm_modulate");
    if (rc != HDIT_OK) return rc;
  }
  return HDIT_OK;
}

extern "C" __attribute__((visibility("default"))) int hdit_layernorm_modulate(const void* x, void* y, const float* shift, const float* scale,
                                       const void* ln_weight, const void* ln_bias, int batch, int tokens, int dim,
                                       int64_t x_sb, int64_t x_st, int64_t y_sb, int64_t y_st, int64_t mod_stride,
                                       float eps, void* stream) {
  hdit_ln_job j;
  memset(&j, 0, sizeof(j));
  j.x = x, j.y = y, j.shift = shift, j.scale = scale;
  j.batch = batch, j.tokens = tokens;
  j.x_f32 = 0, j.pad_ = 0;
  j.x_sb = x_sb, j.x_st = x_st, j.y_sb = y_sb, j.y_st = y_st, j.mod_stride = mod_stride;
  return hdit_layernorm_modulate_jobs(&j, 1, dim, ln_weight, ln_bias, eps, stream);
}

extern "C" __attribute__((visibility("default"))) int hdit_gate_residual(const void* x, const void* y, const float* gate, void* out, int batch, int tokens,
                                  int dim, int64_t x_sb, int64_t x_st, int64_t y_sb, int64_t y_st, int64_t o_sb,
                                  int64_t o_st, int64_t gate_stride, void* stream) {
  if (!x || !y || !gate || !out || batch < 0 || tokens < 0 || dim <= 0) return HDIT_EINVAL;
  if (dim % 8 || x_sb % 8 || x_st % 8 || y_sb % 8 || y_st % 8 || o_sb % 8 || o_st % 8 || gate_stride % 4)
    return HDIT_EINVAL;
  if (!aligned16(x) || !aligned16(y) || !aligned16(out) || !aligned16(gate)) return HDIT_EINVAL;
  int64_t total = (int64_t)batch * tokens * (dim / 8);
  if (total == 0) return HDIT_OK;
  hipLaunchKernelGGL(gate_residual_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __bf16*)x, (const __bf16*)y, gate, (__bf16*)out, total, tokens, dim / 8, x_sb, x_st, y_sb,
                     y_st, o_sb, o_st, gate_stride);
  return hdit_host::check_launch("hdit_gate_residual");
}

extern "C" __attribute__((visibility("default"))) int hdit_gelu_tanh(const void* x, const void* bias, void* y, int64_t rows, int dim, int64_t ldx,
                              int64_t ldy, void* stream) {
  if (!x || !y || rows < 0 || dim <= 0 || dim % 8 || ldx % 8 || ldy % 8) return HDIT_EINVAL;
  if (!aligned16(x) || !aligned16(y) || !aligned16(bias)) return HDIT_EINVAL;
  int64_t total = rows * (dim / 8);
  if (total == 0) return HDIT_OK;
  hipLaunchKernelGGL(gelu_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __bf16*)x, (const __bf16*)bias, (__bf16*)y, total, dim / 8, ldx, ldy);
  return hdit_host::check_launch("hdit_gelu_tanh");
}

extern "C" __attribute__((visibility("default"))) int hdit_ff_activation(const void* x, void* y, int64_t rows, int dim, int64_t ldx, int64_t ldy,
                                  int kind, void* stream) {
  if (!x || !y || rows < 0 || dim <= 0 || dim % 8 || ldx % 8 || ldy % 8) return HDIT_EINVAL;
  if (!aligned16(x) || !aligned16(y)) return HDIT_EINVAL;
  if (kind != HDIT_ACT_GELU_ERF && kind != HDIT_ACT_GEGLU && kind != HDIT_ACT_SILU) return HDIT_EINVAL;
  if (ldx < (kind == HDIT_ACT_GEGLU ? 2 : 1) * (int64_t)dim || ldy < dim) return HDIT_EINVAL;
  // in place only where an element is read by the thread that writes it (not GEGLU: other threads read the gate half)
  if (x == y && kind == HDIT_ACT_GEGLU) return HDIT_EINVAL;
  const int64_t total = rows * (dim / 8);
  if (total == 0) return HDIT_OK;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  hipStream_t s = (hipStream_t)stream;
  if (kind == HDIT_ACT_GELU_ERF)
    hipLaunchKernelGGL(ff_activation_kernel<HDIT_ACT_GELU_ERF>, grid, block, 0, s, (const __bf16*)x, (__bf16*)y, total, dim / 8, ldx, ldy);
  else if (kind == HDIT_ACT_GEGLU)
    hipLaunchKernelGGL(ff_activation_kernel<HDIT_ACT_GEGLU>, grid, block, 0, s, (const __bf16*)x, (__bf16*)y, total, dim / 8, ldx, ldy);
  else
    hipLaunchKernelGGL(ff_activation_kernel<HDIT_ACT_SILU>, grid, block, 0, s, (const __bf16*)x, (__bf16*)y, total, dim / 8, ldx, ldy);
  return hdit_host::check_launch("hdit_ff_activation");
}

extern "C" __attribute__((visibility("default"))) int hdit_adaln_gemv(const void* temb, const void* w, const void* bias, float* out, int batch, int n, int k,
                               void* stream) {
  if (!temb || !w || !out || batch <= 0 || n <= 0 || k <= 0) return HDIT_EINVAL;
  if (batch > 8) return HDIT_EUNSUPPORTED;
  if (k % 8 || !aligned16(temb) || !aligned16(w)) return HDIT_EINVAL;
  if (k > 8 * 512) return HDIT_EUNSUPPORTED;
  dim3 grid((n + 15) / 16), block(256);  // 4 waves x 4 rows
  hipStream_t s = (hipStream_t)stream;
  const int nch = (k / 8 + 63) / 64;
#define GEMV_LAUNCH(MB, NC)                                                                                    \
  hipLaunchKernelGGL((adaln_gemv_kernel<MB, NC>), grid, block, 0, s, (const __bf16*)temb, (const __bf16*)w, \
                     (const __bf16*)bias, out, batch, n, k)
  if (batch <= 2) {
    if (nch <= 1) GEMV_LAUNCH(2, 1);
    else if (nch <= 3) GEMV_LAUNCH(2, 3);
    else if (nch <= 6) GEMV_LAUNCH(2, 6);
    else GEMV_LAUNCH(2, 8);
  } else {
    if (nch <= 1) GEMV_LAUNCH(8, 1);
    else if (nch <= 3) GEMV_LAUNCH(8, 3);
    else if (nch <= 6) GEMV_LAUNCH(8, 6);
    else GEMV_LAUNCH(8, 8);
  }
#undef GEMV_LAUNCH
  return hdit_host::check_launch("hdit_adaln_gemv");
}

extern "C" __attribute__((visibility("default"))) int hdit_qk_norm_rope(const hdit_qknorm_job* jobs, int count, int batch, int heads, int head_dim, float eps,
                                 void* stream) {
  if (!jobs || count <= 0 || count > 4 || batch <= 0 || heads <= 0) return HDIT_EINVAL;
  if (head_dim != 64 && head_dim != 128) return HDIT_EUNSUPPORTED;
  QkJobs tab;
  tab.count = count;
  int64_t max_vec = 0;
  for (int i = 0; i < count; i++) {
    const hdit_qknorm_job& j = jobs[i];
    if (!j.x || j.seq < 0 || j.norm_kind < 0 || j.norm_kind > 2) return HDIT_EINVAL;
    if (j.stride_b % 8 || j.stride_s % 8 || j.stride_h % 8 || !aligned16(j.x)) return HDIT_EINVAL;
    if (!aligned16(j.weight) || !aligned16(j.bias) || !aligned16(j.cos_table) || !aligned16(j.sin_table))
      return HDIT_EINVAL;
    if (j.cos_table && !j.sin_table) return HDIT_EINVAL;
    // the table must cover every row from rope_row0 on: a short table would leave rows silently unrotated
    if (j.cos_table && (j.rope_row0 < 0 || j.seq - j.rope_row0 > j.rope_rows)) return HDIT_EINVAL;
    tab.j[i] = j;
    int64_t nv = (int64_t)batch * j.seq * heads;
    if (nv > max_vec) max_vec = nv;
  }
  if (max_vec == 0) return HDIT_OK;
  const int lph = head_dim / 8;
  const int nh = heads % 4 == 0 ? 4 : heads % 2 == 0 ? 2 : 1;  // head vectors per thread
  const int64_t threads = max_vec / nh * lph;
  dim3 grid((unsigned)((threads + 255) / 256), count), block(256);
#define QK_LAUNCH(HD, NH) \
  hipLaunchKernelGGL((qk_norm_rope_kernel<HD, NH>), grid, block, 0, (hipStream_t)stream, tab, batch, heads, eps)
  if (head_dim == 64) {
    if (nh == 4) QK_LAUNCH(64, 4);
    else if (nh == 2) QK_LAUNCH(64, 2);
    else QK_LAUNCH(64, 1);
  } else {
    if (nh == 4) QK_LAUNCH(128, 4);
    else if (nh == 2) QK_LAUNCH(128, 2);
    else QK_LAUNCH(128, 1);
  }
#undef QK_LAUNCH
  return hdit_host::check_launch("hdit_qk_norm_rope");
}

extern "C" __attribute__((visibility("default"))) int hdit_copy_rows(const void* src, void* dst, int batch, int tokens, int dim, int64_t src_sb,
                              int64_t src_st, int64_t dst_sb, int64_t dst_st, void* stream) {
  if (!src || !dst || batch < 0 || tokens < 0 || dim <= 0 || dim % 8) return HDIT_EINVAL;
  if (src_sb % 8 || src_st % 8 || dst_sb % 8 || dst_st % 8 || !aligned16(src) || !aligned16(dst)) return HDIT_EINVAL;
  int64_t total = (int64_t)batch * tokens * (dim / 8);
  if (total == 0) return HDIT_OK;
  hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __bf16*)src, (__bf16*)dst, total, tokens, dim / 8, src_sb, src_st, dst_sb, dst_st);
  return hdit_host::check_launch("hdit_copy_rows");
}
