// Joint (image + text) flash attention forward for gfx950, bf16 in/out.
//
// Work split: one workgroup = 4 waves = 256 query rows of one (batch, head);
// each wave owns 64 query rows (two 32-row MFMA column blocks) and walks the
// keys in tiles of 64.  K and V tiles are staged global -> registers -> LDS in
// two buffers (one barrier per tile).
//
// The scores are produced transposed, S^T = K . Q^T, with K rows as the MFMA
// "A" operand and the wave's Q rows (held in registers for the whole kernel)
// as the "B" operand.  In the 32x32 accumulator layout a lane then owns ONE
// query column and 16 keys per block, so the online-softmax row max / row sum
// are in-lane reductions plus a single exchange between lane l and l^32, and
// the rescale factor is a per-lane scalar.  The same accumulator registers,
// rounded to bf16, are directly the "B" operand (P^T, 16 keys per step) of
// O^T = V^T . P^T; the matching V^T "A" fragments are fetched from the
// row-major V tile with the LDS transpose read (ds_read_b64_tr_b16), choosing
// key rows in the order the accumulator layout dictates.
//
// Q, K, V, O are each up to two sequence segments in different buffers, so the
// joint [image, text] / [text, image] sequences and the "fresh text + stale
// image buffer" K/V of a PipeFusion patch need no concatenation copy.
#include "hdit_common.h"

namespace {

constexpr int BKV = 64;   // keys per tile
constexpr int WQ = 64;    // query rows per wave
constexpr int NWAVE = 4;
constexpr int BQ = WQ * NWAVE;

struct Seg2 {
  const __bf16* p0;
  const __bf16* p1;
  int64_t sb0, ss0, sh0, sb1, ss1, sh1;
  int len0, len1;
};

__device__ __forceinline__ const __bf16* row_ptr(const Seg2& s, int b, int h, int r) {
  // r must be < len0 + len1
  if (r < s.len0) return s.p0 + b * s.sb0 + (int64_t)r * s.ss0 + h * s.sh0;
  return s.p1 + b * s.sb1 + (int64_t)(r - s.len0) * s.ss1 + h * s.sh1;
}

struct AttnParams {
  Seg2 q, k, v, o;
  int heads, sq, skv;
  float scale_log2;
};

template <int HD>
struct Lds {
  static constexpr int K_ROW = HD * 2 + 16;  // bytes; +16 keeps 8 consecutive rows on distinct banks
  static constexpr int V_ROW = HD * 2 + 32;  // +32: the 4 key rows of one transpose read hit distinct banks
  static constexpr int K_BYTES = BKV * K_ROW;
  static constexpr int V_BYTES = BKV * V_ROW;
  static constexpr int STAGE = K_BYTES + V_BYTES;
  static constexpr int TOTAL = 2 * STAGE;
};

template <int HD>
__global__ void __launch_bounds__(256, (HD == 64 ? 2 : 1)) attn_fwd_kernel(const AttnParams P, int q_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using L = Lds<HD>;
  constexpr int KS = HD / 16;       // k-steps of the S^T MFMA (over head dim)
  constexpr int DB = HD / 32;       // 32-wide d blocks of O^T
  constexpr int CPR = HD / 8;       // 16-byte chunks per row
  constexpr int NCH = BKV * CPR / 256;  // chunks per thread per tile (K and V each)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int qt = blockIdx.x % q_tiles;
  const int bh = blockIdx.x / q_tiles;
  const int b = bh / P.heads, h = bh % P.heads;
  const int q0 = qt * BQ + wave * WQ;

  // ---- Q fragments: lane holds q row (qb*32 + l32), d = 16*ks + 8*lh .. +7
  bf16x8 qf[2][KS];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    int r = min(q0 + qb * 32 + l32, P.sq - 1);
    const __bf16* rp = row_ptr(P.q, b, h, r);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[qb][ks] = *(const bf16x8*)(rp + ks * 16 + lh * 8);
  }

  // ---- K/V tile staging
  i32x4 kreg[NCH], vreg[NCH];
  auto load_tile = [&](int t) {
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      int c = tid + i * 256, row = c / CPR, cc = c % CPR;
      int r = min(t * BKV + row, P.skv - 1);
      kreg[i] = *(const i32x4*)(row_ptr(P.k, b, h, r) + cc * 8);
      vreg[i] = *(const i32x4*)(row_ptr(P.v, b, h, r) + cc * 8);
    }
  };
  auto store_tile = [&](int stage) {
    unsigned char* base = lds + stage * L::STAGE;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      int c = tid + i * 256, row = c / CPR, cc = c % CPR;
      *(i32x4*)(base + row * L::K_ROW + cc * 16) = kreg[i];
      *(i32x4*)(base + L::K_BYTES + row * L::V_ROW + cc * 16) = vreg[i];
    }
  };

  f32x16 oacc[DB][2];
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[i][j][v] = 0.f;
  float m_run[2] = {-INFINITY, -INFINITY};
  float l_run[2] = {0.f, 0.f};

  // lane-constant part of the V^T transpose-read address:
  // 16-lane group G = lane/16, x = lane%16: key row 4*(G/2) + x/4, column 16*(G%2) + 4*(x%4)
  const int vt_off = (4 * (lane >> 5) + ((lane & 15) >> 2)) * L::V_ROW + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

  const int NT = (P.skv + BKV - 1) / BKV;
  load_tile(0);
  store_tile(0);
  __syncthreads();
  if (NT > 1) load_tile(1);

  for (int t = 0; t < NT; t++) {
    const unsigned char* sk = lds + (t & 1) * L::STAGE;
    const unsigned char* sv = sk + L::K_BYTES;

    // ---- S^T[kb][qb] = K_tile . Q^T
    f32x16 sacc[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
#pragma unroll
        for (int v = 0; v < 16; v++) sacc[kb][qb][v] = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; kb++) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        bf16x8 kf = *(const bf16x8*)(sk + (kb * 32 + l32) * L::K_ROW + (ks * 2 + lh) * 16);
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
          sacc[kb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], sacc[kb][qb], 0, 0, 0);
      }
    }

    // ---- mask keys past the end (last tile only)
    if (t == NT - 1 && (P.skv % BKV) != 0) {
      const int valid = P.skv - t * BKV;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          int key = kb * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
          if (key >= valid) {
            sacc[kb][0][v] = -INFINITY;
            sacc[kb][1][v] = -INFINITY;
          }
        }
    }

    // ---- online softmax (log2 domain); P^T rounded to bf16 in place
    bf16x8 pf[2][4];  // [qb][u], u = 2*kb + half: 16 keys per PV k-step
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      float mx = sacc[0][qb][0];
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int v = 0; v < 16; v++) mx = fmaxf(mx, sacc[kb][qb][v]);
      auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(mx), __float_as_int(mx), false, false);
      mx = fmaxf(__int_as_float(sw[0]), __int_as_float(sw[1]));
      const float m_new = fmaxf(m_run[qb], mx * P.scale_log2);
      const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_new);
      m_run[qb] = m_new;
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
          p[v] = __builtin_amdgcn_exp2f(sacc[kb][qb][v] * P.scale_log2 - m_new);
          rs += p[v];
        }
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
          i32x4 pk;
#pragma unroll
          for (int e = 0; e < 4; e++) pk[e] = (int)hdit::pack2(p[hh * 8 + 2 * e], p[hh * 8 + 2 * e + 1]);
          pf[qb][kb * 2 + hh] = __builtin_bit_cast(bf16x8, pk);
        }
      }
      l_run[qb] = l_run[qb] * alpha + rs;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[db][qb][v] *= alpha;
    }

    // ---- O^T[db][qb] += V^T . P^T
#pragma unroll
    for (int u = 0; u < 4; u++) {
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const unsigned char* va = sv + vt_off + (u * 16) * L::V_ROW + db * 64;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(va));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3)))*)(va + 8 * L::V_ROW));
        typedef __attribute__((ext_vector_type(8))) short s16x8;
        s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        bf16x8 vf = __builtin_bit_cast(bf16x8, both);
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
          oacc[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qb][u], oacc[db][qb], 0, 0, 0);
      }
    }

    if (t + 1 < NT) store_tile((t + 1) & 1);
    __syncthreads();
    if (t + 2 < NT) load_tile(t + 2);
  }

  // ---- normalise and write O[q][d]: lane owns q = qb*32 + l32, d = 32*db + 8*(v/4) + 4*lh + v%4
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(l_run[qb]), __float_as_int(l_run[qb]), false, false);
    const float inv = 1.0f / (__int_as_float(sw[0]) + __int_as_float(sw[1]));
    const int r = q0 + qb * 32 + l32;
    if (r >= P.sq) continue;
    __bf16* op = (__bf16*)row_ptr(P.o, b, h, r);
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        i32x2 out;
        out[0] = (int)hdit::pack2(oacc[db][qb][g * 4 + 0] * inv, oacc[db][qb][g * 4 + 1] * inv);
        out[1] = (int)hdit::pack2(oacc[db][qb][g * 4 + 2] * inv, oacc[db][qb][g * 4 + 3] * inv);
        *(i32x2*)(op + db * 32 + g * 8 + lh * 4) = out;
      }
  }
}

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

extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_bf16(const hdit_attn_args* a, void* stream) {
  int rc = hdit_host::attn_validate(a);
  if (rc != HDIT_OK) return rc;
  AttnParams P;
  P.q = make_seg(a->q);
  P.k = make_seg(a->k);
  P.v = make_seg(a->v);
  P.o = make_seg(a->o);
  P.heads = a->heads;
  P.sq = a->q[0].len + a->q[1].len;
  P.skv = a->k[0].len + a->k[1].len;
  if (P.sq == 0) return HDIT_OK;
  float scale = a->scale > 0.f ? a->scale : 1.0f / sqrtf((float)a->head_dim);
  P.scale_log2 = scale * 1.4426950408889634f;
  int q_tiles = (P.sq + BQ - 1) / BQ;
  dim3 grid((unsigned)(q_tiles * a->batch * a->heads)), block(256);
  hipStream_t s = (hipStream_t)stream;
  if (a->head_dim == 64) {
    hipLaunchKernelGGL(attn_fwd_kernel<64>, grid, block, Lds<64>::TOTAL, s, P, q_tiles);
  } else {
    static bool attr = false;
    if (!attr) {
      if (hipFuncSetAttribute((const void*)attn_fwd_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              Lds<128>::TOTAL) != hipSuccess)
        return HDIT_ELAUNCH;
      attr = true;
    }
    hipLaunchKernelGGL(attn_fwd_kernel<128>, grid, block, Lds<128>::TOTAL, s, P, q_tiles);
  }
  return hdit_host::check_launch("hdit_attn_fwd_bf16");
}
