// fp8 (OCP e4m3) variant of the joint flash attention for gfx950.
//
// Same work split and softmax as the bf16 kernel (S^T = K . Q^T so that a lane
// owns one query column; O^T = V^T . P^T), but every MFMA is the 64-deep
// v_mfma_scale_f32_32x32x64_f8f6f4 with unit block scales:
//   * Q, K, V are quantised with one scale per (batch, head):
//     x8 = x * 448 / absmax(x)  (absmax from hdit_attn_absmax, clamped away
//     from zero).  K and V are quantised ONCE by a pre-pass into a caller
//     workspace laid out [batch, head, key (padded to 64), d] (every query
//     tile would otherwise repeat the conversion); Q is quantised as its
//     fragments are loaded;
//   * the scores are de-scaled by the MFMA itself.  With d = 64 the Q scale is chosen (within a factor of two
//     below the full-range one, which costs e4m3 nothing but headroom) so that softmax scale * log2(e) *
//     de-quantisation factor of q and k is an exact power of two, and that power goes into the block-scale
//     operand of the score MFMA; the running reference (and the +7 of the next item) is subtracted by letting
//     the MFMA accumulate onto a vector holding it.  The accumulators then feed exp2 directly: no per-score
//     multiply-add in a loop whose matrix and vector time add up.  (d = 128 has no registers for that vector and
//     keeps the multiply-add.)
//   * P is re-quantised per tile as exp2(s - m + 7): at most 2^8 = 256 < 448
//     with the running maximum allowed to lag by one power of two, so small
//     probabilities keep normal-range e4m3 precision;
//   * O is de-scaled by absmax_v / 448 when it is normalised.
// In the 32x32 accumulator layout a lane's 32 score registers are exactly its
// 32 bytes of the P^T "B" operand; the matching V^T "A" bytes are gathered from
// the row-major fp8 V tile with the byte transpose read (ds_read_b64_tr_b8).
#include <atomic>
#include <type_traits>

#include "hdit_common.h"

typedef __attribute__((ext_vector_type(8))) int i32x8;

namespace {

constexpr int BKV = 64;
constexpr int WQ = 64;
constexpr int NWAVE = 4;
constexpr int BQ = WQ * NWAVE;
constexpr float FP8_MAX = 448.0f;
constexpr float P_SHIFT = 7.0f;            // P is stored as 2^7 * exp2(s - m)
constexpr float RESCALE_THRESHOLD = 1.0f;  // running max may lag by 2^1: P <= 2^8

struct Seg2 {
  const __bf16* p0;
  const __bf16* p1;
  int64_t sb0, ss0, sh0, sb1, ss1, sh1;
  int len0, len1;
};

__device__ __forceinline__ const __bf16* row_ptr(const Seg2& s, int b, int h, int r) {
  if (r < s.len0) return s.p0 + b * s.sb0 + (int64_t)r * s.ss0 + h * s.sh0;
  return s.p1 + b * s.sb1 + (int64_t)(r - s.len0) * s.ss1 + h * s.sh1;
}

struct AttnParams {
  Seg2 q, k, v, o;
  const float* absmax;  // [3][batch][heads]
  unsigned char* k8;    // fp8 [batch][heads][skv_pad][head_dim]
  unsigned char* v8;
  int batch, heads, sq, skv, skv_pad;
  float scale;
};

// 8 bf16 (one 16-byte chunk) -> 8 fp8 in two dwords, scaled and clamped to the finite e4m3 range
__device__ __forceinline__ i32x2 quant8(const i32x4& raw, float s) {
  float f[8];
  hdit::unpack8(raw, f);
#pragma unroll
  for (int e = 0; e < 8; e++) f[e] = fminf(fmaxf(f[e] * s, -FP8_MAX), FP8_MAX);
  i32x2 r;
  int w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w, true);
  r[0] = w;
  w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w, true);
  r[1] = w;
  return r;
}

// K and V tiles (64 keys x HD bytes each) go straight from the pre-quantised workspace into LDS
// (global_load_lds_dwordx4: no staging registers, no ds_write), which lands a wave's 64 x 16 bytes contiguously:
// unpadded rows of HD bytes.  The spread over the 256-byte bank window comes from XOR swizzles of the 16-byte
// chunk index, applied on the source side.  A ds_read_b128 pass covers 16 consecutive K rows, which must fall on
// 16 distinct chunk slots: slot p of K row r holds chunk p ^ xk(r).  A transpose-read pass covers, per half wave,
// key rows {0..3, 8..11} (or {4..7, 12..15}) x 32 bytes, which must fall on distinct 32-byte pieces: slot p of V
// row r holds chunk p ^ xv(r), xv even (it moves whole 32-byte pieces).
template <int HD>
struct Lds8 {
  static constexpr int K_ROW = HD;
  static constexpr int V_ROW = HD;
  static constexpr int K_BYTES = BKV * K_ROW;
  static constexpr int V_BYTES = BKV * V_ROW;
  static constexpr int STAGE = K_BYTES + V_BYTES;
  static constexpr int TOTAL = 2 * STAGE;
  __device__ static constexpr int xk(int r) { return HD == 64 ? ((r >> 2) & 3) : ((r >> 1) & 7); }
  __device__ static constexpr int xv(int r) { return HD == 64 ? 2 * ((r >> 3) & 1) : 2 * (((r >> 1) & 1) | (((r >> 3) & 1) << 1)); }
};

// One wave-wide direct-to-LDS copy: lane l's 16 bytes land at LDS byte address lds_addr + 16*l.  Inline
// assembly, so the compiler's wait-count bookkeeping does not see it; the tile loop waits for it explicitly.
__device__ __forceinline__ void lds_dma16(const unsigned char* base_uniform, unsigned voff, unsigned lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr_uniform), "v"(voff), "s"(base_uniform)
               : "m0", "memory");
}
__device__ __forceinline__ unsigned lds_address(const unsigned char* p) {
  return (unsigned)(uintptr_t)((const __attribute__((address_space(3))) unsigned char*)p);
}

template <int HD>
__global__ void __launch_bounds__(256, (HD == 64 ? 2 : 1)) attn_fp8_kernel(const AttnParams P, int q_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using L = Lds8<HD>;
  constexpr int KS = HD / 64;  // 64-deep k-steps of the score MFMA
  constexpr int DB = HD / 32;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  // Workgroups go to the 8 XCDs round-robin by id, and each XCD has its own L2: all query tiles of one
  // (batch, head) run on one XCD, so that its K and V are fetched into one L2 instead of eight.
  int qt = blockIdx.x % q_tiles;
  int bh = blockIdx.x / q_tiles;
  if ((P.batch * P.heads) % 8 == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    qt = slot % q_tiles;
    bh = (slot / q_tiles) * 8 + xcd;
  }
  const int b = bh / P.heads, h = bh % P.heads;
  const int q0 = qt * BQ + wave * WQ;

  const int nbh = P.batch * P.heads;
  const float amq = fmaxf(P.absmax[bh], 1e-20f);
  const float amk = fmaxf(P.absmax[nbh + bh], 1e-20f);
  const float amv = fmaxf(P.absmax[2 * nbh + bh], 1e-20f);
  constexpr bool FOLD = HD == 64;
  // score = f * (q8 . k8), f = softmax scale * log2(e) * amk / (448 * qs).  FOLD: qs = full-range scale * f0 / 2^e
  // with e = ceil(log2 f0), so that f = 2^e exactly and 2^e rides the MFMA's E8M0 block scale of the Q operand.
  float qs = FP8_MAX / amq;
  float scale_log2 = P.scale * 1.4426950408889634f * (amq / FP8_MAX) * (amk / FP8_MAX);
  int q_block_scale = 0x7f7f7f7f;  // E8M0 127 = 2^0 in every byte
  if constexpr (FOLD) {
    int e = (int)ceilf(log2f(scale_log2));
    e = max(-126, min(127, e));
    const float pow2 = exp2f((float)e);
    qs *= fminf(scale_log2 / pow2, 1.0f);
    scale_log2 = pow2;
    q_block_scale = 0x01010101 * (127 + e);
  }
  const float o_descale = amv / FP8_MAX;

  // ---- Q fragments: lane holds q row qb*32 + l32, bytes d = 64*ks + 32*lh .. +31
  i32x8 qf[2][KS];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    int r = min(q0 + qb * 32 + l32, P.sq - 1);
    const __bf16* rp = row_ptr(P.q, b, h, r);
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        i32x2 q8 = quant8(*(const i32x4*)(rp + ks * 64 + lh * 32 + c * 8), qs);
        qf[qb][ks][2 * c] = q8[0];
        qf[qb][ks][2 * c + 1] = q8[1];
      }
  }

  // K/V tiles come from the pre-quantised workspace, 64 rows x HD bytes each: request i of a wave covers rows
  // RPR * (wave + 4 i) .. + RPR - 1, lane -> (row, slot lane % CPR8); the chunk fetched for a slot is the slot index
  // XORed with the row's swizzle.  Rows past the last key are zero in the workspace.
  constexpr int CPR8 = HD / 16;        // 16-byte chunks per row
  constexpr int RPR = 64 / CPR8;       // rows per request
  constexpr int NREQ = BKV / (RPR * NWAVE);
  const unsigned char* k8 = P.k8 + (size_t)bh * P.skv_pad * HD;
  const unsigned char* v8 = P.v8 + (size_t)bh * P.skv_pad * HD;
  unsigned koff[NREQ], voff[NREQ];
#pragma unroll
  for (int i = 0; i < NREQ; i++) {
    const int row = RPR * (wave + NWAVE * i) + lane / CPR8, slot = lane % CPR8;
    koff[i] = (unsigned)(row * HD + ((slot ^ L::xk(row)) << 4));
    voff[i] = (unsigned)(row * HD + ((slot ^ L::xv(row)) << 4));
  }
  const unsigned lds_base_addr = __builtin_amdgcn_readfirstlane(lds_address(lds));
  const unsigned wave_dst = lds_base_addr + __builtin_amdgcn_readfirstlane(wave) * 1024;
  auto dma_tile = [&](int t, int stage) {
    const unsigned char* kb = k8 + (size_t)t * BKV * HD;
    const unsigned char* vb = v8 + (size_t)t * BKV * HD;
    const unsigned kdst = wave_dst + stage * L::STAGE;
#pragma unroll
    for (int i = 0; i < NREQ; i++) {
      lds_dma16(kb, koff[i], kdst + i * NWAVE * 1024);
      lds_dma16(vb, voff[i], kdst + L::K_BYTES + i * NWAVE * 1024);
    }
  };

  f32x16 oacc[DB][2];
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[i][j][v] = 0.f;
  // FOLD: m_run is the running reference in log2 units (0 until the first tile sets it); the score accumulators
  // start from negm = P_SHIFT - m_run (one value in all 16 entries: a lane owns one query column per qb)
  float m_run[2] = {FOLD ? 0.f : -INFINITY, FOLD ? 0.f : -INFINITY};
  float l_run[2] = {0.f, 0.f};
  f32x16 negm[2];
#pragma unroll
  for (int qb = 0; qb < 2; qb++)
#pragma unroll
    for (int v = 0; v < 16; v++) negm[qb][v] = P_SHIFT;
  bool first = true;

  // byte-transpose read of V^T: in a 16-lane group lane x supplies the address of 8 bytes
  // (row = key of slot x>>1, column half x&1) and lane i receives byte i%8 of the rows of lanes 2j + i/8.
  // Slot jj of read r is key 16r + 8*(jj>>2) + 4*lh + (jj&3): the key order of a lane's accumulator bytes.
  const int jj = (lane & 15) >> 1;
  const int vt_row = 8 * (jj >> 2) + 4 * lh + (jj & 3);  // + 16 r: does not change the row's swizzle
  const int vt_base = vt_row * L::V_ROW + 8 * (lane & 1);
  const int vt_chunk = (lane >> 4) & 1;                  // + 2 db
  const int vt_swz = L::xv(vt_row);
  const int k_base = l32 * L::K_ROW;                       // + 32 kb rows: does not change the row's swizzle
  const int k_swz = L::xk(l32);
  const int unit_scale = 0x7f7f7f7f;  // E8M0 exponent 127 = 2^0 for every block

  auto tile_compute = [&](const unsigned char* sk, auto mask_tag, int valid, auto last_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr bool LAST = decltype(last_tag)::value;
    const unsigned char* sv = sk + L::K_BYTES;
    f32x16 sacc[2][2];
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < 2; kb++) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const unsigned char* ka = sk + k_base + kb * 32 * L::K_ROW;
        const int c0 = ks * 4 + lh * 2;  // this lane's 32 bytes are chunks c0, c0 + 1 of the row
        i32x4 lo = *(const i32x4*)(ka + ((c0 ^ k_swz) << 4)), hi = *(const i32x4*)(ka + (((c0 + 1) ^ k_swz) << 4));
        i32x8 kf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
          sacc[kb][qb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              kf, qf[qb][ks], ks == 0 ? (FOLD ? negm[qb] : zero16) : sacc[kb][qb], 0, 0, 0, unit_scale, 0, q_block_scale);
      }
    }
    if (MASK) {
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
    if constexpr (FOLD) {
      // the accumulators hold s - m + P_SHIFT; their column maxima, minus P_SHIFT, are relative to the reference
      float mrel[2];
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        float mx = fmaxf(sacc[0][qb][0], sacc[1][qb][0]);
#pragma unroll
        for (int v = 1; v < 16; v++) mx = fmaxf(mx, fmaxf(sacc[0][qb][v], sacc[1][qb][v]));
        auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(mx), __float_as_int(mx), false, false);
        mrel[qb] = fmaxf(__int_as_float(sw[0]), __int_as_float(sw[1])) - P_SHIFT;
      }
      const bool grow = first || mrel[0] > RESCALE_THRESHOLD || mrel[1] > RESCALE_THRESHOLD;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
          const float d = first ? mrel[qb] : fmaxf(mrel[qb], 0.f);
          m_run[qb] += d;
          if (!first) {
            const float alpha = __builtin_amdgcn_exp2f(-d);
            l_run[qb] *= alpha;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
              for (int v = 0; v < 16; v++) oacc[db][qb][v] *= alpha;
          }
#pragma unroll
          for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int v = 0; v < 16; v++) sacc[kb][qb][v] -= d;
#pragma unroll
          for (int v = 0; v < 16; v++) negm[qb][v] = P_SHIFT - m_run[qb];
        }
        first = false;
      }
    } else {
    float mcand[2];
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        float mx = fmaxf(sacc[0][qb][0], sacc[1][qb][0]);
#pragma unroll
        for (int v = 1; v < 16; v++) mx = fmaxf(mx, fmaxf(sacc[0][qb][v], sacc[1][qb][v]));
        auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(mx), __float_as_int(mx), false, false);
        mx = fmaxf(__int_as_float(sw[0]), __int_as_float(sw[1]));
        mcand[qb] = fmaxf(m_run[qb], mx * scale_log2);
      }
      const bool grow = (mcand[0] - m_run[0] > RESCALE_THRESHOLD) || (mcand[1] - m_run[1] > RESCALE_THRESHOLD);
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
          const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - mcand[qb]);
          m_run[qb] = mcand[qb];
          l_run[qb] *= alpha;
#pragma unroll
          for (int db = 0; db < DB; db++)
#pragma unroll
            for (int v = 0; v < 16; v++) oacc[db][qb][v] *= alpha;
        }
      }
    }
    i32x8 pf[2];  // [qb]: 32 bytes, byte e = 16*kb + v
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const float moff = m_run[qb] - P_SHIFT;
      float rs = l_run[qb];
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int w4 = 0; w4 < 4; w4++) {
          float p[4];
#pragma unroll
          for (int e = 0; e < 4; e++)
            p[e] = __builtin_amdgcn_exp2f(FOLD ? sacc[kb][qb][w4 * 4 + e] : __builtin_fmaf(sacc[kb][qb][w4 * 4 + e], scale_log2, -moff));
          int w = 0;
          w = __builtin_amdgcn_cvt_pk_fp8_f32(p[0], p[1], w, false);
          w = __builtin_amdgcn_cvt_pk_fp8_f32(p[2], p[3], w, true);
          pf[qb][kb * 4 + w4] = w;
          rs += (p[0] + p[1]) + (p[2] + p[3]);
        }
      l_run[qb] = rs;
    }
#pragma unroll
    for (int db = 0; db < DB; db++) {
      i32x8 vf;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const unsigned char* va = sv + vt_base + (16 * r) * L::V_ROW + (((2 * db + vt_chunk) ^ vt_swz) << 4);
        i32x2 t8 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((i32x2 __attribute__((address_space(3)))*)(va));
        vf[2 * r] = t8[0];
        vf[2 * r + 1] = t8[1];
      }
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
        oacc[db][qb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf, pf[qb], oacc[db][qb], 0, 0, 0, unit_scale, 0,
                                                                       unit_scale);
    }
    if constexpr (LAST) {
      // These PV MFMAs are 16-pass instructions and what follows the last tile reads their accumulators at once
      // (the compiler shuffles them into other registers for the output code).  The no-ops it puts in front of
      // that were seen to be too few for the last two registers of the last accumulator block -- wrong values in
      // exactly those output columns when the masked tile ran last -- so the distance is made explicit here, once
      // per workgroup.
      // (The accumulators are operands of the statement, so it sits behind the MFMAs that write them and in front
      // of every instruction that reads them.)  Regression case: tests/test_gpu_ops.py,
      // test_attention_fp8_masked_last_tile_tail_columns (constant-V outputs, masked last tile, both head sizes).
      // The other reads of an MFMA result in this kernel (the column maxima behind the score MFMAs, the
      // multiply-add of the d = 128 path) rely on the compiler's own wait states.
      if constexpr (DB == 2)
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(oacc[0][0]), "+v"(oacc[0][1]), "+v"(oacc[1][0]), "+v"(oacc[1][1]));
      else
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+v"(oacc[0][0]), "+v"(oacc[0][1]), "+v"(oacc[1][0]), "+v"(oacc[1][1]), "+v"(oacc[2][0]),
                       "+v"(oacc[2][1]), "+v"(oacc[3][0]), "+v"(oacc[3][1]));
    }
  };

  const int NT = (P.skv + BKV - 1) / BKV;
  // Tile t+1 is fetched while tile t is worked on: its requests are issued behind the barrier that published
  // tile t, into the stage tile t-1 vacated; every wave waits for its own requests before the next barrier.
  dma_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  if (NT > 1) dma_tile(1, 1);
  for (int t = 0; t < NT - 1; t++) {
    tile_compute(lds + (t & 1) * L::STAGE, std::false_type{}, BKV, std::false_type{});
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of tile t+1 has landed
    __syncthreads();
    if (t + 2 < NT) dma_tile(t + 2, t & 1);
  }
  {
    const int t = NT - 1;
    const int valid = P.skv - t * BKV;
    if (valid < BKV) tile_compute(lds + (t & 1) * L::STAGE, std::true_type{}, valid, std::true_type{});
    else tile_compute(lds + (t & 1) * L::STAGE, std::false_type{}, BKV, std::true_type{});
  }
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(l_run[qb]), __float_as_int(l_run[qb]), false, false);
    const float inv = o_descale / (__int_as_float(sw[0]) + __int_as_float(sw[1]));
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

// ---------------------------------------------------------------------------
// K, V -> fp8 workspace [batch][heads][skv_pad][HD]; rows past skv are zero.
// ---------------------------------------------------------------------------
template <int HD>
__global__ void __launch_bounds__(256) quantize_kv_kernel(const AttnParams P) {
  constexpr int CPR = HD / 8;
  const int bh = blockIdx.y;
  const int b = bh / P.heads, h = bh % P.heads;
  const int nbh = P.batch * P.heads;
  const float ks = FP8_MAX / fmaxf(P.absmax[nbh + bh], 1e-20f);
  const float vs = FP8_MAX / fmaxf(P.absmax[2 * nbh + bh], 1e-20f);
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int r = c / CPR, cc = c % CPR;
  if (r >= P.skv_pad) return;
  i32x2 k8 = {0, 0}, v8 = {0, 0};
  if (r < P.skv) {
    k8 = quant8(*(const i32x4*)(row_ptr(P.k, b, h, r) + cc * 8), ks);
    v8 = quant8(*(const i32x4*)(row_ptr(P.v, b, h, r) + cc * 8), vs);
  }
  const size_t o = ((size_t)bh * P.skv_pad + r) * HD + cc * 8;
  *(i32x2*)(P.k8 + o) = k8;
  *(i32x2*)(P.v8 + o) = v8;
}

// ---------------------------------------------------------------------------
// absmax per (tensor, batch, head): grid (row chunks, 3 * batch * heads); non-negative floats order like
// their bit patterns, so the partial maxima are merged with an integer atomic max.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(64) absmax_zero_kernel(float* absmax, int n) {
  int i = blockIdx.x * 64 + threadIdx.x;
  if (i < n) absmax[i] = 0.f;
}

template <int HD>
__global__ void __launch_bounds__(256) absmax_kernel(const AttnParams P, float* absmax, int rows_per_wg) {
  constexpr int CPR = HD / 8;
  const int which = blockIdx.y / (P.batch * P.heads);
  const int bh = blockIdx.y % (P.batch * P.heads);
  const int b = bh / P.heads, h = bh % P.heads;
  const Seg2& s = which == 0 ? P.q : (which == 1 ? P.k : P.v);
  const int total = s.len0 + s.len1;
  const int r0 = blockIdx.x * rows_per_wg;
  const int r1 = min(r0 + rows_per_wg, total);
  float m = 0.f;
  for (int c = r0 * CPR + threadIdx.x; c < r1 * CPR; c += 256) {
    const int r = c / CPR, cc = c % CPR;
    float f[8];
    hdit::unpack8(*(const i32x4*)(row_ptr(s, b, h, r) + cc * 8), f);
#pragma unroll
    for (int e = 0; e < 8; e++) m = fmaxf(m, fabsf(f[e]));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  if ((threadIdx.x & 63) == 0 && r0 < r1) atomicMax((int*)absmax + blockIdx.y, __float_as_int(m));
}

// The same maxima when the heads of a row lie side by side in memory (stride_h == HD: column ranges of a packed
// q|k|v tensor, the usual case): a workgroup streams whole rows -- every request a run of full cache lines --
// instead of one 128- or 256-byte piece per row and head.  A 16-byte chunk belongs to one head; the lanes of a
// head's chunks in a row are neighbours, so they reduce among themselves before one lane merges into the
// workgroup's per-head maxima in LDS, and those go out with one atomic per head.
template <int HD>
__global__ void __launch_bounds__(256) absmax_rows_kernel(const AttnParams P, float* absmax, int rows_per_wg) {
  constexpr int CPH = HD / 8;  // chunks per head
  __shared__ int head_max[256];
  const int which = blockIdx.y / P.batch, b = blockIdx.y % P.batch;
  const Seg2& s = which == 0 ? P.q : (which == 1 ? P.k : P.v);
  const int total = s.len0 + s.len1;
  const int cpr = P.heads * CPH;  // chunks per row
  for (int i = threadIdx.x; i < P.heads; i += 256) head_max[i] = 0;
  __syncthreads();
  const int r0 = blockIdx.x * rows_per_wg, r1 = min(r0 + rows_per_wg, total);
  const int64_t chunks = (int64_t)(r1 - r0) * cpr;
  for (int64_t c0 = 0; c0 < chunks; c0 += 256) {
    const int64_t c = c0 + threadIdx.x;
    float m = 0.f;
    int head = 0;
    if (c < chunks) {
      const int r = r0 + (int)(c / cpr), cc = (int)(c % cpr);
      head = cc / CPH;
      float f[8];
      hdit::unpack8(*(const i32x4*)(row_ptr(s, b, 0, r) + cc * 8), f);
#pragma unroll
      for (int e = 0; e < 8; e++) m = fmaxf(m, fabsf(f[e]));
    }
    // cpr and 256 are multiples of CPH, so the CPH lanes of one (row, head) are an aligned group of the wave
#pragma unroll
    for (int off = 1; off < CPH; off <<= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((threadIdx.x & (CPH - 1)) == 0 && c < chunks) atomicMax(&head_max[head], __float_as_int(m));
  }
  __syncthreads();
  for (int i = threadIdx.x; i < P.heads; i += 256)
    if (r0 < r1) atomicMax((int*)absmax + (which * P.batch + b) * P.heads + i, head_max[i]);
}

bool heads_side_by_side(const Seg2& s, int hd) {
  return (s.len0 == 0 || s.sh0 == hd) && (s.len1 == 0 || s.sh1 == hd);
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

size_t kv8_bytes(const hdit_attn_args* a) {
  const int skv = a->k[0].len + a->k[1].len;
  const size_t skv_pad = (size_t)(skv + BKV - 1) / BKV * BKV;
  return (size_t)a->batch * a->heads * skv_pad * a->head_dim;
}

AttnParams make_params(const hdit_attn_args* a, const float* absmax, void* workspace = nullptr) {
  AttnParams P;
  P.q = make_seg(a->q);
  P.k = make_seg(a->k);
  P.v = make_seg(a->v);
  P.o = make_seg(a->o);
  P.absmax = absmax;
  P.batch = a->batch;
  P.heads = a->heads;
  P.sq = a->q[0].len + a->q[1].len;
  P.skv = a->k[0].len + a->k[1].len;
  P.skv_pad = (P.skv + BKV - 1) / BKV * BKV;
  P.k8 = (unsigned char*)workspace;
  P.v8 = workspace ? (unsigned char*)workspace + kv8_bytes(a) : nullptr;
  P.scale = a->scale > 0.f ? a->scale : 1.0f / sqrtf((float)a->head_dim);
  return P;
}

}  // namespace

namespace hdit_host {
int attn_validate(const hdit_attn_args* a);
}

extern "C" __attribute__((visibility("default"))) int hdit_attn_absmax(const hdit_attn_args* a, float* absmax, void* stream) {
  int rc = hdit_host::attn_validate(a);
  if (rc != HDIT_OK) return rc;
  if (!absmax || (((uintptr_t)absmax) & 3)) return HDIT_EINVAL;
  AttnParams P = make_params(a, absmax);
  hipStream_t s = (hipStream_t)stream;
  const int n = 3 * a->batch * a->heads;
  hipLaunchKernelGGL(absmax_zero_kernel, dim3((n + 63) / 64), dim3(64), 0, s, absmax, n);
  const int longest = P.sq > P.skv ? P.sq : P.skv;
  if (longest == 0) return hdit_host::check_launch("hdit_attn_absmax");
  if (a->heads <= 256 && heads_side_by_side(P.q, a->head_dim) && heads_side_by_side(P.k, a->head_dim) &&
      heads_side_by_side(P.v, a->head_dim)) {
    const int rows = 32;
    dim3 grid((longest + rows - 1) / rows, 3 * a->batch);
    if (a->head_dim == 64)
      hipLaunchKernelGGL(absmax_rows_kernel<64>, grid, dim3(256), 0, s, P, absmax, rows);
    else
      hipLaunchKernelGGL(absmax_rows_kernel<128>, grid, dim3(256), 0, s, P, absmax, rows);
    return hdit_host::check_launch("hdit_attn_absmax");
  }
  const int rows_per_wg = 256;
  dim3 grid((longest + rows_per_wg - 1) / rows_per_wg, n);
  if (a->head_dim == 64)
    hipLaunchKernelGGL(absmax_kernel<64>, grid, dim3(256), 0, s, P, absmax, rows_per_wg);
  else
    hipLaunchKernelGGL(absmax_kernel<128>, grid, dim3(256), 0, s, P, absmax, rows_per_wg);
  return hdit_host::check_launch("hdit_attn_absmax");
}

extern "C" __attribute__((visibility("default"))) int64_t hdit_attn_fp8_workspace_bytes(const hdit_attn_args* a) {
  if (hdit_host::attn_validate(a) != HDIT_OK) return -1;
  return (int64_t)(2 * kv8_bytes(a));
}

namespace {

int fwd_fp8_launch(const hdit_attn_args* a, const float* absmax, void* workspace, hipStream_t s, const char* what) {
  AttnParams P = make_params(a, absmax, workspace);
  if (P.sq == 0) return HDIT_OK;
  const int cpr = a->head_dim / 8;
  dim3 qgrid((unsigned)((P.skv_pad * cpr + 255) / 256), (unsigned)(a->batch * a->heads));
  if (a->head_dim == 64)
    hipLaunchKernelGGL(quantize_kv_kernel<64>, qgrid, dim3(256), 0, s, P);
  else
    hipLaunchKernelGGL(quantize_kv_kernel<128>, qgrid, dim3(256), 0, s, P);
  int q_tiles = (P.sq + BQ - 1) / BQ;
  dim3 grid((unsigned)(q_tiles * a->batch * a->heads)), block(256);
  if (a->head_dim == 64)
    hipLaunchKernelGGL(attn_fp8_kernel<64>, grid, block, Lds8<64>::TOTAL, s, P, q_tiles);
  else
    hipLaunchKernelGGL(attn_fp8_kernel<128>, grid, block, Lds8<128>::TOTAL, s, P, q_tiles);
  return hdit_host::check_launch(what);
}

// ---- the entry point that allocates nothing ---------------------------------------------------------
// The quantised K / V copy of hdit_attn_fwd_fp8_static lives in this array instead of a caller workspace.
// Every GPU the library runs on holds its own copy at its own address until the process ends; in host
// code the name below is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t STATIC_SCRATCH_BYTES = HDIT_ATTN_FP8_STATIC_MAX_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_DEVICES];

// Device address of `scratch` on the current device, looked up once per device (the first call on it).
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    hdit_host::set_error(hipGetErrorString(e));
    return HDIT_ELAUNCH;
  }
  if (dev < 0 || dev >= MAX_DEVICES) return HDIT_EUNSUPPORTED;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // the same address for every thread asking on this device
    if (e != hipSuccess || !p) {
      hdit_host::set_error(e != hipSuccess ? hipGetErrorString(e) : "hipGetSymbolAddress returned a null address");
      return HDIT_ELAUNCH;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return HDIT_OK;
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_fp8(const hdit_attn_args* a, const float* absmax, void* workspace,
                                                                         void* stream) {
  int rc = hdit_host::attn_validate(a);
  if (rc != HDIT_OK) return rc;
  if (!absmax || !workspace || (((uintptr_t)workspace) & 15)) return HDIT_EINVAL;
  return fwd_fp8_launch(a, absmax, workspace, (hipStream_t)stream, "hdit_attn_fwd_fp8");
}

extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_fp8_static(const hdit_attn_args* a, const float* absmax,
                                                                                void* stream) {
  int rc = hdit_host::attn_validate(a);
  if (rc != HDIT_OK) return rc;
  if (!absmax) return HDIT_EINVAL;
  if (2 * kv8_bytes(a) > STATIC_SCRATCH_BYTES) {
    hdit_host::set_error("hdit_attn_fwd_fp8_static: batch * heads * keys (padded to 64) * head_dim * 2 exceeds "
                         "HDIT_ATTN_FP8_STATIC_MAX_BYTES; use hdit_attn_fwd_fp8 with a caller workspace");
    return HDIT_ETOOLARGE;
  }
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != HDIT_OK) return rc;
  return fwd_fp8_launch(a, absmax, ws, (hipStream_t)stream, "hdit_attn_fwd_fp8_static");
}
