// Device code of the bf16 flash-attention kernels, shared by the translation units that instantiate them
// (attention_bf16.hip: head dim 64 and the C entry point; attention_bf16_d128.hip: head dim 128): the two are
// compiled with different register-allocation options, see build.py.
//
// Joint (image + text) flash attention forward for gfx950, bf16 in/out.
//
// Work split: one workgroup = 4 waves = 256 query rows of one (batch, head);
// each wave owns 64 query rows (two 32-row MFMA column blocks) and walks the
// keys in tiles of 64.  K and V tiles go straight from global memory into two
// LDS buffers (direct-to-LDS loads, one barrier per tile).
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
#pragma once
#include <atomic>
#include <cstdlib>
#include <type_traits>

#include "hdit_common.h"

namespace hdit_attn {

struct Seg2 {
  const __bf16* p0;
  const __bf16* p1;
  int64_t sb0, ss0, sh0, sb1, ss1, sh1;
  int len0, len1;
};

__device__ __forceinline__ const __bf16* row_ptr(const Seg2& s, int b, int h, int r) {
  // r must be < len0 + len1.  Every field is read and the values are selected: with a branch the compiler may
  // merge the two sides into one load through a selected address, which forces the kernel's parameter block
  // out of the scalar registers into private memory.
  const bool a = r < s.len0;
  const __bf16* p = a ? s.p0 : s.p1;
  const int64_t sb = a ? s.sb0 : s.sb1, ss = a ? s.ss0 : s.ss1, sh = a ? s.sh0 : s.sh1;
  return p + b * sb + (int64_t)(a ? r : r - s.len0) * ss + h * sh;
}

struct AttnParams {
  Seg2 q, k, v, o;
  int heads, sq, skv;
  float scale_log2;
};

// Launch of the kernels for one head dim on an argument block the entry point has validated and converted.
// pipelined: take the software-pipelined kernel (the caller has checked that the problem qualifies).
int launch_d64(const AttnParams& P, int q_tiles, unsigned grid, bool pipelined, hipStream_t stream);
int launch_d128(const AttnParams& P, int q_tiles, unsigned grid, bool pipelined, hipStream_t stream);
// `count` problems of one head dim as one grid of the tracked or of the pipelined kernel
int launch_multi_d64(const AttnParams* P, const int* q_tiles, const int* nblocks, int count, bool pipelined, hipStream_t stream);
int launch_multi_d128(const AttnParams* P, const int* q_tiles, const int* nblocks, int count, bool pipelined, hipStream_t stream);

}  // namespace hdit_attn

namespace {

using hdit_attn::AttnParams;
using hdit_attn::Seg2;

constexpr int BKV = 64;   // keys per tile
constexpr int WQ = 64;    // query rows per wave
constexpr int NWAVE = 4;
constexpr int BQ = WQ * NWAVE;

template <int HD>
struct Lds {
  // K and V tiles come straight from global memory (global_load_lds_dwordx4: no staging registers, no
  // ds_write), which lands a wave's 64 x 16 bytes contiguously -- eight (d = 64) or four (d = 128) unpadded
  // rows.  The spread over the 64-bank (256-byte) LDS window therefore comes from XOR swizzles applied on the
  // source side.  A ds_read_b128 pass covers 16 consecutive K rows, which must land on 16 distinct 16-byte
  // slots; a transpose-read pass covers 4 consecutive V rows x 64 bytes, which must land on 4 distinct 64-byte
  // slots.  d = 64 (rows of 128 bytes): slot p of K row r holds chunk p ^ ((r>>1)&7), slot p of V row r holds
  // chunk p ^ 4*((r>>1)&1).  d = 128 (rows of 256 bytes, a whole bank window): K chunk p ^ (r&15), V chunk
  // p ^ 4*(r&3).
  static constexpr int K_ROW = HD * 2;
  static constexpr int V_ROW = HD * 2;
  static constexpr int K_BYTES = BKV * K_ROW;
  static constexpr int V_BYTES = BKV * V_ROW;
  static constexpr int STAGE = K_BYTES + V_BYTES;
  // d = 128: the Q fragments (64 registers) live in LDS instead, one private region per wave, rows strided like
  // the K rows, and are read per k-step next to the K fragments: the registers they would occupy are what the
  // loop otherwise spills (and reloads from scratch on every tile, with one wave per SIMD to hide nothing).
  static constexpr bool Q_IN_LDS = HD == 128;
  static constexpr int Q_ROW = HD * 2 + 16;
  static constexpr int Q_OFF = 2 * STAGE;
  static constexpr int Q_WAVE_BYTES = WQ * Q_ROW;
  static constexpr int TOTAL = 2 * STAGE + (Q_IN_LDS ? 4 * Q_WAVE_BYTES : 0);
  static_assert(TOTAL <= 160 * 1024, "attention tiles do not fit the LDS");
};

// One wave-wide direct-to-LDS copy: lane l's 16 bytes land at LDS byte address lds_addr + 16*l.  Inline
// assembly, so the compiler's wait-count bookkeeping does not see it; the tile loop waits for it explicitly.
// AGENT: issued at agent scope (sc1), which the CU's L1 never serves.  The pipelined kernel waits for "all but the
// newest n" requests and relies on completion in issue order, and a request that hits in L1 -- the rows of a clamped
// tile, a tile requested again past the end, a short sequence the previous workgroup on the CU has just read --
// completes ahead of older misses; from L2, hits and misses complete in issue order.  The kernels that wait for
// everything (vmcnt(0)) do not care about the order and keep the L1 (2 % faster where two workgroups of a CU read
// the same keys).
template <bool AGENT>
__device__ __forceinline__ void lds_dma16(const unsigned char* base_uniform, unsigned voff, unsigned lds_addr_uniform) {
  // the base is wave-uniform by construction; say so, or a base the compiler keeps in vector registers ends up in
  // the scalar-address operand
  const uint64_t bu = (uint64_t)base_uniform;
  const uint64_t base = ((uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(bu >> 32)) << 32) |
                        (unsigned)__builtin_amdgcn_readfirstlane((int)bu);
  if constexpr (AGENT)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 sc1"
                 :
                 : "s"(lds_addr_uniform), "v"(voff), "s"(base)
                 : "m0", "memory");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr_uniform), "v"(voff), "s"(base)
                 : "m0", "memory");
}
template <bool AGENT>
__device__ __forceinline__ void lds_dma16_ptr(const unsigned char* ptr_per_lane, unsigned lds_addr_uniform) {
  if constexpr (AGENT)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off sc1"
                 :
                 : "s"(lds_addr_uniform), "v"(ptr_per_lane)
                 : "m0", "memory");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_addr_uniform), "v"(ptr_per_lane)
                 : "m0", "memory");
}
__device__ __forceinline__ unsigned lds_address(const unsigned char* p) {
  return (unsigned)(uintptr_t)((const __attribute__((address_space(3))) unsigned char*)p);
}

// s_waitcnt immediate: all but the newest n vector-memory operations have completed, and every LDS operation
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0070; }

// The running row maximum is only raised when some row's maximum grew by more than this many powers of
// two; until then exp2(s - m) may reach 2^8, harmless for the bf16 P operand and the fp32 row sums, and the
// accumulator rescale (the most expensive VALU block after the exponentials) is skipped for most tiles.
constexpr float RESCALE_THRESHOLD = 8.0f;

// The whole kernel for one workgroup: the online softmax with a running reference that follows the column
// maxima.  Also the second pass of the pipelined d = 64 kernel when its fixed reference overflowed.
template <int HD>
__device__ __forceinline__ void attn_tracked_body(const AttnParams& P, int q_tiles, unsigned char* lds, int block_id,
                                                  int nblocks) {
  using L = Lds<HD>;
  constexpr int KS = HD / 16;       // k-steps of the S^T MFMA (over head dim)
  constexpr int DB = HD / 32;       // 32-wide d blocks of O^T
  constexpr int CPR = HD / 8;       // 16-byte chunks per row
  constexpr int NCH = BKV * CPR / 256;  // chunks per thread per tile (K and V each)
  // FOLD: the softmax scale is multiplied into Q once and the running reference m is subtracted inside the
  // score MFMA (its first k-step accumulates onto -m), so the accumulators feed exp2 directly: one FMA less
  // per score in a loop that is bound by the VALU.  Costs 32 registers; the d = 128 kernel has none to spare.
  constexpr bool FOLD = HD == 64;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  // Workgroups go to the 8 XCDs round-robin by id, and each XCD has its own L2: all query tiles of one
  // (batch, head) run on one XCD, so that its K and V are fetched into one L2 instead of eight.  Within that,
  // the partly filled last query tiles (some of their waves have no rows and skip the arithmetic) come after
  // all full ones: workgroups are placed in id order, one per CU first, so when a launch has a few more
  // workgroups than CUs it is the light ones that share a CU with a full one.
  const int nbh = nblocks / q_tiles;
  const bool by_xcd = nbh % 8 == 0;
  const int slot = by_xcd ? (block_id >> 3) : block_id;
  const int nbh_loc = by_xcd ? nbh / 8 : nbh;
  int qt = slot % q_tiles, bhl = slot / q_tiles;
  if (q_tiles > 1 && P.sq % BQ != 0) {
    const int heavy = nbh_loc * (q_tiles - 1);
    if (slot < heavy) {
      qt = slot % (q_tiles - 1);
      bhl = slot / (q_tiles - 1);
    } else {
      qt = q_tiles - 1;
      bhl = slot - heavy;
    }
  }
  const int bh = by_xcd ? bhl * 8 + (block_id & 7) : bhl;
  const int b = bh / P.heads, h = bh % P.heads;
  const int q0 = qt * BQ + wave * WQ;
  // a wave past the last query row still stages K/V tiles and meets the barriers, but does no arithmetic
  const bool active = __builtin_amdgcn_readfirstlane(q0 < P.sq);

  // ---- Q fragments: lane holds q row (qb*32 + l32), d = 16*ks + 8*lh .. +7
  bf16x8 qf[2][L::Q_IN_LDS ? 1 : KS];
  unsigned char* qlds = lds + L::Q_OFF + wave * L::Q_WAVE_BYTES;
  if constexpr (L::Q_IN_LDS) {
    // the wave's 64 query rows, 16 lanes per row (coalesced 256-byte rows), into its private LDS region;
    // only this wave reads them back, so its own wait for the writes is all the synchronisation needed
    constexpr int RPI = 64 / CPR;  // rows per wave-wide load
#pragma unroll
    for (int i = 0; i < WQ / RPI; i++) {
      const int row = i * RPI + lane / CPR, cc = lane % CPR;
      const int r = min(q0 + row, P.sq - 1);
      const i32x4 raw = *(const i32x4*)(row_ptr(P.q, b, h, r) + cc * 8);
      *(i32x4*)(qlds + row * L::Q_ROW + cc * 16) = raw;
    }
  } else
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    int r = min(q0 + qb * 32 + l32, P.sq - 1);
    const __bf16* rp = row_ptr(P.q, b, h, r);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const i32x4 raw = *(const i32x4*)(rp + ks * 16 + lh * 8);
      if constexpr (FOLD) {
        float f[8];
        hdit::unpack8(raw, f);
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] *= P.scale_log2;
        qf[qb][ks] = __builtin_bit_cast(bf16x8, hdit::pack8(f));
      } else {
        qf[qb][ks] = __builtin_bit_cast(bf16x8, raw);
      }
    }
  }

  // ---- K/V tile staging: global -> registers -> LDS.  A tile that lies inside one segment is addressed as
  // (wave-uniform base) + (loop-invariant per-thread offset); the tile that straddles the segment boundary
  // and the last, clamped tile take the per-row path.
  unsigned koff[2][NCH], voff[2][NCH];
  // direct-to-LDS (d = 64): request i of a wave covers rows 8*(wave + 4*i) .. +7, lane -> (row, slot lane%8);
  // the chunk fetched for a slot is the slot index XORed with the row's swizzle (the same for every i)
  constexpr int RPI = 64 / CPR;  // rows per request
  const int dma_row = wave * RPI + lane / CPR;
  const int dma_kc = (lane % CPR) ^ (HD == 64 ? ((dma_row >> 1) & 7) : (dma_row & 15));
  const int dma_vc = (lane % CPR) ^ (4 * (HD == 64 ? ((dma_row >> 1) & 1) : (dma_row & 3)));
  const unsigned lds_base_addr = __builtin_amdgcn_readfirstlane(lds_address(lds));
#pragma unroll
  for (int i = 0; i < NCH; i++) {
    const int row = dma_row + 4 * RPI * i;
    koff[0][i] = (unsigned)((row * P.k.ss0 + dma_kc * 8) * 2);
    koff[1][i] = (unsigned)((row * P.k.ss1 + dma_kc * 8) * 2);
    voff[0][i] = (unsigned)((row * P.v.ss0 + dma_vc * 8) * 2);
    voff[1][i] = (unsigned)((row * P.v.ss1 + dma_vc * 8) * 2);
  }
  const unsigned char* kb0 = (const unsigned char*)(P.k.p0 + b * P.k.sb0 + h * P.k.sh0);
  const unsigned char* kb1 = (const unsigned char*)(P.k.p1 + b * P.k.sb1 + h * P.k.sh1);
  const unsigned char* vb0 = (const unsigned char*)(P.v.p0 + b * P.v.sb0 + h * P.v.sh0);
  const unsigned char* vb1 = (const unsigned char*)(P.v.p1 + b * P.v.sb1 + h * P.v.sh1);
  const int len0 = P.k.len0;
  // tile t straight into LDS stage `stage`
  auto dma_tile = [&](int t, int stage) {
    const int r0 = t * BKV;
    const unsigned kdst = lds_base_addr + stage * L::STAGE + __builtin_amdgcn_readfirstlane(wave) * 1024;
    const unsigned vdst = kdst + L::K_BYTES;
    if (r0 + BKV <= len0) {
      const unsigned char* kb = kb0 + (int64_t)r0 * P.k.ss0 * 2;
      const unsigned char* vb = vb0 + (int64_t)r0 * P.v.ss0 * 2;
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        lds_dma16<false>(kb, koff[0][i], kdst + i * 4096);
        lds_dma16<false>(vb, voff[0][i], vdst + i * 4096);
      }
    } else if (r0 >= len0 && r0 + BKV <= P.skv) {
      const unsigned char* kb = kb1 + (int64_t)(r0 - len0) * P.k.ss1 * 2;
      const unsigned char* vb = vb1 + (int64_t)(r0 - len0) * P.v.ss1 * 2;
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        lds_dma16<false>(kb, koff[1][i], kdst + i * 4096);
        lds_dma16<false>(vb, voff[1][i], vdst + i * 4096);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        const int r = min(r0 + dma_row + 4 * RPI * i, P.skv - 1);
        lds_dma16_ptr<false>((const unsigned char*)(row_ptr(P.k, b, h, r) + dma_kc * 8), kdst + i * 4096);
        lds_dma16_ptr<false>((const unsigned char*)(row_ptr(P.v, b, h, r) + dma_vc * 8), vdst + i * 4096);
      }
    }
  };
  f32x16 oacc[DB][2];
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[i][j][v] = 0.f;
  // running reference m of the online softmax (log2 units) and running sum per query column.  With FOLD the
  // accumulators of a score block start from negm = -m (the same value in all 16 entries: a lane owns one
  // query column per qb) and m starts at 0 until the first tile sets it to that tile's column maxima.
  float m_run[2] = {FOLD ? 0.f : -INFINITY, FOLD ? 0.f : -INFINITY};
  float l_run[2] = {0.f, 0.f};
  f32x16 negm[2];
#pragma unroll
  for (int qb = 0; qb < 2; qb++)
#pragma unroll
    for (int v = 0; v < 16; v++) negm[qb][v] = 0.f;
  bool first = true;

  // lane-constant part of the V^T transpose-read address:
  // 16-lane group G = lane/16, x = lane%16: key row 4*(G/2) + x/4, column 16*(G%2) + 4*(x%4)
  const int vt_row = 4 * (lane >> 5) + ((lane & 15) >> 2);
  const int vt_off = vt_row * L::V_ROW + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  const int vt_swz = HD == 64 ? ((vt_row >> 1) & 1) : (vt_row & 3);  // XORed into the 64-byte piece index
  const int k_off = l32 * L::K_ROW;
  const int k_swz = HD == 64 ? ((l32 >> 1) & 7) : (l32 & 15);  // direct-to-LDS layout: chunk c of K row r sits in slot c ^ this
  const bf16x2 ones2 = {(__bf16)1.0f, (__bf16)1.0f};

  // one K/V tile: scores, online softmax, PV.  MASK: keys >= valid do not exist (last tile only).
  auto tile_compute = [&](const unsigned char* sk, auto mask_tag, int valid) {
    constexpr bool MASK = decltype(mask_tag)::value;
    const unsigned char* sv = sk + L::K_BYTES;
    // ---- S^T[kb][qb] = K_tile . Q^T (first k-step starts from a zero accumulator operand)
    f32x16 sacc[2][2];
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if constexpr (L::Q_IN_LDS) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        bf16x8 qk[2], kf[2];
#pragma unroll
        for (int qb = 0; qb < 2; qb++) qk[qb] = *(const bf16x8*)(qlds + (qb * 32 + l32) * L::Q_ROW + lh * 16 + ks * 32);
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
          kf[kb] = *(const bf16x8*)(sk + k_off + kb * 32 * L::K_ROW + (((ks * 2 + lh) ^ k_swz) << 4));
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int qb = 0; qb < 2; qb++)
            sacc[kb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb], qk[qb], ks == 0 ? zero16 : sacc[kb][qb], 0, 0, 0);
      }
    }
    auto mask_scores = [&]() {
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
    };
    auto scores_from_registers = [&]() {
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          bf16x8 kf = *(const bf16x8*)(sk + k_off + kb * 32 * L::K_ROW +
                                       (((ks * 2 + lh) ^ k_swz) << 4));
#pragma unroll
          for (int qb = 0; qb < 2; qb++)
            sacc[kb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][L::Q_IN_LDS ? 0 : ks], ks == 0 ? (FOLD ? negm[qb] : zero16) : sacc[kb][qb], 0, 0, 0);
        }
      }
      mask_scores();
    };
    if constexpr (L::Q_IN_LDS) mask_scores();
    else scores_from_registers();
    if constexpr (FOLD) {
      // Both key blocks start from the reference vectors.  Reading them once more here keeps them alive past the
      // second block's first MFMA, which the compiler otherwise ties to a copy of them (16 v_mov_b64 per tile)
      // instead of naming them as its addend the way the first block's does.
      asm volatile("" : : "v"(negm[0]), "v"(negm[1]));
    }

    // ---- online softmax in the log2 domain.  A lane owns one query column per qb and 32 of its 64 keys;
    // the other 32 live in lane^32.
    bf16x8 pf[2][4];  // [qb][u], u = 2*kb + half: the 16 keys of PV k-step u
    if constexpr (FOLD) {
      float mrel[2];  // column maxima relative to the running reference
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        float mx = fmaxf(sacc[0][qb][0], sacc[1][qb][0]);
#pragma unroll
        for (int v = 1; v < 16; v++) mx = fmaxf(fmaxf(mx, sacc[0][qb][v]), sacc[1][qb][v]);  // one v_max3 per step
        auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(mx), __float_as_int(mx), false, false);
        mrel[qb] = fmaxf(__int_as_float(sw[0]), __int_as_float(sw[1]));
      }
      // move the reference (and rescale) only if some column outgrew the threshold: wave-uniform branch
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
          for (int v = 0; v < 16; v++) negm[qb][v] = -m_run[qb];
        }
        first = false;
      }
    } else {
      float mcand[2];
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        float mx = fmaxf(sacc[0][qb][0], sacc[1][qb][0]);
#pragma unroll
        for (int v = 1; v < 16; v++) mx = fmaxf(fmaxf(mx, sacc[0][qb][v]), sacc[1][qb][v]);  // one v_max3 per step
        auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(mx), __float_as_int(mx), false, false);
        mx = fmaxf(__int_as_float(sw[0]), __int_as_float(sw[1]));
        mcand[qb] = fmaxf(m_run[qb], mx * P.scale_log2);
      }
      // raise the running maxima (and rescale) only if some row outgrew the threshold: wave-uniform branch
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
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const float m = m_run[qb];
      float rs = l_run[qb];
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
          i32x4 pk;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float s0 = sacc[kb][qb][hh * 8 + 2 * e], s1 = sacc[kb][qb][hh * 8 + 2 * e + 1];
            const float p0 = __builtin_amdgcn_exp2f(FOLD ? s0 : __builtin_fmaf(s0, P.scale_log2, -m));
            const float p1 = __builtin_amdgcn_exp2f(FOLD ? s1 : __builtin_fmaf(s1, P.scale_log2, -m));
            const uint32_t pp = hdit::pack2(p0, p1);
            pk[e] = (int)pp;
            // row sum of exactly the bf16 values that enter the PV product
            rs = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pp), ones2, rs, false);
          }
          pf[qb][kb * 2 + hh] = __builtin_bit_cast(bf16x8, pk);
        }
      }
      l_run[qb] = rs;
    }

    // ---- O^T[db][qb] += V^T . P^T
#pragma unroll
    for (int u = 0; u < 4; u++) {
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const unsigned char* va = sv + vt_off + (u * 16) * L::V_ROW + ((db ^ vt_swz) << 6);
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
  };

  const int NT = (P.skv + BKV - 1) / BKV;
  // Tile t+1 is fetched while tile t is worked on: its requests are issued behind the barrier that published
  // tile t, into the stage tile t-1 vacated; every wave waits for its own requests before the next barrier.
  dma_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  if (NT > 1) dma_tile(1, 1);
  auto next_tile = [&](int t) {  // end of iteration t: publish tile t+1, start fetching tile t+2
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of tile t+1 has landed
    __syncthreads();
    if (t + 2 < NT) dma_tile(t + 2, t & 1);
  };

  if (!active) {
    // no query rows: stage this wave's share of every K/V tile and meet the same barriers, nothing else
    for (int t = 0; t < NT - 1; t++) next_tile(t);
    __builtin_amdgcn_s_waitcnt(0x0f70);
    return;
  }
  for (int t = 0; t < NT - 1; t++) {
    tile_compute(lds + (t & 1) * L::STAGE, std::false_type{}, BKV);
    next_tile(t);
  }
  {
    const int t = NT - 1;
    const int valid = P.skv - t * BKV;
    if (valid < BKV) tile_compute(lds + (t & 1) * L::STAGE, std::true_type{}, valid);
    else tile_compute(lds + (t & 1) * L::STAGE, std::false_type{}, BKV);
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

template <int HD>
__global__ void __launch_bounds__(256, (HD == 64 ? 2 : 1)) attn_fwd_kernel(const AttnParams P, int q_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  attn_tracked_body<HD>(P, q_tiles, lds, (int)blockIdx.x, (int)gridDim.x);
}

// Several independent attention problems of one head dim in one grid (the blocks of neighbouring pipeline patches
// that run side by side): problem i owns the workgroups [start[i], start[i + 1]), each range a multiple of 8 long so
// that a workgroup's position modulo 8 -- the XCD it lands on -- is the same inside its problem as in the launch.
constexpr int ATTN_MAX_MULTI = HDIT_ATTN_MAX_MULTI;
struct AttnMulti {
  AttnParams p[ATTN_MAX_MULTI];
  int q_tiles[ATTN_MAX_MULTI];
  int nblocks[ATTN_MAX_MULTI];   // workgroups that have work (the range may be padded beyond them)
  int start[ATTN_MAX_MULTI + 1];
  int count;
};

template <int HD>
__global__ void __launch_bounds__(256, (HD == 64 ? 2 : 1)) attn_fwd_multi_kernel(const AttnMulti M) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  int i = 0;
#pragma unroll 1
  while (i + 1 < M.count && (int)blockIdx.x >= M.start[i + 1]) i++;
  const int local = (int)blockIdx.x - M.start[i];
  if (local >= M.nblocks[i]) return;
  attn_tracked_body<HD>(M.p[i], M.q_tiles[i], lds, local, M.nblocks[i]);
}

// ---------------------------------------------------------------------------------------------------------
// Software-pipelined inside the wave (both head sizes).
//
// On this chip the matrix pipe and the vector ALU of a SIMD overlap only inside ONE wave's instruction stream
// (an MFMA executes for 32 cycles after it issued, and independent VALU instructions of the same wave issue
// under it); two waves do not overlap each other.  A tile's work is half MFMA and half VALU (exponentials,
// packs, row sums), so the kernel above, whose waves alternate between an MFMA phase and a VALU phase, pays
// the sum.  Here a wave owns its SIMD alone (512 registers) and every instruction between two tile barriers
// is one basic block in which the score MFMAs of tile t+1 and the PV MFMAs of tile t are dealt between the
// softmax instructions of tile t:
//
//   segment A   P.V step 3 of tile t-1 (4 MFMAs) + scores of tile t, keys 32-63, k-steps 0-1 (4)  |  exp/pack/sum of keys  0-15
//   segment B   scores of tile t, keys 32-63, k-steps 2-3 (4) + P.V step 0 of tile t (4)          |  keys 16-31
//   segment C   scores of tile t+1, keys 0-31 (8), into the registers keys 0-31 of tile t vacated  |  keys 32-47
//   segment D   P.V steps 1, 2 of tile t (8)                                                      |  keys 48-63
//
// For the block to have no branch the reference of the online softmax is fixed after the first tile (its column
// maxima plus a margin: p = 2^(s - m) may then grow to PIPE_LIMIT and shrink to nothing without any loss
// of relative precision in fp32 / bf16): no maxima, no rescale in the loop.  A row whose sum ends at or above
// the limit (infinity and NaN included) makes the whole workgroup run the tracked kernel above from the start.
// K tiles are staged one tile ahead of V tiles (the scores run half a tile ahead of P.V), in rings of four LDS slots
// each, requested two tiles before they are read.
constexpr int PIPE_RING = 4;  // LDS slots per operand
// iteration t requests K tile t + PIPE_LEAD and V tile t + PIPE_LEAD - 1 (rings of 8 with leads of 5 and 7 tiles
// were measured: no difference, the requests arrive in time)
constexpr int PIPE_LEAD = 3;
static_assert(PIPE_LEAD >= 3 && PIPE_LEAD < PIPE_RING, "a requested tile must not land in a slot still being read");
constexpr int PIPE_MASK = PIPE_RING - 1;
template <int HD>
struct PipeLds {
  static constexpr int ROW = HD * 2;         // bytes of a K or V row
  static constexpr int TILE = BKV * ROW;     // bytes of one K or V tile
  static constexpr int V_OFF = PIPE_RING * TILE;
  static constexpr int FLAG_OFF = 2 * PIPE_RING * TILE;
  // the launch also covers the tracked kernel's layout, which a workgroup falls back to
  static constexpr int TOTAL = FLAG_OFF + 16 > Lds<HD>::TOTAL ? FLAG_OFF + 16 : Lds<HD>::TOTAL;
  static_assert(TOTAL <= 160 * 1024, "rings do not fit the LDS");
};
constexpr float PIPE_MARGIN = 24.0f;
constexpr float PIPE_LIMIT = 0x1p40f;
constexpr int PIPE_MIN_TILES = 3;

#define SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)

template <int HD>
__device__ __forceinline__ void attn_pipe_body(const AttnParams& P, int q_tiles, unsigned char* lds, int block_id, int nblocks) {
  using PL = PipeLds<HD>;
  constexpr int KS = HD / 16, DB = HD / 32, CPR = HD / 8, NCH = BKV * CPR / 256, RPI = 64 / CPR, ROW = PL::ROW;
  constexpr int PIPE_TILE = PL::TILE, PIPE_V_OFF = PL::V_OFF, PIPE_FLAG_OFF = PL::FLAG_OFF;
  constexpr int NMFMA = 4 * KS + 8 * DB;  // per iteration: two key blocks of scores, four P.V steps
  constexpr int VALU_PER_MFMA = (160 + NMFMA - 1) / NMFMA;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  // same placement of (batch, head, query tile) on workgroups as the kernel above
  const int nbh = nblocks / q_tiles;
  const bool by_xcd = nbh % 8 == 0;
  const int slot = by_xcd ? (block_id >> 3) : block_id;
  const int nbh_loc = by_xcd ? nbh / 8 : nbh;
  int qt = slot % q_tiles, bhl = slot / q_tiles;
  if (q_tiles > 1 && P.sq % BQ != 0) {
    const int heavy = nbh_loc * (q_tiles - 1);
    if (slot < heavy) {
      qt = slot % (q_tiles - 1);
      bhl = slot / (q_tiles - 1);
    } else {
      qt = q_tiles - 1;
      bhl = slot - heavy;
    }
  }
  const int bh = by_xcd ? bhl * 8 + (block_id & 7) : bhl;
  const int b = bh / P.heads, h = bh % P.heads;
  const int q0 = qt * BQ + wave * WQ;
  const bool active = __builtin_amdgcn_readfirstlane(q0 < P.sq);
  const int NT = (P.skv + BKV - 1) / BKV;  // >= PIPE_MIN_TILES (host)

  typedef __attribute__((address_space(3))) int lds_int;
  lds_int* const flag = (lds_int*)(uintptr_t)(lds_address(lds) + PIPE_FLAG_OFF);

  // ---- K / V tile requests, straight into LDS (same source-side swizzles as the kernel above)
  const int dma_row = wave * RPI + lane / CPR;
  const int dma_kc = (lane % CPR) ^ (HD == 64 ? ((dma_row >> 1) & 7) : (dma_row & 15));
  const int dma_vc = (lane % CPR) ^ (4 * (HD == 64 ? ((dma_row >> 1) & 1) : (dma_row & 3)));
  const unsigned lds_base_addr = __builtin_amdgcn_readfirstlane(lds_address(lds));
  // lane offsets of request 0 inside a tile of segment 0 / 1; request i lies 4 * RPI * i rows further down, a
  // scalar step that goes into the request's scalar base
  unsigned koff[2], voff[2];
  koff[0] = (unsigned)((dma_row * P.k.ss0 + dma_kc * 8) * 2);
  koff[1] = (unsigned)((dma_row * P.k.ss1 + dma_kc * 8) * 2);
  voff[0] = (unsigned)((dma_row * P.v.ss0 + dma_vc * 8) * 2);
  voff[1] = (unsigned)((dma_row * P.v.ss1 + dma_vc * 8) * 2);
  // A tile that lies inside one segment is (scalar base of the segment + tile * bytes per tile) + a loop-invariant
  // lane offset: four scalar instructions for the address (the host has checked that a tile step fits 32 bits).
  // The tile that straddles the segment boundary and the clamped last tile take the per-row path.
  const int len0 = P.k.len0;
  const int full0 = len0 / BKV;              // tiles [0, full0) lie in segment 0
  const int first1 = (len0 + BKV - 1) / BKV; // tiles [first1, full_all) lie in segment 1
  const int full_all = P.skv / BKV;
  const unsigned span1 = full_all > first1 ? (unsigned)(full_all - first1) : 0u;
  const uint64_t kb0 = (uint64_t)(P.k.p0 + b * P.k.sb0 + h * P.k.sh0);
  const uint64_t vb0 = (uint64_t)(P.v.p0 + b * P.v.sb0 + h * P.v.sh0);
  // segment 1 bases moved back by the rows of segment 0, so that they too are indexed by the tile number
  const uint64_t kb1 = (uint64_t)(P.k.p1 + b * P.k.sb1 + h * P.k.sh1) - (uint64_t)((int64_t)len0 * P.k.ss1 * 2);
  const uint64_t vb1 = (uint64_t)(P.v.p1 + b * P.v.sb1 + h * P.v.sh1) - (uint64_t)((int64_t)len0 * P.v.ss1 * 2);
  const unsigned krow0 = (unsigned)(P.k.ss0 * 2), krow1 = (unsigned)(P.k.ss1 * 2);  // bytes per row
  const unsigned vrow0 = (unsigned)(P.v.ss0 * 2), vrow1 = (unsigned)(P.v.ss1 * 2);
  const unsigned kstep0 = krow0 * BKV, kstep1 = krow1 * BKV, vstep0 = vrow0 * BKV, vstep1 = vrow1 * BKV;
  const unsigned wave_dst = lds_base_addr + __builtin_amdgcn_readfirstlane(wave) * 1024;
  // tile t (clamped to the last one) into the LDS bytes at dst (this wave's share: two requests 4 KiB apart)
  auto dma_k = [&](int t, unsigned dst) __attribute__((always_inline)) {
    if (t < full0) {
      const unsigned char* kb = (const unsigned char*)(kb0 + (uint64_t)(unsigned)t * kstep0);
#pragma unroll
      for (int i = 0; i < NCH; i++) lds_dma16<true>(kb + i * (4 * RPI) * krow0, koff[0], dst + i * 4096);
    } else if ((unsigned)(t - first1) < span1) {
      const unsigned char* kb = (const unsigned char*)(kb1 + (uint64_t)(unsigned)t * kstep1);
#pragma unroll
      for (int i = 0; i < NCH; i++) lds_dma16<true>(kb + i * (4 * RPI) * krow1, koff[1], dst + i * 4096);
    } else {
      const int r0 = min(t, NT - 1) * BKV;
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        const int r = min(r0 + dma_row + 4 * RPI * i, P.skv - 1);
        const bool in0 = r < len0;
        const uint64_t a = (in0 ? kb0 : kb1) + (uint64_t)(unsigned)r * (in0 ? krow0 : krow1) + dma_kc * 16;
        lds_dma16_ptr<true>((const unsigned char*)a, dst + i * 4096);
      }
    }
  };
  auto dma_v = [&](int t, unsigned dst) __attribute__((always_inline)) {
    if (t < full0) {
      const unsigned char* vb = (const unsigned char*)(vb0 + (uint64_t)(unsigned)t * vstep0);
#pragma unroll
      for (int i = 0; i < NCH; i++) lds_dma16<true>(vb + i * (4 * RPI) * vrow0, voff[0], dst + i * 4096);
    } else if ((unsigned)(t - first1) < span1) {
      const unsigned char* vb = (const unsigned char*)(vb1 + (uint64_t)(unsigned)t * vstep1);
#pragma unroll
      for (int i = 0; i < NCH; i++) lds_dma16<true>(vb + i * (4 * RPI) * vrow1, voff[1], dst + i * 4096);
    } else {
      const int r0 = min(t, NT - 1) * BKV;
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        const int r = min(r0 + dma_row + 4 * RPI * i, P.skv - 1);
        const bool in0 = r < len0;
        const uint64_t a = (in0 ? vb0 : vb1) + (uint64_t)(unsigned)r * (in0 ? vrow0 : vrow1) + dma_vc * 16;
        lds_dma16_ptr<true>((const unsigned char*)a, dst + i * 4096);
      }
    }
  };
  // Iteration t works on the scores of tiles t (keys 32-63) and t+1 (keys 0-31) and the probabilities of tile t.
  // It requests K tile t+3 and V tile t+2 first and, at its end, waits for everything older than those requests
  // (a wave's requests complete in order): K tile t+2 and V tile t+1, which the barrier then publishes.
  // Past the end the last tile is simply requested again (into a slot nobody reads any more): every iteration
  // then issues the same number of requests, its closing wait is one immediate, and the block that holds the
  // arithmetic ends at the barrier without a branch the compiler could sink instructions behind.
  auto stage_begin = [&](int t) __attribute__((always_inline)) {
    dma_k(t + PIPE_LEAD, wave_dst + ((t + PIPE_LEAD) & PIPE_MASK) * PIPE_TILE);
    dma_v(t + PIPE_LEAD - 1, wave_dst + PIPE_V_OFF + ((t + PIPE_LEAD - 1) & PIPE_MASK) * PIPE_TILE);
  };
  auto stage_end = [&]() {
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(2 * NCH * (PIPE_LEAD - 2)));
    __syncthreads();
  };

  // ---- prologue: flag, a zero V tile in the last slot (the lagged P.V of iteration 0 multiplies it by P = 0),
  // tiles K0 | K1 V0 | K2 V1 in request order
  if (tid == 0) *flag = 0;
  {
    const i32x4 z = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < PIPE_TILE / 4096; i++) *(i32x4*)(lds + PIPE_V_OFF + PIPE_MASK * PIPE_TILE + i * 4096 + tid * 16) = z;
  }
  dma_k(0, wave_dst);
#pragma unroll
  for (int j = 1; j < PIPE_LEAD; j++) {
    dma_k(j, wave_dst + j * PIPE_TILE);
    dma_v(j - 1, wave_dst + PIPE_V_OFF + (j - 1) * PIPE_TILE);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(2 * NCH * (PIPE_LEAD - 1)));  // K0 has landed
  __syncthreads();

  const int nb = NT - 1;  // pipelined iterations
  if (!active) {
    // no query rows: this wave's share of every tile and the same barriers, nothing else
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(2 * NCH * (PIPE_LEAD - 2)));
    __syncthreads();
    for (int t = 0; t < nb; t++) {
      stage_begin(t);
      stage_end();
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
    __syncthreads();  // the flag barrier
    if (*(volatile lds_int*)flag) attn_tracked_body<HD>(P, q_tiles, lds, block_id, nblocks);
    return;
  }

  // ---- Q fragments, softmax scale folded in: lane holds q row (qb*32 + l32), d = 16*ks + 8*lh .. +7
  bf16x8 qf[2][KS];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    const int r = min(q0 + qb * 32 + l32, P.sq - 1);
    const __bf16* rp = row_ptr(P.q, b, h, r);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const i32x4 raw = *(const i32x4*)(rp + ks * 16 + lh * 8);
      float f[8];
      hdit::unpack8(raw, f);
#pragma unroll
      for (int e = 0; e < 8; e++) f[e] *= P.scale_log2;
      qf[qb][ks] = __builtin_bit_cast(bf16x8, hdit::pack8(f));
    }
  }

  const int vt_row = 4 * (lane >> 5) + ((lane & 15) >> 2);
  const int vt_off = vt_row * ROW + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  const int vt_swz = HD == 64 ? ((vt_row >> 1) & 1) : (vt_row & 3);
  const int k_off = l32 * ROW;
  const int k_swz = HD == 64 ? ((l32 >> 1) & 7) : (l32 & 15);
  const bf16x2 ones2 = {(__bf16)1.0f, (__bf16)1.0f};
  typedef __attribute__((ext_vector_type(8))) short s16x8;

  auto k_frag = [&](const unsigned char* sk, int kb, int ks) -> bf16x8 {
    return *(const bf16x8*)(sk + k_off + kb * 32 * ROW + (((ks * 2 + lh) ^ k_swz) << 4));
  };
  auto v_frag = [&](const unsigned char* sv, int u, int db) -> bf16x8 {
    const unsigned char* va = sv + vt_off + (u * 16) * ROW + ((db ^ vt_swz) << 6);
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(va));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(va + 8 * ROW));
    return __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  f32x16 oacc[DB][2];
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[i][j][v] = 0.f;
  float l_run[2] = {0.f, 0.f};
  f32x16 negm[2];
  // scores of the tile in work, [key block][query block]; a key block's registers take the next tile's scores as
  // soon as its probabilities are packed
  f32x16 s0[2], s1[2];

  auto score_steps = [&](f32x16 (&sn)[2], const unsigned char* sk, int kb, int ks0, int ks1) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = ks0; ks < ks1; ks++) {
      const bf16x8 kf = k_frag(sk, kb, ks);
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
        sn[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], ks == 0 ? negm[qb] : sn[qb], 0, 0, 0);
    }
  };

  // ---- the first 32 keys set the reference: raw scores, column maxima plus the margin, then the scores again
  // on top of -m
  {
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int v = 0; v < 16; v++) negm[qb][v] = 0.f;
    score_steps(s0, lds, 0, 0, KS);
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      float mx = s0[qb][0];
#pragma unroll
      for (int v = 1; v < 16; v++) mx = fmaxf(mx, s0[qb][v]);
      auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(mx), __float_as_int(mx), false, false);
      const float m = fmaxf(__int_as_float(sw[0]), __int_as_float(sw[1])) + PIPE_MARGIN;
#pragma unroll
      for (int v = 0; v < 16; v++) negm[qb][v] = -m;
    }
    score_steps(s0, lds, 0, 0, KS);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(2 * NCH * (PIPE_LEAD - 2)));  // K1 and V0 have landed
  __syncthreads();

  // probabilities of a tile: pf[qb][u] holds the 16 keys of P.V k-step u; step 3 is multiplied one iteration late
  bf16x8 pf[2][4];
  bf16x8 vf3[DB];  // the V^T fragments of that late step, read before its tile's slot is given away
  bf16x8 k1c[2];   // the first two K fragments of a tile's keys 32-63, read at the end of the iteration before
#pragma unroll
  for (int qb = 0; qb < 2; qb++) pf[qb][3] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int db = 0; db < DB; db++) vf3[db] = v_frag(lds + PIPE_V_OFF + PIPE_MASK * PIPE_TILE, 3, db);
#pragma unroll
  for (int ks = 0; ks < 2; ks++) k1c[ks] = k_frag(lds, 1, ks);

  // exponentials, packs and row sums of the 16 keys of step u: accumulator entries 8*(u%2) .. of key block u/2
  auto chunk = [&](const f32x16 (&sc)[2], int u) __attribute__((always_inline)) {
    const int hh = u & 1;
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      i32x4 pk;
      float rs = l_run[qb];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const float p0 = __builtin_amdgcn_exp2f(sc[qb][hh * 8 + 2 * e]);
        const float p1 = __builtin_amdgcn_exp2f(sc[qb][hh * 8 + 2 * e + 1]);
        const uint32_t pp = hdit::pack2(p0, p1);
        pk[e] = (int)pp;
        rs = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pp), ones2, rs, false);
      }
      pf[qb][u] = __builtin_bit_cast(bf16x8, pk);
      l_run[qb] = rs;
    }
  };
  auto pv_step = [&](const bf16x8 (&vf)[DB], int u) __attribute__((always_inline)) {
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int qb = 0; qb < 2; qb++) oacc[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db], pf[qb][u], oacc[db][qb], 0, 0, 0);
  };
  auto pv_from = [&](const unsigned char* sv, int u) __attribute__((always_inline)) {
    bf16x8 vf[DB];
#pragma unroll
    for (int db = 0; db < DB; db++) vf[db] = v_frag(sv, u, db);
    pv_step(vf, u);
  };
  auto mask_block = [&](f32x16 (&sc)[2], int kb, int valid) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int key = kb * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
      if (key >= valid) {
        sc[0][v] = -INFINITY;
        sc[1][v] = -INFINITY;
      }
    }
  };

  // one pipelined iteration (tile t): s0 holds the scores of its keys 0-31 on entry and those of tile t+1 on exit
  auto score_mfma = [&](f32x16 (&sn)[2], const bf16x8& kf, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
      sn[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], ks == 0 ? negm[qb] : sn[qb], 0, 0, 0);
  };
  // Lane parts of the fragment addresses (32-bit LDS addresses); an iteration adds the ring slot of its tile, the
  // rest is an immediate offset of the LDS instruction.
  typedef __attribute__((address_space(3))) unsigned char lds_byte;
  unsigned kaddr[KS], vaddr[DB];  // 32-bit LDS addresses
#pragma unroll
  for (int ks = 0; ks < KS; ks++) kaddr[ks] = lds_address(lds) + k_off + (((ks * 2 + lh) ^ k_swz) << 4);
#pragma unroll
  for (int db = 0; db < DB; db++) vaddr[db] = lds_address(lds) + PIPE_V_OFF + vt_off + ((db ^ vt_swz) << 6);
  // slot_off: byte offset of the ring slot (a scalar); the rest of the address is an immediate
  auto k_frag_s = [&](unsigned slot_off, int kb, int ks) __attribute__((always_inline)) -> bf16x8 {
    return *(const __attribute__((address_space(3))) bf16x8*)((lds_byte*)(uintptr_t)(kaddr[ks] + slot_off) + kb * 32 * ROW);
  };
  auto v_frag_s = [&](unsigned slot_off, int u, int db) __attribute__((always_inline)) -> bf16x8 {
    lds_byte* va = (lds_byte*)(uintptr_t)(vaddr[db] + slot_off) + (u * 16) * ROW;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(va));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(va + 8 * ROW));
    return __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  for (int t = 0; t < nb; t++) {
    const unsigned S = (unsigned)(t & PIPE_MASK) * PIPE_TILE, SN = (unsigned)((t + 1) & PIPE_MASK) * PIPE_TILE;  // ring slots of tiles t, t+1
    dma_k(t + PIPE_LEAD, wave_dst + (unsigned)((t + PIPE_LEAD) & PIPE_MASK) * PIPE_TILE);
    dma_v(t + PIPE_LEAD - 1, wave_dst + PIPE_V_OFF + (unsigned)((t + PIPE_LEAD - 1) & PIPE_MASK) * PIPE_TILE);
    __builtin_amdgcn_sched_barrier(0);
    // fragment reads in the order the MFMAs consume them
    bf16x8 k1[KS], k0n[KS], vf[3][DB];
    k1[0] = k1c[0];
    k1[1] = k1c[1];
#pragma unroll
    for (int ks = 2; ks < KS; ks++) k1[ks] = k_frag_s(S, 1, ks);
#pragma unroll
    for (int db = 0; db < DB; db++) vf[0][db] = v_frag_s(S, 0, db);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) k0n[ks] = k_frag_s(SN, 0, ks);
#pragma unroll
    for (int u = 1; u < 3; u++)
#pragma unroll
      for (int db = 0; db < DB; db++) vf[u][db] = v_frag_s(S, u, db);
    // MFMAs 0-3: the late P.V step of the previous tile; 4-11: scores of keys 32-63
    pv_step(vf3, 3);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) score_mfma(s1, k1[ks], ks);
    chunk(s0, 0);
    // 12-15: P.V step 0
    pv_step(vf[0], 0);
    chunk(s0, 1);
    // 16-23: scores of the next tile's keys 0-31
#pragma unroll
    for (int ks = 0; ks < KS; ks++) score_mfma(s0, k0n[ks], ks);
    chunk(s1, 2);
    // 24-31: P.V steps 1 and 2
    pv_step(vf[1], 1);
    pv_step(vf[2], 2);
    chunk(s1, 3);
    // for the next iteration
#pragma unroll
    for (int db = 0; db < DB; db++) vf3[db] = v_frag_s(S, 3, db);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) k1c[ks] = k_frag_s(SN, 1, ks);
    // The order above, pinned: every MFMA is followed by a fragment read and its share of the softmax
    // instructions, so that a fragment is requested a few MFMAs before its use and not much earlier.
#pragma unroll
    for (int i = 0; i < NMFMA; i++) {
      SGB(0x008, 1);
      if ((i & 3) != 3) SGB(0x100, 1);  // three fragment reads per four MFMAs: the rate they are consumed at
      SGB(0x402, VALU_PER_MFMA);
    }
    __builtin_amdgcn_sched_barrier(0);
    stage_end();
  }
  // ---- the last tile: nothing to run ahead for
  {
    const int t = NT - 1;
    const int valid = P.skv - t * BKV;
    const unsigned char* sk = lds + (t & PIPE_MASK) * PIPE_TILE;
    const unsigned char* sv = lds + PIPE_V_OFF + (t & PIPE_MASK) * PIPE_TILE;
    pv_step(vf3, 3);
    score_mfma(s1, k1c[0], 0);
    score_mfma(s1, k1c[1], 1);
    score_steps(s1, sk, 1, 2, KS);
    if (valid < BKV) {
      mask_block(s0, 0, valid);
      mask_block(s1, 1, valid);
    }
    chunk(s0, 0);
    pv_from(sv, 0);
    chunk(s0, 1);
    pv_from(sv, 1);
    chunk(s1, 2);
    pv_from(sv, 2);
    chunk(s1, 3);
    pv_from(sv, 3);
  }

  // ---- did the fixed reference hold?
  {
    const bool bad = !(l_run[0] < PIPE_LIMIT) || !(l_run[1] < PIPE_LIMIT);
    if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0) *flag = 1;
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
    __syncthreads();
    if (*(volatile lds_int*)flag) {
      attn_tracked_body<HD>(P, q_tiles, lds, block_id, nblocks);
      return;
    }
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


template <int HD>
__global__ void __launch_bounds__(256, 1) attn_fwd_pipe_kernel(const AttnParams P, int q_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  attn_pipe_body<HD>(P, q_tiles, lds, (int)blockIdx.x, (int)gridDim.x);
}

template <int HD>
__global__ void __launch_bounds__(256, 1) attn_fwd_pipe_multi_kernel(const AttnMulti M) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  int i = 0;
#pragma unroll 1
  while (i + 1 < M.count && (int)blockIdx.x >= M.start[i + 1]) i++;
  const int local = (int)blockIdx.x - M.start[i];
  if (local >= M.nblocks[i]) return;
  attn_pipe_body<HD>(M.p[i], M.q_tiles[i], lds, local, M.nblocks[i]);
}

// Host side of a multi launch: the table of `count` problems, ranges padded to multiples of 8 workgroups.
inline int fill_multi(AttnMulti& M, const AttnParams* P, const int* q_tiles, const int* nblocks, int count) {
  M.count = count;
  int at = 0;
  for (int i = 0; i < ATTN_MAX_MULTI; i++) {
    M.start[i] = at;
    if (i < count) {
      M.p[i] = P[i], M.q_tiles[i] = q_tiles[i], M.nblocks[i] = nblocks[i];
      at += (nblocks[i] + 7) / 8 * 8;
    } else {
      M.p[i] = P[0], M.q_tiles[i] = 1, M.nblocks[i] = 0;
    }
  }
  M.start[ATTN_MAX_MULTI] = at;
  return at;
}

}  // namespace
