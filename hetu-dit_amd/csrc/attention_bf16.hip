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
#include <atomic>
#include <type_traits>

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

// Work split of the balanced launch.  A "unit" is one query tile of one (batch, head) and costs NT key tiles;
// a launch of whole units runs ceil(units / resident workgroups) rounds, the last one partly empty (1.69 -> 2
// for the SD3 shape, 0.38 -> 1 for a PipeFusion patch).  The balanced launch instead lines all (unit, key tile)
// pairs of a group up, unit-major, and gives each of the group's `slots` workgroups an equal contiguous share:
// workgroup s works on pairs [s*I/slots, (s+1)*I/slots), I = units*NT.  A share covers the tail of one unit,
// whole units, and the head of another; a unit that lies inside one share is finished and written as usual,
// the (at most two) incomplete pieces of a share go to a workspace as un-normalised fp32 accumulators with their
// running reference and row sums, and attn_merge_kernel adds the pieces of every divided unit up.  Groups are
// the 8 XCDs when batch*heads divides by 8 (all query tiles of a (batch, head) then share one L2), else one.
struct Balance {
  float* part;   // [groups * slots][2] pieces of PART_FLOATS each
  int groups, slots, units;  // per group: workgroups, units
  int q_tiles, nt;
};

__host__ __device__ inline int64_t share_begin(int s, int slots, int64_t total) { return (int64_t)s * total / slots; }
// the workgroup whose share holds pair i
__host__ __device__ inline int share_of(int64_t i, int slots, int64_t total) {
  int s = (int)(i * slots / total);
  while (s + 1 < slots && share_begin(s + 1, slots, total) <= i) s++;
  while (s > 0 && share_begin(s, slots, total) > i) s--;
  return s;
}
template <int HD>
constexpr int part_floats() { return NWAVE * (2 * (HD / 32) * 16 * 64 + 4 * 64); }

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
__device__ __forceinline__ void lds_dma16(const unsigned char* base_uniform, unsigned voff, unsigned lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr_uniform), "v"(voff), "s"(base_uniform)
               : "m0", "memory");
}
__device__ __forceinline__ void lds_dma16_ptr(const unsigned char* ptr_per_lane, unsigned lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr_uniform), "v"(ptr_per_lane)
               : "m0", "memory");
}
__device__ __forceinline__ unsigned lds_address(const unsigned char* p) {
  return (unsigned)(uintptr_t)((const __attribute__((address_space(3))) unsigned char*)p);
}

// The running row maximum is only raised when some row's maximum grew by more than this many powers of
// two; until then exp2(s - m) may reach 2^8, harmless for the bf16 P operand and the fp32 row sums, and the
// accumulator rescale (the most expensive VALU block after the exponentials) is skipped for most tiles.
constexpr float RESCALE_THRESHOLD = 8.0f;

// normalise and write O[q][d] of one wave: lane owns q = qb*32 + l32, d = 32*db + 8*(v/4) + 4*lh + v%4
template <int DB>
__device__ __forceinline__ void write_output(const AttnParams& P, int b, int h, int q0, int l32, int lh,
                                             const f32x16 (&oacc)[DB][2], const float (&l_run)[2]) {
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

template <int HD, bool BALANCED>
__global__ void __launch_bounds__(256, (HD == 64 ? 2 : 1)) attn_fwd_kernel(const AttnParams P, int q_tiles, const Balance bal) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
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
  const int NT = (P.skv + BKV - 1) / BKV;
  // ---- which (unit, key tile) pairs this workgroup works on
  int group, units_loc;     // group = XCD when workgroups are dealt to XCDs by id
  bool by_xcd;
  int64_t it, it_end;       // pairs [it, it_end) of the group's unit-major list
  if constexpr (BALANCED) {
    by_xcd = bal.groups == 8;
    group = by_xcd ? (int)(blockIdx.x & 7) : 0;
    const int sl = by_xcd ? (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    units_loc = bal.units;
    it = share_begin(sl, bal.slots, (int64_t)bal.units * NT);
    it_end = share_begin(sl + 1, bal.slots, (int64_t)bal.units * NT);
  } else {
    // One unit per workgroup.  Workgroups go to the 8 XCDs round-robin by id, and each XCD has its own L2: all
    // query tiles of one (batch, head) run on one XCD, so that its K and V are fetched into one L2 instead of
    // eight.  Within that, the partly filled last query tiles (some of their waves have no rows and skip the
    // arithmetic) come after all full ones: workgroups are placed in id order, one per CU first, so when a
    // launch has a few more workgroups than CUs it is the light ones that share a CU with a full one.
    const int nbh = gridDim.x / q_tiles;
    by_xcd = nbh % 8 == 0;
    group = by_xcd ? (int)(blockIdx.x & 7) : 0;
    const int slot = by_xcd ? (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const int nbh_loc = by_xcd ? nbh / 8 : nbh;
    units_loc = nbh_loc * q_tiles;
    int unit = slot;
    if (q_tiles > 1 && P.sq % BQ != 0) {
      const int heavy = nbh_loc * (q_tiles - 1);
      unit = slot < heavy ? (slot / (q_tiles - 1)) * q_tiles + slot % (q_tiles - 1) : (slot - heavy) * q_tiles + q_tiles - 1;
    }
    it = (int64_t)unit * NT;
    it_end = it + NT;
  }
  (void)units_loc;
  int b = 0, h = 0, q0 = 0;
  bool active = false;
  // ---- Q fragments: lane holds q row (qb*32 + l32), d = 16*ks + 8*lh .. +7
  bf16x8 qf[2][L::Q_IN_LDS ? 1 : KS];
  unsigned char* qlds = lds + L::Q_OFF + wave * L::Q_WAVE_BYTES;
  auto load_q = [&]() __attribute__((always_inline)) {
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
  };

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
  const unsigned char *kb0 = nullptr, *kb1 = nullptr, *vb0 = nullptr, *vb1 = nullptr;  // K / V of the unit's (b, h)
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
        lds_dma16(kb, koff[0][i], kdst + i * 4096);
        lds_dma16(vb, voff[0][i], vdst + i * 4096);
      }
    } else if (r0 >= len0 && r0 + BKV <= P.skv) {
      const unsigned char* kb = kb1 + (int64_t)(r0 - len0) * P.k.ss1 * 2;
      const unsigned char* vb = vb1 + (int64_t)(r0 - len0) * P.v.ss1 * 2;
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        lds_dma16(kb, koff[1][i], kdst + i * 4096);
        lds_dma16(vb, voff[1][i], vdst + i * 4096);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NCH; i++) {
        const int r = min(r0 + dma_row + 4 * RPI * i, P.skv - 1);
        lds_dma16_ptr((const unsigned char*)(row_ptr(P.k, b, h, r) + dma_kc * 8), kdst + i * 4096);
        lds_dma16_ptr((const unsigned char*)(row_ptr(P.v, b, h, r) + dma_vc * 8), vdst + i * 4096);
      }
    }
  };
  // running reference m of the online softmax (log2 units) and running sum per query column.  With FOLD the
  // accumulators of a score block start from negm = -m (the same value in all 16 entries: a lane owns one
  // query column per qb) and m starts at 0 until the first tile sets it to that tile's column maxima.
  f32x16 oacc[DB][2];
  float m_run[2], l_run[2];
  f32x16 negm[2];
  bool first;
  auto reset_state = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[i][j][v] = 0.f;
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      m_run[qb] = FOLD ? 0.f : -INFINITY;
      l_run[qb] = 0.f;
#pragma unroll
      for (int v = 0; v < 16; v++) negm[qb][v] = 0.f;
    }
    first = true;
  };

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

  bool first_piece = true;
  while (it < it_end) {
    // ---- the next piece: key tiles [ka, kb) of one unit
    const int unit = (int)(it / NT), ka = (int)(it - (int64_t)unit * NT);
    const int kb = (int)min((int64_t)NT, (int64_t)ka + (it_end - it));
    it += kb - ka;
    const int qt = unit % q_tiles, bhl = unit / q_tiles;
    const int bh = by_xcd ? bhl * 8 + group : bhl;
    b = bh / P.heads;
    h = bh % P.heads;
    q0 = qt * BQ + wave * WQ;
    // a wave past the last query row still stages K/V tiles and meets the barriers, but does no arithmetic
    active = __builtin_amdgcn_readfirstlane(q0 < P.sq);
    kb0 = (const unsigned char*)(P.k.p0 + b * P.k.sb0 + h * P.k.sh0);
    kb1 = (const unsigned char*)(P.k.p1 + b * P.k.sb1 + h * P.k.sh1);
    vb0 = (const unsigned char*)(P.v.p0 + b * P.v.sb0 + h * P.v.sh0);
    vb1 = (const unsigned char*)(P.v.p1 + b * P.v.sb1 + h * P.v.sh1);
    if constexpr (BALANCED) __syncthreads();  // every wave is done with the previous piece's tiles
    load_q();
    reset_state();

    // Tile t+1 is fetched while tile t is worked on: its requests are issued behind the barrier that published
    // tile t, into the stage tile t-1 vacated; every wave waits for its own requests before the next barrier.
    dma_tile(ka, ka & 1);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    __syncthreads();
    if (ka + 1 < kb) dma_tile(ka + 1, (ka + 1) & 1);
    auto next_tile = [&](int t) {  // end of iteration t: publish tile t+1, start fetching tile t+2
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of tile t+1 has landed
      __syncthreads();
      if (t + 2 < kb) dma_tile(t + 2, t & 1);
    };

    if (!active) {
      // no query rows: stage this wave's share of every K/V tile and meet the same barriers, nothing else
      for (int t = ka; t < kb - 1; t++) next_tile(t);
      __builtin_amdgcn_s_waitcnt(0x0f70);
      first_piece = false;
      continue;
    }
    for (int t = ka; t < kb - 1; t++) {
      tile_compute(lds + (t & 1) * L::STAGE, std::false_type{}, BKV);
      next_tile(t);
    }
    {
      const int t = kb - 1;
      const int valid = P.skv - t * BKV;
      if (valid < BKV) tile_compute(lds + (t & 1) * L::STAGE, std::true_type{}, valid);
      else tile_compute(lds + (t & 1) * L::STAGE, std::false_type{}, BKV);
    }

    if (!BALANCED || (ka == 0 && kb == NT)) {
      write_output<DB>(P, b, h, q0, l32, lh, oacc, l_run);
    } else {
      // an incomplete piece: accumulators as they lie in the registers ([qb][db][v/4][lane][4], every store a
      // contiguous KiB per wave), then the running reference and this lane's half of the row sum per qb
      float* pw = bal.part + ((int64_t)blockIdx.x * 2 + (first_piece ? 0 : 1)) * part_floats<HD>() + wave * (part_floats<HD>() / NWAVE);
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            f32x4 v4 = {oacc[db][qb][g * 4 + 0], oacc[db][qb][g * 4 + 1], oacc[db][qb][g * 4 + 2], oacc[db][qb][g * 4 + 3]};
            *(f32x4*)(pw + (((qb * DB + db) * 4 + g) * 64 + lane) * 4) = v4;
          }
        pw[2 * DB * 16 * 64 + qb * 64 + lane] = m_run[qb];
        pw[2 * DB * 16 * 64 + (2 + qb) * 64 + lane] = l_run[qb];
      }
    }
    first_piece = false;
  }
}

// Adds the pieces of every unit that the balanced launch divided between workgroups: one workgroup per unit, a
// thread takes the role the same thread of attn_fwd_kernel had (same rows, same accumulator entries).
template <int HD>
__global__ void __launch_bounds__(256) attn_merge_kernel(const AttnParams P, const Balance bal) {
  constexpr int DB = HD / 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, lh = lane >> 5;
  const bool by_xcd = bal.groups == 8;
  const int group = by_xcd ? (int)(blockIdx.x & 7) : 0;
  const int unit = by_xcd ? (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  const int64_t total = (int64_t)bal.units * bal.nt, u0 = (int64_t)unit * bal.nt;
  const int s_first = share_of(u0, bal.slots, total), s_last = share_of(u0 + bal.nt - 1, bal.slots, total);
  if (s_first == s_last) return;  // finished by one workgroup, already written
  const int qt = unit % bal.q_tiles, bhl = unit / bal.q_tiles;
  const int bh = by_xcd ? bhl * 8 + group : bhl;
  const int b = bh / P.heads, h = bh % P.heads;
  const int q0 = qt * BQ + wave * WQ;
  if (q0 >= P.sq) return;
  f32x16 oacc[DB][2];
  float m_all[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
  auto piece = [&](int s) {
    // the piece of this unit in share s: its first piece if the share starts inside the unit, else its last
    const bool is_first = share_begin(s, bal.slots, total) >= u0;
    const int wg = by_xcd ? s * 8 + group : s;
    return bal.part + ((int64_t)wg * 2 + (is_first ? 0 : 1)) * part_floats<HD>() + wave * (part_floats<HD>() / NWAVE);
  };
  for (int s = s_first; s <= s_last; s++) {
    const float* pw = piece(s);
#pragma unroll
    for (int qb = 0; qb < 2; qb++) m_all[qb] = fmaxf(m_all[qb], pw[2 * DB * 16 * 64 + qb * 64 + lane]);
  }
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[i][j][v] = 0.f;
  for (int s = s_first; s <= s_last; s++) {
    const float* pw = piece(s);
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const float w = __builtin_amdgcn_exp2f(pw[2 * DB * 16 * 64 + qb * 64 + lane] - m_all[qb]);
      l_run[qb] += w * pw[2 * DB * 16 * 64 + (2 + qb) * 64 + lane];
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const f32x4 v4 = *(const f32x4*)(pw + (((qb * DB + db) * 4 + g) * 64 + lane) * 4);
#pragma unroll
          for (int e = 0; e < 4; e++) oacc[db][qb][g * 4 + e] += w * v4[e];
        }
    }
  }
  write_output<DB>(P, b, h, q0, l32, lh, oacc, l_run);
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

namespace {
constexpr int NUM_CU = 256;  // MI355X

// The balanced launch is taken when a workspace is there and the equal shares (plus a few tiles of overhead per
// piece: pipeline refill, Q reload, the piece written out and merged) are at least a quarter shorter than the
// rounds of whole units -- in practice launches of less than one round (a PipeFusion patch: 192 units on 512
// resident workgroups, 10-14 % faster).  Between one and two rounds (the SD3 step: 1.69) both launches take the
// same time: the chip runs at its power limit, the CUs that idle in the last round of whole units lend their
// power budget to the busy ones, and the balanced launch only trades that for the traffic of the pieces.
struct Plan {
  bool balanced;
  Balance bal;
  int q_tiles, wgs;
};
Plan make_plan(int batch, int heads, int head_dim, int sq, int skv, bool have_workspace) {
  Plan p;
  p.q_tiles = (sq + BQ - 1) / BQ;
  const int nbh = batch * heads;
  const int64_t units = (int64_t)nbh * p.q_tiles;
  const int nt = (skv + BKV - 1) / BKV;
  const int capacity = NUM_CU * (head_dim == 64 ? 2 : 1);
  const int groups = nbh % 8 == 0 ? 8 : 1;
  const int64_t plain = (units + capacity - 1) / capacity * nt;
  const int64_t shares = (units * nt + capacity - 1) / capacity + 3;
  p.balanced = have_workspace && shares * 4 <= plain * 3 && units / groups * nt >= capacity / groups && units < (1 << 24);
  p.wgs = p.balanced ? capacity : (int)units;
  p.bal.part = nullptr;
  p.bal.groups = groups;
  p.bal.slots = capacity / groups;
  p.bal.units = (int)(units / groups);
  p.bal.q_tiles = p.q_tiles;
  p.bal.nt = nt;
  return p;
}
int64_t plan_workspace_bytes(int head_dim) {
  const int capacity = NUM_CU * (head_dim == 64 ? 2 : 1);
  return (int64_t)capacity * 2 * (head_dim == 64 ? part_floats<64>() : part_floats<128>()) * 4;
}

template <int HD, bool BALANCED>
int set_lds_limit() {
  static std::atomic<bool> done{false};  // setting the attribute twice from two threads is harmless
  if (Lds<HD>::TOTAL > 64 * 1024 && !done.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)attn_fwd_kernel<HD, BALANCED>, hipFuncAttributeMaxDynamicSharedMemorySize, Lds<HD>::TOTAL) != hipSuccess)
      return HDIT_ELAUNCH;
    done.store(true, std::memory_order_release);
  }
  return HDIT_OK;
}

template <int HD>
int launch(const AttnParams& P, const Plan& plan, int units_total, hipStream_t s) {
  if (plan.balanced) {
    if (set_lds_limit<HD, true>() != HDIT_OK) return HDIT_ELAUNCH;
    hipLaunchKernelGGL((attn_fwd_kernel<HD, true>), dim3((unsigned)plan.wgs), dim3(256), Lds<HD>::TOTAL, s, P, plan.q_tiles, plan.bal);
    hipLaunchKernelGGL((attn_merge_kernel<HD>), dim3((unsigned)units_total), dim3(256), 0, s, P, plan.bal);
  } else if constexpr (HD == 128) {
    // one unit per workgroup, expressed as shares of exactly one unit each: this instantiation keeps its tile
    // loop free of scratch reloads, the whole-unit one does not at d = 128
    Balance one = plan.bal;
    one.slots = one.units;
    if (set_lds_limit<HD, true>() != HDIT_OK) return HDIT_ELAUNCH;
    hipLaunchKernelGGL((attn_fwd_kernel<HD, true>), dim3((unsigned)plan.wgs), dim3(256), Lds<HD>::TOTAL, s, P, plan.q_tiles, one);
  } else {
    if (set_lds_limit<HD, false>() != HDIT_OK) return HDIT_ELAUNCH;
    hipLaunchKernelGGL((attn_fwd_kernel<HD, false>), dim3((unsigned)plan.wgs), dim3(256), Lds<HD>::TOTAL, s, P, plan.q_tiles, plan.bal);
  }
  return HDIT_OK;
}

int fwd_bf16(const hdit_attn_args* a, void* workspace, int64_t workspace_bytes, void* stream, const char* what) {
  int rc = hdit_host::attn_validate(a);
  if (rc != HDIT_OK) return rc;
  if (workspace && (((uintptr_t)workspace) & 15)) return HDIT_EINVAL;
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
  Plan plan = make_plan(a->batch, a->heads, a->head_dim, P.sq, P.skv, workspace != nullptr && workspace_bytes >= plan_workspace_bytes(a->head_dim));
  plan.bal.part = (float*)workspace;
  const int units_total = plan.q_tiles * a->batch * a->heads;
  rc = a->head_dim == 64 ? launch<64>(P, plan, units_total, (hipStream_t)stream) : launch<128>(P, plan, units_total, (hipStream_t)stream);
  if (rc != HDIT_OK) return rc;
  return hdit_host::check_launch(what);
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_bf16(const hdit_attn_args* a, void* stream) {
  return fwd_bf16(a, nullptr, 0, stream, "hdit_attn_fwd_bf16");
}

namespace hdit_host {
int64_t attn_workspace_bytes_for(int batch, int heads, int head_dim, int sq, int skv) {
  if (sq <= 0 || skv <= 0) return 0;
  return make_plan(batch, heads, head_dim, sq, skv, true).balanced ? plan_workspace_bytes(head_dim) : 0;
}
}  // namespace hdit_host

extern "C" __attribute__((visibility("default"))) int64_t hdit_attn_workspace_bytes(const hdit_attn_args* a) {
  if (hdit_host::attn_validate(a) != HDIT_OK) return -1;
  return hdit_host::attn_workspace_bytes_for(a->batch, a->heads, a->head_dim, a->q[0].len + a->q[1].len, a->k[0].len + a->k[1].len);
}

extern "C" __attribute__((visibility("default"))) int hdit_attn_fwd_bf16_ws(const hdit_attn_args* a, void* workspace,
                                                                            int64_t workspace_bytes, void* stream) {
  return fwd_bf16(a, workspace, workspace_bytes, stream, "hdit_attn_fwd_bf16_ws");
}
