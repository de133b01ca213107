// Grouped bf16 GEMM for gfx950:  C[m, n] = epilogue(A[m, k] . B[n, k]^T + bias)
//
// Persistent kernel, one 256-thread workgroup (2x2 waves) per CU, walking a
// static list of output tiles of (64*TM) x (64*TN) elements; a wave owns a
// (32*TM) x (32*TN) sub-tile in accumulators (v_mfma_f32_32x32x16_bf16).
//
// Staging.  Both operands are k-contiguous, so A and B tiles are staged the
// same way, in slabs of 64 k (128 bytes per row).  A wave-wide request fetches
// 8 rows x 128 bytes, eight lanes per row: every request covers whole 128-byte
// cache lines (64-byte row pieces were measured at half the L2->CU rate,
// 29 B/clk/CU against 58).  LDS rows are 128 bytes whose 16-byte chunks are
// XOR-swizzled with (row>>1)&7: the 16 lanes of a ds_read_b128 pass (16 rows,
// one chunk) land on 16 distinct 16-byte slots of the 256-byte bank window.
//
// Pipeline.  The k slabs of all tiles of a workgroup form one flat stream; tile
// boundaries are invisible to it, so a tile's first slabs arrive during the
// previous tile's last slab and epilogue.  Fragments are double-buffered in
// registers one k-step ahead; the workgroup barrier sits before the last k-step
// of a slab, whose fragments are already in registers, so that the first
// fragments of the next slab are read under that k-step's MFMAs.
//  * 256-row shapes: direct to LDS (global_load_lds_dwordx4, swizzle applied on
//    the source side), three A slots and two B slots.  During slab g the A rows
//    of slab g+2 are requested (k-steps 0..2) into the slot slab g-1 vacated;
//    behind the barrier that ends slab g, the B rows of slab g+2 go into the B
//    slot just vacated.  Requests retire in order, so the wait in front of the
//    barrier leaves exactly the newest A requests in flight.
//  * 128-row shapes: two LDS stages, register-staged.  While slab h is
//    multiplied out of stage h&1, the registers holding slab h+1 are written
//    to the other stage and immediately refilled with the global loads of slab
//    h+2, one write+load pair every few MFMAs.
//
// Epilogue.  A lane's accumulator holds one output row m and runs of 4
// consecutive n; lanes l and l^32 swap halves (v_permlane32_swap) to own 8
// consecutive n.  bias / GELU-tanh are applied there, the bf16 result is staged
// through a wave-private 8 KiB window inside the LDS stage (the A slot) the last
// slab just vacated and written back with 16 lanes covering 256 contiguous bytes of a row
// (gate and residual are applied in that coalesced layout, in fp32).
//
// One launch covers up to HDIT_GEMM_MAX_PROBLEMS problems.  Tiles are dealt to
// workgroups so that the workgroups of one XCD (workgroup id mod 8; each XCD
// has a private L2) own a contiguous, 8-tile-row-grouped range.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "hdit_common.h"

namespace {

constexpr int BK = 64;           // k elements per LDS stage
constexpr int ROW_BYTES = 128;   // BK * sizeof(bf16)
constexpr int NUM_XCD = 8;
constexpr int GROUP_M = 8;
constexpr int NW = 4;
constexpr int NT = 256;
constexpr int EPI_WAVE_BYTES = 8192;  // 32 rows x 128 columns of bf16

struct GemmTable {
  int count;
  int tile_start[HDIT_GEMM_MAX_PROBLEMS + 1];
  hdit_gemm_problem p[HDIT_GEMM_MAX_PROBLEMS];
};

template <int TM_, int TN_>
struct Cfg {
  static constexpr int TM = TM_, TN = TN_;
  static constexpr int BM = 64 * TM, BN = 64 * TN;
  static constexpr int WM = 32 * TM, WN = 32 * TN;
  static constexpr int A_LOADS = BM / 8 / NW;  // wave-wide loads (8 rows x 128 bytes) per wave per slab
  static constexpr int B_LOADS = BN / 8 / NW;
  static constexpr int LOADS = A_LOADS + B_LOADS;
  static constexpr int A_BYTES = BM * ROW_BYTES;
  static constexpr int B_BYTES = BN * ROW_BYTES;
  static constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
  // DMA: the 256-row shapes take their operand slabs straight from global memory into LDS
  // (global_load_lds_dwordx4: no staging registers, no ds_write).  A has three slots (requested two slabs
  // ahead), B two (requested one slab ahead, first in the queue); the epilogue windows alias the A slot the
  // tile's last slab vacated, which is exactly as large.
  static constexpr bool DMA = TM == 4;
  static constexpr int A_SLOTS = 3, B_SLOTS = 2;
  static constexpr int B_OFF = A_SLOTS * A_BYTES;
  static constexpr int DMA_BYTES = A_SLOTS * A_BYTES + B_SLOTS * B_BYTES;
  // RING: the 128x128 shape takes its slabs the same way into a ring of four stages (A then B, 32 KiB each),
  // requested three slabs ahead: its slabs are short (16 MFMAs per wave), and only a lead of several of them
  // covers the latency of operands that come from HBM.  The epilogue windows alias the stage the tile's last slab
  // vacated.
  static constexpr bool RING = TM == 2 && TN == 2;
  static constexpr int NS = RING ? 4 : 2;
  static constexpr bool DIRECT = DMA || RING;
  static constexpr int LDS_BYTES = DMA ? DMA_BYTES : NS * STAGE_BYTES;
  static_assert(LDS_BYTES <= 160 * 1024, "tile does not fit the LDS");
  static_assert(DMA ? NW * EPI_WAVE_BYTES <= A_BYTES : NW * EPI_WAVE_BYTES <= STAGE_BYTES,
                "the epilogue windows live inside one stage (one A slot)");
  static_assert(TN <= 4, "epilogue staging window is 128 columns wide");
};

struct TileCoord {
  int pi, m0, n0;
};

template <class C>
__device__ __forceinline__ TileCoord locate(const GemmTable& tab, int lid) {
  int pi = 0;
#pragma unroll 1
  while (pi + 1 < tab.count && lid >= tab.tile_start[pi + 1]) pi++;
  const int tiles_m = (tab.p[pi].m + C::BM - 1) / C::BM;
  const int tiles_n = (tab.p[pi].n + C::BN - 1) / C::BN;
  const int t = lid - tab.tile_start[pi];
  const int in_group = GROUP_M * tiles_n;
  const int first_m = (t / in_group) * GROUP_M;
  const int gsz = min(tiles_m - first_m, GROUP_M);
  TileCoord tc;
  tc.pi = pi;
  tc.m0 = (first_m + (t % in_group) % gsz) * C::BM;
  tc.n0 = ((t % in_group) / gsz) * C::BN;
  return tc;
}

// One wave-wide direct-to-LDS copy: lane l's 16 bytes at base + voff land at LDS byte address
// lds_addr + lds_off + 16*l; the sum is formed in M0 itself (one scalar instruction less per request than adding
// first and moving the result: a slab is 16 requests per wave).  Inline assembly, so the compiler's wait-count
// insertion does not see it: an extra operation in flight only makes the waits it computes for its own
// loads stricter than needed.
// Every direct-to-LDS request is issued at agent scope (sc1), which the CU's L1 never serves.  The kernels wait
// for "all but the newest n" requests and rely on completion in issue order; a request that hits in L1 completes
// ahead of older misses (measured: a ragged tile, whose out-of-range lanes all read the problem's last row, then
// multiplied a slab that had not landed).  From L2, hits and misses complete in issue order.
__device__ __forceinline__ void lds_dma16_sum(const unsigned char* base_uniform, unsigned voff, unsigned lds_addr_uniform,
                                              unsigned lds_off_uniform) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 sc1"
               :
               : "s"(lds_addr_uniform), "v"(voff), "s"(base_uniform), "s"(lds_off_uniform)
               : "m0", "scc");
}

__device__ __forceinline__ unsigned lds_address(const unsigned char* p) {
  return (unsigned)(uintptr_t)((const __attribute__((address_space(3))) unsigned char*)p);
}

#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// s_waitcnt immediate that waits for all but the newest n vector-memory operations (and for nothing else)
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0f70; }

// All tiles of one shape that this workgroup owns.
template <class C>
__device__ __forceinline__ void run_tiles(const GemmTable& tab, int total_tiles, int tiles_per_xcd, int wgs_per_xcd,
                                          unsigned char* lds) {
  constexpr int TM = C::TM, TN = C::TN;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  const int wm0 = (wave >> 1) * C::WM;
  const int wn0 = (wave & 1) * C::WN;

  // tiles of this workgroup: XCD x owns logical tiles [x*tiles_per_xcd, (x+1)*tiles_per_xcd),
  // dealt round-robin to that XCD's workgroups
  const int xcd = blockIdx.x % NUM_XCD;
  const int xcd_begin = xcd * tiles_per_xcd;
  const int xcd_end = min(xcd_begin + tiles_per_xcd, total_tiles);
  int lid = xcd_begin + blockIdx.x / NUM_XCD;
  if (lid >= xcd_end) return;

  // ---- producer: the slab stream, two slabs ahead of the MFMAs ------------------
  // A wave-wide load covers rows 8*(wave + NW*i) + lane/8 of the A (or B) tile, chunk lane%8 of the row's
  // 128-byte slab.  Its LDS destination is row*128 + ((chunk ^ ((row>>1)&7)) << 4); (row>>1)&7 does not
  // depend on i, so the destinations of one lane differ by the constant NW*8*128 bytes.
  const int ld_row = lane >> 3;
  const int ld_chunk = lane & 7;
  const int st_row = wave * 8 + ld_row;
  const int st_off = st_row * ROW_BYTES + ((ld_chunk ^ ((st_row >> 1) & 7)) << 4);
  // A direct-to-LDS request lands lane l at byte 16*l of the wave's 1 KiB (row l/8, position l%8), so the
  // swizzle is applied on the source side: position c' of row r receives chunk c' ^ ((r>>1)&7).
  const int src_chunk = C::DIRECT ? (ld_chunk ^ ((st_row >> 1) & 7)) : ld_chunk;
  const unsigned lds_base_addr = __builtin_amdgcn_readfirstlane(lds_address(lds));
  int p_lid = lid;
  bool p_valid = true;
  int p_kt = 0, p_KT = 0;
  const unsigned char* p_abase = nullptr;
  const unsigned char* p_bbase = nullptr;
  unsigned p_off[C::LOADS];
  i32x4 G[C::DIRECT ? 1 : C::LOADS];  // the slab in flight between global memory and LDS (register-staged shapes)
  auto p_setup = [&]() {
    const TileCoord tc = locate<C>(tab, p_lid);
    const hdit_gemm_problem& pr = tab.p[tc.pi];
    p_abase = (const unsigned char*)pr.a;
    p_bbase = (const unsigned char*)pr.b;
    p_KT = pr.k / BK;
    p_kt = 0;
#pragma unroll
    for (int i = 0; i < C::A_LOADS; i++) {
      const int gr = min(tc.m0 + (wave + i * NW) * 8 + ld_row, pr.m - 1);
      unsigned row_off = (unsigned)gr * (unsigned)pr.lda;  // byte offsets stay below 2^32: checked on the host
      asm volatile("" : "+v"(row_off));  // a product of its own: fused with the addition it is a 64-bit multiply-add,
                                         // and the offsets then occupy register pairs for the whole kernel
      p_off[i] = (row_off + (unsigned)(src_chunk * 8)) * 2u;
    }
#pragma unroll
    for (int i = 0; i < C::B_LOADS; i++) {
      const int gr = min(tc.n0 + (wave + i * NW) * 8 + ld_row, pr.n - 1);
      unsigned row_off = (unsigned)gr * (unsigned)pr.ldb;
      asm volatile("" : "+v"(row_off));
      p_off[C::A_LOADS + i] = (row_off + (unsigned)(src_chunk * 8)) * 2u;
    }
  };
  // Once the stream is exhausted the last slab is simply loaded again and written to a stage nobody
  // reads: no branch may split the MFMA stream the loads are interleaved with.
  auto g_load = [&](int i) {
    const unsigned char* base = (i < C::A_LOADS ? p_abase : p_bbase) + (size_t)p_kt * ROW_BYTES;
    G[i] = *(const i32x4*)(base + p_off[i]);
  };
  // direct-to-LDS request i of the slab at the cursor: A rows into A slot `slot`, B rows into B slot `slot`
  const unsigned wave_lds = lds_base_addr + wave * 8 * ROW_BYTES;
  auto dma_a = [&](int slot, int i) {
    lds_dma16_sum(p_abase + (size_t)p_kt * ROW_BYTES, p_off[i], wave_lds + slot * C::A_BYTES, i * (NW * 8 * ROW_BYTES));
  };
  auto dma_b = [&](int slot, int i) {
    lds_dma16_sum(p_bbase + (size_t)p_kt * ROW_BYTES, p_off[C::A_LOADS + i], wave_lds + C::B_OFF + slot * C::B_BYTES,
                  i * (NW * 8 * ROW_BYTES));
  };
  // ring shapes: request i (A rows, then B rows) of the slab at the cursor into stage `slot`
  auto dma_ring = [&](int slot, int i) {
    if (i < C::A_LOADS)
      lds_dma16_sum(p_abase + (size_t)p_kt * ROW_BYTES, p_off[i], wave_lds + slot * C::STAGE_BYTES, i * (NW * 8 * ROW_BYTES));
    else
      lds_dma16_sum(p_bbase + (size_t)p_kt * ROW_BYTES, p_off[i], wave_lds + slot * C::STAGE_BYTES,
                    C::A_BYTES + (i - C::A_LOADS) * (NW * 8 * ROW_BYTES));
  };
  auto l_store = [&](int stage, int i) {
    const int tile_off = i < C::A_LOADS ? i * (NW * 8 * ROW_BYTES) : C::A_BYTES + (i - C::A_LOADS) * (NW * 8 * ROW_BYTES);
    *(i32x4*)(lds + stage * C::STAGE_BYTES + tile_off + st_off) = G[i];
  };
  auto p_advance = [&]() {
    if (!p_valid) return;
    if (++p_kt == p_KT) {
      p_lid += wgs_per_xcd;
      p_valid = p_lid < xcd_end;
      if (p_valid) p_setup();
      else p_kt = p_KT - 1;
    }
  };

  // ---- consumer ------------------------------------------------------------
  // fragment read offsets: row r, logical chunk c -> r*128 + ((c ^ ((r>>1)&7)) << 4); fragment rows are
  // l32 plus a multiple of 32, so (r>>1)&7 == (l32>>1)&7.  k-step ks uses chunk 2*ks + lh.
  const int swz = (l32 >> 1) & 7;
  const int a_row = (wm0 + l32) * ROW_BYTES;
  const int b_row = (wn0 + l32) * ROW_BYTES;
  bf16x8 fa[2][TM], fb[2][TN];
  auto read_frags2 = [&](const unsigned char* abase, const unsigned char* bbase, int ks, int buf) {
    const int ch = ((ks * 2 + lh) ^ swz) << 4;
#pragma unroll
    for (int i = 0; i < TM; i++) fa[buf][i] = *(const bf16x8*)(abase + a_row + ch + i * 32 * ROW_BYTES);
#pragma unroll
    for (int j = 0; j < TN; j++) fb[buf][j] = *(const bf16x8*)(bbase + b_row + ch + j * 32 * ROW_BYTES);
  };
  auto read_frags = [&](const unsigned char* sbase, int ks, int buf) { read_frags2(sbase, sbase + C::A_BYTES, ks, buf); };

  // The bias enters through the accumulators: a tile's accumulators start as bias (x) ones -- one MFMA per 32-column
  // block, whose A operand holds bias[n] at k = 0 and whose B operand holds 1 at k = 0 -- instead of zero.  The
  // epilogue then needs neither bias registers (the 256 x 256 shape could only find its 32 by spilling accumulators)
  // nor an LDS slot, and every shape forms bias + sum of products in the same order, so results do not depend on the
  // shape a problem is given.  Lane l < 32 fetches the bias of column l of each of the wave's column blocks; the
  // values of the next tile are requested at the start of the current tile's epilogue, in front of its stores.
  unsigned short bnext[TN];
  auto fetch_bias = [&](const TileCoord& tc) {
    const hdit_gemm_problem& pr = tab.p[tc.pi];
    const unsigned short* bsrc = (const unsigned short*)pr.bias;
#pragma unroll
    for (int j = 0; j < TN; j++) {
      bnext[j] = 0;
      if (bsrc) bnext[j] = bsrc[min(tc.n0 + wn0 + j * 32 + l32, pr.n - 1)];
    }
  };
  fetch_bias(locate<C>(tab, lid));

  // prologue: slab 0 into stage 0, slab 1 into the registers
  p_setup();
  int stage = 0;
  int sa = 0, sb = 0;  // DMA: the A and B slots of the slab being multiplied
  if constexpr (C::DMA) {
    // slab 0 into slots (0, 0), slab 1 into slots (1, 1); slab 0 has landed before the first fragment read
#pragma unroll
    for (int i = 0; i < C::A_LOADS; i++) dma_a(0, i);
#pragma unroll
    for (int i = 0; i < C::B_LOADS; i++) dma_b(0, i);
    p_advance();
#pragma unroll
    for (int i = 0; i < C::A_LOADS; i++) dma_a(1, i);
#pragma unroll
    for (int i = 0; i < C::B_LOADS; i++) dma_b(1, i);
    p_advance();
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(C::LOADS));
    __syncthreads();
    read_frags2(lds, lds + C::B_OFF, 0, 0);
  } else if constexpr (C::RING) {
    // slabs 0 .. NS-2 into stages 0 .. NS-2; slab 0 has landed before the first fragment read
#pragma unroll
    for (int s = 0; s < C::NS - 1; s++) {
#pragma unroll
      for (int i = 0; i < C::LOADS; i++) dma_ring(s, i);
      p_advance();
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((C::NS - 2) * C::LOADS));
    __syncthreads();
    read_frags(lds, 0, 0);
  } else {
#pragma unroll
    for (int i = 0; i < C::LOADS; i++) g_load(i);
    p_advance();
#pragma unroll
    for (int i = 0; i < C::LOADS; i++) l_store(0, i);
#pragma unroll
    for (int i = 0; i < C::LOADS; i++) g_load(i);
    p_advance();
    __syncthreads();
    read_frags(lds, 0, 0);
  }

  constexpr int NMMA = TM * TN;
  constexpr int NRD = TM + TN;            // fragment reads per k-step
  constexpr int RD_MFMA = (NRD + 1) / 2;  // MFMAs that are followed by two fragment reads
  constexpr int SLOTS = NMMA - RD_MFMA;   // MFMAs per k-step that can carry a write+load pair
  constexpr int CP = (C::LOADS + 2) / 3;  // pairs per k-step (k-steps 0..2 of a slab)
  static_assert(RD_MFMA < NMMA, "not enough MFMAs to place the fragment reads");

  bool first_tile = true;
  while (true) {
    const TileCoord tc = locate<C>(tab, lid);
    const hdit_gemm_problem& pr = tab.p[tc.pi];
    const int KT = pr.k / BK;
    if (!first_tile) {
      __syncthreads();  // every wave has left the previous epilogue, whose staging windows the next writes reuse
    }
    first_tile = false;

    f32x16 acc[TM][TN];
    {
      const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      i32x4 ones_bits = {lh == 0 ? 0x3f80 : 0, 0, 0, 0};  // bf16 1.0 at k = 0 (lanes < 32 hold k = 0..7)
      bf16x8 ones;
      __builtin_memcpy(&ones, &ones_bits, 16);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        i32x4 bb = {lh == 0 ? (int)bnext[j] : 0, 0, 0, 0};
        bf16x8 bfr;
        __builtin_memcpy(&bfr, &bb, 16);
#pragma unroll
        for (int i = 0; i < TM; i++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr, ones, zero, 0, 0, 0);
      }
    }

    // One k-step: the MFMAs on fragment buffer `buf`.  Under them, pinned in this order: two reads per MFMA
    // of the fragments the next k-step needs (an MFMA goes first, so that its wait for its own fragments
    // is placed while no younger read is outstanding), then the write+load pairs [cp_first, cp_last)
    // spread over the remaining MFMAs: registers of slab h+1 to LDS stage `wstage`, then the same
    // registers refilled with slab h+2.
    auto k_step = [&](int buf, const unsigned char* rd_base, int rd_ks, int wstage, int cp_first, int cp_last) {
      read_frags(rd_base, rd_ks, buf ^ 1);
#pragma unroll
      for (int t = 0; t < NMMA; t++) {
        acc[t / TN][t % TN] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][t % TN], fa[buf][t / TN], acc[t / TN][t % TN], 0, 0, 0);
        if (t == RD_MFMA - 1) {
#pragma unroll
          for (int u = 0; u < RD_MFMA; u++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                        // MFMA
            if (2 * u + 2 <= NRD) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // DS reads
            else __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          SCHED_FENCE();
        }
        if (t >= RD_MFMA) {
#pragma unroll
          for (int j = 0; j < CP; j++)
            if (RD_MFMA + (j * SLOTS) / CP == t && cp_first + j < cp_last) {
              l_store(wstage, cp_first + j);
              g_load(cp_first + j);
            }
          SCHED_FENCE();
        }
      }
    };

    // The same k-step for the direct-to-LDS shapes: under the MFMAs that carry no fragment reads, requests
    // [first, last) of the slab at the cursor -- A rows (kind 0) or B rows (kind 1) -- into slot `slot`.
    auto k_step_dma = [&](int buf, const unsigned char* rd_a, const unsigned char* rd_b, int rd_ks, int kind, int first,
                          int last, int slot) {
      read_frags2(rd_a, rd_b, rd_ks, buf ^ 1);
#pragma unroll
      for (int t = 0; t < NMMA; t++) {
        acc[t / TN][t % TN] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][t % TN], fa[buf][t / TN], acc[t / TN][t % TN], 0, 0, 0);
        if (t == RD_MFMA - 1) {
#pragma unroll
          for (int u = 0; u < RD_MFMA; u++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                        // MFMA
            if (2 * u + 2 <= NRD) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // DS reads
            else __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          SCHED_FENCE();
        }
        if (t >= RD_MFMA) {
          const int n = last - first;
#pragma unroll
          for (int j = 0; j < C::LOADS; j++)
            if (j < n && RD_MFMA + (j * SLOTS) / (n > 0 ? n : 1) == t) {
              if (kind == 0) dma_a(slot, first + j);
              else if (kind == 1) dma_b(slot, first + j);
              else dma_ring(slot, first + j);
            }
          SCHED_FENCE();
        }
      }
    };
    constexpr int CPA = (C::A_LOADS + 2) / 3;  // A requests per k-step (k-steps 0..2 of a slab)

    if constexpr (C::DMA) {
      for (int kt = 0; kt < KT; kt++) {
        const unsigned char* ab = lds + sa * C::A_BYTES;
        const unsigned char* bb = lds + C::B_OFF + sb * C::B_BYTES;
        // A rows of the slab after next go to the slot the previous slab vacated
        const int sa_req = sa == 0 ? C::A_SLOTS - 1 : sa - 1;
        k_step_dma(0, ab, bb, 1, 0, 0, CPA, sa_req);
        k_step_dma(1, ab, bb, 2, 0, CPA, 2 * CPA, sa_req);
        k_step_dma(0, ab, bb, 3, 0, 2 * CPA, C::A_LOADS, sa_req);
        // ---- turn over: everything but the A requests just issued has landed (the next slab is complete),
        // and the fragments of the last k-step are in registers
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(C::A_LOADS) & 0xf0ff);  // and lgkmcnt(0)
        __syncthreads();
        const int sb_req = sb;  // the B slot this slab vacates takes the B rows of the slab after next
        sa = sa == C::A_SLOTS - 1 ? 0 : sa + 1;
        sb ^= 1;
        k_step_dma(1, lds + sa * C::A_BYTES, lds + C::B_OFF + sb * C::B_BYTES, 0, 1, 0, C::B_LOADS, sb_req);
        p_advance();
      }
    } else if constexpr (C::RING) {
      constexpr int RQ = C::LOADS / 4;  // requests per k-step
      static_assert(C::LOADS % 4 == 0, "ring requests are dealt evenly to the four k-steps");
      for (int kt = 0; kt < KT; kt++) {
        const unsigned char* sbase = lds + stage * C::STAGE_BYTES;
        // the slab NS-1 ahead goes to the stage the previous slab vacated
        const int rq = stage == 0 ? C::NS - 1 : stage - 1;
        k_step_dma(0, sbase, sbase + C::A_BYTES, 1, 2, 0, RQ, rq);
        k_step_dma(1, sbase, sbase + C::A_BYTES, 2, 2, RQ, 2 * RQ, rq);
        k_step_dma(0, sbase, sbase + C::A_BYTES, 3, 2, 2 * RQ, 3 * RQ, rq);
        // ---- turn over: the next slab has landed -- everything but the slab after it (NS-3 whole slabs in
        // general) and the requests just issued
        __builtin_amdgcn_s_waitcnt(waitcnt_vm((C::NS - 3) * C::LOADS + 3 * RQ) & 0xf0ff);  // and lgkmcnt(0)
        __syncthreads();
        stage = stage == C::NS - 1 ? 0 : stage + 1;
        const unsigned char* nbase = lds + stage * C::STAGE_BYTES;
        k_step_dma(1, nbase, nbase + C::A_BYTES, 0, 2, 3 * RQ, C::LOADS, rq);
        p_advance();
      }
    } else
    for (int kt = 0; kt < KT; kt++) {
      const unsigned char* sbase = lds + stage * C::STAGE_BYTES;
      const int wstage = stage ^ 1;  // held slab h-1; every wave passed the barrier of that slab
      k_step(0, sbase, 1, wstage, 0, CP);
      k_step(1, sbase, 2, wstage, CP, 2 * CP);
      k_step(0, sbase, 3, wstage, 2 * CP, C::LOADS);
      p_advance();
      // ---- turn the stages over: the fragments of the last k-step are in registers, slab h+1 is written
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __syncthreads();
      stage ^= 1;
      k_step(1, lds + stage * C::STAGE_BYTES, 0, wstage, 0, 0);
    }
    // staging window of this wave: inside the stage (the A slot) the tile's last slab vacated
    unsigned char* epi = lds + wave * EPI_WAVE_BYTES +
                         (C::DMA    ? (sa == 0 ? C::A_SLOTS - 1 : sa - 1) * C::A_BYTES
                          : C::RING ? (stage == 0 ? C::NS - 1 : stage - 1) * C::STAGE_BYTES
                                    : (stage ^ 1) * C::STAGE_BYTES);

    // ---- epilogue ---------------------------------------------------------
    auto epilogue = [&](auto mode_tag) {
      constexpr int MODE = decltype(mode_tag)::value;
      constexpr bool GATED = MODE == HDIT_EPI_GATE_RESIDUAL;
      // The lane-dependent addresses of the epilogue are recomputed per tile from an opaque copy of the lane id:
      // otherwise the compiler hoists some fifty of them out of the tile loop and, the main loop having no registers
      // to spare, spills them around it -- reloads that wait for every operand request in flight.
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      const int l32 = lane_e & 31, lh = lane_e >> 5;
      // all addressing below is a uniform base plus a 32-bit byte offset per lane (checked on the host)
      unsigned char* __restrict__ Cb = (unsigned char*)pr.c;
      const unsigned char* __restrict__ Rb = (const unsigned char*)pr.resid;
      const float* __restrict__ gate = pr.gate;
      const int M = pr.m, N = pr.n;
      const int ldc = (int)pr.ldc, ldr = (int)pr.ldr;
      const int ncol0 = tc.n0 + wn0;

      // Write-back layout: 16 lanes cover one 256-byte row segment, a wave covers 4 rows per pass, 8 passes
      // per 32-row block, done as two halves of 4.  The residual rows and the gate columns are requested one
      // block ahead, before the stores in front of them: vector memory operations retire in order, so a load
      // placed behind stores would wait for the stores' round trip.
      const int rchunk = lane_e & 15;
      const int wr_row = lane_e >> 4;
      const int wr_n = ncol0 + rchunk * 8;
      const int wr_nc = min(wr_n, N - 8);
      const bool wr_ok = rchunk < 4 * TN && wr_n < N;
      // The residual stream may be carried in fp32 (HDIT_EPI_RESID_F32 / HDIT_EPI_OUT_F32): a lane's 8 columns
      // are then 32 bytes, moved as two 16-byte accesses.
      const bool rf32 = GATED && (pr.epilogue & HDIT_EPI_RESID_F32) != 0;
      const bool of32 = GATED && (pr.epilogue & HDIT_EPI_OUT_F32) != 0;
      i32x4 rres[8], rres_hi[GATED ? 8 : 1];
      f32x4 gte0, gte1;
      bool straddle = false;
      auto prefetch_rows = [&](int i, int half) {
        const int mrow0 = tc.m0 + wm0 + i * 32;
#pragma unroll
        for (int it = half * 4; it < half * 4 + 4; it++) {
          const int mm = min(mrow0 + it * 4 + wr_row, M - 1);
          if (rf32) {
            const unsigned char* rp = Rb + (unsigned)((mm * ldr + wr_nc) * 4);
            rres[it] = *(const i32x4*)rp;
            rres_hi[GATED ? it : 0] = *(const i32x4*)(rp + 16);
          } else {
            rres[it] = *(const i32x4*)(Rb + (unsigned)((mm * ldr + wr_nc) * 2));
          }
        }
      };
      auto prefetch_gate = [&](int i) {
        const int mrow0 = tc.m0 + wm0 + i * 32;
        const int b_lo = min(mrow0, M - 1) / pr.rows_per_batch;
        straddle = min(mrow0 + 31, M - 1) >= (b_lo + 1) * pr.rows_per_batch;
        const float* g = gate + (int64_t)b_lo * pr.gate_stride + wr_nc;
        gte0 = *(const f32x4*)g;
        gte1 = *(const f32x4*)(g + 4);
      };
      {
        // bias of the next tile of this workgroup (this tile's is inside its accumulators: see the tile start)
        const int next_lid = lid + wgs_per_xcd;
        if (next_lid < xcd_end) fetch_bias(locate<C>(tab, next_lid));
      }
      if (GATED) {
        prefetch_rows(0, 0);
        prefetch_rows(0, 1);
        prefetch_gate(0);
      }

      typedef __attribute__((address_space(3))) i32x4 lds_i32x4;
#pragma unroll
      for (int i = 0; i < TM; i++) {
        const int mrow0 = tc.m0 + wm0 + i * 32;
        // Staging addresses: the XOR swizzle only touches bits 4-7, which are zero in the 256-byte aligned row
        // base, so slot (chunk ^ (row & 15)) of a row is (row base + ((row & 15) << 4)) ^ (chunk << 4): one register
        // and one v_xor per access, made opaque per block so that the sixteen write and eight read addresses are not
        // computed ahead and spilled.
        unsigned wa = lds_address(epi) + l32 * 256 + ((l32 & 15) << 4);
        unsigned ra = lds_address(epi) + wr_row * 256 + ((rchunk ^ wr_row) << 4);
        asm volatile("" : "+v"(wa), "+v"(ra));
#pragma unroll
        for (int j = 0; j < TN; j++) {
#pragma unroll
          for (int gp = 0; gp < 2; gp++) {
            // accumulator groups g = 2gp (even) and 2gp+1 (odd) hold columns 8g + 4*lh + e.  After the swap
            // lanes < 32 own the 8 columns of the even group, lanes >= 32 those of the odd group.
            float v[8];
#pragma unroll
            for (int e = 0; e < 4; e++) {
              auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(acc[i][j][(2 * gp) * 4 + e]),
                                                         __float_as_int(acc[i][j][(2 * gp + 1) * 4 + e]), false, false);
              v[e] = __int_as_float(sw[0]);
              v[4 + e] = __int_as_float(sw[1]);
            }
            const int chunk = j * 4 + 2 * gp + lh;  // 16-byte chunk inside the wave's 256-byte row
            if (MODE == HDIT_EPI_BIAS_GELU) {
#pragma unroll
              for (int e = 0; e < 8; e++) v[e] = hdit::gelu_tanh_f(v[e]);
            }
            *(lds_i32x4*)(uintptr_t)(wa ^ (unsigned)(chunk << 4)) = hdit::pack8(v);
          }
          SCHED_FENCE();  // keeps the scheduler from pulling whole accumulator tiles into VGPRs at once
        }
        // coalesced write-back of this 32 x (32*TN) block
#pragma unroll
        for (int half = 0; half < 2; half++) {
          i32x4 outv[4], outv_hi[GATED ? 4 : 1];
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int it = half * 4 + q;
            const int r = it * 4 + wr_row;
            // row r = 4 it + wr_row: slot rchunk ^ (r & 15) = (rchunk ^ wr_row) ^ 4 (it & 3)
            i32x4 val = *(const lds_i32x4*)(uintptr_t)((ra ^ (unsigned)(((it & 3) * 4) << 4)) + it * 1024);
            if (GATED) {
              f32x4 g0 = gte0, g1 = gte1;
              if (straddle) {  // rows of this block belong to different batch elements: fetch the gate per row
                const int mm = min(mrow0 + r, M - 1);
                const float* g = gate + (int64_t)(mm / pr.rows_per_batch) * pr.gate_stride + wr_nc;
                g0 = *(const f32x4*)g;
                g1 = *(const f32x4*)(g + 4);
              }
              float u[8], rf[8];
              hdit::unpack8(val, u);
              if (rf32) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                  rf[e] = __int_as_float(rres[it][e]);
                  rf[4 + e] = __int_as_float(rres_hi[GATED ? it : 0][e]);
                }
              } else {
                hdit::unpack8(rres[it], rf);
              }
#pragma unroll
              for (int e = 0; e < 4; e++) {
                u[e] = __builtin_fmaf(g0[e], u[e], rf[e]);
                u[4 + e] = __builtin_fmaf(g1[e], u[4 + e], rf[4 + e]);
              }
              if (of32) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                  val[e] = __float_as_int(u[e]);
                  outv_hi[GATED ? q : 0][e] = __float_as_int(u[4 + e]);
                }
              } else {
                val = hdit::pack8(u);
              }
            }
            outv[q] = val;
          }
          SCHED_FENCE();
          if (GATED && i + 1 < TM) {
            prefetch_rows(i + 1, half);
            if (half == 1) prefetch_gate(i + 1);
          }
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int mm = mrow0 + (half * 4 + q) * 4 + wr_row;
            if (wr_ok && mm < M) {
              if (of32) {
                unsigned char* cp = Cb + (unsigned)((mm * ldc + wr_n) * 4);
                *(i32x4*)cp = outv[q];
                *(i32x4*)(cp + 16) = outv_hi[GATED ? q : 0];
              } else {
                *(i32x4*)(Cb + (unsigned)((mm * ldc + wr_n) * 2)) = outv[q];
              }
            }
          }
          SCHED_FENCE();
        }
      }
    };
    if ((pr.epilogue & HDIT_EPI_MODE_MASK) == HDIT_EPI_BIAS) epilogue(std::integral_constant<int, HDIT_EPI_BIAS>{});
    else if ((pr.epilogue & HDIT_EPI_MODE_MASK) == HDIT_EPI_BIAS_GELU) epilogue(std::integral_constant<int, HDIT_EPI_BIAS_GELU>{});
    else epilogue(std::integral_constant<int, HDIT_EPI_GATE_RESIDUAL>{});

    // Leave nothing of the epilogue in flight.  The compiler's bookkeeping of pending loads is path-insensitive:
    // one epilogue load it believes may still be pending makes it place a small vmcnt wait where the main loop
    // first reuses that register, and that wait drains the operand stream on every slab (the direct-to-LDS
    // requests are invisible to it, and the register-staged loads of the slab after next are younger).
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    lid += wgs_per_xcd;
    if (lid >= xcd_end) break;
  }
  // requests past the end of the stream are still in flight: nothing may land in LDS after this returns
  if constexpr (C::DIRECT) __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
}

template <class C>
__global__ void __launch_bounds__(NT) gemm_kernel(const GemmTable tab, int total_tiles, int tiles_per_xcd,
                                                  int wgs_per_xcd) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  run_tiles<C>(tab, total_tiles, tiles_per_xcd, wgs_per_xcd, lds);
}

// Two tile shapes in one launch: the large tiles of the tall problems first, then the small tiles of the
// short ones (the text stream of a joint block), which a workgroup starts as soon as its large tiles are
// done: no second launch, and the small tiles fill the tail of the large ones.
template <class C1, class C2>
__global__ void __launch_bounds__(NT) gemm_kernel2(const GemmTable tab1, int total1, int per_xcd1, const GemmTable tab2,
                                                   int total2, int per_xcd2, int wgs_per_xcd) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  run_tiles<C1>(tab1, total1, per_xcd1, wgs_per_xcd, lds);
  __syncthreads();  // the second phase reuses the LDS of the first
  run_tiles<C2>(tab2, total2, per_xcd2, wgs_per_xcd, lds);
}

std::atomic<int> g_num_cus{0};

int max_workgroups() {
  if (g_num_cus.load(std::memory_order_acquire) == 0) {
    int dev = 0, n = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) {
      hdit_host::set_error(hipGetErrorString(e));
      return -1;
    }
    g_num_cus.store(n, std::memory_order_release);
  }
  int max_wgs = g_num_cus.load(std::memory_order_relaxed) / NUM_XCD * NUM_XCD;  // one workgroup per CU: a wave may use the whole register file
  return max_wgs < NUM_XCD ? NUM_XCD : max_wgs;
}

template <class C>
int launch(const GemmTable& tab, int total_tiles, hipStream_t stream) {
  static std::atomic<bool> attr_set{false};  // setting the attribute twice from two threads is harmless
  if (!attr_set.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) {
      hdit_host::set_error(hipGetErrorString(e));
      return HDIT_ELAUNCH;
    }
    attr_set.store(true, std::memory_order_release);
  }
  const int max_wgs = max_workgroups();
  if (max_wgs < 0) return HDIT_ELAUNCH;
  const int tiles_per_xcd = (total_tiles + NUM_XCD - 1) / NUM_XCD;
  int wgs_per_xcd = max_wgs / NUM_XCD;
  if (wgs_per_xcd > tiles_per_xcd) wgs_per_xcd = tiles_per_xcd;
  hipLaunchKernelGGL(gemm_kernel<C>, dim3(wgs_per_xcd * NUM_XCD), dim3(NT), C::LDS_BYTES, stream, tab, total_tiles,
                     tiles_per_xcd, wgs_per_xcd);
  return hdit_host::check_launch("hdit_gemm_bf16");
}

template <class C>
int fill_table(GemmTable& tab, const hdit_gemm_problem* problems, int count) {
  tab.count = count;
  int total = 0;
  for (int i = 0; i < count; i++) {
    tab.p[i] = problems[i];
    tab.tile_start[i] = total;
    total += ((problems[i].m + C::BM - 1) / C::BM) * ((problems[i].n + C::BN - 1) / C::BN);
  }
  for (int i = count; i <= HDIT_GEMM_MAX_PROBLEMS; i++) tab.tile_start[i] = total;
  return total;
}

template <class C1, class C2>
int launch2(const hdit_gemm_problem* p1, int n1, const hdit_gemm_problem* p2, int n2, hipStream_t stream) {
  constexpr int LDS = C1::LDS_BYTES > C2::LDS_BYTES ? C1::LDS_BYTES : C2::LDS_BYTES;
  static std::atomic<bool> attr_set{false};  // setting the attribute twice from two threads is harmless
  if (!attr_set.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_kernel2<C1, C2>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (e != hipSuccess) {
      hdit_host::set_error(hipGetErrorString(e));
      return HDIT_ELAUNCH;
    }
    attr_set.store(true, std::memory_order_release);
  }
  const int max_wgs = max_workgroups();
  if (max_wgs < 0) return HDIT_ELAUNCH;
  GemmTable t1, t2;
  const int total1 = fill_table<C1>(t1, p1, n1), total2 = fill_table<C2>(t2, p2, n2);
  const int per1 = (total1 + NUM_XCD - 1) / NUM_XCD, per2 = (total2 + NUM_XCD - 1) / NUM_XCD;
  int wgs_per_xcd = max_wgs / NUM_XCD;
  const int need = per1 > per2 ? per1 : per2;
  if (wgs_per_xcd > need) wgs_per_xcd = need;
  hipLaunchKernelGGL((gemm_kernel2<C1, C2>), dim3(wgs_per_xcd * NUM_XCD), dim3(NT), LDS, stream, t1, total1, per1, t2,
                     total2, per2, wgs_per_xcd);
  return hdit_host::check_launch("hdit_gemm_bf16");
}

template <class C>
int count_tiles(const hdit_gemm_problem* problems, int count) {
  int total = 0;
  for (int i = 0; i < count; i++)
    total += ((problems[i].m + C::BM - 1) / C::BM) * ((problems[i].n + C::BN - 1) / C::BN);
  return total;
}

template <class C>
int build_and_launch(const hdit_gemm_problem* problems, int count, hipStream_t stream) {
  GemmTable tab;
  const int total = fill_table<C>(tab, problems, count);
  if (total == 0) return HDIT_OK;
  return launch<C>(tab, total, stream);
}

using Cfg256x256 = Cfg<4, 4>;
using Cfg256x192 = Cfg<4, 3>;
using Cfg128x256 = Cfg<2, 4>;
using Cfg128x128 = Cfg<2, 2>;
using Cfg128x192 = Cfg<2, 3>;

std::atomic<int> g_force_cfg{-1};

// ---- launch planning ---------------------------------------------------------
// A launch runs ceil(tiles / CUs) rounds of tiles; a tile costs (k / 64) slab times plus an epilogue.
// Problems of very different heights (the 8192-row image stream and the 666-row text stream of a joint
// block) are badly served by one tile shape: the small problem's few large tiles add a nearly empty
// round.  The planner therefore gives every problem the shape that is cheapest for it alone, launches
// one kernel per shape, and falls back to a single shape when that is cheaper.
constexpr int NCFG = 5;
constexpr int kBM[NCFG] = {256, 128, 128, 256, 128};
constexpr int kBN[NCFG] = {192, 256, 128, 256, 192};
// measured on MI355X: microseconds per 64-wide slab and per epilogue of one tile
constexpr double kSlabUs[NCFG] = {1.21, 0.72, 0.44, 1.40, 0.68};
constexpr double kEpiUs[NCFG] = {13.0, 12.4, 8.0, 16.0, 7.1};  // epilogue plus the pipeline fill of a tile
constexpr double kLaunchUs = 3.0;
constexpr int kSlots = 256;

int tiles_of(const hdit_gemm_problem& p, int c) { return ((p.m + kBM[c] - 1) / kBM[c]) * ((p.n + kBN[c] - 1) / kBN[c]); }

// time of all tiles of `ps` under shape c, without launch overhead
double tiles_time(const hdit_gemm_problem* const* ps, int count, int c) {
  int tiles = 0;
  double work = 0;
  for (int i = 0; i < count; i++) {
    const int t = tiles_of(*ps[i], c);
    tiles += t;
    work += t * ((ps[i]->k / BK) * kSlabUs[c] + kEpiUs[c]);
  }
  if (tiles == 0) return 0;
  const int rounds = (tiles + kSlots - 1) / kSlots;
  return rounds * (work / tiles);
}

double launch_time(const hdit_gemm_problem* const* ps, int count, int c) {
  return count == 0 ? 0.0 : kLaunchUs + tiles_time(ps, count, c);
}

int launch_cfg(int cfg, const hdit_gemm_problem* problems, int count, hipStream_t s) {
  switch (cfg) {
    case 0: return build_and_launch<Cfg256x192>(problems, count, s);
    case 1: return build_and_launch<Cfg128x256>(problems, count, s);
    case 4: return build_and_launch<Cfg128x192>(problems, count, s);
    case 3: return build_and_launch<Cfg256x256>(problems, count, s);
    default: return build_and_launch<Cfg128x128>(problems, count, s);
  }
}

}  // namespace

extern "C" __attribute__((visibility("default"))) void hdit_gemm_force_config(int cfg) { g_force_cfg.store(cfg, std::memory_order_relaxed); }

extern "C" __attribute__((visibility("default"))) int hdit_gemm_bf16(const hdit_gemm_problem* problems, int count, void* stream) {
  if (!problems || count < 0 || count > HDIT_GEMM_MAX_PROBLEMS) return HDIT_EINVAL;
  hdit_gemm_problem live[HDIT_GEMM_MAX_PROBLEMS];
  int nlive = 0;
  for (int i = 0; i < count; i++) {
    const hdit_gemm_problem& p = problems[i];
    if (p.m < 0 || p.n <= 0 || p.k <= 0) return HDIT_EINVAL;
    if (p.m == 0) continue;
    if (!p.a || !p.b || !p.c) return HDIT_EINVAL;
    if (p.k % BK != 0 || p.n % 8 != 0) return HDIT_EUNSUPPORTED;
    if (p.lda % 8 || p.ldb % 8 || p.ldc % 8) return HDIT_EINVAL;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uintptr_t)p.c | (uintptr_t)p.bias) & 15) return HDIT_EINVAL;
    // rows are addressed with 32-bit byte offsets from the operand base
    if ((int64_t)p.m * p.lda * 2 >= (1ll << 32) || (int64_t)p.n * p.ldb * 2 >= (1ll << 32)) return HDIT_EUNSUPPORTED;
    const int mode = p.epilogue & HDIT_EPI_MODE_MASK;
    const int c_bytes = (p.epilogue & HDIT_EPI_OUT_F32) ? 4 : 2, r_bytes = (p.epilogue & HDIT_EPI_RESID_F32) ? 4 : 2;
    if (p.epilogue & ~(HDIT_EPI_MODE_MASK | HDIT_EPI_RESID_F32 | HDIT_EPI_OUT_F32)) return HDIT_EINVAL;
    if (mode > HDIT_EPI_GATE_RESIDUAL) return HDIT_EINVAL;
    // the fp32 residual stream only exists in the gated-residual epilogue
    if (mode != HDIT_EPI_GATE_RESIDUAL && (p.epilogue & (HDIT_EPI_RESID_F32 | HDIT_EPI_OUT_F32))) return HDIT_EINVAL;
    if ((int64_t)p.m * p.ldc * c_bytes >= (1ll << 31)) return HDIT_EUNSUPPORTED;
    if (mode == HDIT_EPI_GATE_RESIDUAL) {
      if (!p.resid || !p.gate || p.rows_per_batch <= 0 || p.ldr % 8) return HDIT_EINVAL;
      if ((int64_t)p.m * p.ldr * r_bytes >= (1ll << 31)) return HDIT_EUNSUPPORTED;
      if (((uintptr_t)p.resid & 15) || ((uintptr_t)p.gate & 15) || p.gate_stride % 4) return HDIT_EINVAL;
    }
    live[nlive++] = p;
  }
  if (nlive == 0) return HDIT_OK;
  hipStream_t s = (hipStream_t)stream;
  const int forced = g_force_cfg.load(std::memory_order_relaxed);
  if (forced >= 0) return launch_cfg(forced, live, nlive, s);

  // every problem's own best shape
  int own[HDIT_GEMM_MAX_PROBLEMS];
  const hdit_gemm_problem* ptr[HDIT_GEMM_MAX_PROBLEMS];
  for (int i = 0; i < nlive; i++) {
    const hdit_gemm_problem* one = &live[i];
    own[i] = 0;
    double best = launch_time(&one, 1, 0);
    for (int c = 1; c < NCFG; c++) {
      const double t = launch_time(&one, 1, c);
      if (t < best) best = t, own[i] = c;
    }
  }
  // plan A: one shape for everything
  for (int i = 0; i < nlive; i++) ptr[i] = &live[i];
  int single = 0;
  double single_cost = launch_time(ptr, nlive, 0);
  for (int c = 1; c < NCFG; c++) {
    const double t = launch_time(ptr, nlive, c);
    if (t < single_cost) single_cost = t, single = c;
  }
  // plan B: one launch, two shapes -- the problems that want 256-row tiles on the better of the two large
  // shapes, the others on the better of the two 128-row shapes
  hdit_gemm_problem big[HDIT_GEMM_MAX_PROBLEMS], small[HDIT_GEMM_MAX_PROBLEMS];
  const hdit_gemm_problem* pb[HDIT_GEMM_MAX_PROBLEMS];
  const hdit_gemm_problem* psm[HDIT_GEMM_MAX_PROBLEMS];
  int nb = 0, ns = 0;
  for (int i = 0; i < nlive; i++) {
    if (own[i] == 0 || own[i] == 3) big[nb] = live[i], pb[nb] = &live[i], nb++;
    else small[ns] = live[i], psm[ns] = &live[i], ns++;
  }
  double two_cost = 1e30;
  int big_cfg = 0, small_cfg = 2;
  if (nb > 0 && ns > 0) {
    const double t0 = tiles_time(pb, nb, 0), t3 = tiles_time(pb, nb, 3);
    big_cfg = t3 < t0 ? 3 : 0;
    // the short problems on 128x128 or, when that needs a second round, on 128x256
    const double s2 = tiles_time(psm, ns, 2), s1 = tiles_time(psm, ns, 1);
    small_cfg = s1 < s2 ? 1 : 2;
    two_cost = kLaunchUs + (t3 < t0 ? t3 : t0) + (s1 < s2 ? s1 : s2);
  }
  static const bool debug = getenv("HDIT_GEMM_DEBUG") != nullptr;
  if (debug) {
    fprintf(stderr, "hdit_gemm_bf16 plan:");
    for (int i = 0; i < nlive; i++) fprintf(stderr, " [%dx%dx%d epi%d own%d]", live[i].m, live[i].n, live[i].k, live[i].epilogue, own[i]);
    fprintf(stderr, " single cfg%d %.1f us, two-shape(big cfg%d, small cfg%d) %.1f us\n", single, single_cost, big_cfg,
            small_cfg, two_cost);
  }
  if (two_cost < single_cost) {
    if (big_cfg == 0 && small_cfg == 2) return launch2<Cfg256x192, Cfg128x128>(big, nb, small, ns, s);
    if (big_cfg == 0) return launch2<Cfg256x192, Cfg128x256>(big, nb, small, ns, s);
    if (small_cfg == 2) return launch2<Cfg256x256, Cfg128x128>(big, nb, small, ns, s);
    return launch2<Cfg256x256, Cfg128x256>(big, nb, small, ns, s);
  }
  return launch_cfg(single, live, nlive, s);
}
