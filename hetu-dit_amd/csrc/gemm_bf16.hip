// Grouped bf16 GEMM for gfx950:  C[m, n] = epilogue(A[m, k] . B[n, k]^T + bias)
//
// Persistent kernel: one 512-thread workgroup per CU walks a static list of
// 256x256 (or smaller) output tiles.  Both operands are k-contiguous, so A and
// B tiles are staged the same way: `global_load_lds_dwordx4` copies 64-wide k
// slabs straight from global memory into LDS (no VGPR staging, no ds_write),
// two LDS stages, one barrier per slab.  A wave-wide direct load writes 1 KiB
// of LDS in lane order, i.e. 8 rows x 128 bytes; the XOR swizzle that keeps
// the later ds_read_b128 fragment reads conflict-free is applied on the global
// side (lane l fetches 16-byte chunk (l%8)^(l/8) of row l/8), which stays
// inside one 128-byte line, so the global access remains fully coalesced.
// The first slab of the NEXT tile is requested before the epilogue of the
// current one, so tile prologues are hidden behind stores.
//
// MFMA mapping: v_mfma_f32_32x32x16_bf16 with the weight fragment as "A" (rows
// = n) and the activation fragment as "B" (columns = m): a lane's accumulator
// holds one output row m and runs of 4 consecutive n.  Lanes l and l^32 swap
// halves (v_permlane32_swap) so that each lane stores 16 contiguous bytes; the
// epilogue fuses bias, GELU-tanh or the gated residual.
//
// One launch covers up to HDIT_GEMM_MAX_PROBLEMS problems.  Tiles are dealt to
// workgroups so that the workgroups of one XCD (workgroup id mod 8; each XCD
// has a private L2) own a contiguous, 8-tile-row-grouped range.
#include "hdit_common.h"

namespace {

constexpr int BK = 64;          // k elements per LDS stage
constexpr int ROW_BYTES = 128;  // BK * sizeof(bf16)
constexpr int NUM_XCD = 8;
constexpr int GROUP_M = 8;

struct GemmTable {
  int count;
  int tile_start[HDIT_GEMM_MAX_PROBLEMS + 1];
  hdit_gemm_problem p[HDIT_GEMM_MAX_PROBLEMS];
};

template <int BM_, int BN_, int WGM_, int WGN_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
  static constexpr int NW = WGM * WGN;
  static constexpr int NT = NW * 64;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int A_LOADS = BM / 8 / NW;  // direct-to-LDS wave loads per wave per stage (8 rows each)
  static constexpr int B_LOADS = BN / 8 / NW;
  static constexpr int A_BYTES = BM * ROW_BYTES;
  static constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile/waves mismatch");
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

__device__ __forceinline__ void lds_dma16(const void* gptr, unsigned char* lds_dst_uniform) {
  __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)gptr,
                                   (void __attribute__((address_space(3)))*)lds_dst_uniform, 16, 0, 0);
}

template <class C>
__global__ void __launch_bounds__(C::NT) gemm_kernel(const GemmTable tab, int total_tiles, int tiles_per_xcd,
                                                      int wgs_per_xcd) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  const int wm0 = (wave / C::WGN) * C::WM;
  const int wn0 = (wave % C::WGN) * C::WN;

  // tiles of this workgroup: XCD x owns logical tiles [x*tiles_per_xcd, (x+1)*tiles_per_xcd),
  // dealt round-robin to that XCD's workgroups
  const int xcd = blockIdx.x % NUM_XCD;
  const int wg_in_xcd = blockIdx.x / NUM_XCD;
  const int xcd_begin = xcd * tiles_per_xcd;
  const int xcd_end = min(xcd_begin + tiles_per_xcd, total_tiles);

  // lane-constant parts of the direct-to-LDS copy: row-in-group l/8, swizzled chunk
  const int ld_row = lane >> 3;
  const int ld_chunk = (lane & 7) ^ ld_row;

  auto issue_stage = [&](const TileCoord& tc, int kt, int stage) {
    const hdit_gemm_problem& pr = tab.p[tc.pi];
    const __bf16* A = (const __bf16*)pr.a;
    const __bf16* B = (const __bf16*)pr.b;
    unsigned char* base = lds + stage * C::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < C::A_LOADS; i++) {
      const int grp = wave + i * C::NW;  // 8-row group inside the tile
      const int gr = min(tc.m0 + grp * 8 + ld_row, pr.m - 1);
      lds_dma16(A + (int64_t)gr * pr.lda + kt * BK + ld_chunk * 8, base + grp * 1024);
    }
#pragma unroll
    for (int i = 0; i < C::B_LOADS; i++) {
      const int grp = wave + i * C::NW;
      const int gr = min(tc.n0 + grp * 8 + ld_row, pr.n - 1);
      lds_dma16(B + (int64_t)gr * pr.ldb + kt * BK + ld_chunk * 8, base + C::A_BYTES + grp * 1024);
    }
  };

  // fragment read offsets: row r, logical chunk c -> r*128 + ((c ^ (r&7)) << 4); r&7 == l32&7 for every fragment
  const int swz = l32 & 7;
  int a_off[4], b_off[4];  // per k-step (chunk = 2*ks + lh)
#pragma unroll
  for (int ks = 0; ks < 4; ks++) {
    a_off[ks] = (wm0 + l32) * ROW_BYTES + (((ks * 2 + lh) ^ swz) << 4);
    b_off[ks] = C::A_BYTES + (wn0 + l32) * ROW_BYTES + (((ks * 2 + lh) ^ swz) << 4);
  }

  int lid = xcd_begin + wg_in_xcd;
  if (lid >= xcd_end) return;
  TileCoord tc = locate<C>(tab, lid);
  int stage = 0;
  issue_stage(tc, 0, stage);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();

  while (true) {
    const hdit_gemm_problem& pr = tab.p[tc.pi];
    const int KT = pr.k / BK;
    const int next_lid = lid + wgs_per_xcd;
    const bool has_next = next_lid < xcd_end;
    TileCoord ntc = tc;
    if (has_next) ntc = locate<C>(tab, next_lid);

    f32x16 acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    for (int kt = 0; kt < KT; kt++) {
      // request the next slab (or the next tile's first slab) into the other stage
      if (kt + 1 < KT) issue_stage(tc, kt + 1, stage ^ 1);
      else if (has_next) issue_stage(ntc, 0, stage ^ 1);

      const unsigned char* sbase = lds + stage * C::STAGE_BYTES;
      bf16x8 fa[2][C::TM], fb[2][C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; i++) fa[0][i] = *(const bf16x8*)(sbase + a_off[0] + i * 32 * ROW_BYTES);
#pragma unroll
      for (int j = 0; j < C::TN; j++) fb[0][j] = *(const bf16x8*)(sbase + b_off[0] + j * 32 * ROW_BYTES);
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        const int cur = ks & 1, nxt = cur ^ 1;
        if (ks + 1 < 4) {
#pragma unroll
          for (int i = 0; i < C::TM; i++) fa[nxt][i] = *(const bf16x8*)(sbase + a_off[ks + 1] + i * 32 * ROW_BYTES);
#pragma unroll
          for (int j = 0; j < C::TN; j++) fb[nxt][j] = *(const bf16x8*)(sbase + b_off[ks + 1] + j * 32 * ROW_BYTES);
        }
#pragma unroll
        for (int i = 0; i < C::TM; i++)
#pragma unroll
          for (int j = 0; j < C::TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's direct-to-LDS copies have landed
      __syncthreads();
      stage ^= 1;
    }

    // ---- epilogue ---------------------------------------------------------
    __bf16* __restrict__ Cp = (__bf16*)pr.c;
    const __bf16* __restrict__ bias = (const __bf16*)pr.bias;
    const __bf16* __restrict__ resid = (const __bf16*)pr.resid;
    const float* __restrict__ gate = pr.gate;
    const int epi = pr.epilogue;
    const int M = pr.m, N = pr.n;
    const int64_t ldc = pr.ldc, ldr = pr.ldr;
#pragma unroll
    for (int i = 0; i < C::TM; i++) {
      const int m = tc.m0 + wm0 + i * 32 + l32;
      const float* grow = nullptr;
      if (epi == HDIT_EPI_GATE_RESIDUAL) grow = gate + (int64_t)(min(m, M - 1) / pr.rows_per_batch) * pr.gate_stride;
#pragma unroll
      for (int j = 0; j < C::TN; j++) {
#pragma unroll
        for (int gp = 0; gp < 2; gp++) {
          // accumulator groups g = 2gp (even) and 2gp+1 (odd): columns 8g + 4*lh + e.  After the swap
          // lanes < 32 hold the 8 columns of the even group, lanes >= 32 those of the odd group.
          float v[8];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            auto sw = __builtin_amdgcn_permlane32_swap(__float_as_int(acc[i][j][(2 * gp) * 4 + e]),
                                                       __float_as_int(acc[i][j][(2 * gp + 1) * 4 + e]), false, false);
            v[e] = __int_as_float(sw[0]);
            v[4 + e] = __int_as_float(sw[1]);
          }
          const int n = tc.n0 + wn0 + j * 32 + (2 * gp + lh) * 8;
          if (m >= M || n >= N) continue;
          if (bias) {
            float bf[8];
            hdit::unpack8(*(const i32x4*)(bias + n), bf);
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] += bf[e];
          }
          if (epi == HDIT_EPI_BIAS_GELU) {
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = hdit::gelu_tanh_f(v[e]);
          } else if (epi == HDIT_EPI_GATE_RESIDUAL) {
            float rf[8];
            hdit::unpack8(*(const i32x4*)(resid + (int64_t)m * ldr + n), rf);
            f32x4 g0 = *(const f32x4*)(grow + n), g1 = *(const f32x4*)(grow + n + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
              v[e] = rf[e] + g0[e] * v[e];
              v[4 + e] = rf[4 + e] + g1[e] * v[4 + e];
            }
          }
          *(i32x4*)(Cp + (int64_t)m * ldc + n) = hdit::pack8(v);
        }
      }
    }

    if (!has_next) break;
    lid = next_lid;
    tc = ntc;
  }
}

template <class C>
int launch(const GemmTable& tab, int total_tiles, hipStream_t stream) {
  static bool attr_set = false;
  static int num_cus = 0;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e == hipSuccess) {
      int dev = 0;
      e = hipGetDevice(&dev);
      if (e == hipSuccess) e = hipDeviceGetAttribute(&num_cus, hipDeviceAttributeMultiprocessorCount, dev);
    }
    if (e != hipSuccess) {
      hdit_host::set_error(hipGetErrorString(e));
      return HDIT_ELAUNCH;
    }
    attr_set = true;
  }
  const int per_cu = (2 * C::LDS_BYTES <= 160 * 1024 && C::NT <= 256) ? 2 : 1;
  int max_wgs = (num_cus * per_cu) / NUM_XCD * NUM_XCD;
  if (max_wgs < NUM_XCD) max_wgs = NUM_XCD;
  const int tiles_per_xcd = (total_tiles + NUM_XCD - 1) / NUM_XCD;
  int wgs_per_xcd = max_wgs / NUM_XCD;
  if (wgs_per_xcd > tiles_per_xcd) wgs_per_xcd = tiles_per_xcd;
  hipLaunchKernelGGL(gemm_kernel<C>, dim3(wgs_per_xcd * NUM_XCD), dim3(C::NT), C::LDS_BYTES, stream, tab, total_tiles,
                     tiles_per_xcd, wgs_per_xcd);
  return hdit_host::check_launch("hdit_gemm_bf16");
}

template <class C>
int build_and_launch(const hdit_gemm_problem* problems, int count, hipStream_t stream) {
  GemmTable tab;
  tab.count = count;
  int total = 0;
  for (int i = 0; i < count; i++) {
    tab.p[i] = problems[i];
    tab.tile_start[i] = total;
    total += ((problems[i].m + C::BM - 1) / C::BM) * ((problems[i].n + C::BN - 1) / C::BN);
  }
  for (int i = count; i <= HDIT_GEMM_MAX_PROBLEMS; i++) tab.tile_start[i] = total;
  if (total == 0) return HDIT_OK;
  return launch<C>(tab, total, stream);
}

using Cfg256x256 = Cfg<256, 256, 2, 4>;
using Cfg256x128 = Cfg<256, 128, 4, 2>;
using Cfg128x128 = Cfg<128, 128, 2, 2>;

int g_force_cfg = -1;

}  // namespace

extern "C" __attribute__((visibility("default"))) void hdit_gemm_force_config(int cfg) { g_force_cfg = cfg; }

extern "C" __attribute__((visibility("default"))) int hdit_gemm_bf16(const hdit_gemm_problem* problems, int count, void* stream) {
  if (!problems || count < 0 || count > HDIT_GEMM_MAX_PROBLEMS) return HDIT_EINVAL;
  hdit_gemm_problem live[HDIT_GEMM_MAX_PROBLEMS];
  int nlive = 0;
  int64_t tiles256 = 0, tiles_mid = 0;
  for (int i = 0; i < count; i++) {
    const hdit_gemm_problem& p = problems[i];
    if (p.m < 0 || p.n <= 0 || p.k <= 0) return HDIT_EINVAL;
    if (p.m == 0) continue;
    if (!p.a || !p.b || !p.c) return HDIT_EINVAL;
    if (p.k % BK != 0 || p.n % 8 != 0) return HDIT_EUNSUPPORTED;
    if (p.lda % 8 || p.ldb % 8 || p.ldc % 8) return HDIT_EINVAL;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uintptr_t)p.c | (uintptr_t)p.bias) & 15) return HDIT_EINVAL;
    if (p.epilogue < HDIT_EPI_BIAS || p.epilogue > HDIT_EPI_GATE_RESIDUAL) return HDIT_EINVAL;
    if (p.epilogue == HDIT_EPI_GATE_RESIDUAL) {
      if (!p.resid || !p.gate || p.rows_per_batch <= 0 || p.ldr % 8) return HDIT_EINVAL;
      if (((uintptr_t)p.resid & 15) || ((uintptr_t)p.gate & 15) || p.gate_stride % 4) return HDIT_EINVAL;
    }
    tiles256 += (int64_t)((p.m + 255) / 256) * ((p.n + 255) / 256);
    tiles_mid += (int64_t)((p.m + 255) / 256) * ((p.n + 127) / 128);
    live[nlive++] = p;
  }
  if (nlive == 0) return HDIT_OK;
  hipStream_t s = (hipStream_t)stream;
  int cfg = g_force_cfg;
  if (cfg < 0) {
    // Prefer the largest tile that still gives every CU (256 of them) work for
    // about two rounds; small launches fall back to smaller tiles.
    if (tiles256 >= 2 * 256) cfg = 0;
    else if (tiles_mid >= 256) cfg = 1;
    else cfg = 2;
  }
  switch (cfg) {
    case 0: return build_and_launch<Cfg256x256>(live, nlive, s);
    case 1: return build_and_launch<Cfg256x128>(live, nlive, s);
    default: return build_and_launch<Cfg128x128>(live, nlive, s);
  }
}
