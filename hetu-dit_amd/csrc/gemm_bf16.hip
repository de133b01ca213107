// Grouped bf16 GEMM for gfx950:  C[m, n] = epilogue(A[m, k] . B[n, k]^T + bias)
//
// Both operands are k-contiguous, so A and B tiles are staged identically:
// 16-byte global loads -> registers -> LDS (XOR-swizzled 16-byte chunks, two
// buffers), one barrier per 64-wide k step, v_mfma_f32_32x32x16_bf16 from
// ds_read_b128 fragments.  The MFMA "A" operand is the weight fragment (rows =
// n) and the "B" operand the activation fragment (columns = m), so a lane's
// accumulator holds one output row m and runs of 4 consecutive n: the epilogue
// (bias, GELU-tanh, gated residual) writes 8-byte bf16 packets along the row.
//
// One launch covers up to HDIT_GEMM_MAX_PROBLEMS problems; workgroup ids are
// first de-interleaved over the 8 XCDs (hardware round-robins consecutive
// workgroups over XCDs, each with a private L2) and then walked in groups of 8
// tile rows so that the tiles resident on one XCD share A and B panels.
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
  static constexpr int A_CHUNKS = BM * 8 / NT;  // 16-byte chunks per thread per stage
  static constexpr int B_CHUNKS = BN * 8 / NT;
  static constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile/threads mismatch");
};

__device__ __forceinline__ int swz(int row, int chunk) { return row * ROW_BYTES + ((chunk ^ (row & 7)) << 4); }

template <class C>
__global__ void __launch_bounds__(C::NT) gemm_kernel(const GemmTable tab, int total_tiles, int tiles_per_xcd) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  // ---- which tile -------------------------------------------------------
  const int bid = blockIdx.x;
  const int lid = (bid % NUM_XCD) * tiles_per_xcd + bid / NUM_XCD;
  if (lid >= total_tiles) return;
  int pi = 0;
#pragma unroll 1
  while (pi + 1 < tab.count && lid >= tab.tile_start[pi + 1]) pi++;
  const hdit_gemm_problem& pr = tab.p[pi];
  const int M = pr.m, N = pr.n, K = pr.k;
  const int tiles_m = (M + C::BM - 1) / C::BM;
  const int tiles_n = (N + C::BN - 1) / C::BN;
  int t = lid - tab.tile_start[pi];
  const int in_group = GROUP_M * tiles_n;
  const int group = t / in_group;
  const int first_m = group * GROUP_M;
  const int gsz = min(tiles_m - first_m, GROUP_M);
  const int tm = first_m + (t % in_group) % gsz;
  const int tn = (t % in_group) / gsz;
  const int m0 = tm * C::BM, n0 = tn * C::BN;

  const __bf16* __restrict__ A = (const __bf16*)pr.a;
  const __bf16* __restrict__ B = (const __bf16*)pr.b;
  const int64_t lda = pr.lda, ldb = pr.ldb;

  // ---- global -> register staging ----------------------------------------
  // chunk id c = tid + i*NT: row = c / 8, kc = c % 8 (8 threads cover one 128-byte row)
  const __bf16* a_src[C::A_CHUNKS];
  const __bf16* b_src[C::B_CHUNKS];
  int a_dst[C::A_CHUNKS], b_dst[C::B_CHUNKS];
#pragma unroll
  for (int i = 0; i < C::A_CHUNKS; i++) {
    int c = tid + i * C::NT, row = c >> 3, kc = c & 7;
    int gr = min(m0 + row, M - 1);
    a_src[i] = A + (int64_t)gr * lda + kc * 8;
    a_dst[i] = swz(row, kc);
  }
#pragma unroll
  for (int i = 0; i < C::B_CHUNKS; i++) {
    int c = tid + i * C::NT, row = c >> 3, kc = c & 7;
    int gr = min(n0 + row, N - 1);
    b_src[i] = B + (int64_t)gr * ldb + kc * 8;
    b_dst[i] = C::BM * ROW_BYTES + swz(row, kc);
  }
  i32x4 a_reg[C::A_CHUNKS], b_reg[C::B_CHUNKS];

  auto load_global = [&](int kt) {
#pragma unroll
    for (int i = 0; i < C::A_CHUNKS; i++) a_reg[i] = *(const i32x4*)(a_src[i] + kt * BK);
#pragma unroll
    for (int i = 0; i < C::B_CHUNKS; i++) b_reg[i] = *(const i32x4*)(b_src[i] + kt * BK);
  };
  auto store_lds = [&](int stage) {
    unsigned char* base = lds + stage * C::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < C::A_CHUNKS; i++) *(i32x4*)(base + a_dst[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < C::B_CHUNKS; i++) *(i32x4*)(base + b_dst[i]) = b_reg[i];
  };

  // ---- per-wave fragment addressing ---------------------------------------
  const int wm0 = (wave / C::WGN) * C::WM;
  const int wn0 = (wave % C::WGN) * C::WN;
  const int l32 = lane & 31, lh = lane >> 5;

  f32x16 acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; i++)
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  const int KT = K / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  if (KT > 1) load_global(1);

  for (int kt = 0; kt < KT; kt++) {
    const unsigned char* sa = lds + (kt & 1) * C::STAGE_BYTES;
    const unsigned char* sb = sa + C::BM * ROW_BYTES;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      bf16x8 fa[C::TM], fb[C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; i++) fa[i] = *(const bf16x8*)(sa + swz(wm0 + i * 32 + l32, ks * 2 + lh));
#pragma unroll
      for (int j = 0; j < C::TN; j++) fb[j] = *(const bf16x8*)(sb + swz(wn0 + j * 32 + l32, ks * 2 + lh));
#pragma unroll
      for (int i = 0; i < C::TM; i++)
#pragma unroll
        for (int j = 0; j < C::TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) store_lds((kt + 1) & 1);
    __syncthreads();
    if (kt + 2 < KT) load_global(kt + 2);
  }

  // ---- epilogue -----------------------------------------------------------
  __bf16* __restrict__ Cp = (__bf16*)pr.c;
  const __bf16* __restrict__ bias = (const __bf16*)pr.bias;
  const __bf16* __restrict__ resid = (const __bf16*)pr.resid;
  const float* __restrict__ gate = pr.gate;
  const int epi = pr.epilogue;
  const int64_t ldc = pr.ldc, ldr = pr.ldr;
#pragma unroll
  for (int i = 0; i < C::TM; i++) {
    const int m = m0 + wm0 + i * 32 + l32;
    if (m >= M) continue;
    const float* grow = nullptr;
    if (epi == HDIT_EPI_GATE_RESIDUAL) grow = gate + (int64_t)(m / pr.rows_per_batch) * pr.gate_stride;
#pragma unroll
    for (int j = 0; j < C::TN; j++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int n = n0 + wn0 + j * 32 + g * 8 + lh * 4;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = acc[i][j][g * 4 + e];
        if (bias) {
          i32x2 braw = *(const i32x2*)(bias + n);
          v[0] += __uint_as_float((uint32_t)braw[0] << 16);
          v[1] += __uint_as_float((uint32_t)braw[0] & 0xffff0000u);
          v[2] += __uint_as_float((uint32_t)braw[1] << 16);
          v[3] += __uint_as_float((uint32_t)braw[1] & 0xffff0000u);
        }
        if (epi == HDIT_EPI_BIAS_GELU) {
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = hdit::gelu_tanh_f(v[e]);
        } else if (epi == HDIT_EPI_GATE_RESIDUAL) {
          i32x2 rraw = *(const i32x2*)(resid + (int64_t)m * ldr + n);
          f32x4 gv = *(const f32x4*)(grow + n);
          v[0] = __uint_as_float((uint32_t)rraw[0] << 16) + gv[0] * v[0];
          v[1] = __uint_as_float((uint32_t)rraw[0] & 0xffff0000u) + gv[1] * v[1];
          v[2] = __uint_as_float((uint32_t)rraw[1] << 16) + gv[2] * v[2];
          v[3] = __uint_as_float((uint32_t)rraw[1] & 0xffff0000u) + gv[3] * v[3];
        }
        i32x2 out;
        out[0] = (int)hdit::pack2(v[0], v[1]);
        out[1] = (int)hdit::pack2(v[2], v[3]);
        *(i32x2*)(Cp + (int64_t)m * ldc + n) = out;
      }
    }
  }
}

template <class C>
int launch(const GemmTable& tab, int total_tiles, hipStream_t stream) {
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) {
      hdit_host::set_error(hipGetErrorString(e));
      return HDIT_ELAUNCH;
    }
    attr_set = true;
  }
  int per_xcd = (total_tiles + NUM_XCD - 1) / NUM_XCD;
  hipLaunchKernelGGL(gemm_kernel<C>, dim3(per_xcd * NUM_XCD), dim3(C::NT), C::LDS_BYTES, stream, tab, total_tiles, per_xcd);
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
  int64_t tiles256 = 0, tiles_mid = 0;
  for (int i = 0; i < count; i++) {
    const hdit_gemm_problem& p = problems[i];
    if (p.m < 0 || p.n <= 0 || p.k <= 0) return HDIT_EINVAL;
    if (p.m == 0) continue;
    if (!p.a || !p.b || !p.c) return HDIT_EINVAL;
    if (p.k % BK != 0 || p.n % 8 != 0) return HDIT_EUNSUPPORTED;
    if (p.lda % 8 || p.ldb % 8 || p.ldc % 4) return HDIT_EINVAL;
    if (((uintptr_t)p.a | (uintptr_t)p.b) & 15) return HDIT_EINVAL;
    if (((uintptr_t)p.c | (uintptr_t)p.bias) & 7) return HDIT_EINVAL;
    if (p.epilogue < HDIT_EPI_BIAS || p.epilogue > HDIT_EPI_GATE_RESIDUAL) return HDIT_EINVAL;
    if (p.epilogue == HDIT_EPI_GATE_RESIDUAL) {
      if (!p.resid || !p.gate || p.rows_per_batch <= 0 || p.ldr % 4) return HDIT_EINVAL;
      if (((uintptr_t)p.resid & 7) || ((uintptr_t)p.gate & 15) || p.gate_stride % 4) return HDIT_EINVAL;
    }
    tiles256 += (int64_t)((p.m + 255) / 256) * ((p.n + 255) / 256);
    tiles_mid += (int64_t)((p.m + 255) / 256) * ((p.n + 127) / 128);
  }
  hipStream_t s = (hipStream_t)stream;
  int cfg = g_force_cfg;
  if (cfg < 0) {
    // Prefer the largest tile that still gives every CU (256 of them) work for
    // at least ~2 rounds; small launches fall back to smaller tiles.
    if (tiles256 >= 2 * 256) cfg = 0;
    else if (tiles_mid >= 256) cfg = 1;
    else cfg = 2;
  }
  switch (cfg) {
    case 0: return build_and_launch<Cfg256x256>(problems, count, s);
    case 1: return build_and_launch<Cfg256x128>(problems, count, s);
    default: return build_and_launch<Cfg128x128>(problems, count, s);
  }
}
