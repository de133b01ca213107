// Head and tail of a denoise step around the block stack: patchify / unpatchify of the latent, the
// sinusoidal timestep projection, SiLU, and classifier-free guidance fused with the flow-match Euler
// update.  All of them touch about a megabyte per step; one thread per element (or per 8) is plenty.
#include "hdit_common.h"

namespace {

using hdit::pack8;
using hdit::unpack8;

inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// out[b, hy*w + wx, (c*p + py)*p + px] = latent[b, c, hy*p + py, wx*p + px]: the im2col of a p x p, stride p
// convolution, columns in the order of the flattened conv weight [out, c, py, px]
__global__ void __launch_bounds__(256) patchify_kernel(const __bf16* __restrict__ latent, __bf16* __restrict__ out,
                                                       int64_t total, int C, int H, int W, int p) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int K = C * p * p, w = W / p, h = H / p;
  const int col = (int)(i % K);
  const int64_t tok = i / K;
  const int px = col % p, py = (col / p) % p, c = col / (p * p);
  const int wx = (int)(tok % w), hy = (int)((tok / w) % h);
  const int64_t b = tok / ((int64_t)w * h);
  out[i] = latent[((b * C + c) * H + hy * p + py) * W + wx * p + px];
}

// out[b, c, hy*p + py, wx*p + px] = x[b, hy*w + wx, (py*p + px)*C + c]   (channel innermost), or
//                                 = x[b, hy*w + wx, (c*p + py)*p + px]   (CHANNEL_MAJOR)
template <bool CHANNEL_MAJOR>
__global__ void __launch_bounds__(256) unpatchify_kernel(const __bf16* __restrict__ x, __bf16* __restrict__ out,
                                                         int64_t total, int C, int H, int W, int p) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int w = W / p, h = H / p;
  const int X = (int)(i % W), Y = (int)((i / W) % H), c = (int)((i / ((int64_t)W * H)) % C);
  const int64_t b = i / ((int64_t)W * H * C);
  const int wx = X / p, px = X % p, hy = Y / p, py = Y % p;
  const int col = CHANNEL_MAJOR ? (c * p + py) * p + px : (py * p + px) * C + c;
  out[i] = x[((b * h + hy) * w + wx) * (int64_t)(p * p * C) + col];
}

// out[b, :half] = cos(t[b] * f_i), out[b, half:] = sin(t[b] * f_i), f_i = exp(-ln(max_period) * i / half)
__global__ void __launch_bounds__(256) timestep_embedding_kernel(const float* __restrict__ t, __bf16* __restrict__ out,
                                                                 int batch, int dim, float max_period) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int half = dim / 2;
  if (i >= batch * half) return;
  const int b = i / half, k = i % half;
  const float freq = expf(-logf(max_period) * (float)k / (float)half);
  const float arg = t[b] * freq;
  out[(int64_t)b * dim + k] = (__bf16)cosf(arg);
  out[(int64_t)b * dim + half + k] = (__bf16)sinf(arg);
}

__global__ void __launch_bounds__(256) silu_kernel(const __bf16* __restrict__ x, __bf16* __restrict__ y, int64_t chunks) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= chunks) return;
  float f[8];
  unpack8(*(const i32x4*)(x + i * 8), f);
#pragma unroll
  for (int e = 0; e < 8; e++) f[e] = f[e] / (1.0f + expf(-f[e]));
  *(i32x4*)(y + i * 8) = pack8(f);
}

struct RopeAxes {
  int n;
  int dim[HDIT_ROPE_MAX_AXES];
};

// cos/sin[row, off_a + 2i] = cos/sin[row, off_a + 2i + 1] = cos/sin(pos[row, a] * theta^(-2i / dim_a)), in float64
// like the table it replaces, stored as f32; one thread per rotation pair
__global__ void __launch_bounds__(256) rope_table_kernel(const float* __restrict__ pos, float* __restrict__ cos_out,
                                                         float* __restrict__ sin_out, int rows, RopeAxes ax, int width,
                                                         double theta) {
  const int pairs = width / 2;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)rows * pairs) return;
  const int row = (int)(i / pairs);
  int pr = (int)(i % pairs), a = 0;
  while (pr >= ax.dim[a] / 2) pr -= ax.dim[a++] / 2;  // ax.dim sums to width, so a stays below ax.n
  const double freq = 1.0 / pow(theta, (double)(2 * pr) / (double)ax.dim[a]);
  const double ang = (double)pos[(int64_t)row * ax.n + a] * freq;
  const float c = (float)cos(ang), sn = (float)sin(ang);
  const int64_t o = (int64_t)row * width + (i % pairs) * 2;
  *(float2*)(cos_out + o) = make_float2(c, c);
  *(float2*)(sin_out + o) = make_float2(sn, sn);
}

__device__ __forceinline__ float round_bf16(float v) { return (float)(__bf16)v; }

// Classifier-free guidance and the flow-match Euler update, in the rounding sequence of the bf16 tensor
// expressions they replace:
//   noise = uncond + s * (cond - uncond)                      (three bf16 tensor operations)
//   x32 = float(sample); denoised = x32 - bf16(noise * sigma); derivative = (x32 - denoised) / sigma
//   prev = bf16(x32 + derivative * (sigma_next - sigma))       (fp32 arithmetic, no fused multiply-add)
__global__ void __launch_bounds__(256) cfg_euler_kernel(const __bf16* __restrict__ uncond, const __bf16* __restrict__ cond,
                                                        const __bf16* __restrict__ sample, __bf16* __restrict__ out,
                                                        int64_t total, float guidance, float sigma, float sigma_next) {
#pragma clang fp contract(off)
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const float u = (float)uncond[i], c = (float)cond[i];
  const float diff = round_bf16(c - u);
  const float scaled = round_bf16(guidance * diff);
  const float noise = round_bf16(u + scaled);
  const float x = (float)sample[i];
  const float denoised = x - round_bf16(noise * sigma);
  const float derivative = (x - denoised) / sigma;
  const float dt = sigma_next - sigma;
  out[i] = (__bf16)(x + derivative * dt);
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_patchify(const void* latent, void* out, int batch, int channels, int height, int width,
                                             int patch, void* stream) {
  if (batch < 0 || channels <= 0 || height <= 0 || width <= 0 || patch <= 0) return HDIT_EINVAL;
  if (height % patch || width % patch) return HDIT_EINVAL;
  const int64_t total = (int64_t)batch * channels * height * width;
  if (total == 0) return HDIT_OK;
  if (!latent || !out) return HDIT_EINVAL;
  hipLaunchKernelGGL(patchify_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __bf16*)latent, (__bf16*)out, total, channels, height, width, patch);
  return hdit_host::check_launch("hdit_patchify");
}

extern "C" __attribute__((visibility("default"))) int hdit_unpatchify(const void* x, void* out, int batch, int channels, int height, int width,
                                               int patch, int channel_major, void* stream) {
  if (batch < 0 || channels <= 0 || height <= 0 || width <= 0 || patch <= 0) return HDIT_EINVAL;
  if (height % patch || width % patch) return HDIT_EINVAL;
  const int64_t total = (int64_t)batch * channels * height * width;
  if (total == 0) return HDIT_OK;
  if (!x || !out) return HDIT_EINVAL;
  if (channel_major)
    hipLaunchKernelGGL(unpatchify_kernel<true>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const __bf16*)x, (__bf16*)out, total, channels, height, width, patch);
  else
    hipLaunchKernelGGL(unpatchify_kernel<false>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const __bf16*)x, (__bf16*)out, total, channels, height, width, patch);
  return hdit_host::check_launch("hdit_unpatchify");
}

extern "C" __attribute__((visibility("default"))) int hdit_timestep_embedding(const float* timesteps, void* out, int batch, int dim,
                                                       float max_period, void* stream) {
  if (batch < 0 || dim <= 0 || dim % 2 || max_period <= 1.0f) return HDIT_EINVAL;
  if (batch == 0) return HDIT_OK;
  if (!timesteps || !out) return HDIT_EINVAL;
  const int n = batch * (dim / 2);
  hipLaunchKernelGGL(timestep_embedding_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     timesteps, (__bf16*)out, batch, dim, max_period);
  return hdit_host::check_launch("hdit_timestep_embedding");
}

extern "C" __attribute__((visibility("default"))) int hdit_silu(const void* x, void* y, int64_t count, void* stream) {
  if (count < 0 || count % 8) return HDIT_EINVAL;
  if (count == 0) return HDIT_OK;
  if (!x || !y || !aligned16(x) || !aligned16(y)) return HDIT_EINVAL;
  const int64_t chunks = count / 8;
  hipLaunchKernelGGL(silu_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __bf16*)x, (__bf16*)y, chunks);
  return hdit_host::check_launch("hdit_silu");
}

extern "C" __attribute__((visibility("default"))) int hdit_cfg_euler_step(const void* noise_uncond, const void* noise_cond, const void* sample,
                                                   void* out, int64_t count, float guidance, float sigma,
                                                   float sigma_next, void* stream) {
  if (count < 0 || !(sigma > 0.0f)) return HDIT_EINVAL;
  if (count == 0) return HDIT_OK;
  if (!noise_uncond || !noise_cond || !sample || !out) return HDIT_EINVAL;
  hipLaunchKernelGGL(cfg_euler_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __bf16*)noise_uncond, (const __bf16*)noise_cond, (const __bf16*)sample, (__bf16*)out, count,
                     guidance, sigma, sigma_next);
  return hdit_host::check_launch("hdit_cfg_euler_step");
}

extern "C" __attribute__((visibility("default"))) int hdit_rope_table(const float* positions, int rows, const int* axes_dim, int n_axes,
                                               double theta, float* cos_out, float* sin_out, void* stream) {
  if (rows < 0 || !axes_dim || n_axes <= 0 || n_axes > HDIT_ROPE_MAX_AXES || !(theta > 1.0)) return HDIT_EINVAL;
  RopeAxes ax{};
  ax.n = n_axes;
  int width = 0;
  for (int a = 0; a < n_axes; a++) {
    if (axes_dim[a] <= 0 || axes_dim[a] % 2) return HDIT_EINVAL;
    ax.dim[a] = axes_dim[a];
    width += axes_dim[a];
  }
  if (rows == 0) return HDIT_OK;
  if (!positions || !cos_out || !sin_out || (((uintptr_t)cos_out | (uintptr_t)sin_out) & 7)) return HDIT_EINVAL;
  const int64_t n = (int64_t)rows * (width / 2);
  hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, positions,
                     cos_out, sin_out, rows, ax, width, theta);
  return hdit_host::check_launch("hdit_rope_table");
}
