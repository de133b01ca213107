// Head-dim-128 instantiations of the bf16 flash-attention kernels (device code: attention_bf16_kernels.h).  A
// translation unit of its own because it is compiled without the VGPR-form MFMA option the head-dim-64 kernels
// take: with 128 output accumulator registers per lane the P.V accumulators have to live in the AGPR half.
#include "attention_bf16_kernels.h"

namespace hdit_attn {
int launch_d128(const AttnParams& P, int q_tiles, unsigned grid, bool pipelined, hipStream_t stream) {
  static std::atomic<bool> attr{false};  // setting the attributes twice from two threads is harmless
  if (!attr.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)attn_fwd_pipe_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            PipeLds<128>::TOTAL) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_fwd_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            Lds<128>::TOTAL) != hipSuccess)
      return HDIT_ELAUNCH;
    attr.store(true, std::memory_order_release);
  }
  if (pipelined)
    hipLaunchKernelGGL(attn_fwd_pipe_kernel<128>, dim3(grid), dim3(256), PipeLds<128>::TOTAL, stream, P, q_tiles);
  else
    hipLaunchKernelGGL(attn_fwd_kernel<128>, dim3(grid), dim3(256), Lds<128>::TOTAL, stream, P, q_tiles);
  return HDIT_OK;
}

int launch_multi_d128(const AttnParams* P, const int* q_tiles, const int* nblocks, int count, bool pipelined, hipStream_t stream) {
  AttnMulti M;
  const int grid = fill_multi(M, P, q_tiles, nblocks, count);
  static std::atomic<bool> attr{false};  // setting the attributes twice from two threads is harmless
  if (!attr.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)attn_fwd_pipe_multi_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            PipeLds<128>::TOTAL) != hipSuccess ||
        hipFuncSetAttribute((const void*)attn_fwd_multi_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            Lds<128>::TOTAL) != hipSuccess)
      return HDIT_ELAUNCH;
    attr.store(true, std::memory_order_release);
  }
  if (pipelined)
    hipLaunchKernelGGL(attn_fwd_pipe_multi_kernel<128>, dim3((unsigned)grid), dim3(256), PipeLds<128>::TOTAL, stream, M);
  else
    hipLaunchKernelGGL(attn_fwd_multi_kernel<128>, dim3((unsigned)grid), dim3(256), Lds<128>::TOTAL, stream, M);
  return HDIT_OK;
}
}  // namespace hdit_attn
