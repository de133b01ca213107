// Host-side plumbing shared by the C-ABI entry points: ABI version, per-thread
// error string, launch check.
#include <string.h>

#include <atomic>

#include "hdit_common.h"

namespace {
thread_local char g_err[256] = "";
}

namespace hdit_host {
void set_error(const char* msg) {
  strncpy(g_err, msg ? msg : "", sizeof(g_err) - 1);
  g_err[sizeof(g_err) - 1] = 0;
}
int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return HDIT_OK;
  char buf[256];
  snprintf(buf, sizeof(buf), "%s: %s", what, hipGetErrorString(e));
  set_error(buf);
  return HDIT_ELAUNCH;
}
// Compute units of the current device (cached for the first device asked about; 0 if the query fails).
int num_cus() {
  static std::atomic<int> cached{0};
  int n = cached.load(std::memory_order_acquire);
  if (n == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      return 0;
    cached.store(n, std::memory_order_release);
  }
  return n;
}
}  // namespace hdit_host

extern "C" __attribute__((visibility("default"))) int hdit_abi_version(void) { return 5; }
extern "C" __attribute__((visibility("default"))) const char* hdit_last_error(void) { return g_err; }

namespace {
// Lane 0 of every workgroup stores {shader-clock counter, constant 100 MHz counter, XCD id, hardware id}.
// Every CU counts its own shader clock, so samples can only be paired within one CU.
__global__ void clock_sample_kernel(unsigned long long* out) {
  if (threadIdx.x == 0) {
    unsigned long long* o = out + 4 * blockIdx.x;
    o[0] = __builtin_amdgcn_s_memtime();
    o[1] = __builtin_amdgcn_s_memrealtime();
    o[2] = __builtin_amdgcn_s_getreg((3 << 11) | 20);   // HW_REG_XCC_ID, bits 3:0
    o[3] = __builtin_amdgcn_s_getreg((31 << 11) | 4);   // HW_REG_HW_ID
  }
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_clock_sample(void* out, int slots, void* stream) {
  if (!out || (((uintptr_t)out) & 7) || slots <= 0 || slots > 1024) return HDIT_EINVAL;
  hipLaunchKernelGGL(clock_sample_kernel, dim3(slots), dim3(64), 0, (hipStream_t)stream, (unsigned long long*)out);
  return hdit_host::check_launch("hdit_clock_sample");
}
