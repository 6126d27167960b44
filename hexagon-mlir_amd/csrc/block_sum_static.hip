// hexmi_block_sum_static: hexmi_block_sum_ws for callers that cannot allocate (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc). The fp32 partial sums of the two-pass form live in a fixed
// device array of this library instead of a workspace argument; the kernels are the ones hexmi_block_sum_ws
// launches (elementwise.hip) and take the array's address as their argument.
#include <mutex>
#include "hexmi_common.h"

namespace hexmi {
namespace {

// Room for the partial sums of 2^30 elements (one per run of kSumRun). Every GPU the library runs on holds its own
// copy, at its own address, until the process ends. In host code the name below is only a handle for
// hipGetSymbolAddress: it is never passed to a kernel or a memory call.
constexpr int64_t kStaticPartials = 1 << 18;                 // 1 MiB
static __device__ __align__(256) float scratch[kStaticPartials];

// Device address of `scratch` on the current device, looked up once per device. nullptr if the lookup fails.
float* static_scratch() {
  constexpr int kMaxDevices = 64;
  static float* ptr[kMaxDevices];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
    ptr[dev] = static_cast<float*>(p);
  }
  return ptr[dev];
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

extern "C" int64_t hexmi_block_sum_static_max_n(void) { return kStaticPartials * kSumRun; }

extern "C" int hexmi_block_sum_static(const void* x, void* out, int64_t n, int64_t block, int dtype,
                                      hexmi_stream_t stream) {
  if (n < 0 || block <= 0) return HEXMI_EINVAL;
  if (n == 0) return HEXMI_OK;
  if (!x || !out) return HEXMI_EINVAL;
  if (n > kStaticPartials * kSumRun) return HEXMI_ETOOBIG;
  begin_call();
  float* partials = nullptr;
  if (two_pass_sum(n, block)) {
    partials = static_scratch();
    if (!partials) return HEXMI_ELAUNCH;
  }
  // The first pass writes every partial sum the second pass reads, so nothing in the array has to start at zero;
  // what an earlier call left there is never read.
  return block_sum_any(x, out, n, block, dtype, partials, as_stream(stream));
}
