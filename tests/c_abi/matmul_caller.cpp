// A compiled caller of the C ABI in the shape of the reference's device wrapper for `hexkl.matmul`
// (test/python/mlir/hexkl_linalg_matmul/wrapper.cpp:31-81): fp16 activations [1024, 64] x fp16 weights [64, 512] ->
// fp32 [1024, 512] through hexmi_matmul_f16f16_f32, checked element by element against a scalar fp32 loop with the
// wrapper's MAX_DIFF of 1e-2. Inputs and output cross the process boundary as raw tensor files.
//   usage: matmul_caller act.bin w.bin out.bin        exit status 0 = pass
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>
#include <vector>
#include "hexmi.h"
#include "tensor_io.h"

#define MAX_DIFF 1e-2

static bool check(const float* out, const _Float16* act, const _Float16* w, int64_t rows, int64_t inner, int64_t cols) {
  for (int64_t row = 0; row < rows; row++) {
    for (int64_t col = 0; col < cols; col++) {
      float acc = 0;
      for (int64_t k = 0; k < inner; k++) acc += (float)act[row * inner + k] * (float)w[k * cols + col];
      const float diff = out[row * cols + col] - acc;
      if (!(diff <= MAX_DIFF && diff >= -MAX_DIFF)) {
        std::printf("mismatch at [%lld, %lld]: scalar loop %f, hexmi_matmul_f16f16_f32 %f\n", (long long)row,
                    (long long)col, acc, out[row * cols + col]);
        return false;
      }
    }
  }
  return true;
}

#define HIP_OK(call)                                                                 \
  do {                                                                               \
    hipError_t e_ = (call);                                                          \
    if (e_ != hipSuccess) {                                                          \
      std::printf("%s failed: %s\n", #call, hipGetErrorString(e_));                  \
      return 2;                                                                      \
    }                                                                                \
  } while (0)

int main(int argc, char** argv) {
  if (argc != 4) {
    std::printf("usage: %s act.bin w.bin out.bin\n", argv[0]);
    return 2;
  }
  RawTensor act, w;
  if (!read_tensor(argv[1], act) || !read_tensor(argv[2], w) || act.dtype != 1 || w.dtype != 1 ||
      act.shape.size() != 2 || w.shape.size() != 2 || act.shape[1] != w.shape[0]) {
    std::printf("expected fp16 [rows, inner] and fp16 [inner, cols] tensor files\n");
    return 2;
  }
  const int64_t rows = act.shape[0], inner = act.shape[1], cols = w.shape[1];
  void *d_act = nullptr, *d_w = nullptr, *d_out = nullptr;
  HIP_OK(hipMalloc(&d_act, act.bytes.size()));
  HIP_OK(hipMalloc(&d_w, w.bytes.size()));
  HIP_OK(hipMalloc(&d_out, (size_t)(rows * cols) * sizeof(float)));
  HIP_OK(hipMemcpy(d_act, act.bytes.data(), act.bytes.size(), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_w, w.bytes.data(), w.bytes.size(), hipMemcpyHostToDevice));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  std::printf("%s\n", hexmi_version());
  const int rc = hexmi_matmul_f16f16_f32(rows, cols, inner, static_cast<float*>(d_out), d_act, d_w, stream);
  if (rc != HEXMI_OK) {
    std::printf("hexmi_matmul_f16f16_f32: %s\n", hexmi_strerror(rc));
    return 1;
  }
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<float> out((size_t)(rows * cols));
  HIP_OK(hipMemcpy(out.data(), d_out, out.size() * sizeof(float), hipMemcpyDeviceToHost));
  const bool pass = check(out.data(), reinterpret_cast<const _Float16*>(act.bytes.data()),
                          reinterpret_cast<const _Float16*>(w.bytes.data()), rows, inner, cols);
  if (!write_tensor(argv[3], 2, {rows, cols}, out.data())) return 2;
  // a bad argument comes back as a status, not as a crash
  if (hexmi_matmul_f16f16_f32(rows, cols, inner, nullptr, d_act, d_w, stream) != HEXMI_EINVAL) return 1;
  (void)hipFree(d_act);
  (void)hipFree(d_w);
  (void)hipFree(d_out);
  (void)hipStreamDestroy(stream);
  std::printf("hexkl_linalg_matmul shape [%lld x %lld] x [%lld x %lld]: %s\n", (long long)rows, (long long)inner,
              (long long)inner, (long long)cols, pass ? "Pass" : "Fail");
  return pass ? 0 : 1;
}
