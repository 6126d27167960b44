// A compiled caller of the C ABI in the shape of the reference's device wrapper for its attention kernel
// (test/python/mlir/hexkl_attention/wrapper.cpp:151-221): fp16 Q, K, V [Z, H, N_CTX, D_HEAD] -> fp32 output through
// hexmi_flash_attn_fwd with scale 0.5, checked against a scalar pipeline of the same steps as the wrapper's check()
// (S = Q K^T with fp32 sums of fp16 products, S * 0.5, row softmax in fp32, P rounded to fp16 as the kernel's
// input.mlir:140-145 does, P V in fp32) with its MAX_DIFF of 1e-3. Tensors cross the process boundary as raw files.
//   usage: attention_caller q.bin k.bin v.bin out.bin        exit status 0 = pass
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <limits>
#include <vector>
#include "hexmi.h"
#include "tensor_io.h"

#define MAX_DIFF 1e-3

static bool check(const _Float16* Q, const _Float16* K, const _Float16* V, const float* out, int64_t ZH, int64_t n_ctx,
                  int64_t d_head, float scale) {
  std::vector<float> s((size_t)n_ctx), o((size_t)d_head);
  for (int64_t zh = 0; zh < ZH; ++zh) {
    const _Float16* q = Q + zh * n_ctx * d_head;
    const _Float16* k = K + zh * n_ctx * d_head;
    const _Float16* v = V + zh * n_ctx * d_head;
    for (int64_t i = 0; i < n_ctx; ++i) {
      float max_val = -std::numeric_limits<float>::infinity();
      for (int64_t j = 0; j < n_ctx; ++j) {
        float acc = 0.0f;
        for (int64_t d = 0; d < d_head; ++d) acc += (float)q[i * d_head + d] * (float)k[j * d_head + d];
        s[(size_t)j] = acc * scale;
        max_val = std::max(max_val, s[(size_t)j]);
      }
      float exp_sum = 0.0f;
      for (int64_t j = 0; j < n_ctx; ++j) exp_sum += std::exp(s[(size_t)j] - max_val);
      std::fill(o.begin(), o.end(), 0.0f);
      for (int64_t j = 0; j < n_ctx; ++j) {
        const _Float16 p = (_Float16)(std::exp(s[(size_t)j] - max_val) / exp_sum);
        for (int64_t d = 0; d < d_head; ++d) o[(size_t)d] += (float)p * (float)v[j * d_head + d];
      }
      for (int64_t d = 0; d < d_head; ++d) {
        const float got = out[(zh * n_ctx + i) * d_head + d];
        const float diff = got - o[(size_t)d];
        if (!(diff <= MAX_DIFF && diff >= -MAX_DIFF)) {
          std::printf("mismatch at index %lld: scalar pipeline %f, hexmi_flash_attn_fwd %f\n",
                      (long long)((zh * n_ctx + i) * d_head + d), o[(size_t)d], got);
          return false;
        }
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
  if (argc != 5) {
    std::printf("usage: %s q.bin k.bin v.bin out.bin\n", argv[0]);
    return 2;
  }
  RawTensor q, k, v;
  if (!read_tensor(argv[1], q) || !read_tensor(argv[2], k) || !read_tensor(argv[3], v) || q.dtype != 1 || k.dtype != 1 ||
      v.dtype != 1 || q.shape.size() != 4 || k.shape != q.shape || v.shape != q.shape) {
    std::printf("expected three fp16 [Z, H, N_CTX, D_HEAD] tensor files of one shape\n");
    return 2;
  }
  const int64_t Z = q.shape[0], H = q.shape[1], n_ctx = q.shape[2], d_head = q.shape[3];
  const float scale = 0.5f;                                  // the wrapper's multiplySoftmaxInputByScalar(.., 0.5)
  void *dq = nullptr, *dk = nullptr, *dv = nullptr, *dout = nullptr;
  HIP_OK(hipMalloc(&dq, q.bytes.size()));
  HIP_OK(hipMalloc(&dk, k.bytes.size()));
  HIP_OK(hipMalloc(&dv, v.bytes.size()));
  HIP_OK(hipMalloc(&dout, (size_t)q.count() * sizeof(float)));
  HIP_OK(hipMemcpy(dq, q.bytes.data(), q.bytes.size(), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dk, k.bytes.data(), k.bytes.size(), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dv, v.bytes.data(), v.bytes.size(), hipMemcpyHostToDevice));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  const int rc = hexmi_flash_attn_fwd(dq, dk, dv, dout, Z, H, n_ctx, d_head, scale, /*causal=*/0, HEXMI_F16, HEXMI_F32,
                                      stream);
  if (rc != HEXMI_OK) {
    std::printf("hexmi_flash_attn_fwd: %s\n", hexmi_strerror(rc));
    return 1;
  }
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<float> out((size_t)q.count());
  HIP_OK(hipMemcpy(out.data(), dout, out.size() * sizeof(float), hipMemcpyDeviceToHost));
  const bool pass = check(reinterpret_cast<const _Float16*>(q.bytes.data()), reinterpret_cast<const _Float16*>(k.bytes.data()),
                          reinterpret_cast<const _Float16*>(v.bytes.data()), out.data(), Z * H, n_ctx, d_head, scale);
  if (!write_tensor(argv[4], 2, q.shape, out.data())) return 2;
  (void)hipFree(dq);
  (void)hipFree(dk);
  (void)hipFree(dv);
  (void)hipFree(dout);
  (void)hipStreamDestroy(stream);
  std::printf("hexkl_attention shape [%lld, %lld, %lld, %lld]: %s\n", (long long)Z, (long long)H, (long long)n_ctx,
              (long long)d_head, pass ? "Pass" : "Fail");
  return pass ? 0 : 1;
}
