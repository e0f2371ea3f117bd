// Example user kernel for call_custom_kernel: out = in + 1 on a float tensor.
// Same job as the reference's example (tests/mojo/kernels/custom_kernel.mojo:12-26),
// written against the nbk_custom_fn contract of include/nbk.h.
#include <hip/hip_runtime.h>
#include "nbk.h"

__global__ void add_one_kernel(const float* in, float* out, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = in[i] + 1.0f;
}

extern "C" int my_kernel(const nbk_tensor* in, int n_in, nbk_tensor* out, int n_out, void* stream) {
  if (n_in != 1 || n_out != 1) return 1;
  if (in[0].dtype != NBK_F32 || out[0].dtype != NBK_F32) return 2;
  int64_t n = 1;
  for (int i = 0; i < in[0].rank; ++i) n *= in[0].shape[i];
  if (n == 0) return 0;
  hipLaunchKernelGGL(add_one_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, (const float*)in[0].ptr, (float*)out[0].ptr, n);
  return 0;
}
