// SwiGLU's elementwise half: y = T( T(silu(g)) * u ) with g = gu[:, :I], u = gu[:, I:],
// silu(g) = g / (1 + exp(-g)) evaluated in float
// (reference: engine/dryft_qwen3/model.py:44-46, kernels/silu_mul.py:23-32).
#include "common.h"

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ y, int inter, int64_t gu_stride) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const float g = load_as_float(gu + row * gu_stride + i);
  const float u = load_as_float(gu + row * gu_stride + inter + i);
  const float s = rounded_as<T>(g / (1.f + expf(-g)));
  store_from_float(y + row * inter + i, s * u);
}

DRYFT_API int dryft_silu_mul(const void* gu, void* y, int n_rows, int inter, int64_t gu_stride, int is_f32,
                             hipStream_t stream) {
  if (n_rows <= 0) return 0;
  dim3 grid(n_rows, (inter + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)y, inter, gu_stride);
  else
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)y, inter,
                       gu_stride);
  return DRYFT_LAUNCH_CHECK();
}
