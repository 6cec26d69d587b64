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

// Eight values per thread with 16-byte loads and stores, for widths and strides that are multiples of 8.
typedef __attribute__((ext_vector_type(4))) uint32_t au4;

__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ y,
                                                           int inter, int64_t gu_stride) {
  const int64_t row = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= inter) return;
  const au4 g4 = *(const au4*)(gu + row * gu_stride + i);
  const au4 u4 = *(const au4*)(gu + row * gu_stride + inter + i);
  au4 o4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float g0 = __uint_as_float(g4[j] << 16), g1 = __uint_as_float(g4[j] & 0xffff0000u);
    const float u0 = __uint_as_float(u4[j] << 16), u1 = __uint_as_float(u4[j] & 0xffff0000u);
    const float s0 = rounded_as<bf16_t>(g0 / (1.f + expf(-g0))), s1 = rounded_as<bf16_t>(g1 / (1.f + expf(-g1)));
    o4[j] = (uint32_t)float_to_bf16(s0 * u0).bits | ((uint32_t)float_to_bf16(s1 * u1).bits << 16);
  }
  *(au4*)(y + row * inter + i) = o4;
}

DRYFT_API int dryft_silu_mul(const void* gu, void* y, int n_rows, int inter, int64_t gu_stride, int is_f32,
                             hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!is_f32 && inter % 8 == 0 && gu_stride % 8 == 0 && (((uintptr_t)gu | (uintptr_t)y) & 15) == 0) {
    dim3 vgrid(n_rows, (inter / 8 + 255) / 256);
    hipLaunchKernelGGL(silu_mul_vec_kernel, vgrid, dim3(256), 0, stream, (const bf16_t*)gu, (bf16_t*)y, inter, gu_stride);
    return DRYFT_LAUNCH_CHECK();
  }
  dim3 grid(n_rows, (inter + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)y, inter, gu_stride);
  else
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)y, inter,
                       gu_stride);
  return DRYFT_LAUNCH_CHECK();
}
