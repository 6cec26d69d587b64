// RMSNorm and residual-add + RMSNorm over rows of any width.
//
//   res_new = T(res + sum_p delta[p])          (the sum in float, rounded once)
//   y       = T( T(res_new * rsqrt(mean(res_new^2) + eps)) * w )
//
// Statistics are float; the normalised value is rounded to the activation
// dtype before the weight multiply, as the reference does
// (engine/dryft_qwen3/model.py:28-32, kernels/rmsnorm.py:21-39). With T = float
// every rounding is the identity. `delta` may be given as several float
// partial sums (the split-K outputs of a matrix product), which are added here
// instead of in a pass of their own.
#include "common.h"

template <typename T, typename D>
__global__ void add_rmsnorm_kernel(const T* __restrict__ res, const D* __restrict__ delta, int n_partials,
                                   int64_t partial_stride, const void* __restrict__ w, int w_f32,
                                   T* __restrict__ res_out, T* __restrict__ y, int width, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const T* r_in = res + row * width;
  T* r_out = res_out + row * width;
  T* y_row = y + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = load_as_float(r_in + i);
    if (n_partials > 0) {
      float d = 0.f;
      for (int p = 0; p < n_partials; ++p) d += load_as_float(delta + p * partial_stride + row * width + i);
      v = rounded_as<T>(v + d);
      store_from_float(r_out + i, v);
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
  const T* r_back = n_partials > 0 ? r_out : r_in;   // each thread re-reads what it wrote itself
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = load_as_float(r_back + i);
    const float n = rounded_as<T>(v * inv);
    store_from_float(y_row + i, n * load_vector(w, i, w_f32));
  }
}

// The same for rows whose width is a multiple of 8 and at most 8 * 8 * blockDim: a thread owns runs of 8
// contiguous values, reads them with 16-byte loads issued together, and keeps them in registers between the
// two passes. This is the kernel that decoding steps use: few rows, so latency rather than bandwidth counts: the
// weights are asked for together with the row, so that nothing has to come from memory after the reduction.
#define NORM_VEC_RUNS 8   // runs of 8 values a thread may hold

template <typename T, typename D, int RUNS>
__global__ __launch_bounds__(512) void add_rmsnorm_vec_kernel(const T* __restrict__ res, const D* __restrict__ delta,
                                                              int n_partials, int64_t partial_stride,
                                                              const void* __restrict__ w, int w_f32,
                                                              T* __restrict__ res_out, T* __restrict__ y, int width,
                                                              float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int64_t base = row * width;
  float v[RUNS][8], wv[RUNS][8];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    const int i = (r * blockDim.x + threadIdx.x) * 8;
    if (i < width) {
      load8_as_float(res + base + i, v[r]);
      if (w_f32) load8_as_float((const float*)w + i, wv[r]);
      else load8_as_float((const bf16_t*)w + i, wv[r]);
      if (n_partials > 0) {
        float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        int p = 0;
        for (; p + 4 <= n_partials; p += 4) {             // four loads in flight; added in the order 0, 1, ...
          float t[4][8];
#pragma unroll
          for (int u = 0; u < 4; ++u) load8_as_float(delta + (p + u) * partial_stride + base + i, t[u]);
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < 8; ++j) d[j] += t[u][j];
        }
        for (; p < n_partials; ++p) {
          float t[8];
          load8_as_float(delta + p * partial_stride + base + i, t);
#pragma unroll
          for (int j = 0; j < 8; ++j) d[j] += t[j];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[r][j] = rounded_as<T>(v[r][j] + d[j]);
        store8_from_float(res_out + base + i, v[r]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[r][j] * v[r][j];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    const int i = (r * blockDim.x + threadIdx.x) * 8;
    if (i < width) {
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = rounded_as<T>(v[r][j] * inv) * wv[r][j];
      store8_from_float(y + base + i, o);
    }
  }
}

template <typename T, typename D>
static void launch_norm_vec(const void* res, const void* delta, int n_partials, int64_t partial_stride, const void* w,
                            int w_f32, void* res_out, void* y, int n_rows, int width, float eps, hipStream_t stream) {
  const int runs_total = width / 8;
  int threads = 64;
  // few rows: latency counts, one run a thread; many rows: throughput counts, fuller threads in fewer waves
  const int per_thread = n_rows >= 256 ? 2 : 1;
  while (threads < 512 && per_thread * threads < runs_total) threads *= 2;
  const int runs = (runs_total + threads - 1) / threads;
  dim3 grid(n_rows), block(threads);
#define NV(R)                                                                                                        \
  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, D, R>), grid, block, 0, stream, (const T*)res, (const D*)delta,      \
                     n_partials, partial_stride, w, w_f32, (T*)res_out, (T*)y, width, eps)
  if (runs <= 1) NV(1);
  else if (runs <= 2) NV(2);
  else if (runs <= 4) NV(4);
  else NV(8);
#undef NV
}

// delta_kind: 0 = none (plain norm), 1 = same dtype as the activations, 2 = float partial sums
DRYFT_API int dryft_add_rmsnorm(const void* res, const void* delta, int delta_kind, int n_partials,
                                int64_t partial_stride, const void* w, int w_f32, void* res_out, void* y,
                                int n_rows, int width, float eps, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  const int threads = width >= 2048 ? 512 : 256;
  dim3 grid(n_rows), block(threads);
  if (delta_kind == 0) n_partials = 0;
  const bool aligned = (((uintptr_t)res | (uintptr_t)delta | (uintptr_t)res_out | (uintptr_t)y | (uintptr_t)w) & 15) == 0 &&
                       (partial_stride % 4) == 0;
  if (width % 8 == 0 && width <= 8 * NORM_VEC_RUNS * 512 && aligned) {
    if (is_f32)
      launch_norm_vec<float, float>(res, delta, n_partials, partial_stride, w, w_f32, res_out, y, n_rows, width, eps, stream);
    else if (delta_kind == 2)
      launch_norm_vec<bf16_t, float>(res, delta, n_partials, partial_stride, w, w_f32, res_out, y, n_rows, width, eps, stream);
    else
      launch_norm_vec<bf16_t, bf16_t>(res, delta, n_partials, partial_stride, w, w_f32, res_out, y, n_rows, width, eps, stream);
    return DRYFT_LAUNCH_CHECK();
  }
  if (is_f32) {
    hipLaunchKernelGGL((add_rmsnorm_kernel<float, float>), grid, block, 0, stream, (const float*)res,
                       (const float*)delta, n_partials, partial_stride, w, w_f32, (float*)res_out, (float*)y, width,
                       eps);
  } else if (delta_kind == 2) {
    hipLaunchKernelGGL((add_rmsnorm_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)res,
                       (const float*)delta, n_partials, partial_stride, w, w_f32, (bf16_t*)res_out, (bf16_t*)y,
                       width, eps);
  } else {
    hipLaunchKernelGGL((add_rmsnorm_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (const bf16_t*)res,
                       (const bf16_t*)delta, n_partials, partial_stride, w, w_f32, (bf16_t*)res_out, (bf16_t*)y,
                       width, eps);
  }
  return DRYFT_LAUNCH_CHECK();
}

// res_out = T(res + delta): the last residual sum of a stack that is not followed by a norm.
template <typename T>
__global__ void add_rows_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) store_from_float(out + i, load_as_float(a + i) + load_as_float(b + i));
}

DRYFT_API int dryft_add_rows(const void* a, const void* b, void* out, int64_t n, int is_f32, hipStream_t stream) {
  if (n <= 0) return 0;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (is_f32)
    hipLaunchKernelGGL(add_rows_kernel<float>, grid, block, 0, stream, (const float*)a, (const float*)b, (float*)out, n);
  else
    hipLaunchKernelGGL(add_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)a, (const bf16_t*)b,
                       (bf16_t*)out, n);
  return DRYFT_LAUNCH_CHECK();
}
