// Shared device helpers for the gfx950 kernels: storage types, exact
// float <-> bfloat16 conversion, wave and block reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define DRYFT_API extern "C" __attribute__((visibility("default")))
#define WAVE 64
#define PAGE_TOKENS 64

// bfloat16 kept as its 16 bits; arithmetic is always done in float.
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

// round to nearest, ties to even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  const __bf16 h = (__bf16)f;
  bf16_t r;
  r.bits = __builtin_bit_cast(uint16_t, h);
  return r;
}

template <typename T> __device__ __forceinline__ float load_as_float(const T* p);
template <> __device__ __forceinline__ float load_as_float<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_as_float<bf16_t>(const bf16_t* p) { return bf16_to_float(*p); }

template <typename T> __device__ __forceinline__ void store_from_float(T* p, float v);
template <> __device__ __forceinline__ void store_from_float<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_from_float<bf16_t>(bf16_t* p, float v) { *p = float_to_bf16(v); }

// The value a float takes when it is stored as T and read back: the rounding
// boundaries of the bfloat16 path; the identity in the float32 path.
template <typename T> __device__ __forceinline__ float rounded_as(float v);
template <> __device__ __forceinline__ float rounded_as<float>(float v) { return v; }
template <> __device__ __forceinline__ float rounded_as<bf16_t>(float v) { return bf16_to_float(float_to_bf16(v)); }

// Eight contiguous values at a 16-byte aligned address, as floats.
typedef __attribute__((ext_vector_type(4))) float vf4;
typedef __attribute__((ext_vector_type(4))) uint32_t vu4;

__device__ __forceinline__ void load8_as_float(const float* p, float (&v)[8]) {
  const vf4 a = *(const vf4*)p, b = *(const vf4*)(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
}
__device__ __forceinline__ void load8_as_float(const bf16_t* p, float (&v)[8]) {
  const vu4 a = *(const vu4*)p;
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(a[i] << 16); v[2 * i + 1] = __uint_as_float(a[i] & 0xffff0000u); }
}
__device__ __forceinline__ void store8_from_float(float* p, const float (&v)[8]) {
  *(vf4*)p = vf4{v[0], v[1], v[2], v[3]};
  *(vf4*)(p + 4) = vf4{v[4], v[5], v[6], v[7]};
}
__device__ __forceinline__ void store8_from_float(bf16_t* p, const float (&v)[8]) {
  vu4 a;
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = (uint32_t)float_to_bf16(v[2 * i]).bits | ((uint32_t)float_to_bf16(v[2 * i + 1]).bits << 16);
  *(vu4*)p = a;
}

// A vector whose dtype is only known at run time (norm weights: bfloat16, or float32 if stored so).
__device__ __forceinline__ float load_vector(const void* p, int i, int is_f32) {
  return is_f32 ? ((const float*)p)[i] : bf16_to_float(((const bf16_t*)p)[i]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of LDS; the call synchronises the block.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, waves = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < waves; ++w) t += scratch[w];
  return t;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, waves = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
  for (int w = 1; w < waves; ++w) t = fmaxf(t, scratch[w]);
  return t;
}

// Where position `pos` of the sequence in `slot` lives: index of its page, or -1.
__device__ __forceinline__ int page_of(const int* page_table, int max_pages, int slot, int pos) {
  return page_table[(int64_t)slot * max_pages + pos / PAGE_TOKENS];
}

// A page of values is [head_dim][64]: a row per feature, a column per position of the page, with the positions
// of each block of 32 in the order in which the matrix cores want them. The first attention product leaves a
// lane group g with the scores of positions 4g..4g+3 and 16+4g..16+4g+3 of a block, and the second product
// takes the values of exactly those positions from one lane; in this order they are 16 contiguous bytes.
// Position 16a + 4g + i of a block (a in 0..1, g in 0..3, i in 0..3) sits in column 8g + 4a + i of it.
__host__ __device__ __forceinline__ int value_column(int pos_in_page) {
  const int o = pos_in_page & 31;
  return (pos_in_page & 32) + 8 * ((o >> 2) & 3) + 4 * (o >> 4) + (o & 3);
}

#define DRYFT_LAUNCH_CHECK() (int)hipGetLastError()
