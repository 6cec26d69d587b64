// Matrix products y[M,N] = x[M,K] . W[N,K]^T (weights in their checkpoint layout [out, in], no bias;
// reference: F.linear at engine/dryft_qwen3/model.py:153, 179-180, 237, 258-261).
//
//  * gemm_tiled:  any M, N, K, float accumulation by plain fused multiply-adds. With float inputs it
//    is the true 32-bit product (no reduced-precision matrix mode); with bfloat16 inputs it takes the
//    sizes the matrix-core kernel refuses.
//  * gemm_stream (M <= 16) and gemm_wide (M <= 64): bfloat16, few rows (decoding, output head): every
//    weight is read once and multiplied on the matrix cores; K may be split across workgroups into
//    float partial sums that the consumer adds in a fixed order. gemm_panel (M <= 64) is the fused gate/up
//    product, gemm_mid (M <= 256) the projections back to the hidden width for short prompts.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// ------------------------------------------------------------------------------------------ tiled
#define TILE 64
#define TILE_K 16

template <typename T, typename O>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const T* __restrict__ x, int64_t x_stride,
                                                         const T* __restrict__ w, O* __restrict__ y, int M, int N,
                                                         int K) {
  __shared__ float xs[TILE_K][TILE + 1];
  __shared__ float ws[TILE_K][TILE + 1];
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * TILE, n0 = blockIdx.x * TILE;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  const int lr = tid / 4, lk = (tid % 4) * 4;   // this thread stages row lr, k lk..lk+3 of both tiles
  for (int k0 = 0; k0 < K; k0 += TILE_K) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      const int m = m0 + lr, n = n0 + lr;
      xs[lk + i][lr] = (m < M && k < K) ? load_as_float(x + (int64_t)m * x_stride + k) : 0.f;
      ws[lk + i][lr] = (n < N && k < K) ? load_as_float(w + (int64_t)n * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) store_from_float(y + (int64_t)m * N + n, acc[i][j]);
    }
  }
}

// out_f32: the result is stored as float whatever the inputs are (logits)
DRYFT_API int dryft_gemm_tiled(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K,
                               int is_f32, int out_f32, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return -1;
  dim3 grid((N + TILE - 1) / TILE, (M + TILE - 1) / TILE), block(256);
  if (grid.y > 65535) return -1;
  if (is_f32)
    hipLaunchKernelGGL((gemm_tiled_kernel<float, float>), grid, block, 0, stream, (const float*)x, x_stride,
                       (const float*)w, (float*)y, M, N, K);
  else if (out_f32)
    hipLaunchKernelGGL((gemm_tiled_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)x, x_stride,
                       (const bf16_t*)w, (float*)y, M, N, K);
  else
    hipLaunchKernelGGL((gemm_tiled_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (const bf16_t*)x, x_stride,
                       (const bf16_t*)w, (bf16_t*)y, M, N, K);
  return DRYFT_LAUNCH_CHECK();
}

// ----------------------------------------------------------------------------------------- few rows
__device__ __forceinline__ bf16x8 zero8g() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// gemm_stream: at most 16 activation rows. A wave computes C^T[n, m] = W[n, :] . x[m, :] for 16 weight rows
// with v_mfma_f32_16x16x32_bf16 over its share of K; the four waves of a workgroup split K, and further
// workgroups may split it again into float partial sums. Every weight is read once, and the memory traffic
// is shaped for the cache in front of the matrix cores: loading the operands straight into the matrix-core
// layout touches 16 rows, 64 bytes of each (half a cache line), per instruction, for the weights and again for
// the activations, and the rate at which the vector cache looks lines up, not HBM, then bounds the kernel as
// soon as there are several activation rows. So a wave reads whole lines (GB * 128 contiguous bytes of a row
// per group of GB blocks of K, four or eight rows per instruction), parks them in its own piece of LDS and
// takes the matrix-core operands from there. With SWIGLU the two weight tiles of a wave are rows [n0, n0+16)
// of the first half (gate) and of the second half (up) of W, and the epilogue stores T(T(silu(gate)) * up)
// for the N = rows/2 outputs (reference: kernels/silu_mul.py:29-32). The next group's loads are in flight
// while the current one is multiplied. Rows beyond N or M are read from a clamped, valid row and never
// stored; values beyond the wave's share of K are zeros.
template <int GB, int NW>
struct StreamShape {
  static constexpr int ROW_BYTES = GB * 128;            // of one row in one group
  static constexpr int STRIDE = ROW_BYTES + 16;         // in LDS: rows 16 bytes apart in the banks
  static constexpr int ROWS_PER_LOAD = 1024 / ROW_BYTES;
  static constexpr int LANES_PER_ROW = WAVE / ROWS_PER_LOAD;
  static constexpr int LOADS = 16 / ROWS_PER_LOAD;      // instructions per tile of 16 rows
  static constexpr int TILE_BYTES = 16 * STRIDE;
  static constexpr int WAVE_BYTES = (NW + 1) * TILE_BYTES;
  static constexpr int LDS_BYTES = 4 * WAVE_BYTES;
};

template <int I>
struct StaticIndex {
  static constexpr int value = I;
};
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(StaticIndex<I>{});
    static_for<N, I + 1>(f);
  }
}

template <int GB, int NW, int DEPTH, bool SWIGLU, typename O>
__global__ __launch_bounds__(256) void gemm_stream_kernel(const bf16_t* __restrict__ x, int64_t x_stride,
                                                          const bf16_t* __restrict__ w, O* __restrict__ y,
                                                          float* __restrict__ partials, int M, int N, int K) {
  typedef StreamShape<GB, NW> S;
  extern __shared__ __align__(16) unsigned char stream_lds[];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int lr = lane / S::LANES_PER_ROW, lp = lane % S::LANES_PER_ROW;   // row within a load, 16-byte piece of it
  const int n0 = blockIdx.x * 16;
  const int splits = gridDim.y, units = splits * 4, unit = blockIdx.y * 4 + wave;
  const int kblocks = (K + 63) / 64, per = (kblocks + units - 1) / units;
  const int kb0 = min(kblocks, unit * per), kb1 = min(kblocks, kb0 + per);
  const int k_begin = kb0 * 64, k_end = min(kb1 * 64, K);
  unsigned char* mine = stream_lds + wave * S::WAVE_BYTES;
  f32x4 acc[NW];
#pragma unroll
  for (int t = 0; t < NW; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  // where each load instruction of this lane starts (element offsets at k = 0)
  int64_t w_at[NW][S::LOADS], x_at[S::LOADS];
#pragma unroll
  for (int i = 0; i < S::LOADS; ++i) {
    const int r = S::ROWS_PER_LOAD * i + lr;
#pragma unroll
    for (int t = 0; t < NW; ++t) w_at[t][i] = (int64_t)((SWIGLU ? t * N : 0) + min(n0 + r, N - 1)) * K + 8 * lp;
    x_at[i] = (int64_t)min(r, M - 1) * x_stride + 8 * lp;
  }
  const int x_loads = (M + S::ROWS_PER_LOAD - 1) / S::ROWS_PER_LOAD;
  // DEPTH groups are in flight: slot d of the registers holds group d, d + DEPTH, ... of the wave's share
  bf16x8 wa[DEPTH][NW][S::LOADS], xa[DEPTH][S::LOADS];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
#pragma unroll
    for (int i = 0; i < S::LOADS; ++i) xa[d][i] = zero8g();
  auto fetch = [&](auto slot, int k0) {
    constexpr int d = decltype(slot)::value;
    if (k0 + GB * 64 <= k_end) {
#pragma unroll
      for (int i = 0; i < S::LOADS; ++i) {
#pragma unroll
        for (int t = 0; t < NW; ++t) wa[d][t][i] = *(const bf16x8*)(w + w_at[t][i] + k0);
        if (i < x_loads) xa[d][i] = *(const bf16x8*)(x + x_at[i] + k0);
      }
    } else {                                            // the wave's last, partial group
      const bool in = k0 + 8 * lp < k_end;
#pragma unroll
      for (int i = 0; i < S::LOADS; ++i) {
#pragma unroll
        for (int t = 0; t < NW; ++t) wa[d][t][i] = in ? *(const bf16x8*)(w + w_at[t][i] + k0) : zero8g();
        if (i < x_loads) xa[d][i] = in ? *(const bf16x8*)(x + x_at[i] + k0) : zero8g();
      }
    }
  };
  auto multiply = [&](auto slot, int k0) {
    constexpr int d = decltype(slot)::value;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");   // the previous group's operand reads are done
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < S::LOADS; ++i) {
      const int at = (S::ROWS_PER_LOAD * i + lr) * S::STRIDE + 16 * lp;
#pragma unroll
      for (int t = 0; t < NW; ++t) *(bf16x8*)(mine + t * S::TILE_BYTES + at) = wa[d][t][i];
      *(bf16x8*)(mine + NW * S::TILE_BYTES + at) = xa[d][i];
    }
    if (k0 + DEPTH * GB * 64 < k_end) fetch(slot, k0 + DEPTH * GB * 64);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int u = 0; u < 2 * GB; ++u) {                   // 32 values of K at a time
      const int at = c * S::STRIDE + 64 * u + 16 * g;
      const bf16x8 b = *(const bf16x8*)(mine + NW * S::TILE_BYTES + at);
#pragma unroll
      for (int t = 0; t < NW; ++t) {
        const bf16x8 a = *(const bf16x8*)(mine + t * S::TILE_BYTES + at);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
      }
    }
  };
  static_for<DEPTH>([&](auto slot) {
    const int k0 = k_begin + decltype(slot)::value * GB * 64;
    if (k0 < k_end) fetch(slot, k0);
  });
  for (int k0 = k_begin; k0 < k_end; k0 += DEPTH * GB * 64)
    static_for<DEPTH>([&](auto slot) {
      const int kk = k0 + decltype(slot)::value * GB * 64;
      if (kk < k_end) multiply(slot, kk);
    });
  __syncthreads();                                        // every wave is done with its staging area
  f32x4 (*red)[NW][WAVE] = (f32x4 (*)[NW][WAVE])stream_lds;
#pragma unroll
  for (int t = 0; t < NW; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();
  if (wave != 0) return;
  const int m = c;
  if (SWIGLU) {
    // gate and up of the same (n, m) sit in the same lane
    f32x4 gate = red[0][0][lane], up = red[0][NW - 1][lane];
#pragma unroll
    for (int wv = 1; wv < 4; ++wv) {
      gate += red[wv][0][lane];
      up += red[wv][NW - 1][lane];
    }
    if (m >= M) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g + i;
      if (n >= N) continue;
      const float gv = rounded_as<bf16_t>(gate[i]), uv = rounded_as<bf16_t>(up[i]);
      const float sv = rounded_as<bf16_t>(gv / (1.f + expf(-gv)));
      store_from_float(y + (int64_t)m * N + n, sv * uv);
    }
    return;
  }
  f32x4 s = red[0][0][lane];                              // waves in the order 0..3
  s += red[1][0][lane];
  s += red[2][0][lane];
  s += red[3][0][lane];
  if (m >= M) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = n0 + 4 * g + i;
    if (n >= N) continue;
    if (splits > 1)
      partials[((int64_t)blockIdx.y * M + m) * N + n] = s[i];
    else
      store_from_float(y + (int64_t)m * N + n, s[i]);
  }
}

template <int GB, int NW, int DEPTH, bool SWIGLU, typename O>
static int launch_stream(const void* x, int64_t x_stride, const void* w, void* y, float* partials, int M, int N, int K,
                         int splits, hipStream_t stream) {
  typedef StreamShape<GB, NW> S;
  static bool raised = false;                             // more dynamic LDS than the default limit allows
  auto kernel = gemm_stream_kernel<GB, NW, DEPTH, SWIGLU, O>;
  if (!raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, S::LDS_BYTES) != hipSuccess)
      return -2;
    raised = true;
  }
  dim3 grid((N + 15) / 16, splits), block(256);
  hipLaunchKernelGGL(kernel, grid, block, S::LDS_BYTES, stream, (const bf16_t*)x, x_stride, (const bf16_t*)w, (O*)y,
                     partials, M, N, K);
  return DRYFT_LAUNCH_CHECK();
}

// M <= 16. splits > 1: float partial sums go to partials[splits, M, N] and y is not written.
DRYFT_API int dryft_gemm_stream_bf16(const void* x, int64_t x_stride, const void* w, void* y, float* partials, int M,
                                     int N, int K, int group_blocks, int depth, int splits, int out_f32, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K <= 0 || K % 8 || x_stride % 8 || splits < 1 || splits > 64) return -1;
  if (splits > 1 && partials == nullptr) return -1;
#define ST(GBV, DV)                                                                                               \
  return out_f32 ? launch_stream<GBV, 1, DV, false, float>(x, x_stride, w, y, partials, M, N, K, splits, stream)  \
                 : launch_stream<GBV, 1, DV, false, bf16_t>(x, x_stride, w, y, partials, M, N, K, splits, stream)
  switch (depth * 10 + group_blocks) {
    case 11: ST(1, 1);
    case 12: ST(2, 1);
    case 21: ST(1, 2);
    case 22: ST(2, 2);
    default: return -1;
  }
#undef ST
}

// M <= 16. y[M, N] = T(T(silu(x . Wg^T)) * (x . Wu^T)) with W = [Wg; Wu] of 2N rows
DRYFT_API int dryft_gemm_stream_swiglu_bf16(const void* x, int64_t x_stride, const void* w, void* y, int M, int N,
                                            int K, int group_blocks, int depth, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K <= 0 || K % 8 || x_stride % 8) return -1;
#define SW(GBV, DV) return launch_stream<GBV, 2, DV, true, bf16_t>(x, x_stride, w, y, nullptr, M, N, K, 1, stream)
  switch (depth * 10 + group_blocks) {
    case 11: SW(1, 1);
    case 12: SW(2, 1);
    case 21: SW(1, 2);
    case 22: SW(2, 2);
    default: return -1;
  }
#undef SW
}

// ------------------------------------------------------------------------------------------- wide
// The same product for 17 to 64 activation rows (decoding at larger batch). Here the activations weigh as much
// as the weights, so a workgroup shares them: its four waves stage the rows of x for one group of K in LDS once
// (double-buffered, one barrier per group), each wave streams 16 weight rows of its own through its own piece of
// LDS (whole cache lines per load, as in gemm_stream) and multiplies them with all MT tiles of 16 rows of x.
// K is split across workgroups only (float partial sums for the consumer to add), never across the waves of one.
// With SWIGLU a workgroup owns 32 outputs: waves 0 and 1 hold their gate rows, waves 2 and 3 their up rows, and
// the two halves meet through LDS for T(T(silu(gate)) * up) (reference: kernels/silu_mul.py:29-32).
template <int MT, int GB, int DEPTH, bool SWIGLU, typename O>
__global__ __launch_bounds__(256) void gemm_wide_kernel(const bf16_t* __restrict__ x, int64_t x_stride,
                                                        const bf16_t* __restrict__ w, O* __restrict__ y,
                                                        float* __restrict__ partials, int M, int N, int K) {
  typedef StreamShape<GB, 1> S;
  constexpr int GROUP = GB * 64;                           // values of K in one group
  extern __shared__ __align__(16) unsigned char wide_lds[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  unsigned char* mine = wide_lds + wave * S::TILE_BYTES;                          // this wave's weight tile
  unsigned char* shared = wide_lds + 4 * S::TILE_BYTES;                           // [2][4 tiles] of x
  const int lr = lane / S::LANES_PER_ROW, lp = lane % S::LANES_PER_ROW;
  const int cols = SWIGLU ? 32 : 64;                       // outputs a workgroup owns
  const int n0 = blockIdx.x * cols + 16 * (SWIGLU ? wave % 2 : wave);             // first output of this wave
  const int w_row0 = (SWIGLU && wave >= 2 ? N : 0) + n0;   // its first weight row (W = [Wg; Wu] with SWIGLU)
  const int w_last = (SWIGLU && wave >= 2 ? 2 * N : N) - 1;
  const int splits = gridDim.y;
  const int kblocks = (K + 63) / 64, per = (kblocks + splits - 1) / splits;
  const int kb0 = min(kblocks, (int)blockIdx.y * per), kb1 = min(kblocks, kb0 + per);
  const int k_begin = kb0 * 64, k_end = min(kb1 * 64, K);
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16_t* w_row[S::LOADS];
  const bf16_t* x_row[S::LOADS];
#pragma unroll
  for (int i = 0; i < S::LOADS; ++i) {
    const int r = S::ROWS_PER_LOAD * i + lr;
    w_row[i] = w + (int64_t)min(w_row0 + r, w_last) * K;
    x_row[i] = x + (int64_t)min(16 * wave + r, M - 1) * x_stride;   // a wave beyond the last row stages copies of it
  }
  // DEPTH groups are in flight: slot d of the registers holds group d, d + DEPTH, ... Nothing in the walk is
  // conditional, so that the compiler counts the loads in flight exactly and waits for one slot's only: a
  // group beyond the workgroup's share of K is read from the share's last piece (a line that is in the cache
  // already) and its activations are replaced by zeros.
  bf16x8 wa[DEPTH][S::LOADS], xa[DEPTH][S::LOADS];
  auto fetch = [&](auto slot, int k0) {
    constexpr int d = decltype(slot)::value;
    const int kk = min(k0 + 8 * lp, k_end - 8);
#pragma unroll
    for (int i = 0; i < S::LOADS; ++i) {
      wa[d][i] = *(const bf16x8*)(w_row[i] + kk);
      xa[d][i] = *(const bf16x8*)(x_row[i] + kk);
    }
  };
  int buf = 0;
  auto step = [&](auto slot, int k0) {
    constexpr int d = decltype(slot)::value;
    const bool in = k0 + 8 * lp < k_end;
    unsigned char* xs = shared + buf * 4 * S::TILE_BYTES;
    buf ^= 1;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");   // this wave's reads of its weight tile come first
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < S::LOADS; ++i) {
      const int at = (S::ROWS_PER_LOAD * i + lr) * S::STRIDE + 16 * lp;
      *(bf16x8*)(mine + at) = wa[d][i];
      *(bf16x8*)(xs + wave * S::TILE_BYTES + at) = in ? xa[d][i] : zero8g();
    }
    fetch(slot, k0 + DEPTH * GROUP);
    __syncthreads();                                         // all tiles of x of this group are in place
    // every operand of the group is asked for before the first product: the reads overlap one another
    // instead of each product waiting a whole LDS round trip for its own
    bf16x8 a[2 * GB], b[2 * GB][MT];
#pragma unroll
    for (int u = 0; u < 2 * GB; ++u) {
      const int at = c * S::STRIDE + 64 * u + 16 * g;
      a[u] = *(const bf16x8*)(mine + at);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = *(const bf16x8*)(xs + mt * S::TILE_BYTES + at);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < 2 * GB; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][mt], acc[mt], 0, 0, 0);
  };
  if (k_begin < k_end) {
    static_for<DEPTH>([&](auto slot) {
      fetch(slot, k_begin + decltype(slot)::value * GROUP);
      __builtin_amdgcn_sched_barrier(0);                   // slot after slot, the order in which they are waited for
    });
    for (int k0 = k_begin; k0 < k_end; k0 += DEPTH * GROUP)
      static_for<DEPTH>([&](auto slot) { step(slot, k0 + decltype(slot)::value * GROUP); });
  }
  // acc[mt][i] is output n0 + 4g + i of activation row 16 mt + c
  if (SWIGLU) {
    __syncthreads();                                         // the buffers of x are free: up passes through them
    f32x4 (*pass)[MT][WAVE] = (f32x4 (*)[MT][WAVE])shared;
    if (wave >= 2) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) pass[wave - 2][mt][lane] = acc[mt];
    }
    __syncthreads();
    if (wave >= 2) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const f32x4 up = pass[wave][mt][lane];
      const int m = 16 * mt + c;
      if (m >= M) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * g + i;
        if (n >= N) continue;
        const float gv = rounded_as<bf16_t>(acc[mt][i]), uv = rounded_as<bf16_t>(up[i]);
        const float sv = rounded_as<bf16_t>(gv / (1.f + expf(-gv)));
        store_from_float(y + (int64_t)m * N + n, sv * uv);
      }
    }
    return;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + c;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g + i;
      if (n >= N) continue;
      if (splits > 1)
        partials[((int64_t)blockIdx.y * M + m) * N + n] = acc[mt][i];
      else
        store_from_float(y + (int64_t)m * N + n, acc[mt][i]);
    }
  }
}

template <int MT, int GB, int DEPTH, bool SWIGLU, typename O>
static int launch_wide(const void* x, int64_t x_stride, const void* w, void* y, float* partials, int M, int N, int K,
                       int splits, hipStream_t stream) {
  typedef StreamShape<GB, 1> S;
  constexpr int lds = 12 * S::TILE_BYTES;                  // four weight tiles, two buffers of four tiles of x
  static bool raised = false;                              // more dynamic LDS than the default limit allows
  auto kernel = gemm_wide_kernel<MT, GB, DEPTH, SWIGLU, O>;
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -2;
    raised = true;
  }
  const int cols = SWIGLU ? 32 : 64;
  dim3 grid((N + cols - 1) / cols, splits), block(256);
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, (const bf16_t*)x, x_stride, (const bf16_t*)w, (O*)y, partials, M,
                     N, K);
  return DRYFT_LAUNCH_CHECK();
}

// M <= 64. splits > 1: float partial sums go to partials[splits, M, N] and y is not written.
template <int MT, int GB>
static int wide_depth(const void* x, int64_t x_stride, const void* w, void* y, float* partials, int M, int N, int K,
                      int depth, int splits, int out_f32, hipStream_t stream) {
#define WD(DV)                                                                                                    \
  return out_f32 ? launch_wide<MT, GB, DV, false, float>(x, x_stride, w, y, partials, M, N, K, splits, stream)    \
                 : launch_wide<MT, GB, DV, false, bf16_t>(x, x_stride, w, y, partials, M, N, K, splits, stream)
  switch (depth) {
    case 1: WD(1);
    case 2: WD(2);
    case 3: WD(3);
    default: return -1;
  }
#undef WD
}

template <int MT, int GB>
static int wide_swiglu_depth(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K, int depth,
                             hipStream_t stream) {
  switch (depth) {
    case 1: return launch_wide<MT, GB, 1, true, bf16_t>(x, x_stride, w, y, nullptr, M, N, K, 1, stream);
    case 2: return launch_wide<MT, GB, 2, true, bf16_t>(x, x_stride, w, y, nullptr, M, N, K, 1, stream);
    case 3: return launch_wide<MT, GB, 3, true, bf16_t>(x, x_stride, w, y, nullptr, M, N, K, 1, stream);
    default: return -1;
  }
}

DRYFT_API int dryft_gemm_wide_bf16(const void* x, int64_t x_stride, const void* w, void* y, float* partials, int M,
                                   int N, int K, int group_blocks, int depth, int splits, int out_f32,
                                   hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 || x_stride % 8 || splits < 1 || splits > 64) return -1;
  if (splits > 1 && partials == nullptr) return -1;
#define WD(MTV, GBV) return wide_depth<MTV, GBV>(x, x_stride, w, y, partials, M, N, K, depth, splits, out_f32, stream)
  switch (((M + 15) / 16) * 10 + group_blocks) {
    case 11: WD(1, 1);
    case 12: WD(1, 2);
    case 21: WD(2, 1);
    case 22: WD(2, 2);
    case 31: WD(3, 1);
    case 32: WD(3, 2);
    case 41: WD(4, 1);
    case 42: WD(4, 2);
    default: return -1;
  }
#undef WD
}

// M <= 64. y[M, N] = T(T(silu(x . Wg^T)) * (x . Wu^T)) with W = [Wg; Wu] of 2N rows
DRYFT_API int dryft_gemm_wide_swiglu_bf16(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K,
                                          int group_blocks, int depth, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 || x_stride % 8) return -1;
#define WS(MTV, GBV) return wide_swiglu_depth<MTV, GBV>(x, x_stride, w, y, M, N, K, depth, stream)
  switch (((M + 15) / 16) * 10 + group_blocks) {
    case 11: WS(1, 1);
    case 12: WS(1, 2);
    case 21: WS(2, 1);
    case 22: WS(2, 2);
    case 31: WS(3, 1);
    case 32: WS(3, 2);
    case 41: WS(4, 1);
    case 42: WS(4, 2);
    default: return -1;
  }
#undef WS
}

// ------------------------------------------------------------------------------------------- panel
// The fused gate/up product with its activation for steps of up to 64 rows, with the operands going from memory straight
// into LDS (global_load_lds_dwordx4: 16 bytes a lane, no registers in between and nothing for the waves to store),
// two groups of K ahead of the one that is multiplied. A workgroup of four to eight waves owns 8 outputs a wave
// (each wave the gate rows and the up rows of its own) and all MT tiles of 16 rows of x. A group is
// 128 values of K: 256 bytes of every row, 16 pieces of 16 bytes, piece p of row r at place p ^ (r % 16), so that
// operand reads meet no bank twice without padding; which piece a lane fetches is what places it. One instruction
// fills 1 KB (four rows); a wave fetches its own 16 weight rows (four instructions) and its share of the rows of x
// (dealt to the waves in turn; every wave issues the same number, the last piece again if need be). Three groups
// have room in LDS (120 KB at 64 rows and six waves: one workgroup a compute unit). Every wave issues the same number of loads
// per group, also past the end of K (the last group again, into a buffer nobody reads), so one constant says how
// many may still be in flight when a group is needed. K must be a multiple of 128. The compiler does not know
// that these loads write LDS; each wave waits for its own, then a barrier.
// Measured beside it on Qwen3-4B's gate/up at 64 rows (26 us, 24.4 since the operand reads are ordered by hand; the
// vendor library plus the activation kernel 30 to 31):
// four waves and 32 outputs (304 workgroups, two rounds or shallow stages: 32 to 38 us), eight waves (28 to 34),
// groups of 64 values (27 to 36), four or five stages (the same), weights and activations fetched by different waves
// with depths of their own (26 at best). The plain product of the same form was no faster than what serves it now.
// Walking K from a different starting group in every workgroup took Qwen3-8B's gate/up (rows 8,192 bytes apart)
// from 44 to 38 us at 8 to 40 rows; at Qwen3-4B's 5,120 bytes it changes nothing.
__device__ __forceinline__ void panel_load16(const void* base, uint32_t offset, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
}

// s_waitcnt vmcnt(N) alone (vmcnt sits in bits 3:0 and 15:14 of the immediate, the other counters stay at their
// maxima); as a builtin, so that the compiler's own count of loads in flight takes it into account
template <int N>
__device__ __forceinline__ void panel_wait() {
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
  asm volatile("" ::: "memory");
}

// silu for the epilogues whose result is rounded to bfloat16 at once: the hardware's exp2 and reciprocal (about an
// ulp of float each) instead of the library's exp and an exact division, a fifth of the instructions; the ends of
// the range come out right (exp2 = inf gives -0, exp2 = 0 gives g).
__device__ __forceinline__ float silu_for_bf16(float g) {
  return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
}

// The end of the fused gate/up products: of one row, a lane with g < 2 holds the gates of four neighbouring outputs
// n .. n + 3 (n = first + 4 g), the lane 32 further on their ups. The two lanes share the work: the first takes
// outputs n and n + 1, the second n + 2 and n + 3, each after one exchange of two values.
// y[n + i] = T(T(silu(gate)) * up), two values in one store where N is even.
__device__ __forceinline__ void swiglu_store4(bf16_t* __restrict__ y_row, int first, int N, int g, const f32x4& acc,
                                              bool row_there) {
  const bool second = g >= 2;
  const float got0 = __shfl_xor(second ? acc[0] : acc[2], 32, WAVE);
  const float got1 = __shfl_xor(second ? acc[1] : acc[3], 32, WAVE);
  const float gate0 = second ? got0 : acc[0], gate1 = second ? got1 : acc[1];
  const float up0 = second ? acc[2] : got0, up1 = second ? acc[3] : got1;
  const int n = first + 4 * (g & 1) + (second ? 2 : 0);
  const bf16_t v0 = float_to_bf16(rounded_as<bf16_t>(silu_for_bf16(rounded_as<bf16_t>(gate0))) * rounded_as<bf16_t>(up0));
  const bf16_t v1 = float_to_bf16(rounded_as<bf16_t>(silu_for_bf16(rounded_as<bf16_t>(gate1))) * rounded_as<bf16_t>(up1));
  if (!row_there || n >= N) return;
  if (N % 2 == 0) {                                        // then n + 1 < N too, and the address is a multiple of 4
    *(uint32_t*)(y_row + n) = (uint32_t)v0.bits | ((uint32_t)v1.bits << 16);
    return;
  }
  y_row[n] = v0;
  if (n + 1 < N) y_row[n + 1] = v1;
}

#define PANEL_GROUP 128                      // values of K in a group; K must be a multiple of it
#define PANEL_STAGES 3

// WAVES waves, 8 outputs each: a wave's 16 weight rows are the gate rows of its 8 outputs and then their up rows, so
// that gate and up of an output meet in lanes 32 apart and no LDS pass is needed at the end. The launcher picks
// WAVES so that the workgroups are about as many as the compute units and all run at once.
template <int MT, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemm_panel_swiglu_kernel(const bf16_t* __restrict__ x, int64_t x_stride,
                                                                       const bf16_t* __restrict__ w,
                                                                       bf16_t* __restrict__ y, int M, int N, int K) {
  extern __shared__ __align__(16) unsigned char panel_lds[];
  constexpr int STAGES = PANEL_STAGES;
  constexpr int RB = 2 * PANEL_GROUP;                      // bytes of a row in a group
  constexpr int X_ALL = 4 * MT;                            // 1 KB pieces of x in a group, dealt to the waves in turn
  constexpr int X_LOADS = (X_ALL + WAVES - 1) / WAVES;     // every wave issues this many
  constexpr int LOADS = 4 + X_LOADS;                       // per wave and group
  constexpr int W_BYTES = 16 * WAVES * RB, X_BYTES = 16 * MT * RB, STAGE_BYTES = W_BYTES + X_BYTES;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.x * WAVES + wave) * 8;          // first output of this wave
  const int groups = K / PANEL_GROUP;
  // where this lane fetches: its place within an instruction's 1 KB is fixed, the piece that belongs there follows
  uint32_t w_from[4], x_from[X_LOADS];
  int x_piece[X_LOADS];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * i + lane / 16;                       // row within the wave's 16: 0..7 gate, 8..15 up
    const int row = (r < 8 ? 0 : N) + min(n0 + (r & 7), N - 1);
    w_from[i] = (uint32_t)row * (uint32_t)K * 2u + (((lane % 16) ^ r) << 4);
  }
#pragma unroll
  for (int i = 0; i < X_LOADS; ++i) {
    x_piece[i] = min(wave + WAVES * i, X_ALL - 1);
    const int r = 4 * x_piece[i] + lane / 16;              // row of x
    x_from[i] = (uint32_t)min(r, M - 1) * (uint32_t)x_stride * 2u + (((lane % 16) ^ (r & 15)) << 4);
  }
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)panel_lds);
  // Workgroups walk K from different starting groups (and wrap around): at a row stride that is a multiple of the
  // memory channels' interleave, all of them asking for the same columns at the same time would queue on one channel.
  const int first_group = (int)((blockIdx.x * 5u) % (unsigned)groups);
  auto fetch = [&](int group, int stage) {
    int gk = min(group, groups - 1) + first_group;         // past the end: the last group again, into a free buffer
    gk = gk >= groups ? gk - groups : gk;
    const unsigned char* wb = (const unsigned char*)w + (int64_t)gk * RB;
    const unsigned char* xb = (const unsigned char*)x + (int64_t)gk * RB;
    const uint32_t at = lds0 + stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < 4; ++i) panel_load16(wb, w_from[i], at + (16 * wave + 4 * i) * RB);
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) panel_load16(xb, x_from[i], at + W_BYTES + x_piece[i] * 1024);
  };
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) fetch(s, s);
  int stage = 0;
  for (int group = 0; group < groups; ++group) {
    panel_wait<(STAGES - 2) * LOADS>();                    // this group has arrived; the later ones may be on their way
    __syncthreads();                                       // everybody's part of it too; the group before is done with
    fetch(group + STAGES - 1, stage == 0 ? STAGES - 1 : stage - 1);
    const unsigned char* ws = panel_lds + stage * STAGE_BYTES + (16 * wave + c) * RB;
    const unsigned char* xs = panel_lds + stage * STAGE_BYTES + W_BYTES + c * RB;
    constexpr int US = PANEL_GROUP / 32;                   // 32 values of K at a time
    bf16x8 a[US], b[US][MT];
#pragma unroll
    for (int u = 0; u < US; ++u) {
      const int place = ((4 * u + g) ^ c) << 4;            // row 16 t + c of any tile is swizzled like row c
      a[u] = *(const bf16x8*)(ws + place);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = *(const bf16x8*)(xs + 16 * mt * RB + place);
    }
#pragma unroll
    for (int u = 0; u < US; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][mt], acc[mt], 0, 0, 0);
    // The order the scheduler is to keep (left alone it reads two operands, waits, multiplies, and so on, and every
    // wait shows): the first quarter's reads; each quarter's matrix instructions with the next quarter's reads
    // between them; the last quarter's matrix instructions. 0x100: LDS reads, 0x008: matrix instructions.
    // With one or two tiles of rows all reads of the group go first.
    if (MT <= 2) {
      __builtin_amdgcn_sched_group_barrier(0x100, US * (MT + 1), 0);
      __builtin_amdgcn_sched_group_barrier(0x008, US * MT, 0);
    } else {
      __builtin_amdgcn_sched_group_barrier(0x100, MT + 1, 0);
#pragma unroll
      for (int u = 0; u + 1 < US; ++u) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, MT, 0);
    }
    stage = stage + 1 == STAGES ? 0 : stage + 1;
  }
  panel_wait<0>();                                         // the loads past the end have landed before the waves leave
  // acc[mt][i] is row 4g + i of the wave's 16 for activation row 16 mt + c: gate of output 4g + i in lanes with
  // g < 2, its up 32 lanes further on
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + c;
    swiglu_store4(y + (int64_t)min(m, M - 1) * N, n0, N, g, acc[mt], m < M);
  }
}

template <int MT, int WAVES>
static int launch_panel_swiglu(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K,
                               hipStream_t stream) {
  constexpr int lds = PANEL_STAGES * (16 * WAVES + 16 * MT) * 2 * PANEL_GROUP;
  static_assert(lds <= 160 * 1024, "the stages must fit a compute unit's LDS");
  static bool raised = false;                              // more dynamic LDS than the default limit allows
  auto kernel = gemm_panel_swiglu_kernel<MT, WAVES>;
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -2;
    raised = true;
  }
  dim3 grid((N + 8 * WAVES - 1) / (8 * WAVES)), block(64 * WAVES);
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, (const bf16_t*)x, x_stride, (const bf16_t*)w, (bf16_t*)y, M, N, K);
  return DRYFT_LAUNCH_CHECK();
}

template <int MT>
static int panel_waves(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K, int waves,
                       hipStream_t stream) {
  switch (waves) {
    case 4: return launch_panel_swiglu<MT, 4>(x, x_stride, w, y, M, N, K, stream);
    case 5: return launch_panel_swiglu<MT, 5>(x, x_stride, w, y, M, N, K, stream);
    case 6: return launch_panel_swiglu<MT, 6>(x, x_stride, w, y, M, N, K, stream);
    case 7: return launch_panel_swiglu<MT, 7>(x, x_stride, w, y, M, N, K, stream);
    case 8: return launch_panel_swiglu<MT, 8>(x, x_stride, w, y, M, N, K, stream);
    default: return -1;
  }
}

// How many waves a workgroup gets for N outputs (8 outputs a wave): from four to eight, the count whose workgroups
// fill whole rounds of the 256 compute units best (one workgroup runs on a unit at a time); among equals the fewest.
// Qwen3-4B's 9,728 outputs: 5 waves, 244 workgroups; Qwen3-8B's 12,288: 6 waves, 256; Qwen3-32B's 25,600: 7 waves,
// 458 in two rounds (measured best in each case).
DRYFT_API int dryft_gemm_panel_waves(int N) {
  int best = 4;
  double best_fill = 0.0;
  for (int waves = 4; waves <= 8; ++waves) {
    const int groups = (N + 8 * waves - 1) / (8 * waves), rounds = (groups + 255) / 256;
    const double fill = (double)groups / (256.0 * rounds);
    if (fill > best_fill + 1e-9) {
      best_fill = fill;
      best = waves;
    }
  }
  return best;
}

// M <= 64. y[M, N] = T(T(silu(x . Wg^T)) * (x . Wu^T)) with W = [Wg; Wu] of 2N rows; K a multiple of 128; x and W
// within reach of 32-bit byte offsets; waves: 4 to 8, or 0 for dryft_gemm_panel_waves' choice.
DRYFT_API int dryft_gemm_panel_swiglu_bf16(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K,
                                           int waves, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % PANEL_GROUP || x_stride % 8 || (((uintptr_t)x | (uintptr_t)w) & 15) ||
      (int64_t)2 * N * K * 2 >= (int64_t)4 << 30 || (int64_t)M * x_stride * 2 >= (int64_t)4 << 30)
    return -1;
  if (waves == 0) waves = dryft_gemm_panel_waves(N);
  switch ((M + 15) / 16) {
    case 1: return panel_waves<1>(x, x_stride, w, y, M, N, K, waves, stream);
    case 2: return panel_waves<2>(x, x_stride, w, y, M, N, K, waves, stream);
    case 3: return panel_waves<3>(x, x_stride, w, y, M, N, K, waves, stream);
    default: return panel_waves<4>(x, x_stride, w, y, M, N, K, waves, stream);
  }
}

// --------------------------------------------------------------------------------------------- mid
// The projections back to the hidden width (few outputs, a long K) for short prompts, 65 to 256 rows: there the
// vendor library takes 20 to 50 us for matrices that stream in 4 to 10 (Qwen3-4B: o 20 to 25 us, down 27 to 53),
// because its tiles are too few for the chip. Here a workgroup of four waves owns 64 outputs (16 rows of W a wave)
// and all rows of x, K is split over workgroups into float partial sums that the consumer adds in a fixed order,
// and the operands go from memory straight into LDS as in the panel product (groups of 64 values of K: rows of
// 128 bytes, piece p of row r at place p ^ ((r / 2) % 8); three groups in LDS; a wave fetches its own 16 rows of W
// and its share of the rows of x; every workgroup walks its part of K from a starting group of its own). Every
// workgroup reads all of x (from L2), which is why this form stops paying at about 250 rows and never pays for the
// products with many outputs (q/k/v, gate/up). Measured, weights from memory, us at 80 / 128 / 192 rows against the
// vendor library: Qwen3-4B's o 10.9 / 12.8 / 17.3 (21 / 25 / 19), down 19.1 / 21.0 / 28.5 (27 / 53 / 34); Qwen3-8B's o
// 13.5 / 15.4 / 20.6 (21 / 25 / 34), down 29 / 38 / 53 (38 / 67 / 90); Qwen3-32B's o 26 / 29 / 39 (30 / 45 / 61), down
// 72 / 88 / 111 (173 / 181 / 209). Since the tall product below took the steps of 65 to 256 rows (its workgroups take
// in fewer bytes of x for a row of W), this one serves those of 33 to 64 rows.
#define MID_GROUP 64
#define MID_STAGES 3
#define MID_WAVES 4

template <int MT>
__global__ __launch_bounds__(64 * MID_WAVES) void gemm_mid_kernel(const bf16_t* __restrict__ x, int64_t x_stride,
                                                                  const bf16_t* __restrict__ w,
                                                                  float* __restrict__ partials, int M, int N, int K,
                                                                  int groups_per_split) {
  extern __shared__ __align__(16) unsigned char mid_lds[];
  constexpr int STAGES = MID_STAGES, WAVES = MID_WAVES;
  constexpr int RB = 2 * MID_GROUP;                        // bytes of a row in a group
  constexpr int X_ALL = 2 * MT;                            // 1 KB pieces (8 rows) of x in a group
  constexpr int X_LOADS = (X_ALL + WAVES - 1) / WAVES;     // every wave issues this many
  constexpr int LOADS = 2 + X_LOADS;
  constexpr int W_BYTES = 16 * WAVES * RB, X_BYTES = 16 * MT * RB, STAGE_BYTES = W_BYTES + X_BYTES;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.x * WAVES + wave) * 16;         // first output of this wave
  const int group0 = blockIdx.y * groups_per_split;
  const int groups = min(groups_per_split, K / MID_GROUP - group0);
  uint32_t w_from[2], x_from[X_LOADS];
  int x_piece[X_LOADS];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = 8 * i + lane / 8;                        // row within the wave's 16
    w_from[i] = (uint32_t)min(n0 + r, N - 1) * (uint32_t)K * 2u + (((lane % 8) ^ ((r >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int i = 0; i < X_LOADS; ++i) {
    x_piece[i] = min(wave + WAVES * i, X_ALL - 1);
    const int r = 8 * x_piece[i] + lane / 8;               // row of x
    x_from[i] = (uint32_t)min(r, M - 1) * (uint32_t)x_stride * 2u + (((lane % 8) ^ ((r >> 1) & 7)) << 4);
  }
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)mid_lds);
  const int first_group = (int)((blockIdx.x * 5u) % (unsigned)groups);
  auto fetch = [&](int group, int stage) {
    int gk = min(group, groups - 1) + first_group;         // past the end: the last group again, into a free buffer
    gk = (gk >= groups ? gk - groups : gk) + group0;
    const unsigned char* wb = (const unsigned char*)w + (int64_t)gk * RB;
    const unsigned char* xb = (const unsigned char*)x + (int64_t)gk * RB;
    const uint32_t at = lds0 + stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < 2; ++i) panel_load16(wb, w_from[i], at + (16 * wave + 8 * i) * RB);
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) panel_load16(xb, x_from[i], at + W_BYTES + x_piece[i] * 1024);
  };
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) fetch(s, s);
  int stage = 0;
  const int sw = (c >> 1) & 7;                             // row 16 t + c of any tile is swizzled like row c
  for (int group = 0; group < groups; ++group) {
    panel_wait<(STAGES - 2) * LOADS>();                    // this group has arrived; the later ones may be on their way
    __syncthreads();                                       // everybody's part of it too; the group before is done with
    fetch(group + STAGES - 1, stage == 0 ? STAGES - 1 : stage - 1);
    const unsigned char* ws = mid_lds + stage * STAGE_BYTES + (16 * wave + c) * RB;
    const unsigned char* xs = mid_lds + stage * STAGE_BYTES + W_BYTES + c * RB;
    bf16x8 a[2], b[2][MT];
#pragma unroll
    for (int u = 0; u < 2; ++u) {                          // 32 values of K at a time
      const int place = ((4 * u + g) ^ sw) << 4;
      a[u] = *(const bf16x8*)(ws + place);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = *(const bf16x8*)(xs + 16 * mt * RB + place);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][mt], acc[mt], 0, 0, 0);
    // the order the scheduler is to keep: the first half's reads; its matrix instructions with one read of the
    // second half after each; the second half's matrix instructions (0x100: LDS reads, 0x008: matrix instructions)
    __builtin_amdgcn_sched_group_barrier(0x100, MT + 1, 0);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, MT, 0);
    stage = stage + 1 == STAGES ? 0 : stage + 1;
  }
  panel_wait<0>();                                         // the loads past the end have landed before the waves leave
  // acc[mt][i] is output n0 + 4g + i of activation row 16 mt + c
  float* out = partials + (int64_t)blockIdx.y * M * N;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + c, n = n0 + 4 * g;
    if (m >= M) continue;
    if (n + 3 < N && (N & 3) == 0) {
      *(f32x4*)(out + (int64_t)m * N + n) = acc[mt];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < N) out[(int64_t)m * N + n + i] = acc[mt][i];
    }
  }
}

template <int MT>
static int launch_mid(const void* x, int64_t x_stride, const void* w, float* partials, int M, int N, int K, int splits,
                      int groups_per_split, hipStream_t stream) {
  constexpr int lds = MID_STAGES * (16 * MID_WAVES + 16 * MT) * 2 * MID_GROUP;
  static_assert(lds <= 160 * 1024, "the stages must fit a compute unit's LDS");
  static bool raised = false;                              // more dynamic LDS than the default limit allows
  auto kernel = gemm_mid_kernel<MT>;
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -2;
    raised = true;
  }
  dim3 grid((N + 16 * MID_WAVES - 1) / (16 * MID_WAVES), splits), block(64 * MID_WAVES);
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, (const bf16_t*)x, x_stride, (const bf16_t*)w, partials, M, N, K,
                     groups_per_split);
  return DRYFT_LAUNCH_CHECK();
}

// M <= 256. partials[splits, M, N] = float partial sums of x . W^T over `splits` equal runs of groups of 64 values of K
// (the last run may be shorter, none may be empty); K a multiple of 64; x and W within reach of 32-bit byte offsets.
DRYFT_API int dryft_gemm_mid_bf16(const void* x, int64_t x_stride, const void* w, float* partials, int M, int N, int K,
                                  int splits, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 256 || K <= 0 || K % MID_GROUP || splits < 1 || x_stride % 8 || (((uintptr_t)x | (uintptr_t)w) & 15) ||
      ((uintptr_t)partials & 15) || (int64_t)N * K * 2 >= (int64_t)4 << 30 || (int64_t)M * x_stride * 2 >= (int64_t)4 << 30)
    return -1;
  const int groups = K / MID_GROUP, per = (groups + splits - 1) / splits;
  if ((groups + per - 1) / per != splits) return -1;       // a run would be empty
  if (M <= 32) return launch_mid<2>(x, x_stride, w, partials, M, N, K, splits, per, stream);
  if (M <= 48) return launch_mid<3>(x, x_stride, w, partials, M, N, K, splits, per, stream);
  if (M <= 64) return launch_mid<4>(x, x_stride, w, partials, M, N, K, splits, per, stream);
  if (M <= 96) return launch_mid<6>(x, x_stride, w, partials, M, N, K, splits, per, stream);
  if (M <= 128) return launch_mid<8>(x, x_stride, w, partials, M, N, K, splits, per, stream);
  if (M <= 192) return launch_mid<12>(x, x_stride, w, partials, M, N, K, splits, per, stream);
  return launch_mid<16>(x, x_stride, w, partials, M, N, K, splits, per, stream);
}

// -------------------------------------------------------------------------------------------- tall
// Products of 65 to 256 rows (short prompts, decoding at large batch), cut the other way than the panel and mid
// products above, whose waves each read every row of x from LDS for only 16 rows of W (one LDS read a matrix
// instruction). Here a workgroup of eight multiplying waves owns T tiles of 16 rows of W and all rows of x; wave w
// owns R tiles of 16 rows of x (rows 16 R w ...) and multiplies them with all T tiles of W: R + T reads for R T
// instructions. Operands go from memory straight into LDS in groups of 64 values of K (rows of 128 bytes, piece p of
// row r at place p ^ ((r / 2) % 8), as in gemm_mid). Two forms:
//   the fused gate/up product with its activation (a tile of W is 8 gate rows and the 8 up rows of the same outputs,
//     as in the panel product, so a workgroup owns 8 T outputs over all of K), rounded to bfloat16;
//   the plain product as float partial sums over runs of K (a tile is 16 outputs).
// What bounds it, by the cycle counter inside the kernel at Qwen3-4B's gate/up (100 MB, 244 workgroups of 80 rows
// of W): the waves never wait for data, they wait to issue loads. A compute unit takes in about 46 bytes a cycle of
// activations from the L2 on top of the time its share of the weights takes to stream from memory (16.5 us), and
// every workgroup takes in all of x over its run of K: 1.3 MB at 256 rows, 12 us. So the time grows with the rows
// (20 us inside the loop at 64 rows, 23 at 128, 29 at 256), deeper rings change nothing, and what pays is fewer
// bytes of x a compute unit: more rows of W a workgroup, shorter runs of K.
// x and W within reach of 32-bit offsets.
#define TALL_GROUP 64
#define TALL_WAVES 8
#define TALL_LDS (160 * 1024)

// Weights come from memory (about 2 us away: a compute unit's share of the memory rate wants some 44 KB of them in
// flight), activations from the L2 (nearer, but 16 R / T times as many bytes): each has a ring of its own in LDS, the
// activations' of X_STAGES groups, the weights' as deep as the rest of LDS allows. A wave's loads are counted off in
// the order of their issue, so a wave that fetched both would wait for its newest weights whenever it waits for its
// activations: a ninth wave fetches the weights and does nothing else, the eight that multiply fetch their own rows
// of x. The weights' ring is no deeper than the 63 loads a wave can count.
template <int R, int T>
struct TallPlan {
  static constexpr int RB = 2 * TALL_GROUP;                             // bytes of a row in a group
  static constexpr int W_BYTES = 16 * T * RB, X_BYTES = 16 * R * TALL_WAVES * RB;
  static constexpr int X_STAGES = R == 1 ? 4 : 3;
  static constexpr int w_fit = (TALL_LDS - X_STAGES * X_BYTES) / W_BYTES, w_count = 63 / (2 * T) + 2;
  static constexpr int W_STAGES = w_fit < w_count ? (w_fit < 8 ? w_fit : 8) : (w_count < 8 ? w_count : 8);
  static constexpr int LDS = W_STAGES * W_BYTES + X_STAGES * X_BYTES;
  static_assert(W_STAGES >= 3, "two groups of weights in flight at least");
};

// SWIGLU: y is bf16 [M, N], w is [2N, K]. Otherwise y is float [splits, M, N], w is [N, K], and a workgroup sums
// over one run of `per` groups of K. Workgroups go to the eight dies in turn, each die with an L2 of its own: the
// (run, tile) pairs are dealt so that a die gets neighbouring ones, and with them few runs of K, whose columns of x
// are all of x that its L2 has to hold and to fetch (a prompt's 256 rows of Qwen3-4B's down projection are 5 MB,
// more than one L2). The grid is 8 * ceil(pairs / 8) workgroups; those beyond the last pair leave at once.
template <int R, int T, bool SWIGLU>
__global__ __launch_bounds__(64 * (TALL_WAVES + 1)) void gemm_tall_kernel(
    const bf16_t* __restrict__ x, int64_t x_stride, const bf16_t* __restrict__ w, void* __restrict__ y, int M, int N,
    int K, int per, int blocks, int splits) {
  extern __shared__ __align__(16) unsigned char tall_lds[];
  using Plan = TallPlan<R, T>;
  constexpr int WAVES = TALL_WAVES, RB = Plan::RB, W_BYTES = Plan::W_BYTES, X_BYTES = Plan::X_BYTES;
  constexpr int WS = Plan::W_STAGES, XS = Plan::X_STAGES, DW = WS - 1, DX = XS - 1;
  constexpr int W_LOADS = 2 * T;                           // 1 KB pieces (8 rows) of W in a group
  constexpr int X_LOADS = 2 * R;                           // a wave's own 16 R rows of x
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int pairs = blocks * splits, a_die = (pairs + 7) / 8;
  const int pair = (int)(blockIdx.x % 8) * a_die + (int)(blockIdx.x / 8);
  if (pair >= pairs) return;
  const int run = pair / blocks, block = pair % blocks;
  const int tile0 = block * T;                             // first tile of this workgroup
  const int group0 = run * per;                            // its run of K
  const int groups = min(per, K / TALL_GROUP - group0);
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)tall_lds);
  const int first_group = (int)(((unsigned)block * 5u) % (unsigned)groups);   // workgroups walk K from different places
  auto group_at = [&](int group) {
    const int gk = group + first_group;
    return (int64_t)(group0 + (gk >= groups ? gk - groups : gk)) * RB;
  };
  // Nothing is fetched past the end of the run, so near the end fewer loads follow a group's than the waits count on:
  // there a wave waits for all it has issued.
  if (wave == WAVES) {                                     // the wave that fetches the weights
    uint32_t w_from[W_LOADS];
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      const int r = 8 * i + lane / 8;                      // row among the workgroup's 16 T rows of W
      int row;
      if (SWIGLU) {                                        // 0..7: gate rows of the tile's outputs, 8..15: their up rows
        const int tile = tile0 + r / 16, in_tile = r % 16;
        row = (in_tile < 8 ? 0 : N) + min(8 * tile + (in_tile & 7), N - 1);
      } else {
        row = min(16 * tile0 + r, N - 1);
      }
      w_from[i] = (uint32_t)row * (uint32_t)K * 2u + (((lane % 8) ^ ((r >> 1) & 7)) << 4);
    }
    auto fetch_w = [&](int group, int stage) {
      const unsigned char* wb = (const unsigned char*)w + group_at(group);
#pragma unroll
      for (int i = 0; i < W_LOADS; ++i) panel_load16(wb, w_from[i], lds0 + stage * W_BYTES + i * 1024);
    };
#pragma unroll
    for (int j = 0; j < DW; ++j)
      if (j < groups) fetch_w(j, j);
    int w_stage = 0;
    for (int group = 0; group < groups; ++group) {
      if (group + DW <= groups) panel_wait<(DW - 1) * W_LOADS>();      // this group's weights have arrived
      else panel_wait<0>();
      __syncthreads();                                     // the others hear of it; they are done with the group before
      if (group + DW < groups) fetch_w(group + DW, w_stage == 0 ? WS - 1 : w_stage - 1);
      w_stage = w_stage + 1 == WS ? 0 : w_stage + 1;
    }
    return;
  }
  uint32_t x_from[X_LOADS];
#pragma unroll
  for (int i = 0; i < X_LOADS; ++i) {
    const int r = 16 * R * wave + 8 * i + lane / 8;        // row of x
    x_from[i] = (uint32_t)min(r, M - 1) * (uint32_t)x_stride * 2u + (((lane % 8) ^ ((r >> 1) & 7)) << 4);
  }
  const uint32_t x_lds0 = lds0 + WS * W_BYTES;
  auto fetch_x = [&](int group, int stage) {
    const unsigned char* xb = (const unsigned char*)x + group_at(group);
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) panel_load16(xb, x_from[i], x_lds0 + stage * X_BYTES + (2 * R * wave + i) * 1024);
  };
  f32x4 acc[R][T];
#pragma unroll
  for (int m = 0; m < R; ++m)
#pragma unroll
    for (int t = 0; t < T; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < DX; ++j)
    if (j < groups) fetch_x(j, j);
  int w_stage = 0, x_stage = 0;
  const int sw = (c >> 1) & 7;                             // row 16 t + c of any tile is swizzled like row c
  // Operands are read from LDS half a group (32 values of K) ahead of the matrix instructions that use them, into one
  // of two sets of registers, so that the reads of one half run under the instructions of the half before.
  bf16x8 a[2][T], b[2][R];
  auto read_half = [&](int u) {
    const unsigned char* ws = tall_lds + w_stage * W_BYTES + c * RB;
    const unsigned char* xs = tall_lds + WS * W_BYTES + x_stage * X_BYTES + (16 * R * wave + c) * RB;
    const int place = ((4 * u + g) ^ sw) << 4;
#pragma unroll
    for (int t = 0; t < T; ++t) a[u][t] = *(const bf16x8*)(ws + 16 * t * RB + place);
#pragma unroll
    for (int m = 0; m < R; ++m) b[u][m] = *(const bf16x8*)(xs + 16 * m * RB + place);
  };
  auto multiply_half = [&](int u) {
#pragma unroll
    for (int m = 0; m < R; ++m)
#pragma unroll
      for (int t = 0; t < T; ++t) acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], b[u][m], acc[m][t], 0, 0, 0);
  };
  for (int group = 0; group < groups; ++group) {
    if (group + DX <= groups) panel_wait<(DX - 1) * X_LOADS>();        // this group's rows of x have arrived (nobody
    else panel_wait<0>();                                              // else reads them)
    __syncthreads();                                       // its weights too; everybody has read the group before
    if (group + DX < groups) fetch_x(group + DX, x_stage == 0 ? XS - 1 : x_stage - 1);
    read_half(0);
    __builtin_amdgcn_sched_barrier(0);
    if (group > 0) multiply_half(1);                       // the second half of the group before
    __builtin_amdgcn_sched_barrier(0);
    read_half(1);
    __builtin_amdgcn_sched_barrier(0);
    multiply_half(0);
    __builtin_amdgcn_sched_barrier(0);
    w_stage = w_stage + 1 == WS ? 0 : w_stage + 1;
    x_stage = x_stage + 1 == XS ? 0 : x_stage + 1;
  }
  multiply_half(1);
  // acc[m][t][i] is row 4g + i of W tile t for activation row 16 (R wave + m) + c
#pragma unroll
  for (int m = 0; m < R; ++m) {
    const int row = 16 * (R * wave + m) + c;
    if (SWIGLU) {                                          // the gate of output 4g + i of the tile in lanes with g < 2,
      bf16_t* y_row = (bf16_t*)y + (int64_t)min(row, M - 1) * N;                    // its up 32 lanes further on
#pragma unroll
      for (int t = 0; t < T; ++t) swiglu_store4(y_row, 8 * (tile0 + t), N, g, acc[m][t], row < M);
    } else if (row < M) {
      float* y_row = (float*)y + ((int64_t)run * M + row) * N;
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const int n = 16 * (tile0 + t) + 4 * g;
        if (N % 4 == 0) {                                  // then n + 3 < N where n < N, and the address is a multiple of 16
          if (n < N) *(f32x4*)(y_row + n) = acc[m][t];
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) y_row[n + i] = acc[m][t][i];
        }
      }
    }
  }
}

template <int R, int T, bool SWIGLU>
static int launch_tall(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K, int splits, int per,
                       hipStream_t stream) {
  constexpr int lds = TallPlan<R, T>::LDS;
  static_assert(lds <= TALL_LDS, "the rings must fit a compute unit's LDS");
  static bool raised = false;                              // more dynamic LDS than the default limit allows
  auto kernel = gemm_tall_kernel<R, T, SWIGLU>;
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -2;
    raised = true;
  }
  const int outputs = (SWIGLU ? 8 : 16) * T, blocks = (N + outputs - 1) / outputs;
  dim3 grid(8 * ((blocks * splits + 7) / 8)), block(64 * (TALL_WAVES + 1));
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, (const bf16_t*)x, x_stride, (const bf16_t*)w, y, M, N, K, per, blocks,
                     splits);
  return DRYFT_LAUNCH_CHECK();
}

// How many tiles of 8 outputs a workgroup of the fused gate/up form gets for N outputs: from four to eight, the count
// whose workgroups fill whole rounds of the 256 compute units best (one workgroup runs on a unit at a time); among
// equals the most.
DRYFT_API int dryft_gemm_tall_tiles(int N) {
  int best = 4;
  double best_fill = 0.0;
  for (int tiles = 4; tiles <= 8; ++tiles) {
    const int groups = (N + 8 * tiles - 1) / (8 * tiles), rounds = (groups + 255) / 256;
    const double fill = (double)groups / (256.0 * rounds);
    if (fill >= best_fill - 1e-9) {
      best_fill = fill > best_fill ? fill : best_fill;
      best = tiles;
    }
  }
  return best;
}

template <int R, bool SWIGLU>
static int tall_tiles(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K, int tiles, int splits,
                      int per, hipStream_t stream) {
  switch (tiles) {
    case 4: return launch_tall<R, 4, SWIGLU>(x, x_stride, w, y, M, N, K, splits, per, stream);
    case 5: return launch_tall<R, 5, SWIGLU>(x, x_stride, w, y, M, N, K, splits, per, stream);
    case 6: return launch_tall<R, 6, SWIGLU>(x, x_stride, w, y, M, N, K, splits, per, stream);
    case 7: return launch_tall<R, 7, SWIGLU>(x, x_stride, w, y, M, N, K, splits, per, stream);
    case 8: return launch_tall<R, 8, SWIGLU>(x, x_stride, w, y, M, N, K, splits, per, stream);
    default: return -1;
  }
}

static bool tall_operands_ok(const void* x, int64_t x_stride, const void* w, int M, int64_t w_rows, int K) {
  return M <= 256 && K > 0 && K % TALL_GROUP == 0 && x_stride % 8 == 0 && !(((uintptr_t)x | (uintptr_t)w) & 15) &&
         w_rows * K * 2 < (int64_t)4 << 30 && (int64_t)M * x_stride * 2 < (int64_t)4 << 30;
}

// M <= 256. y[M, N] = T(T(silu(x . Wg^T)) * (x . Wu^T)) with W = [Wg; Wu] of 2N rows; K a multiple of 64; x and W
// within reach of 32-bit byte offsets; tiles: 4 to 8, or 0 for dryft_gemm_tall_tiles' choice.
DRYFT_API int dryft_gemm_tall_swiglu_bf16(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K,
                                          int tiles, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!tall_operands_ok(x, x_stride, w, M, (int64_t)2 * N, K)) return -1;
  if (tiles == 0) tiles = dryft_gemm_tall_tiles(N);
  const int groups = K / TALL_GROUP;
  if (M <= 128) return tall_tiles<1, true>(x, x_stride, w, y, M, N, K, tiles, 1, groups, stream);
  return tall_tiles<2, true>(x, x_stride, w, y, M, N, K, tiles, 1, groups, stream);
}

// M <= 256. partials[s, M, N] = x . W^T over the s-th of `splits` runs of ceil(K / 64 / splits) groups of K (the last
// run may be shorter, none may be empty: dryft_gemm_mid_splits gives a count that fits); a workgroup owns 16 `tiles`
// outputs (tiles 4 to 8); K a multiple of 64; x and W within reach of 32-bit byte offsets.
DRYFT_API int dryft_gemm_tall_bf16(const void* x, int64_t x_stride, const void* w, float* partials, int M, int N, int K,
                                   int splits, int tiles, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!tall_operands_ok(x, x_stride, w, M, N, K) || splits < 1 || ((uintptr_t)partials & 15)) return -1;
  const int groups = K / TALL_GROUP, per = (groups + splits - 1) / splits;
  if ((groups + per - 1) / per != splits) return -1;       // a run would be empty
  if (M <= 128) return tall_tiles<1, false>(x, x_stride, w, partials, M, N, K, tiles, splits, per, stream);
  return tall_tiles<2, false>(x, x_stride, w, partials, M, N, K, tiles, splits, per, stream);
}

// ------------------------------------------------------------------------------------------- block
// Many rows: a workgroup owns a block of rows by outputs (128 x 128 with four waves, 256 x 256 with eight) and
// walks K in steps of 64. Its threads copy the block's rows of x and of W for one step into LDS (whole cache
// lines per load; rows 32 bytes past a multiple of 64 apart, the stride at which operand reads reach LDS's full
// rate), the next step's rows wait in registers meanwhile; each wave multiplies its part of the block (64 x 64 or
// 128 x 64) with v_mfma_f32_16x16x32_bf16. Rows beyond M or N are read from a clamped, valid row and never
// stored; K is padded with zeros. What bounds it is the rate at which the caches deliver the blocks' rows (a
// 128 x 128 block multiplies 64 flops per byte staged, a 256 x 256 block 128): 0.4-0.6 PFLOP/s at 2,048 rows,
// 0.8-1.0 at 16,384. The vendor library is faster on the sizes it takes; this kernel takes the others (outputs
// that are no multiple of 8, results wanted in float32 for many rows). With SWIGLU the rows of W in a block are
// gate rows and the up rows of the same outputs (W = [Wg; Wu]), and the epilogue stores T(T(silu(gate)) * up)
// (reference: kernels/silu_mul.py:29-32).
#define BLOCK_STRIDE 160      // bytes between rows of a step in LDS: 128 of data

// WM x WN waves, each with MT x NT tiles of 16 x 16: a block of WM*MT*16 rows by WN*NT*16 rows of W.
// T = float: the same kernel on 32-bit values with v_mfma_f32_16x16x4_f32, which multiplies and adds in full
// float precision (a step is then 32 values of K, and a lane's 16 bytes are 4 of them, one per instruction).
template <typename T>
struct BlockElem;
template <>
struct BlockElem<bf16_t> {
  static constexpr int PER_PIECE = 8, STEP = 64;           // values per 16 bytes, values of K per step
};
template <>
struct BlockElem<float> {
  static constexpr int PER_PIECE = 4, STEP = 32;
};

template <typename T>
__device__ __forceinline__ f32x4 block_mfma(f32x4 a, f32x4 b, f32x4 acc) {
  if constexpr (sizeof(T) == 2) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[i], acc, 0, 0, 0);
    return acc;
  }
}

template <typename T, int WM, int WN, int MT, int NT, bool SWIGLU, typename O>
__global__ __launch_bounds__(64 * WM * WN, WM * WN <= 4 ? 2 : 1) void gemm_block_kernel(const T* __restrict__ x,
                                                                                      int64_t x_stride,
                                                                                      const T* __restrict__ w,
                                                                                      O* __restrict__ y, int M, int N,
                                                                                      int K) {
  typedef BlockElem<T> E;
  constexpr int THREADS = 64 * WM * WN, BM = WM * MT * 16, BN = WN * NT * 16;
  constexpr int ROWS_PER_PASS = THREADS / 8, XP = BM / ROWS_PER_PASS, WP = BN / ROWS_PER_PASS;
  static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0 && (!SWIGLU || NT % 2 == 0), "block shape");
  extern __shared__ __align__(16) unsigned char block_lds[];
  unsigned char* const xs = block_lds;
  unsigned char* const ws = block_lds + BM * BLOCK_STRIDE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE;
  const int c = lane % 16, g = lane / 16;
  const int wm = wave / WN, wn = wave % WN;                // the wave's part of the block
  constexpr int OUTS = SWIGLU ? BN / 2 : BN;               // outputs a block owns
  constexpr int WAVE_OUTS = OUTS / WN;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * OUTS;
  // the rows this thread copies: row lr + ROWS_PER_PASS * i of the block, 16-byte piece lp of the step
  const int lr = threadIdx.x / 8, lp = threadIdx.x % 8;
  const T* x_row[XP];
  const T* w_row[WP];
#pragma unroll
  for (int i = 0; i < XP; ++i) x_row[i] = x + (int64_t)min(m0 + lr + ROWS_PER_PASS * i, M - 1) * x_stride;
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int r = lr + ROWS_PER_PASS * i;
    int wr;                                                // row of W behind row r of the block
    if (SWIGLU) wr = r < BN / 2 ? min(n0 + r, N - 1) : N + min(n0 + r - BN / 2, N - 1);
    else wr = min(n0 + r, N - 1);
    w_row[i] = w + (int64_t)wr * K;
  }
  f32x4 acc[MT][NT];                                       // [tile of 16 rows][tile of 16 outputs]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x4 xa[XP], wa[WP];                                    // 16 bytes each, whatever they hold
  auto fetch = [&](int k0) {                               // nothing conditional: a piece beyond K is read from the
    const int kk = min(k0 + E::PER_PIECE * lp, K - E::PER_PIECE);   // row's last piece and stored as zeros
#pragma unroll
    for (int i = 0; i < XP; ++i) xa[i] = *(const f32x4*)(x_row[i] + kk);
#pragma unroll
    for (int i = 0; i < WP; ++i) wa[i] = *(const f32x4*)(w_row[i] + kk);
  };
  // rows of W behind the wave's tiles of outputs, as rows of the block
  int w_tile[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    w_tile[nt] = SWIGLU ? (nt < NT / 2 ? WAVE_OUTS * wn + 16 * nt : BN / 2 + WAVE_OUTS * wn + 16 * (nt - NT / 2))
                        : WAVE_OUTS * wn + 16 * nt;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += E::STEP) {
    const bool in = k0 + E::PER_PIECE * lp < K;
    __syncthreads();                                       // every wave is done with the step before
#pragma unroll
    for (int i = 0; i < XP; ++i)
      *(f32x4*)(xs + (lr + ROWS_PER_PASS * i) * BLOCK_STRIDE + 16 * lp) = in ? xa[i] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < WP; ++i) *(f32x4*)(ws + (lr + ROWS_PER_PASS * i) * BLOCK_STRIDE + 16 * lp) = wa[i];
    fetch(k0 + E::STEP);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      f32x4 a[NT], b[MT];
#pragma unroll
      for (int t = 0; t < NT; ++t) a[t] = *(const f32x4*)(ws + (w_tile[t] + c) * BLOCK_STRIDE + 64 * u + 16 * g);
#pragma unroll
      for (int t = 0; t < MT; ++t) b[t] = *(const f32x4*)(xs + (MT * 16 * wm + 16 * t + c) * BLOCK_STRIDE + 64 * u + 16 * g);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = block_mfma<T>(a[nt], b[mt], acc[mt][nt]);
    }
  }
  // acc[mt][nt][i] is output (tile nt) + 4g + i of row m0 + MT*16*wm + 16 mt + c
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + MT * 16 * wm + 16 * mt + c;
    if (m >= M) continue;
    if (SWIGLU) {
#pragma unroll
      for (int nt = 0; nt < NT / 2; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + WAVE_OUTS * wn + 16 * nt + 4 * g + i;
          if (n >= N) continue;
          const float gv = rounded_as<T>(acc[mt][nt][i]), uv = rounded_as<T>(acc[mt][nt + NT / 2][i]);
          const float sv = rounded_as<T>(gv / (1.f + expf(-gv)));
          store_from_float(y + (int64_t)m * N + n, sv * uv);
        }
    } else {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + WAVE_OUTS * wn + 16 * nt + 4 * g + i;
          if (n < N) store_from_float(y + (int64_t)m * N + n, acc[mt][nt][i]);
        }
    }
  }
}

template <typename T, int WM, int WN, int MT, int NT, bool SWIGLU, typename O>
static int launch_block(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K, hipStream_t stream) {
  constexpr int BM = WM * MT * 16, BN = WN * NT * 16, OUTS = SWIGLU ? BN / 2 : BN;
  constexpr int lds = (BM + BN) * BLOCK_STRIDE;
  auto kernel = gemm_block_kernel<T, WM, WN, MT, NT, SWIGLU, O>;
  static bool raised = false;                              // more dynamic LDS than the default limit allows
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -2;
    raised = true;
  }
  dim3 grid((N + OUTS - 1) / OUTS, (M + BM - 1) / BM), block(64 * WM * WN);
  if (grid.y > 65535) return -1;
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, (const T*)x, x_stride, (const T*)w, (O*)y, M, N, K);
  return DRYFT_LAUNCH_CHECK();
}

// Any M. y[M, N] = x . w^T (w of N rows), or with swiglu y[M, N] = T(T(silu(x . Wg^T)) * (x . Wu^T)) (w of 2N rows).
// shape: 0 = blocks of 128 x 128 (four waves), 1 = 256 x 256 (eight waves; twice the flops per byte staged)
DRYFT_API int dryft_gemm_block_bf16(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K,
                                    int swiglu, int out_f32, int shape, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8 || x_stride % 8 || (swiglu && out_f32)) return -1;
#define BLK(WMV, WNV, MTV, NTV)                                                                                        \
  return swiglu    ? launch_block<bf16_t, WMV, WNV, MTV, NTV, true, bf16_t>(x, x_stride, w, y, M, N, K, stream)        \
         : out_f32 ? launch_block<bf16_t, WMV, WNV, MTV, NTV, false, float>(x, x_stride, w, y, M, N, K, stream)        \
                   : launch_block<bf16_t, WMV, WNV, MTV, NTV, false, bf16_t>(x, x_stride, w, y, M, N, K, stream)
  switch (shape) {
    case 0: BLK(2, 2, 4, 4);
    case 1: BLK(2, 4, 8, 4);
    default: return -1;
  }
#undef BLK
}

// The same on 32-bit values: y[M, N] = x . w^T in full float precision. K and x_stride multiples of 4.
DRYFT_API int dryft_gemm_block_f32(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K, int shape,
                                   hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 4 || x_stride % 4) return -1;
  switch (shape) {
    case 0: return launch_block<float, 2, 2, 4, 4, false, float>(x, x_stride, w, y, M, N, K, stream);
    case 1: return launch_block<float, 2, 4, 8, 4, false, float>(x, x_stride, w, y, M, N, K, stream);
    default: return -1;
  }
}

// ------------------------------------------------------------------------------------------- rows of 32-bit values
// At most 16 rows of 32-bit values (decoding in the float32 path): bound by reading W once. A workgroup owns 8
// weight rows, two per wave, and walks K in chunks of 256: the rows of x for a chunk are staged in LDS once for all
// four waves (double-buffered, one barrier per chunk), a lane takes four consecutive values of each of its weight
// rows (16-byte loads, a wave reads 1 KB of a row per instruction; the next chunk's are in flight while this one is
// multiplied) and the matching four of every row of x, and multiplies with plain fused multiply-adds. At the end
// the 64 lanes' sums are added. K must be a multiple of 4; rows beyond N are read from a clamped row, never stored.
#define ROWS_CHUNK 256
template <int MR>
__global__ __launch_bounds__(256) void gemm_rows_f32_kernel(const float* __restrict__ x, int64_t x_stride,
                                                            const float* __restrict__ w, float* __restrict__ y, int M,
                                                            int N, int K) {
  __shared__ __align__(16) float xs[2][MR][ROWS_CHUNK + 4];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int n0 = blockIdx.x * 8 + 2 * wave;
  const float* w_row[2] = {w + (int64_t)min(n0, N - 1) * K, w + (int64_t)min(n0 + 1, N - 1) * K};
  float acc[2][MR];
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;
  float xr[MR];                                            // thread t brings value k0 + t of every row of x
  auto fetch_x = [&](int k0) {                             // beyond K or M: a valid address, stored as zero
    const int k = min(k0 + (int)threadIdx.x, K - 1);
#pragma unroll
    for (int m = 0; m < MR; ++m) xr[m] = x[(int64_t)min(m, M - 1) * x_stride + k];
  };
  auto store_x = [&](int buf, int k0) {
    const bool in = k0 + (int)threadIdx.x < K;
#pragma unroll
    for (int m = 0; m < MR; ++m) xs[buf][m][threadIdx.x] = (in && m < M) ? xr[m] : 0.f;
  };
  f32x4 wv[2], wn[2];
  auto fetch = [&](f32x4 (&v)[2], int k0) {                // beyond K: the row's last four values, multiplied by zeros
    const int kk = min(k0 + 4 * lane, K - 4);
    v[0] = *(const f32x4*)(w_row[0] + kk);
    v[1] = *(const f32x4*)(w_row[1] + kk);
  };
  fetch_x(0);
  fetch(wv, 0);
  store_x(0, 0);
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += ROWS_CHUNK, buf ^= 1) {
    __syncthreads();                                       // the chunk is staged; the other buffer is free again
    fetch_x(k0 + ROWS_CHUNK);                              // the next chunk's loads are in flight during the products
    fetch(wn, k0 + ROWS_CHUNK);
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const f32x4 xv = *(const f32x4*)&xs[buf][m][4 * lane];   // zeros beyond K
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[r][m] = fmaf(wv[r][i], xv[i], acc[r][m]);
    }
    store_x(buf ^ 1, k0 + ROWS_CHUNK);
    wv[0] = wn[0];
    wv[1] = wn[1];
  }
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float s = wave_sum(acc[r][m]);
      if (lane == 0 && m < M && n0 + r < N) y[(int64_t)m * N + n0 + r] = s;
    }
}

// M <= 16, K % 4 == 0
DRYFT_API int dryft_gemm_rows_f32(const void* x, int64_t x_stride, const void* w, void* y, int M, int N, int K,
                                  hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K <= 0 || K % 4) return -1;
  dim3 grid((N + 7) / 8), block(256);
#define RW(MRV)                                                                                                \
  hipLaunchKernelGGL(gemm_rows_f32_kernel<MRV>, grid, block, 0, stream, (const float*)x, x_stride, (const float*)w, \
                     (float*)y, M, N, K)
  if (M <= 1) RW(1);
  else if (M <= 2) RW(2);
  else if (M <= 4) RW(4);
  else if (M <= 8) RW(8);
  else RW(16);
#undef RW
  return DRYFT_LAUNCH_CHECK();
}

// y = T(sum_s partials[s]) in the order s = 0, 1, ...
template <typename O>
__global__ void sum_partials_kernel(const float* __restrict__ partials, O* __restrict__ y, int64_t n, int splits) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int p = 0; p < splits; ++p) s += partials[p * n + i];
  store_from_float(y + i, s);
}

DRYFT_API int dryft_sum_partials(const float* partials, void* y, int64_t n, int splits, int out_f32,
                                 hipStream_t stream) {
  if (n <= 0) return 0;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (out_f32)
    hipLaunchKernelGGL(sum_partials_kernel<float>, grid, block, 0, stream, partials, (float*)y, n, splits);
  else
    hipLaunchKernelGGL(sum_partials_kernel<bf16_t>, grid, block, 0, stream, partials, (bf16_t*)y, n, splits);
  return DRYFT_LAUNCH_CHECK();
}
