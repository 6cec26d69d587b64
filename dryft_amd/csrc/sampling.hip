// Choosing the next token from float logits, one workgroup per row.
//  * greedy: the largest logit, the lowest index among equals (reference: logits.argmax at
//    engine/dryft_qwen3/model.py:187, 262; tie rule AGENTS.md:174-175).
//  * temperature: p = softmax(logits / T); the token is the first index whose running sum of p
//    reaches u * sum(p), u in [0,1) given per row by the caller. The reference has no temperature
//    sampling; this is this library's own.
#include "common.h"
#include "sampling.h"
#include <mutex>
#include <stdio.h>

#define SAMPLE_THREADS 1024

__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_rows_kernel(const float* __restrict__ logits, int vocab,
                                                                     int64_t row_stride, int* __restrict__ out) {
  __shared__ float best_v[SAMPLE_THREADS / WAVE];
  __shared__ int best_i[SAMPLE_THREADS / WAVE];
  const float* row = logits + blockIdx.x * row_stride;
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float x = row[i];
    if (x > v || (x == v && i < idx)) {  // a NaN never wins a comparison
      v = x;
      idx = i;
    }
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, WAVE);
    const int oi = __shfl_xor(idx, o, WAVE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  if (lane == 0) { best_v[wave] = v; best_i[wave] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SAMPLE_THREADS / WAVE; ++w)
      if (best_v[w] > v || (best_v[w] == v && best_i[w] < idx)) { v = best_v[w]; idx = best_i[w]; }
    out[blockIdx.x] = idx < vocab ? idx : 0;
  }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits, int vocab,
                                                                     int64_t row_stride, float inv_temperature,
                                                                     const float* __restrict__ uniforms,
                                                                     int* __restrict__ out) {
  __shared__ float scratch[16];
  __shared__ float seg_sum[SAMPLE_THREADS];
  __shared__ int chosen;
  const float* row = logits + blockIdx.x * row_stride;
  const int tid = threadIdx.x;
  float mx = -INFINITY;
  for (int i = tid; i < vocab; i += blockDim.x) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, scratch);
  // each thread owns one contiguous segment, so that running sums follow the index order
  const int seg = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int i0 = min(vocab, tid * seg), i1 = min(vocab, i0 + seg);
  float s = 0.f;
  for (int i = i0; i < i1; ++i) s += expf((row[i] - mx) * inv_temperature);
  seg_sum[tid] = s;
  if (tid == 0) chosen = vocab - 1;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int t = 0; t < SAMPLE_THREADS; ++t) total += seg_sum[t];
    const float target = uniforms[blockIdx.x] * total;
    float run = 0.f;
    int t = 0;
    for (; t < SAMPLE_THREADS - 1; ++t) {
      if (run + seg_sum[t] > target) break;
      run += seg_sum[t];
    }
    // walk the segment that holds the target
    const int a = min(vocab, t * seg), b = min(vocab, a + seg);
    int pick = -1;
    for (int i = a; i < b; ++i) {
      run += expf((row[i] - mx) * inv_temperature);
      if (run > target) { pick = i; break; }
    }
    if (pick < 0) {  // rounding left the target just beyond the sum: take the last token with weight
      pick = vocab - 1;
      while (pick > 0 && !(expf((row[pick] - mx) * inv_temperature) > 0.f)) --pick;
    }
    chosen = pick;
  }
  __syncthreads();
  if (tid == 0) out[blockIdx.x] = chosen;
}

// Greedy choice in two stages for wide rows: `chunks` workgroups per row each find the best of their
// stretch, then one wave per row picks among them (lower index wins on equal values in both stages).
__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, int vocab,
                                                            int64_t row_stride, int chunks, float* __restrict__ best_v,
                                                            int* __restrict__ best_i) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int row = blockIdx.x, chunk = blockIdx.y;
  const int per = (vocab + chunks - 1) / chunks;
  const int i0 = chunk * per, i1 = min(vocab, i0 + per);
  const float* r = logits + row * row_stride;
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) {
    const float x = r[i];
    if (x > v || (x == v && i < idx)) { v = x; idx = i; }
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, WAVE);
    const int oi = __shfl_xor(idx, o, WAVE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  if (lane == 0) { sv[wave] = v; si[wave] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (sv[w] > v || (sv[w] == v && si[w] < idx)) { v = sv[w]; idx = si[w]; }
    best_v[row * chunks + chunk] = v;
    best_i[row * chunks + chunk] = idx;
  }
}

__global__ __launch_bounds__(64) void argmax_pick_kernel(const float* __restrict__ best_v, const int* __restrict__ best_i,
                                                         int chunks, int vocab, int* __restrict__ out) {
  const int row = blockIdx.x;
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += WAVE) {
    const float x = best_v[row * chunks + c];
    const int i = best_i[row * chunks + c];
    if (x > v || (x == v && i < idx)) { v = x; idx = i; }
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, WAVE);
    const int oi = __shfl_xor(idx, o, WAVE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
  if (threadIdx.x == 0) out[row] = idx < vocab ? idx : 0;
}

// Temperature sampling in two stages for wide rows. Stage one: `chunks` workgroups per row each find the maximum
// of their stretch and the sum of exp((x - max) / T) over it. Stage two, one workgroup per row: the stretches'
// sums, brought to the row's maximum, are added in index order until the stretch that holds u * total is found;
// that stretch is then walked in index order, each thread summing a run of its own and one thread finishing
// inside the run that holds the target. The token is the first index whose running sum exceeds the target, as
// in the one-stage kernel; the sums are added in another order, so a draw within rounding of a boundary between
// two tokens may fall on the other side.
#define PICK_THREADS 256

__global__ __launch_bounds__(256) void sample_chunks_kernel(const float* __restrict__ logits, int vocab,
                                                            int64_t row_stride, int chunks, float inv_temperature,
                                                            float* __restrict__ chunk_max, float* __restrict__ chunk_sum) {
  __shared__ float scratch[16];
  const int row = blockIdx.x, chunk = blockIdx.y;
  const int per = (vocab + chunks - 1) / chunks;
  const int i0 = min(vocab, chunk * per), i1 = min(vocab, i0 + per);
  const float* r = logits + row * row_stride;
  float mx = -INFINITY;
  for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) mx = fmaxf(mx, r[i]);
  mx = block_max(mx, scratch);
  float s = 0.f;
  if (mx > -INFINITY)
    for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) s += expf((r[i] - mx) * inv_temperature);
  s = block_sum(s, scratch);
  if (threadIdx.x == 0) {
    chunk_max[row * chunks + chunk] = mx;
    chunk_sum[row * chunks + chunk] = s;
  }
}

__global__ __launch_bounds__(PICK_THREADS) void sample_pick_kernel(const float* __restrict__ logits, int vocab,
                                                                   int64_t row_stride, int chunks, float inv_temperature,
                                                                   const float* __restrict__ chunk_max,
                                                                   const float* __restrict__ chunk_sum,
                                                                   const float* __restrict__ uniforms,
                                                                   int* __restrict__ out) {
  __shared__ float scratch[16];
  __shared__ float weight[PICK_THREADS];                   // of a stretch, later of a thread's run
  __shared__ float s_target, s_before;
  __shared__ int s_chunk, s_thread;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* r = logits + row * row_stride;
  // chunks <= PICK_THREADS: one stretch per thread
  const float cm = tid < chunks ? chunk_max[row * chunks + tid] : -INFINITY;
  const float mx = block_max(cm, scratch);
  weight[tid] = tid < chunks && cm > -INFINITY ? chunk_sum[row * chunks + tid] * expf((cm - mx) * inv_temperature) : 0.f;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int c = 0; c < chunks; ++c) total += weight[c];
    const float target = uniforms[row] * total;
    float run = 0.f;
    int c = 0;
    for (; c < chunks - 1; ++c) {
      if (run + weight[c] > target) break;
      run += weight[c];
    }
    s_target = target;
    s_before = run;
    s_chunk = c;
  }
  __syncthreads();
  const int per = (vocab + chunks - 1) / chunks;
  const int i0 = min(vocab, s_chunk * per), i1 = min(vocab, i0 + per);
  const int run_len = (per + PICK_THREADS - 1) / PICK_THREADS;
  const int a = min(i1, i0 + tid * run_len), b = min(i1, a + run_len);
  float mine = 0.f;
  for (int i = a; i < b; ++i) mine += expf((r[i] - mx) * inv_temperature);
  __syncthreads();                                         // the stretches' weights have been read
  weight[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float run = s_before;
    int t = 0;
    for (; t < PICK_THREADS - 1; ++t) {
      if (run + weight[t] > s_target) break;
      run += weight[t];
    }
    s_before = run;
    s_thread = t;
  }
  __syncthreads();
  if (tid != s_thread) return;
  float run = s_before;
  int pick = -1;
  for (int i = a; i < b; ++i) {
    run += expf((r[i] - mx) * inv_temperature);
    if (run > s_target) { pick = i; break; }
  }
  if (pick < 0) {  // rounding left the target just beyond the sums: the last token with weight, from here down
    pick = max((b > a ? b : i1) - 1, 0);
    while (pick > 0 && !(expf((r[pick] - mx) * inv_temperature) > 0.f)) --pick;
  }
  out[row] = pick;
}

// scratch_v / scratch_i: room for n_rows * chunks entries each when chunks > 1
DRYFT_API int dryft_argmax_rows(const float* logits, int n_rows, int vocab, int64_t row_stride, int* out, int chunks,
                                float* scratch_v, int* scratch_i, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (chunks <= 1) {
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, vocab, row_stride, out);
    return DRYFT_LAUNCH_CHECK();
  }
  if (chunks > 65535 || scratch_v == nullptr || scratch_i == nullptr) return -1;
  hipLaunchKernelGGL(argmax_chunks_kernel, dim3(n_rows, chunks), dim3(256), 0, stream, logits, vocab, row_stride, chunks,
                     scratch_v, scratch_i);
  int rc = DRYFT_LAUNCH_CHECK();
  if (rc) return rc;
  hipLaunchKernelGGL(argmax_pick_kernel, dim3(n_rows), dim3(64), 0, stream, scratch_v, scratch_i, chunks, vocab, out);
  return DRYFT_LAUNCH_CHECK();
}

// chunk_max / chunk_sum: room for n_rows * chunks floats each when chunks > 1 (chunks <= 256)
DRYFT_API int dryft_sample_rows(const float* logits, int n_rows, int vocab, int64_t row_stride, float temperature,
                                const float* uniforms, int* out, int chunks, float* chunk_max, float* chunk_sum,
                                hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!(temperature > 0.f) || vocab <= 0) return -1;
  if (chunks <= 1) {
    hipLaunchKernelGGL(sample_rows_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, vocab, row_stride,
                       1.f / temperature, uniforms, out);
    return DRYFT_LAUNCH_CHECK();
  }
  if (chunks > PICK_THREADS || chunk_max == nullptr || chunk_sum == nullptr) return -1;
  hipLaunchKernelGGL(sample_chunks_kernel, dim3(n_rows, chunks), dim3(256), 0, stream, logits, vocab, row_stride, chunks,
                     1.f / temperature, chunk_max, chunk_sum);
  int rc = DRYFT_LAUNCH_CHECK();
  if (rc) return rc;
  hipLaunchKernelGGL(sample_pick_kernel, dim3(n_rows), dim3(PICK_THREADS), 0, stream, logits, vocab, row_stride, chunks,
                     1.f / temperature, chunk_max, chunk_sum, uniforms, out);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The greedy choice with the library's own scratch memory (see sampling.h). `scratch` is a host-side stand-in
// in host code, not a device address: the address on each device is looked up once and kept, and only that
// pointer is handed to kernels.
static __device__ __align__(256) unsigned char scratch[DRYFT_ARGMAX_NOALLOC_ENTRIES * (sizeof(float) + sizeof(int))];

#define NOALLOC_MAX_DEVICES 64
static void* scratch_on_device[NOALLOC_MAX_DEVICES];   // address of `scratch` on each device, null until looked up
static std::mutex scratch_lock;

// The current device's copy of the array. Returns 0 or a HIP error code.
static int scratch_of_current_device(void** ptr) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return (int)err;
  if (device < 0 || device >= NOALLOC_MAX_DEVICES) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_on_device[device] == nullptr) {
    void* found = nullptr;
    err = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (found == nullptr) return (int)hipErrorInvalidSymbol;
    scratch_on_device[device] = found;
  }
  *ptr = scratch_on_device[device];
  return 0;
}

int dryft_argmax_rows_noalloc(const float* logits, int n_rows, int vocab, int64_t row_stride, int* out, int chunks,
                              hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (logits == nullptr || out == nullptr || vocab <= 0 || chunks > 65535) return -1;
  if (chunks <= 1) return dryft_argmax_rows(logits, n_rows, vocab, row_stride, out, 1, nullptr, nullptr, stream);
  const long long entries = (long long)n_rows * chunks;
  if (entries > DRYFT_ARGMAX_NOALLOC_ENTRIES) {
    fprintf(stderr, "dryft_argmax_rows_noalloc: %d rows x %d stretches = %lld entries exceed the library's scratch of "
                    "%d entries; use fewer stretches or rows, or dryft_argmax_rows with buffers of your own\n",
            n_rows, chunks, entries, DRYFT_ARGMAX_NOALLOC_ENTRIES);
    return -2;
  }
  void* base = nullptr;
  const int rc = scratch_of_current_device(&base);
  if (rc) return rc;
  float* best_v = (float*)base;                                   // [entries] floats, then [entries] ints
  int* best_i = (int*)((unsigned char*)base + DRYFT_ARGMAX_NOALLOC_ENTRIES * sizeof(float));
  return dryft_argmax_rows(logits, n_rows, vocab, row_stride, out, chunks, best_v, best_i, stream);
}
