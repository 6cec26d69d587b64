// Per-head RMSNorm of q and k, rotary positions, and the append to the paged cache, in one pass
// over the fused projection output (reference: engine/dryft_qwen3/kernels/rope_qknorm.py:33-99,
// model.py:165-171):
//
//   n  = T( T(x * rsqrt(mean(x^2) + eps)) * w )                 (q and k heads; v is copied)
//   o1 = T( T(n1 * cos) + T(-n2 * sin) ),  o2 = T( T(n2 * cos) + T(n1 * sin) )
//
// for the pair (j, j + rot/2), j < rot/2 ("rotate half"); lanes at or above `rot` pass through.
// cos/sin tables are [positions, rot/2] in the activation dtype. Row r belongs to cache slot
// row_slot[r] (-1: the row takes no part) at position row_pos[r]. Keys go to
// k_pages[page, kv_head, pos % 64, :], values transposed to v_pages[page, kv_head, :, pos % 64],
// so that both matrix products of attention read 16-byte runs along their contraction index.
#include "common.h"

#define MAX_HEAD_DIM 512

// Eight values of the projection's output at element `at`: from the output itself, or, where the product was left as
// `parts` float partial sums (each `part_stride` elements after the other, `qkv` pointing at the first), their sum
// rounded as the output would have been.
template <typename T>
__device__ __forceinline__ void load8_projected(const T* __restrict__ qkv, int64_t at, int parts, int64_t part_stride,
                                                float (&v)[8]) {
  if (parts == 0) {
    load8_as_float(qkv + at, v);
    return;
  }
  const float* f = (const float*)qkv + at;
  load8_as_float(f, v);
  for (int s = 1; s < parts; ++s) {
    float more[8];
    load8_as_float(f + s * part_stride, more);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] += more[j];
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = rounded_as<T>(v[j]);
}

template <typename T>
__global__ void qk_norm_rope_kv_kernel(const T* __restrict__ qkv, int64_t qkv_stride, const void* __restrict__ q_w,
                                       const void* __restrict__ k_w, int w_f32, int has_norm, float eps,
                                       const T* __restrict__ cos_t, const T* __restrict__ sin_t, int rot,
                                       const int* __restrict__ row_slot, const int* __restrict__ row_pos,
                                       T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                       const int* __restrict__ page_table, int max_pages, int write_kv, int n_heads,
                                       int n_kv, int head_dim, int skip_v, int first_job) {
  __shared__ float normed[4][MAX_HEAD_DIM];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int64_t row = blockIdx.x;
  const int job = first_job + blockIdx.y * 4 + wave;  // [0,nH): q heads; [nH,nH+nKV): k heads; then v heads
  if (job >= n_heads + (skip_v ? 1 : 2) * n_kv) return;
  const int slot = row_slot[row];
  const int pos = row_pos[row];
  const bool is_q = job < n_heads, is_k = !is_q && job < n_heads + n_kv;
  const T* src = qkv + row * qkv_stride + (int64_t)job * head_dim;
  if (is_q && q_out == nullptr) return;                // the caller takes the queries from the projection itself
  if (is_q) {
    T* dst = q_out + (row * n_heads + job) * head_dim;
    if (slot < 0) {
      for (int i = lane; i < head_dim; i += WAVE) store_from_float(dst + i, 0.f);
      return;
    }
  } else if (slot < 0 || !write_kv) {
    return;
  }
  int page = 0, in_page = 0;
  if (!is_q) {
    page = page_of(page_table, max_pages, slot, pos);
    in_page = pos % PAGE_TOKENS;
    if (page < 0) return;  // no page: the host reserves one before the step; never write through a bad index
  }
  if (!is_q && !is_k) {
    const int kvh = job - n_heads - n_kv;
    T* dst = v_pages + ((int64_t)page * n_kv + kvh) * head_dim * PAGE_TOKENS + value_column(in_page);
    for (int i = lane; i < head_dim; i += WAVE) dst[(int64_t)i * PAGE_TOKENS] = src[i];
    return;
  }
  // q or k head: norm, then rotation through LDS (a pair's halves may sit in different lanes)
  float ss = 0.f;
  for (int i = lane; i < head_dim; i += WAVE) {
    const float x = load_as_float(src + i);
    normed[wave][i] = x;
    ss += x * x;
  }
  if (has_norm) {
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / (float)head_dim + eps);
    const void* w = is_q ? q_w : k_w;
    for (int i = lane; i < head_dim; i += WAVE)
      normed[wave][i] = rounded_as<T>(rounded_as<T>(normed[wave][i] * inv) * load_vector(w, i, w_f32));
  }
  // the wave's own LDS writes must be visible to its other lanes before the pairs are read
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  __builtin_amdgcn_wave_barrier();
  T* dst = is_q ? q_out + (row * n_heads + job) * head_dim
                : k_pages + (((int64_t)page * n_kv + (job - n_heads)) * PAGE_TOKENS + in_page) * head_dim;
  const int half = rot / 2;
  for (int i = lane; i < head_dim; i += WAVE) {
    float o = normed[wave][i];
    if (i < rot) {
      const int j = i < half ? i : i - half;
      const float c = load_as_float(cos_t + (int64_t)pos * half + j);
      const float s = load_as_float(sin_t + (int64_t)pos * half + j);
      const float other = normed[wave][i < half ? i + half : i - half];
      // first half: x1*c - x2*s ; second half: x2*c + x1*s
      const float a = rounded_as<T>(o * c);
      const float b = rounded_as<T>(other * s);
      o = i < half ? a - b : a + b;
    }
    store_from_float(dst + i, o);
  }
}

// The same for head widths of 32, 64, 128 or 256 rotated over their full width: a head is spread over
// head_dim / 8 lanes that hold 8 contiguous values each, moved with 16-byte loads and stores; the sum of squares
// and the exchange with the rotation partner (the lane head_dim / 16 away) go through lane shuffles. Value
// heads are not handled here.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_vec_kernel(const T* __restrict__ qkv, int64_t qkv_stride,
                                                               const void* __restrict__ q_w, const void* __restrict__ k_w,
                                                               int w_f32, int has_norm, float eps,
                                                               const T* __restrict__ cos_t, const T* __restrict__ sin_t,
                                                               const int* __restrict__ row_slot,
                                                               const int* __restrict__ row_pos, T* __restrict__ q_out,
                                                               T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                               const int* __restrict__ page_table, int max_pages,
                                                               int write_kv, int with_v, int n_heads, int n_kv,
                                                               int head_dim) {
  const int lph = head_dim / 8;                        // lanes per head: 4, 8, 16 or 32
  const int64_t row = blockIdx.x;
  const int job = blockIdx.y * (256 / lph) + threadIdx.x / lph;
  const int part = threadIdx.x % lph;
  const int jobs = n_heads + (write_kv ? (with_v ? 2 : 1) * n_kv : 0);   // q heads, k heads, then v heads
  // lanes of a dead job still take part in the shuffles; without q_out the query heads are dead jobs
  const bool live_job = job < jobs && (q_out != nullptr || job >= n_heads);
  const bool is_v = job >= n_heads + n_kv;
  const int slot = row_slot[row], pos = row_pos[row];
  const bool is_q = job < n_heads;
  float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (live_job && slot >= 0) load8_as_float(qkv + row * qkv_stride + (int64_t)job * head_dim + 8 * part, v);
  if (has_norm) {                                      // (value heads run through it too; their result is not used)
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
    for (int o = lph / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);
    const float inv = rsqrtf(ss / (float)head_dim + eps);
    const void* w = is_q ? q_w : k_w;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      v[j] = rounded_as<T>(rounded_as<T>(v[j] * inv) * (live_job ? load_vector(w, 8 * part + j, w_f32) : 0.f));
  }
  float other[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) other[j] = __shfl_xor(v[j], lph / 2, WAVE);
  if (!live_job) return;
  if (is_v) {                                          // copied as it is, transposed into its page
    if (slot < 0) return;
    const int page = page_of(page_table, max_pages, slot, pos);
    if (page < 0) return;
    T* vd = v_pages + (((int64_t)page * n_kv + (job - n_heads - n_kv)) * head_dim + 8 * part) * PAGE_TOKENS +
            value_column(pos % PAGE_TOKENS);
    const T* vs = qkv + row * qkv_stride + (int64_t)job * head_dim + 8 * part;
#pragma unroll
    for (int j = 0; j < 8; ++j) vd[(int64_t)j * PAGE_TOKENS] = vs[j];
    return;
  }
  T* dst;
  if (is_q) {
    dst = q_out + (row * n_heads + job) * head_dim + 8 * part;
    if (slot < 0) {
      const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      store8_from_float(dst, z);
      return;
    }
  } else {
    if (slot < 0) return;
    const int page = page_of(page_table, max_pages, slot, pos);
    if (page < 0) return;
    dst = k_pages + (((int64_t)page * n_kv + (job - n_heads)) * PAGE_TOKENS + pos % PAGE_TOKENS) * head_dim + 8 * part;
  }
  const int half_lanes = lph / 2;
  const bool first = part < half_lanes;
  float c[8], sn[8];
  const int64_t at = (int64_t)pos * (head_dim / 2) + 8 * (first ? part : part - half_lanes);
  load8_as_float(cos_t + at, c);
  load8_as_float(sin_t + at, sn);
  float o[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float a = rounded_as<T>(v[j] * c[j]), b = rounded_as<T>(other[j] * sn[j]);
    o[j] = first ? a - b : a + b;                       // x1*c - x2*s ; x2*c + x1*s
  }
  store8_from_float(dst, o);
}

// The same for steps of many rows: one workgroup per row. A thread keeps the rotation factors and norm weights
// of its 8 features, which are the same for every head, and walks over the row's q and k heads four at a time,
// so that it issues about a quarter of the loads per head of the kernel above. Value heads are not handled here.
template <typename T, int LPH>   // lanes per head: head_dim / 8
__device__ __forceinline__ void qk_norm_rope_row(int64_t row, const T* __restrict__ qkv, int64_t qkv_stride,
                                                 const void* __restrict__ q_w, const void* __restrict__ k_w, int w_f32,
                                                 int has_norm, float eps, const T* __restrict__ cos_t,
                                                 const T* __restrict__ sin_t, const int* __restrict__ row_slot,
                                                 const int* __restrict__ row_pos, T* __restrict__ q_out,
                                                 T* __restrict__ k_pages, const int* __restrict__ page_table,
                                                 int max_pages, int write_kv, int n_heads, int n_kv, int parts,
                                                 int64_t part_stride) {
  constexpr int D = 8 * LPH, PER = 256 / LPH;           // heads a workgroup handles side by side
  const int part = threadIdx.x % LPH, lane_head = threadIdx.x / LPH;
  const int slot = row_slot[row], pos = row_pos[row];
  if (slot < 0) {                                       // a dead row: its q is zero, nothing is cached
    const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (q_out != nullptr)
      for (int job = lane_head; job < n_heads; job += PER) store8_from_float(q_out + (row * n_heads + job) * D + 8 * part, z);
    return;
  }
  const bool first = part < LPH / 2;
  const int64_t at = (int64_t)pos * (D / 2) + 8 * (first ? part : part - LPH / 2);
  float c[8], sn[8], wq[8], wk[8];
  load8_as_float(cos_t + at, c);
  load8_as_float(sin_t + at, sn);
  if (has_norm) {
    if (w_f32) {
      load8_as_float((const float*)q_w + 8 * part, wq);
      load8_as_float((const float*)k_w + 8 * part, wk);
    } else {
      load8_as_float((const bf16_t*)q_w + 8 * part, wq);
      load8_as_float((const bf16_t*)k_w + 8 * part, wk);
    }
  }
  const int page = write_kv ? page_of(page_table, max_pages, slot, pos) : -1;
  const int jobs = n_heads + (page >= 0 ? n_kv : 0);    // q heads, then k heads
  const int64_t src = row * qkv_stride + 8 * part;
  for (int j0 = (q_out != nullptr ? 0 : n_heads) + lane_head; j0 < jobs; j0 += 4 * PER) {   // without q_out: keys only
    float v[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (j0 + u * PER < jobs) load8_projected(qkv, src + (int64_t)(j0 + u * PER) * D, parts, part_stride, v[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int job = j0 + u * PER;                      // the same for the LPH lanes that share a head
      if (job >= jobs) continue;
      const bool is_q = job < n_heads;
      if (has_norm) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += v[u][j] * v[u][j];
#pragma unroll
        for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);
        const float inv = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[u][j] = rounded_as<T>(rounded_as<T>(v[u][j] * inv) * (is_q ? wq[j] : wk[j]));
      }
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float other = __shfl_xor(v[u][j], LPH / 2, WAVE);
        const float a = rounded_as<T>(v[u][j] * c[j]), b = rounded_as<T>(other * sn[j]);
        o[j] = first ? a - b : a + b;                    // x1*c - x2*s ; x2*c + x1*s
      }
      T* dst = is_q ? q_out + (row * n_heads + job) * D + 8 * part
                    : k_pages + (((int64_t)page * n_kv + (job - n_heads)) * PAGE_TOKENS + pos % PAGE_TOKENS) * D + 8 * part;
      store8_from_float(dst, o);
    }
  }
}

// Values of a step with many rows: a workgroup takes 64 consecutive rows of one kv head and turns the tile in
// LDS. Where 32 consecutive rows are one aligned block of 32 positions of one page (the usual case in a long
// prompt), a thread writes 8 columns of a feature's row with one 16-byte store: they are two runs of four
// consecutive positions (see value_column). Otherwise values go one by one. (The per-row kernel above writes a
// row's values 128 bytes apart.) head_dim must be a multiple of 8.
#define V_TILE_ROWS 64
#define V_TILE_LD (V_TILE_ROWS + 8)
extern __shared__ __attribute__((aligned(16))) unsigned char v_tile_raw[];

template <typename T>
__device__ __forceinline__ void v_tile_write(int tile_index, int kvh, const T* __restrict__ qkv, int64_t qkv_stride,
                                             int v_col0, const int* __restrict__ row_slot,
                                             const int* __restrict__ row_pos, T* __restrict__ v_pages,
                                             const int* __restrict__ page_table, int max_pages, int n_rows, int n_kv,
                                             int head_dim, int parts, int64_t part_stride) {
  __shared__ int64_t base[V_TILE_ROWS];                     // start of the row's page for this kv head, or -1
  __shared__ int in_page[V_TILE_ROWS];                      // the row's position within its page
  __shared__ int block_ok[V_TILE_ROWS / 32];
  T* tile = (T*)v_tile_raw;                                 // [head_dim][V_TILE_LD]: already transposed
  const int r0 = tile_index * V_TILE_ROWS;
  const int rows = min(V_TILE_ROWS, n_rows - r0);
  const int chunks = head_dim / 8;
  for (int e = threadIdx.x; e < V_TILE_ROWS * chunks; e += blockDim.x) {
    const int t = e / chunks, ch = e % chunks;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (t < rows) load8_projected(qkv, (int64_t)(r0 + t) * qkv_stride + v_col0 + kvh * head_dim + 8 * ch, parts, part_stride, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) store_from_float(tile + (8 * ch + j) * V_TILE_LD + t, v[j]);
  }
  if (threadIdx.x < V_TILE_ROWS) {
    int64_t where = -1;
    int at = 0;
    if ((int)threadIdx.x < rows) {
      const int slot = row_slot[r0 + threadIdx.x], pos = row_pos[r0 + threadIdx.x];
      if (slot >= 0) {
        const int page = page_of(page_table, max_pages, slot, pos);
        if (page >= 0) where = ((int64_t)page * n_kv + kvh) * head_dim * PAGE_TOKENS;
        at = pos % PAGE_TOKENS;
      }
    }
    base[threadIdx.x] = where;
    in_page[threadIdx.x] = at;
  }
  __syncthreads();
  if (threadIdx.x < V_TILE_ROWS / 32) {                     // is this block of 32 rows one aligned block of a page?
    const int t0 = 32 * threadIdx.x;
    bool ok = base[t0] >= 0 && in_page[t0] % 32 == 0;
    for (int j = 1; j < 32; ++j) ok = ok && base[t0 + j] == base[t0] && in_page[t0 + j] == in_page[t0] + j;
    block_ok[threadIdx.x] = ok;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < head_dim * (V_TILE_ROWS / 8); e += blockDim.x) {
    const int d = e / (V_TILE_ROWS / 8), piece = e % (V_TILE_ROWS / 8);   // 8 columns of feature d
    const int blk = piece / 4, g = piece % 4, t0 = 32 * blk;
    if (block_ok[blk]) {
      const T* src = tile + d * V_TILE_LD + t0 + 4 * g;     // positions 4g.. and 16+4g.. of the block
      float v[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = load_as_float(src + i);
        v[4 + i] = load_as_float(src + 16 + i);
      }
      store8_from_float(v_pages + base[t0] + (int64_t)d * PAGE_TOKENS + in_page[t0] + 8 * g, v);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int t = t0 + 8 * g + j;
        if (base[t] >= 0) v_pages[base[t] + (int64_t)d * PAGE_TOKENS + value_column(in_page[t])] = tile[d * V_TILE_LD + t];
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void v_tile_write_kernel(const T* __restrict__ qkv, int64_t qkv_stride, int v_col0,
                                                           const int* __restrict__ row_slot,
                                                           const int* __restrict__ row_pos, T* __restrict__ v_pages,
                                                           const int* __restrict__ page_table, int max_pages,
                                                           int n_rows, int n_kv, int head_dim) {
  v_tile_write<T>(blockIdx.x, blockIdx.y, qkv, qkv_stride, v_col0, row_slot, row_pos, v_pages, page_table, max_pages,
                  n_rows, n_kv, head_dim, 0, 0);
}

// One launch for a step of many rows: the first workgroups turn the tiles of values (few, and waiting on memory
// most of their time), the others take a row each for q and k; both read the same projection output.
template <typename T, int LPH>
__global__ __launch_bounds__(256) void rows_to_cache_kernel(const T* __restrict__ qkv, int64_t qkv_stride,
                                                            const void* __restrict__ q_w, const void* __restrict__ k_w,
                                                            int w_f32, int has_norm, float eps,
                                                            const T* __restrict__ cos_t, const T* __restrict__ sin_t,
                                                            const int* __restrict__ row_slot,
                                                            const int* __restrict__ row_pos, T* __restrict__ q_out,
                                                            T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                            const int* __restrict__ page_table, int max_pages,
                                                            int write_kv, int n_rows, int n_heads, int n_kv, int v_tiles,
                                                            int parts, int64_t part_stride) {
  const int v_blocks = v_tiles * n_kv;                      // none when nothing is cached
  if ((int)blockIdx.x < v_blocks) {
    v_tile_write<T>(blockIdx.x % v_tiles, blockIdx.x / v_tiles, qkv, qkv_stride, (n_heads + n_kv) * 8 * LPH, row_slot,
                    row_pos, v_pages, page_table, max_pages, n_rows, n_kv, 8 * LPH, parts, part_stride);
    return;
  }
  qk_norm_rope_row<T, LPH>((int64_t)blockIdx.x - v_blocks, qkv, qkv_stride, q_w, k_w, w_f32, has_norm, eps, cos_t, sin_t,
                           row_slot, row_pos, q_out, k_pages, page_table, max_pages, write_kv, n_heads, n_kv, parts,
                           part_stride);
}

template <typename T>
static int launch_rows_to_cache(const void* qkv, int64_t qkv_stride, const void* q_w, const void* k_w, int w_f32,
                                int has_norm, float eps, const void* cos_t, const void* sin_t, const int* row_slot,
                                const int* row_pos, void* q_out, void* k_pages, void* v_pages, const int* page_table,
                                int max_pages, int write_kv, int n_rows, int n_heads, int n_kv, int head_dim,
                                hipStream_t stream, int parts = 0, int64_t part_stride = 0) {
  const int v_tiles = write_kv ? (n_rows + V_TILE_ROWS - 1) / V_TILE_ROWS : 0;
  const size_t lds = (size_t)head_dim * V_TILE_LD * sizeof(T);
#define ROWS(LPHV)                                                                                                     \
  {                                                                                                                    \
    auto kernel = rows_to_cache_kernel<T, LPHV>;                                                                       \
    if (lds > 64 * 1024 &&                                                                                             \
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)  \
      return -2;                                                                                                       \
    hipLaunchKernelGGL(kernel, dim3(v_tiles * n_kv + n_rows), dim3(256), lds, stream, (const T*)qkv, qkv_stride, q_w,  \
                       k_w, w_f32, has_norm, eps, (const T*)cos_t, (const T*)sin_t, row_slot, row_pos, (T*)q_out,       \
                       (T*)k_pages, (T*)v_pages, page_table, max_pages, write_kv, n_rows, n_heads, n_kv, v_tiles,       \
                       parts, part_stride);                                                                            \
  }
  switch (head_dim) {
    case 32: ROWS(4); break;
    case 64: ROWS(8); break;
    case 128: ROWS(16); break;
    default: ROWS(32); break;
  }
#undef ROWS
  return DRYFT_LAUNCH_CHECK();
}

// The many-row form of dryft_qk_norm_rope_kv below for a projection left as `parts` float partial sums
// [parts, n_rows, qkv_stride] (bfloat16 activations, weights and cache): every value is the sum of its parts rounded
// to bfloat16, then treated as there. For steps that write the cache, a full rotation and a head size of 32, 64, 128
// or 256: dryft_rows_to_cache_takes says whether a step qualifies.
DRYFT_API int dryft_rows_to_cache_takes(int n_rows, int head_dim, int rot, int write_kv) {
  return write_kv && n_rows >= 1 && rot == head_dim && (head_dim == 32 || head_dim == 64 || head_dim == 128 || head_dim == 256);
}

DRYFT_API int dryft_rows_to_cache_parts(const float* qkv_parts, int parts, int64_t qkv_stride, const void* q_w,
                                        const void* k_w, int w_f32, int has_norm, float eps, const void* cos_t,
                                        const void* sin_t, int rot, const int* row_slot, const int* row_pos, void* q_out,
                                        void* k_pages, void* v_pages, const int* page_table, int max_pages, int n_rows,
                                        int n_heads, int n_kv, int head_dim, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (parts < 1 || !dryft_rows_to_cache_takes(n_rows, head_dim, rot, 1)) return -1;
  if ((((uintptr_t)qkv_parts | (uintptr_t)q_out | (uintptr_t)k_pages | (uintptr_t)v_pages | (uintptr_t)cos_t |
        (uintptr_t)sin_t) & 15) || qkv_stride % 8)
    return -1;
  return launch_rows_to_cache<bf16_t>(qkv_parts, qkv_stride, q_w, k_w, w_f32, has_norm, eps, cos_t, sin_t, row_slot,
                                      row_pos, q_out, k_pages, v_pages, page_table, max_pages, 1, n_rows, n_heads, n_kv,
                                      head_dim, stream, parts, (int64_t)n_rows * qkv_stride);
}

DRYFT_API int dryft_qk_norm_rope_kv(const void* qkv, int64_t qkv_stride, const void* q_w, const void* k_w, int w_f32,
                                    int has_norm, float eps, const void* cos_t, const void* sin_t, int rot,
                                    const int* row_slot, const int* row_pos, void* q_out, void* k_pages,
                                    void* v_pages, const int* page_table, int max_pages, int write_kv, int n_rows,
                                    int n_heads, int n_kv, int head_dim, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (head_dim > MAX_HEAD_DIM || rot > head_dim || (rot & 1)) return -1;
  const bool aligned = (((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_pages | (uintptr_t)v_pages |
                         (uintptr_t)cos_t | (uintptr_t)sin_t) & 15) == 0 && qkv_stride % 8 == 0;
  // many rows: the values go through the tile kernel
  const int skip_v = (write_kv && n_rows >= 32 && head_dim % 8 == 0 && aligned) ? 1 : 0;
  const bool vec = aligned && rot == head_dim && (head_dim == 32 || head_dim == 64 || head_dim == 128 || head_dim == 256);
  if (vec && skip_v && n_rows >= 64) {                  // many rows: a workgroup per row, and the values' tiles beside
    return is_f32 ? launch_rows_to_cache<float>(qkv, qkv_stride, q_w, k_w, w_f32, has_norm, eps, cos_t, sin_t, row_slot,
                                                row_pos, q_out, k_pages, v_pages, page_table, max_pages, write_kv, n_rows,
                                                n_heads, n_kv, head_dim, stream)
                  : launch_rows_to_cache<bf16_t>(qkv, qkv_stride, q_w, k_w, w_f32, has_norm, eps, cos_t, sin_t, row_slot,
                                                 row_pos, q_out, k_pages, v_pages, page_table, max_pages, write_kv, n_rows,
                                                 n_heads, n_kv, head_dim, stream);
  } else if (vec) {
    const int lph = head_dim / 8, per_block = 256 / lph;
    const int with_v = (write_kv && !skip_v) ? 1 : 0;
    const int qk_jobs = n_heads + (write_kv ? (with_v ? 2 : 1) * n_kv : 0);
    dim3 qgrid(n_rows, (qk_jobs + per_block - 1) / per_block);
    if (is_f32)
      hipLaunchKernelGGL(qk_norm_rope_vec_kernel<float>, qgrid, dim3(256), 0, stream, (const float*)qkv, qkv_stride, q_w,
                         k_w, w_f32, has_norm, eps, (const float*)cos_t, (const float*)sin_t, row_slot, row_pos,
                         (float*)q_out, (float*)k_pages, (float*)v_pages, page_table, max_pages, write_kv, with_v, n_heads, n_kv,
                         head_dim);
    else
      hipLaunchKernelGGL(qk_norm_rope_vec_kernel<bf16_t>, qgrid, dim3(256), 0, stream, (const bf16_t*)qkv, qkv_stride,
                         q_w, k_w, w_f32, has_norm, eps, (const bf16_t*)cos_t, (const bf16_t*)sin_t, row_slot, row_pos,
                         (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, page_table, max_pages, write_kv, with_v, n_heads,
                         n_kv, head_dim);
    int rc = DRYFT_LAUNCH_CHECK();
    if (rc) return rc;
  }
  // the per-row kernel takes everything when the vector kernel does not apply
  const int first_job = 0;
  const int jobs = n_heads + (skip_v ? 1 : 2) * n_kv;
  if (!vec) {
  dim3 grid(n_rows, (jobs - first_job + 3) / 4), block(256);
  if (is_f32)
    hipLaunchKernelGGL(qk_norm_rope_kv_kernel<float>, grid, block, 0, stream, (const float*)qkv, qkv_stride, q_w, k_w,
                       w_f32, has_norm, eps, (const float*)cos_t, (const float*)sin_t, rot, row_slot, row_pos,
                       (float*)q_out, (float*)k_pages, (float*)v_pages, page_table, max_pages, write_kv, n_heads, n_kv,
                       head_dim, skip_v, first_job);
  else
    hipLaunchKernelGGL(qk_norm_rope_kv_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)qkv, qkv_stride, q_w,
                       k_w, w_f32, has_norm, eps, (const bf16_t*)cos_t, (const bf16_t*)sin_t, rot, row_slot, row_pos,
                       (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, page_table, max_pages, write_kv, n_heads,
                       n_kv, head_dim, skip_v, first_job);
  }
  int rc = DRYFT_LAUNCH_CHECK();
  if (rc || !skip_v) return rc;
  dim3 vgrid((n_rows + V_TILE_ROWS - 1) / V_TILE_ROWS, n_kv);
  const int v_col0 = (n_heads + n_kv) * head_dim;
  if (is_f32)
    hipLaunchKernelGGL(v_tile_write_kernel<float>, vgrid, dim3(256), head_dim * V_TILE_LD * 4, stream,
                       (const float*)qkv, qkv_stride, v_col0, row_slot, row_pos, (float*)v_pages, page_table, max_pages,
                       n_rows, n_kv, head_dim);
  else
    hipLaunchKernelGGL(v_tile_write_kernel<bf16_t>, vgrid, dim3(256), head_dim * V_TILE_LD * 2, stream,
                       (const bf16_t*)qkv, qkv_stride, v_col0, row_slot, row_pos, (bf16_t*)v_pages, page_table,
                       max_pages, n_rows, n_kv, head_dim);
  return DRYFT_LAUNCH_CHECK();
}
