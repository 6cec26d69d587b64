// Causal grouped-query attention over the paged cache, one workgroup per (row, query head), with
// float arithmetic throughout. It serves the float32 path of the model and, in bfloat16, head
// sizes the matrix-core kernels do not take. Formula (reference: engine/dryft_qwen3/model.py:172-177,
// 254-257; kernels/attn_decode.py:180-196):
//
//   s[j] = (q . k[j]) * scale  for  lo <= j <= pos,   p = softmax(s),   o = sum_j p[j] v[j]
//
// with lo = 0, or pos - window + 1 for a windowed mixer; query head h reads kv head h / group.
// Probabilities are rounded to the storage dtype before they weigh the values, as the
// matrix-core kernels must (attn_decode.py:12-14, 89); with float storage that is the identity.
#include "common.h"

#define ROWS_THREADS 256
#define ROWS_MAX_HEAD_DIM 256

template <typename T>
__global__ void attn_rows_kernel(const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                                 const int* __restrict__ page_table, int max_pages, const int* __restrict__ row_slot,
                                 const int* __restrict__ row_pos, T* __restrict__ out, int n_heads, int n_kv,
                                 int head_dim, float scale, int window, int vec) {
  __shared__ float qs[ROWS_MAX_HEAD_DIM];
  __shared__ float ps[ROWS_THREADS];
  __shared__ int pages[ROWS_THREADS / PAGE_TOKENS];
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int head = blockIdx.y, tid = threadIdx.x;
  const int slot = row_slot[row];
  T* o = out + (row * n_heads + head) * head_dim;
  if (slot < 0) {
    if (tid < head_dim) store_from_float(o + tid, 0.f);
    return;
  }
  const int pos = row_pos[row];
  const int kvh = head / (n_heads / n_kv);
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  if (tid < head_dim) qs[tid] = load_as_float(q + (row * n_heads + head) * head_dim + tid);
  float m = -INFINITY, l = 0.f, acc = 0.f;
  for (int c = (lo / PAGE_TOKENS) * PAGE_TOKENS; c <= pos; c += ROWS_THREADS) {
    __syncthreads();  // qs written; previous chunk's ps and pages no longer read
    if (tid < ROWS_THREADS / PAGE_TOKENS) {
      const int p0 = c + tid * PAGE_TOKENS;
      pages[tid] = p0 <= pos ? page_of(page_table, max_pages, slot, p0) : -1;
    }
    __syncthreads();
    const int j = c + tid;
    const int page = pages[tid / PAGE_TOKENS];
    const bool seen = j >= lo && j <= pos && page >= 0;
    float s = -INFINITY;
    if (seen) {
      const T* kp = k_pages + (((int64_t)page * n_kv + kvh) * PAGE_TOKENS + j % PAGE_TOKENS) * head_dim;
      float d = 0.f;
      if (vec) {                                           // head_dim % 8 == 0, 16-byte aligned: 8 values a load
        for (int i = 0; i < head_dim; i += 8) {
          float kv[8];
          load8_as_float(kp + i, kv);
#pragma unroll
          for (int u = 0; u < 8; ++u) d += qs[i + u] * kv[u];
        }
      } else {
        for (int i = 0; i < head_dim; ++i) d += qs[i] * load_as_float(kp + i);
      }
      s = d * scale;
    }
    const float m_new = fmaxf(m, block_max(s, scratch));  // finite: every chunk holds a key the row sees
    const float alpha = expf(m - m_new);                   // first chunk: exp(-inf) = 0
    const float p = seen ? expf(s - m_new) : 0.f;
    l = l * alpha + block_sum(p, scratch);
    ps[tid] = rounded_as<T>(p);
    __syncthreads();
    if (tid < head_dim) {
      acc *= alpha;
      const int n = min(ROWS_THREADS, pos - c + 1);
      if (vec) {
        // a feature's 64 values of a page in the order they are stored, 8 a load: columns 8g..8g+3 of a block of
        // 32 are positions 4g..4g+3, columns 8g+4..8g+7 positions 16+4g.. (value_column); keys the row does not
        // see have weight 0 and their values, whatever was stored there before, are finite
        for (int pi = 0; pi * PAGE_TOKENS < n; ++pi) {
          const int pg = pages[pi];
          if (pg < 0) continue;
          const T* vrow = v_pages + (((int64_t)pg * n_kv + kvh) * head_dim + tid) * PAGE_TOKENS;
          const float* pw = ps + pi * PAGE_TOKENS;
#pragma unroll
          for (int c8 = 0; c8 < PAGE_TOKENS / 8; ++c8) {
            float vv[8];
            load8_as_float(vrow + 8 * c8, vv);
            const int at = 32 * (c8 / 4) + 4 * (c8 % 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc += pw[at + i] * vv[i] + pw[at + 16 + i] * vv[4 + i];
          }
        }
      } else {
        for (int jj = 0; jj < n; ++jj) {
          const int pg = pages[jj / PAGE_TOKENS];
          if (pg < 0) continue;
          const T* vp = v_pages + (((int64_t)pg * n_kv + kvh) * head_dim + tid) * PAGE_TOKENS + value_column(jj % PAGE_TOKENS);
          acc += ps[jj] * load_as_float(vp);
        }
      }
    }
    m = m_new;
  }
  if (tid < head_dim) store_from_float(o + tid, acc / l);
}

DRYFT_API int dryft_attn_rows(const void* q, const void* k_pages, const void* v_pages, const int* page_table,
                              int max_pages, const int* row_slot, const int* row_pos, void* out, int n_rows,
                              int n_heads, int n_kv, int head_dim, float scale, int window, int is_f32,
                              hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (head_dim > ROWS_MAX_HEAD_DIM || n_kv <= 0 || n_heads % n_kv) return -1;
  dim3 grid(n_rows, n_heads), block(ROWS_THREADS);
  const int vec = head_dim % 8 == 0 && (((uintptr_t)k_pages | (uintptr_t)v_pages) & 15) == 0;
  if (is_f32)
    hipLaunchKernelGGL(attn_rows_kernel<float>, grid, block, 0, stream, (const float*)q, (const float*)k_pages,
                       (const float*)v_pages, page_table, max_pages, row_slot, row_pos, (float*)out, n_heads, n_kv,
                       head_dim, scale, window, vec);
  else
    hipLaunchKernelGGL(attn_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q, (const bf16_t*)k_pages,
                       (const bf16_t*)v_pages, page_table, max_pages, row_slot, row_pos, (bf16_t*)out, n_heads, n_kv,
                       head_dim, scale, window, vec);
  return DRYFT_LAUNCH_CHECK();
}
