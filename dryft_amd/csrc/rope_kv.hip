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

template <typename T>
__global__ void qk_norm_rope_kv_kernel(const T* __restrict__ qkv, int64_t qkv_stride, const void* __restrict__ q_w,
                                       const void* __restrict__ k_w, int w_f32, int has_norm, float eps,
                                       const T* __restrict__ cos_t, const T* __restrict__ sin_t, int rot,
                                       const int* __restrict__ row_slot, const int* __restrict__ row_pos,
                                       T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                       const int* __restrict__ page_table, int max_pages, int write_kv, int n_heads,
                                       int n_kv, int head_dim) {
  __shared__ float normed[4][MAX_HEAD_DIM];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int64_t row = blockIdx.x;
  const int job = blockIdx.y * 4 + wave;  // [0,nH): q heads; [nH,nH+nKV): k heads; then v heads
  if (job >= n_heads + 2 * n_kv) return;
  const int slot = row_slot[row];
  const int pos = row_pos[row];
  const bool is_q = job < n_heads, is_k = !is_q && job < n_heads + n_kv;
  const T* src = qkv + row * qkv_stride + (int64_t)job * head_dim;
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
    T* dst = v_pages + ((int64_t)page * n_kv + kvh) * head_dim * PAGE_TOKENS + in_page;
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

DRYFT_API int dryft_qk_norm_rope_kv(const void* qkv, int64_t qkv_stride, const void* q_w, const void* k_w, int w_f32,
                                    int has_norm, float eps, const void* cos_t, const void* sin_t, int rot,
                                    const int* row_slot, const int* row_pos, void* q_out, void* k_pages,
                                    void* v_pages, const int* page_table, int max_pages, int write_kv, int n_rows,
                                    int n_heads, int n_kv, int head_dim, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (head_dim > MAX_HEAD_DIM || rot > head_dim || (rot & 1)) return -1;
  const int jobs = n_heads + 2 * n_kv;
  dim3 grid(n_rows, (jobs + 3) / 4), block(256);
  if (is_f32)
    hipLaunchKernelGGL(qk_norm_rope_kv_kernel<float>, grid, block, 0, stream, (const float*)qkv, qkv_stride, q_w, k_w,
                       w_f32, has_norm, eps, (const float*)cos_t, (const float*)sin_t, rot, row_slot, row_pos,
                       (float*)q_out, (float*)k_pages, (float*)v_pages, page_table, max_pages, write_kv, n_heads, n_kv,
                       head_dim);
  else
    hipLaunchKernelGGL(qk_norm_rope_kv_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)qkv, qkv_stride, q_w,
                       k_w, w_f32, has_norm, eps, (const bf16_t*)cos_t, (const bf16_t*)sin_t, rot, row_slot, row_pos,
                       (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, page_table, max_pages, write_kv, n_heads,
                       n_kv, head_dim);
  return DRYFT_LAUNCH_CHECK();
}
