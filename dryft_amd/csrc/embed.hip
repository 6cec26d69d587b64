// Token embedding: out[r, :] = table[tokens[r], :] (a row copy, no scaling;
// reference: engine/dryft_qwen3/model.py:132, 226). With `tables` > 1 the table is that many tables of `vocab` rows one
// after the other and the same rows are taken from each: out[t * n_rows + r, :] = table[t * vocab + tokens[r], :] (the
// wanted rows of a product left as partial sums).
#include "common.h"

template <typename T>
__global__ void embed_rows_kernel(const int* __restrict__ tokens, const T* __restrict__ table, T* __restrict__ out,
                                  int hidden, int vocab, int n_rows) {
  const int r = blockIdx.x % n_rows, t = blockIdx.x / n_rows;
  int tok = tokens[r];
  // Ids are checked on the host before a step; the clamp only keeps a bad id from reading outside the table.
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const T* src = table + ((int64_t)t * vocab + tok) * hidden;
  T* dst = out + (int64_t)blockIdx.x * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
}

DRYFT_API int dryft_embed_rows(const int* tokens, const void* table, void* out, int n_rows, int hidden, int vocab,
                               int tables, int is_f32, hipStream_t stream) {
  if (n_rows <= 0 || tables <= 0) return 0;
  if (is_f32)
    hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(n_rows * tables), dim3(256), 0, stream, tokens,
                       (const float*)table, (float*)out, hidden, vocab, n_rows);
  else
    hipLaunchKernelGGL(embed_rows_kernel<bf16_t>, dim3(n_rows * tables), dim3(256), 0, stream, tokens,
                       (const bf16_t*)table, (bf16_t*)out, hidden, vocab, n_rows);
  return DRYFT_LAUNCH_CHECK();
}
