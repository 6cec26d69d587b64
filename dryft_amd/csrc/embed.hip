// Token embedding: out[r, :] = table[tokens[r], :] (a row copy, no scaling;
// reference: engine/dryft_qwen3/model.py:132, 226).
#include "common.h"

template <typename T>
__global__ void embed_rows_kernel(const int* __restrict__ tokens, const T* __restrict__ table, T* __restrict__ out,
                                  int hidden, int vocab) {
  const int r = blockIdx.x;
  int tok = tokens[r];
  // Ids are checked on the host before a step; the clamp only keeps a bad id from reading outside the table.
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const T* src = table + (int64_t)tok * hidden;
  T* dst = out + (int64_t)r * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
}

DRYFT_API int dryft_embed_rows(const int* tokens, const void* table, void* out, int n_rows, int hidden, int vocab,
                               int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (is_f32)
    hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(n_rows), dim3(256), 0, stream, tokens, (const float*)table,
                       (float*)out, hidden, vocab);
  else
    hipLaunchKernelGGL(embed_rows_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, stream, tokens, (const bf16_t*)table,
                       (bf16_t*)out, hidden, vocab);
  return DRYFT_LAUNCH_CHECK();
}
