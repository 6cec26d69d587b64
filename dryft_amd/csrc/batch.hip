// Turns a step's per-sequence facts into per-row facts, on the device, so that
// a captured decode step can be replayed at any position: everything that
// varies is read from memory (the reference keeps positions in a device
// tensor for the same reason, engine/dryft_qwen3/cache.py:8-10).
#include "common.h"

#define PREPARE_THREADS 256

// One block. Inputs: seq_slot[B] (-1 = not taking part), q_len[B] (new tokens of
// each sequence), lengths[slots] (cached tokens per slot). Outputs: cu_rows[B+1]
// (prefix sums of rows), kv_len[B] (cached tokens after this step),
// row_seq/row_slot/row_pos[n_rows]. Advances lengths.
__global__ void prepare_batch_kernel(const int* __restrict__ seq_slot, const int* __restrict__ q_len,
                                     int* __restrict__ lengths, int n_seqs, int n_rows,
                                     int* __restrict__ cu_rows,
                                     int* __restrict__ kv_len, int* __restrict__ seq_start,
                                     int* __restrict__ row_seq, int* __restrict__ row_slot,
                                     int* __restrict__ row_pos) {
  // prefix sums over the sequences: every thread sums a run of them, the runs' sums are added up in LDS
  __shared__ int run_rows[PREPARE_THREADS];
  const int per = (n_seqs + PREPARE_THREADS - 1) / PREPARE_THREADS;
  const int s0 = min(n_seqs, (int)threadIdx.x * per), s1 = min(n_seqs, s0 + per);
  int rows = 0;
  for (int s = s0; s < s1; ++s) rows += q_len[s];     // rows of a sequence that sits out still occupy their places
  run_rows[threadIdx.x] = rows;
  __syncthreads();
  rows = 0;
  const int runs = (n_seqs + per - 1) / per;              // threads beyond them have summed nothing
  for (int t = 0; t < min((int)threadIdx.x, runs); ++t) rows += run_rows[t];
  for (int s = s0; s < s1; ++s) {
    cu_rows[s] = rows;
    const int slot = seq_slot[s];
    const int q = slot >= 0 ? q_len[s] : 0;
    const int past = slot >= 0 ? lengths[slot] : 0;
    seq_start[s] = past;
    kv_len[s] = past + q;
    rows += q_len[s];
    if (slot >= 0) lengths[slot] = past + q;
  }
  if (threadIdx.x == PREPARE_THREADS - 1) cu_rows[n_seqs] = rows;   // its runs come last: what it has summed is the total
  __syncthreads();
  for (int r = threadIdx.x; r < n_rows; r += blockDim.x) {
    int lo = 0, hi = n_seqs;                      // last s with cu_rows[s] <= r
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (cu_rows[mid] <= r) lo = mid; else hi = mid;
    }
    // skip over empty sequences that share the same start
    while (lo + 1 < n_seqs && cu_rows[lo + 1] <= r) ++lo;
    const int slot = (r < cu_rows[n_seqs]) ? seq_slot[lo] : -1;
    row_seq[r] = lo;
    row_slot[r] = slot;
    row_pos[r] = slot >= 0 ? seq_start[lo] + (r - cu_rows[lo]) : 0;
  }
}

DRYFT_API int dryft_prepare_batch(const int* seq_slot, const int* q_len, int* lengths, int n_seqs, int n_rows,
                                  int* cu_rows, int* kv_len, int* seq_start, int* row_seq,
                                  int* row_slot, int* row_pos, hipStream_t stream) {
  hipLaunchKernelGGL(prepare_batch_kernel, dim3(1), dim3(PREPARE_THREADS), 0, stream, seq_slot, q_len, lengths, n_seqs, n_rows,
                     cu_rows, kv_len, seq_start, row_seq, row_slot, row_pos);
  return DRYFT_LAUNCH_CHECK();
}

// tile_cu[B+1]: prefix sums over the sequences of the tiles of `tile_rows` rows their rows of this step fill
// (a sequence that sits out has none), for a kernel that walks a step tile by tile. One block.
__global__ void tile_prefix_kernel(const int* __restrict__ seq_slot, const int* __restrict__ q_len, int n_seqs,
                                   int tile_rows, int* __restrict__ tile_cu) {
  __shared__ int run_tiles[PREPARE_THREADS];
  const int per = (n_seqs + PREPARE_THREADS - 1) / PREPARE_THREADS;
  const int s0 = min(n_seqs, (int)threadIdx.x * per), s1 = min(n_seqs, s0 + per);
  int tiles = 0;
  for (int s = s0; s < s1; ++s) tiles += seq_slot[s] >= 0 ? (q_len[s] + tile_rows - 1) / tile_rows : 0;
  run_tiles[threadIdx.x] = tiles;
  __syncthreads();
  tiles = 0;
  const int runs = (n_seqs + per - 1) / per;
  for (int t = 0; t < min((int)threadIdx.x, runs); ++t) tiles += run_tiles[t];
  for (int s = s0; s < s1; ++s) {
    tile_cu[s] = tiles;
    tiles += seq_slot[s] >= 0 ? (q_len[s] + tile_rows - 1) / tile_rows : 0;
  }
  if (threadIdx.x == PREPARE_THREADS - 1) tile_cu[n_seqs] = tiles;
}

DRYFT_API int dryft_tile_prefix(const int* seq_slot, const int* q_len, int n_seqs, int tile_rows, int* tile_cu,
                                hipStream_t stream) {
  if (tile_rows <= 0) return -1;
  hipLaunchKernelGGL(tile_prefix_kernel, dim3(1), dim3(PREPARE_THREADS), 0, stream, seq_slot, q_len, n_seqs, tile_rows,
                     tile_cu);
  return DRYFT_LAUNCH_CHECK();
}
