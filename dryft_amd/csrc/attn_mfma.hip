// bfloat16 attention on the matrix cores (v_mfma_f32_16x16x32_bf16), reading keys and values from
// the paged cache: a causal kernel for steps that bring many rows per sequence, and a split
// kernel plus a combine for steps that bring one row per sequence. They stand where the reference
// uses a library's flash attention for prompts (engine/dryft_qwen3/model.py:172-177) and its
// split-KV kernel for decoding (kernels/attn_decode.py:36-118). Scores, running maximum, exponentials,
// row sums and the output accumulator are float; probabilities are rounded to bfloat16 for the
// second product (attn_decode.py:12-14, 89).
//
// A wave owns 16 query rows. It forms transposed tiles so that no operand has to be moved between
// lanes:   S^T[key, row] = K[key, :] . Q[row, :]        (A = K from its page, B = Q from registers)
//          O^T[d, row]  += V^T[d, key] * P^T[key, row]  (A = V^T from its page, B = P^T = S^T's own layout)
// In the 16x16 result layout lane l holds column l%16 and rows 4*(l/16)..+3, while a B operand of the
// 32-deep product wants 8 consecutive contraction indices per lane. Since a sum does not care about the
// order of its terms, contraction index 8*(l/16)+i of the second product stands for key 4*(l/16)+i of the
// first 16-key tile when i < 4 and for key 16+4*(l/16)+(i-4) of the second tile otherwise; V^T is fetched
// in the same order.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16((a), (b), (c), 0, 0, 0)

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *(const bf16x8*)p; }

__device__ __forceinline__ __bf16 to_bf16(float f) { return (__bf16)f; }

// 2^x by the hardware instruction alone: arguments here are <= 0 or -inf, results below the normal range may flush to 0
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// State of one wave's 16 rows while it walks over pages of keys.
template <int KB>  // KB = ceil(head_dim / 32)
struct RowBlock {
  bf16x8 q[KB];          // B operand of the first product, per 32 features
  f32x4 o[2 * KB];       // O^T tiles of 16 features each
  // Running reference maximum of the lane's own row (lane % 16), the same in the four lanes that share a row,
  // and this lane's part of the row's running sum: the four parts are only added up by row_sum() at the end.
  float m, l;
};

// The row's sum of probabilities from its four lanes' parts (all lanes of the wave must call it).
template <int KB>
__device__ __forceinline__ float row_sum(const RowBlock<KB>& st) {
  float l = st.l;
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  return l;
}

template <int KB>
__device__ __forceinline__ void init_rows(RowBlock<KB>& st, const bf16_t* q_row, bool row_valid, int head_dim) {
  const int g = (threadIdx.x % WAVE) / 16;
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int d = 32 * kb + 8 * g;
    st.q[kb] = (row_valid && d < head_dim) ? load8(q_row + d) : zero8();
  }
#pragma unroll
  for (int dt = 0; dt < 2 * KB; ++dt) st.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m = -INFINITY;
  st.l = 0.f;
}

// ---------------------------------------------------------------------------------------------------
// One page of 64 keys for one wave: loads, scores, online softmax and the second product.
template <int KB>
struct PageK {
  bf16x8 k[4][KB];
};
template <int KB>
struct PageV {
  bf16x8 v[2 * KB][2];      // [tile of 16 features][block of 32 positions]: the lane's 8 values, see value_column
};

// FULL: head_dim == 32 * KB. Otherwise features at or beyond head_dim are read from a clamped, valid address:
// the query holds zeros there, so whatever finite value is read adds nothing to a score, and output
// features beyond head_dim are computed but never stored. This keeps every load unconditional.
template <int KB, bool FULL>
__device__ __forceinline__ void load_page_k(PageK<KB>& f, const bf16_t* __restrict__ k_page, int head_dim) {
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int d = FULL ? 32 * kb + 8 * g : min(32 * kb + 8 * g, head_dim - 8);
      f.k[t][kb] = load8(k_page + (16 * t + c) * head_dim + d);
    }
}

template <int KB, bool FULL>
__device__ __forceinline__ void load_page_v(PageV<KB>& f, const bf16_t* __restrict__ v_page, int head_dim) {
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
#pragma unroll
  for (int dt = 0; dt < 2 * KB; ++dt)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int d = FULL ? 16 * dt + c : min(16 * dt + c, head_dim - 1);
      f.v[dt][h] = load8(v_page + d * PAGE_TOKENS + 32 * h + 8 * g);
    }
}

// scores of one page from its loaded keys: s[t][i] for key 16t + 4g + i, in units of log2(e) so that exp2 serves
template <int KB>
__device__ __forceinline__ void page_scores(f32x4 (&s)[4], const PageK<KB>& f, const RowBlock<KB>& st) {
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) s[t] = MFMA16(f.k[t][kb], st.q[kb], s[t]);
  }
}

// Online softmax over the page's scores, in the form that keeps lanes from talking to each other: the row's
// reference maximum st.m only moves when some row of the wave has met a score more than MAX_SLACK above it, so
// in the steady state a lane neither exchanges maxima nor rescales; probabilities are 2^(s - m) with m at most
// that much below the true maximum (they stay far inside float and bfloat16 range), and each lane adds its own
// scores to its own part of the sum. Leaves the probabilities in `p` as the second product's B operand and
// returns the factor by which the row's accumulator must shrink; `moved` tells (the same for the whole wave)
// whether any factor differs from 1. `scale_log2` turns a raw score into units of log2(e); st.m is kept in those
// units. MASKED: some key of the page may be hidden from some row (the page of the diagonal, a window's edge,
// the end of the sequence).
#define MAX_SLACK 8.f
template <int KB, bool MASKED>
__device__ __forceinline__ float page_softmax(RowBlock<KB>& st, f32x4 (&s)[4], bf16x8 (&p)[2], float scale_log2,
                                              int key0, int lo_row, int hi_row, bool& moved) {
  const int g = (threadIdx.x % WAVE) / 16;
  float lane_max = -INFINITY;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (MASKED) {
        const int j = key0 + 16 * t + 4 * g + i;
        if (!(j >= lo_row && j <= hi_row)) s[t][i] = -INFINITY;
      }
      lane_max = fmaxf(lane_max, s[t][i]);
    }
  lane_max *= scale_log2;                                     // scale > 0, so the maximum commutes with it
  float alpha = 1.f;
  moved = __any(lane_max > st.m + MAX_SLACK);                 // also true for a row's first visible key (m = -inf)
  if (moved) {
    float row_max = fmaxf(lane_max, __shfl_xor(lane_max, 16, WAVE));
    row_max = fmaxf(row_max, __shfl_xor(row_max, 32, WAVE));
    const float m_new = fmaxf(st.m, row_max);
    alpha = m_new == -INFINITY ? 1.f : fast_exp2(st.m - m_new);   // exp2(-inf) = 0: nothing was summed before
    st.l *= alpha;
    st.m = m_new;
  }
  const float m_ref = st.m == -INFINITY ? 0.f : st.m;          // a row that has seen no key yet stays empty
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float e = fast_exp2(fmaf(s[t][i], scale_log2, -m_ref));   // -inf stays -inf: e = 0
      s[t][i] = e;
      sum += e;
    }
  st.l += sum;
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[h][i] = to_bf16(s[2 * h][i]);
      p[h][4 + i] = to_bf16(s[2 * h + 1][i]);
    }
  return alpha;
}

// O^T = alpha * O^T + V^T P^T
template <int KB>
__device__ __forceinline__ void page_values(RowBlock<KB>& st, const bf16x8 (&p)[2], float alpha, bool moved,
                                            const PageV<KB>& f) {
  if (moved) {                                                // rare once the maxima have settled
#pragma unroll
    for (int dt = 0; dt < 2 * KB; ++dt) st.o[dt] *= alpha;
  }
#pragma unroll
  for (int dt = 0; dt < 2 * KB; ++dt)
#pragma unroll
    for (int h = 0; h < 2; ++h) st.o[dt] = MFMA16(f.v[dt][h], p[h], st.o[dt]);
}

template <int KB, bool MASKED>
__device__ __forceinline__ void page_update_impl(RowBlock<KB>& st, f32x4 (&s)[4], const PageV<KB>& f, float scale_log2,
                                                 int key0, int lo_row, int hi_row) {
  bf16x8 p[2];
  bool moved;
  const float alpha = page_softmax<KB, MASKED>(st, s, p, scale_log2, key0, lo_row, hi_row, moved);
  page_values<KB>(st, p, alpha, moved, f);
}

// `masked` must be the same for all lanes of the wave.
template <int KB>
__device__ __forceinline__ void page_update(RowBlock<KB>& st, f32x4 (&s)[4], const PageV<KB>& f, int head_dim,
                                            float scale_log2, int key0, int lo_row, int hi_row, bool masked = true) {
  if (masked)
    page_update_impl<KB, true>(st, s, f, scale_log2, key0, lo_row, hi_row);
  else
    page_update_impl<KB, false>(st, s, f, scale_log2, key0, lo_row, hi_row);
}

// ---------------------------------------------------------------------------------------------------
// Many rows per sequence. Grid: (pairs of 64-position query tiles, query heads / 2) with two heads per wave,
// (query heads, tiles) with one; 4 waves of 16 positions each.
// A wave serves GP query heads that share one kv head. The workgroup copies each page of keys and values
// from the cache into LDS once (the next page's loads are in flight while the current one is used), every
// wave reads its operands from there into registers once per page and uses them for each of its heads.
// LDS rows are padded by 16 bytes so that the 16 lanes that read 16 different rows hit different banks.
#define K_PAD 8
#define V_PAD 8

template <int KB, bool FULL>
__device__ __forceinline__ void lds_page_k(PageK<KB>& f, const bf16_t* k_lds, int head_dim) {
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int d = FULL ? 32 * kb + 8 * g : min(32 * kb + 8 * g, head_dim - 8);
      f.k[t][kb] = load8(k_lds + (16 * t + c) * (head_dim + K_PAD) + d);
    }
}

template <int KB, bool FULL>
__device__ __forceinline__ void lds_page_v(PageV<KB>& f, const bf16_t* v_lds, int head_dim) {
  const int lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
#pragma unroll
  for (int dt = 0; dt < 2 * KB; ++dt)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int d = FULL ? 16 * dt + c : min(16 * dt + c, head_dim - 1);
      f.v[dt][h] = load8(v_lds + d * (PAGE_TOKENS + V_PAD) + 32 * h + 8 * g);
    }
}

// a page is 8 * head_dim pieces of 16 bytes for the keys and as many for the values; thread t moves pieces t, t+256, ...
template <int KB>
struct PageStage {
  bf16x8 k[KB], v[KB];
};

template <int KB>
__device__ __forceinline__ void stage_load(PageStage<KB>& st, const bf16_t* __restrict__ k_page,
                                           const bf16_t* __restrict__ v_page, int head_dim) {
  const int pieces = 8 * head_dim;
#pragma unroll
  for (int i = 0; i < KB; ++i) {
    const int j = threadIdx.x + 256 * i;
    if (j < pieces) {
      st.k[i] = load8(k_page + 8 * j);
      st.v[i] = load8(v_page + 8 * j);
    }
  }
}

template <int KB>
__device__ __forceinline__ void stage_store_k(const PageStage<KB>& st, bf16_t* k_lds, int head_dim) {
  const int pieces = 8 * head_dim;
#pragma unroll
  for (int i = 0; i < KB; ++i) {
    const int j = threadIdx.x + 256 * i;
    if (j < pieces) {
      const int e = 8 * j;                                   // element index within the page
      *(bf16x8*)(k_lds + (e / head_dim) * (head_dim + K_PAD) + e % head_dim) = st.k[i];
    }
  }
}

template <int KB>
__device__ __forceinline__ void stage_store_v(const PageStage<KB>& st, bf16_t* v_lds, int head_dim) {
  const int pieces = 8 * head_dim;
#pragma unroll
  for (int i = 0; i < KB; ++i) {
    const int j = threadIdx.x + 256 * i;
    if (j < pieces) {
      const int e = 8 * j;
      *(bf16x8*)(v_lds + (e / PAGE_TOKENS) * (PAGE_TOKENS + V_PAD) + e % PAGE_TOKENS) = st.v[i];
    }
  }
}

// Tiles of 64 * RP rows over all sequences of the step, and the sequence and place of one of them. A sequence that
// sits out (slot < 0) keeps its rows in cu_rows but has no tiles. tile_cu holds the prefix sums for 64-row tiles.
template <int RP>
__device__ __forceinline__ int count_tiles(const int* __restrict__ seq_slot, const int* __restrict__ cu_rows,
                                           const int* __restrict__ tile_cu, int n_seqs) {
  if (RP == 1) return tile_cu[n_seqs];
  int n_tiles = 0;
  for (int sq = 0; sq < n_seqs; ++sq)
    if (seq_slot[sq] >= 0) n_tiles += (cu_rows[sq + 1] - cu_rows[sq] + 64 * RP - 1) / (64 * RP);
  return n_tiles;
}

template <int RP>
__device__ __forceinline__ void locate_tile(int tile, const int* __restrict__ seq_slot, const int* __restrict__ cu_rows,
                                            const int* __restrict__ tile_cu, int n_seqs, int& seq, int& tile_in_seq) {
  if (RP == 1) {
    int lo = 0, hi = n_seqs;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (tile_cu[mid] <= tile) lo = mid; else hi = mid;
    }
    while (lo + 1 < n_seqs && tile_cu[lo + 1] <= tile) ++lo;
    seq = lo;
    tile_in_seq = tile - tile_cu[seq];
  } else {
    seq = 0;
    tile_in_seq = tile;
    for (;;) {
      const int cnt = seq_slot[seq] >= 0 ? (cu_rows[seq + 1] - cu_rows[seq] + 64 * RP - 1) / (64 * RP) : 0;
      if (tile_in_seq < cnt || seq + 1 >= n_seqs) break;
      tile_in_seq -= cnt;
      ++seq;
    }
  }
}

// A wave serves U = GP * RP units: GP query heads of one kv group, each over RP tiles of 16 consecutive rows. Every
// piece of a page that a wave reads from LDS is used for all its units, so two units halve the LDS reads per
// matrix instruction. A workgroup's tile is 64 * RP rows.
template <int KB, bool FULL, int GP, int RP>
__global__ __launch_bounds__(256, (GP * RP * KB <= 8 && KB <= 4) ? (GP * RP == 1 ? 3 : 2) : 1) void attn_causal_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ page_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_rows, const int* __restrict__ tile_cu, const int* __restrict__ seq_start, int n_seqs,
    bf16_t* __restrict__ out, int n_heads, int n_kv, int head_dim, float scale, int window) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  constexpr int U = GP * RP, TILE_ROWS = 64 * RP, WAVE_ROWS = 16 * RP;
  // Two heads per wave: a workgroup takes one tile from each end of the list (grid: pairs of tiles x heads / 2).
  // Otherwise: one tile per workgroup, the ones with the most pages first, heads fastest (grid: heads x tiles),
  // so that the short tiles fill the compute units that the long ones leave.
  constexpr bool PAIRED = GP != 1;
  const int head0 = (PAIRED ? blockIdx.y : blockIdx.x) * GP;
  const int first_tile = PAIRED ? blockIdx.x : blockIdx.y;
  const int n_tiles = count_tiles<RP>(seq_slot, cu_rows, tile_cu, n_seqs);   // tiles of TILE_ROWS rows over all sequences
  // A tile late in a sequence sees many keys, an early one few. With pairs every workgroup takes one tile from
  // each end of the list, so all of them have about the same work.
  for (int half = 0; half < 2; ++half) {
  if (!PAIRED && half == 1) break;
  const int tile = half == 0 ? n_tiles - 1 - first_tile : first_tile;
  if (tile < 0 || tile >= n_tiles || (half == 1 && tile >= n_tiles - 1 - first_tile)) continue;
  int seq, tile_in_seq;                                       // the sequence whose tiles include `tile`
  locate_tile<RP>(tile, seq_slot, cu_rows, tile_cu, n_seqs, seq, tile_in_seq);
  const int slot = seq_slot[seq];
  if (slot < 0) continue;                                     // the whole workgroup skips the tile together
  __syncthreads();                                            // the previous tile's pages are no longer read
  const int k_elems = PAGE_TOKENS * (head_dim + K_PAD), v_elems = head_dim * (PAGE_TOKENS + V_PAD);
  bf16_t* const smem = (bf16_t*)lds_raw;    // [2][64][D+8] keys, then [2][D][64+8] values
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int q_len = cu_rows[seq + 1] - cu_rows[seq];
  const int tile_first = tile_in_seq * TILE_ROWS;             // first row of the tile within the sequence
  const int wave_first = tile_first + WAVE_ROWS * wave;       // first of the wave's rows
  const int wave_rows = max(0, min(WAVE_ROWS, q_len - wave_first));   // a wave past the sequence's end has none
  const int pos_tile = seq_start[seq] + tile_first;           // position of the tile's first row
  const int pos_wave = pos_tile + WAVE_ROWS * wave;
  // per tile of 16 rows
  int rows[RP], pos0[RP], pos_row[RP], lo_row[RP];
  bool row_valid[RP];
  int64_t row[RP];
#pragma unroll
  for (int rt = 0; rt < RP; ++rt) {
    const int first = wave_first + 16 * rt;
    rows[rt] = max(0, min(16, q_len - first));
    row_valid[rt] = c < rows[rt];
    row[rt] = (int64_t)cu_rows[seq] + first + c;
    pos0[rt] = pos_wave + 16 * rt;
    pos_row[rt] = row_valid[rt] ? pos0[rt] + c : -1;          // an absent row sees nothing
    lo_row[rt] = window > 0 ? max(0, pos_row[rt] - window + 1) : 0;
  }
  const int kvh = head0 / (n_heads / n_kv);
  RowBlock<KB> st[U];                                         // unit u: head u % GP, rows of tile u / GP
#pragma unroll
  for (int u = 0; u < U; ++u)
    init_rows<KB>(st[u], q + (row[u / GP] * n_heads + head0 + u % GP) * head_dim, row_valid[u / GP], head_dim);
  const int lo_wave = window > 0 ? max(0, pos_wave - window + 1) : 0;
  const int hi_wave = pos_wave + wave_rows - 1;               // below lo_wave for a wave without rows
  const int lo_tile = window > 0 ? max(0, pos_tile - window + 1) : 0;
  const int hi_tile = pos_tile + min(TILE_ROWS, q_len - tile_first) - 1;
  const float scale_log2 = scale * 1.44269504088896340736f;
  const int64_t page_elems = (int64_t)PAGE_TOKENS * head_dim;
  const int* table = page_table + (int64_t)slot * max_pages;
  const int pg_first = lo_tile / PAGE_TOKENS, pg_last = hi_tile / PAGE_TOKENS;
  PageStage<KB> stage;
  int page = table[pg_first];
  if (page >= 0)
    stage_load<KB>(stage, k_pages + ((int64_t)page * n_kv + kvh) * page_elems,
                   v_pages + ((int64_t)page * n_kv + kvh) * page_elems, head_dim);
  for (int pg = pg_first; pg <= pg_last; ++pg) {
    const int buf = (pg - pg_first) & 1;
    bf16_t* const k_lds = smem + buf * k_elems;
    // With one unit per wave the values have one buffer only: three workgroups then fit a compute unit, and
    // the third wave per SIMD covers more of the latency than the second barrier per page costs.
    constexpr bool V_DOUBLE = U != 1;
    bf16_t* const v_lds = smem + 2 * k_elems + (V_DOUBLE ? buf * v_elems : 0);
    if (page >= 0) {
      stage_store_k<KB>(stage, k_lds, head_dim);
      if (V_DOUBLE) stage_store_v<KB>(stage, v_lds, head_dim);
    }
    __syncthreads();   // the keys are in LDS; every wave is done with the page before (and the buffers it used)
    if (!V_DOUBLE && page >= 0) stage_store_v<KB>(stage, v_lds, head_dim);
    const int page_now = page;
    page = pg < pg_last ? table[pg + 1] : -1;
    if (page >= 0)
      stage_load<KB>(stage, k_pages + ((int64_t)page * n_kv + kvh) * page_elems,
                     v_pages + ((int64_t)page * n_kv + kvh) * page_elems, head_dim);
    const int key0 = pg * PAGE_TOKENS;
    const bool sees = page_now >= 0 && key0 <= hi_wave && key0 + PAGE_TOKENS > lo_wave;   // some row sees some key
    bf16x8 p[U][2];
    if (sees) {
      // Every piece of a page is read from LDS once and used at once for each of the wave's units, so that no
      // whole page of operands has to sit in registers.
      float alpha[U];
      bool moved[U];
      f32x4 s[U][4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int u = 0; u < U; ++u) s[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          const int d = FULL ? 32 * kb + 8 * g : min(32 * kb + 8 * g, head_dim - 8);
          const bf16x8 a = load8(k_lds + (16 * t + c) * (head_dim + K_PAD) + d);
#pragma unroll
          for (int u = 0; u < U; ++u) s[u][t] = MFMA16(a, st[u].q[kb], s[u][t]);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int rt = u / GP;
        // every key of the page is seen by every row of the tile unless the page reaches past the tile's first
        // row, starts before a window's edge, or the tile has fewer than 16 rows
        const bool masked = key0 + PAGE_TOKENS - 1 > pos0[rt] || rows[rt] < 16 ||
                            (window > 0 && key0 < pos0[rt] + 15 - window + 1);
        alpha[u] = masked ? page_softmax<KB, true>(st[u], s[u], p[u], scale_log2, key0, lo_row[rt], pos_row[rt], moved[u])
                          : page_softmax<KB, false>(st[u], s[u], p[u], scale_log2, key0, lo_row[rt], pos_row[rt], moved[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (moved[u]) {                                       // rare once the maxima have settled
#pragma unroll
          for (int dt = 0; dt < 2 * KB; ++dt) st[u].o[dt] *= alpha[u];
        }
    }
    if (!V_DOUBLE) __syncthreads();                          // the values are in LDS
    if (sees) {
#pragma unroll
      for (int dt = 0; dt < 2 * KB; ++dt)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int d = FULL ? 16 * dt + c : min(16 * dt + c, head_dim - 1);
          const bf16x8 a = load8(v_lds + d * (PAGE_TOKENS + V_PAD) + 32 * h + 8 * g);
#pragma unroll
          for (int u = 0; u < U; ++u) st[u].o[dt] = MFMA16(a, p[u][h], st[u].o[dt]);
        }
    }
  }
  float row_l[U];
#pragma unroll
  for (int u = 0; u < U; ++u) row_l[u] = row_sum<KB>(st[u]);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (!row_valid[u / GP]) continue;
    const float inv = 1.f / row_l[u];
    bf16_t* o = out + (row[u / GP] * n_heads + head0 + u % GP) * head_dim;
#pragma unroll
    for (int dt = 0; dt < 2 * KB; ++dt) {
      if (FULL || 16 * dt < head_dim) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[16 * dt + 4 * g + i] = float_to_bf16(st[u].o[dt][i] * inv);
      }
    }
  }
  }  // the two tiles of the workgroup
}

// ---------------------------------------------------------------------------------------------------
// The same kernel for head size 128 with one head per wave, with the pages going from the cache straight into
// LDS (global_load_lds_dwordx4: 16 bytes a lane, no registers in between and nothing for the waves to store;
// about a quarter of the staged kernel's time goes into that copying). One instruction fills 1,024 contiguous
// bytes of LDS, lane l at byte 16 l. Which 16 bytes of the page a lane fetches is free, and that choice
// swizzles the layout so that operand reads meet no bank twice without padding:
//   keys   [64 positions][16 pieces of 16 bytes]: piece p of row r sits at place p ^ (r % 16);
//   values [128 features][8 pieces]:              piece p of row d sits at place p ^ ((d / 2) % 8).
// The compiler does not know that these loads write LDS (it would otherwise wait for all of them before every
// LDS read that follows one): each wave waits for its own (s_waitcnt vmcnt(0)) before the barrier after which
// the page is read. The LDS address of an instruction goes through M0.
#define DIRECT_D 128
#define DIRECT_PAGE_BYTES (PAGE_TOKENS * DIRECT_D * 2)

// 16 bytes from base + offset (a base the whole wave shares, an offset per lane) to LDS byte lds_base + 16 * lane
__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t offset, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
}

// s_waitcnt vmcnt(0), leaving the other counters alone (vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8). As a
// builtin rather than text, so that the compiler's own count of loads in flight takes it into account: it would
// otherwise wait again, inside the loop, for the query loads of the prologue, and with them for the page on its way.
__device__ __forceinline__ void wait_direct_loads() {
  __builtin_amdgcn_s_waitcnt(0x0f70);
  asm volatile("" ::: "memory");
}

// A wave's quarter of a page of keys or of values: a page is 16 KB, an instruction moves 1 KB, and wave w takes the
// pieces of 1 KB number w, 4 + w, 8 + w and 12 + w. They are 4,096 bytes apart in the page and in LDS, and the
// swizzle repeats with that period (16 rows of keys, 32 rows of values), so one offset per lane serves all four:
// where the lane reads within the first of them (`lane_offset`); `lds_wave` is the LDS address of the page's
// buffer plus 1,024 w. Base addresses are the wave's, in scalar registers: no vector arithmetic per page.
__device__ __forceinline__ void direct_page(const bf16_t* page, uint32_t lane_offset, uint32_t lds_wave) {
#pragma unroll
  for (int i = 0; i < 4; ++i) load_to_lds16((const unsigned char*)page + 4096 * i, lane_offset, lds_wave + 4096 * i);
}

// Where a lane reads within its wave's first piece of a page of keys: row 4 w + lane / 16 of 256 bytes, and the
// 16-byte piece that belongs at place lane % 16 of that row; of values: row 8 w + lane / 8 of 128 bytes, place lane % 8.
__device__ __forceinline__ uint32_t direct_offset_k(int wave, int lane) {
  const int row = 4 * wave + lane / 16, place = lane % 16;
  return row * (2 * DIRECT_D) + ((place ^ (row & 15)) << 4);
}

__device__ __forceinline__ uint32_t direct_offset_v(int wave, int lane) {
  const int row = 8 * wave + lane / 8, place = lane % 8;
  return row * (2 * PAGE_TOKENS) + ((place ^ ((row >> 1) & 7)) << 4);
}

// What the kernel needs to take a row's query heads straight from the fused projection: per-head RMSNorm
// (optional) and the rotation of pairs (j, j + 64) over the full head, with the roundings of the stand-alone kernel
// (rope_kv.hip). Saves writing the queries out and reading them back.
struct ProjectedQ {
  const bf16_t* qkv;       // [rows, stride]: the row's query heads come first; null: q is given ready
  int64_t stride;
  const void* q_w;
  int w_f32, has_norm;
  float eps;
  const bf16_t* cos_t;     // [positions, 64]
  const bf16_t* sin_t;
};

// A lane holds 8 features 32 kb + 8 g .. of its row for kb = 0..3 (the first product's B operand): the four lanes
// of a row add up their sums of squares, and a feature's rotation partner (64 further on) sits in the same lane.
__device__ __forceinline__ void init_rows_projected(RowBlock<4>& st, const ProjectedQ& pq, int64_t row, int head,
                                                    int pos, bool row_valid) {
  const int g = (threadIdx.x % WAVE) / 16;
  float x[4][8];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    if (row_valid) {
      load8_as_float(pq.qkv + row * pq.stride + (int64_t)head * DIRECT_D + 32 * kb + 8 * g, x[kb]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[kb][i] = 0.f;
    }
  }
  if (pq.has_norm) {
    float ss = 0.f;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += x[kb][i] * x[kb][i];
    ss += __shfl_xor(ss, 16, WAVE);
    ss += __shfl_xor(ss, 32, WAVE);
    const float inv = rsqrtf(ss / (float)DIRECT_D + pq.eps);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      float w[8];
      if (pq.w_f32) load8_as_float((const float*)pq.q_w + 32 * kb + 8 * g, w);
      else load8_as_float((const bf16_t*)pq.q_w + 32 * kb + 8 * g, w);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[kb][i] = rounded_as<bf16_t>(rounded_as<bf16_t>(x[kb][i] * inv) * w[i]);
    }
  }
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    float c[8], sn[8];
    if (row_valid) {
      load8_as_float(pq.cos_t + (int64_t)pos * (DIRECT_D / 2) + 32 * kb + 8 * g, c);
      load8_as_float(pq.sin_t + (int64_t)pos * (DIRECT_D / 2) + 32 * kb + 8 * g, sn);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) { c[i] = 1.f; sn[i] = 0.f; }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float x1 = x[kb][i], x2 = x[kb + 2][i];
      const float o1 = rounded_as<bf16_t>(x1 * c[i]) - rounded_as<bf16_t>(x2 * sn[i]);   // x1*c - x2*s
      const float o2 = rounded_as<bf16_t>(x2 * c[i]) + rounded_as<bf16_t>(x1 * sn[i]);   // x2*c + x1*s
      st.q[kb][i] = to_bf16(o1);
      st.q[kb + 2][i] = to_bf16(o2);
    }
  }
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) st.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m = -INFINITY;
  st.l = 0.f;
}

// RP tiles of 16 consecutive rows per wave; a workgroup's tile is 64 * RP rows. Grid: (heads, tiles), the
// tiles with the most pages first. With 16 rows a wave, keys and values have one buffer each and a page takes two
// barriers (the values arrive during the first product and the softmax, the next keys during the second
// product): 32 KB of LDS and under 128 registers put four workgroups on a compute unit, which covers more
// latency than a second buffer would (0.67 against 0.63 PFLOP/s at 3,000 positions, 0.76 against 0.70 at 4,096,
// the same at 2,048). With 32 rows a wave the registers allow two workgroups a unit anyway, so both have two
// buffers and a page takes one barrier.
template <int RP>
__global__ __launch_bounds__(256, RP == 1 ? 4 : 2) void attn_causal_direct_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ page_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_rows, const int* __restrict__ tile_cu, const int* __restrict__ seq_start, int n_seqs,
    bf16_t* __restrict__ out, int n_heads, int n_kv, float scale, int window, ProjectedQ projected) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  constexpr int KB = DIRECT_D / 32, TILE_ROWS = 64 * RP, WAVE_ROWS = 16 * RP, head_dim = DIRECT_D;
  constexpr bool TWO = RP != 1;                               // two buffers each for keys and values
  const int head = blockIdx.x;
  const int n_tiles = count_tiles<RP>(seq_slot, cu_rows, tile_cu, n_seqs);
  const int tile = n_tiles - 1 - (int)blockIdx.y;
  if (tile < 0) return;
  int seq, tile_in_seq;
  locate_tile<RP>(tile, seq_slot, cu_rows, tile_cu, n_seqs, seq, tile_in_seq);
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int q_len = cu_rows[seq + 1] - cu_rows[seq];
  const int tile_first = tile_in_seq * TILE_ROWS;
  const int wave_first = tile_first + WAVE_ROWS * wave;
  const int wave_rows = max(0, min(WAVE_ROWS, q_len - wave_first));
  const int pos_tile = seq_start[seq] + tile_first;
  const int pos_wave = pos_tile + WAVE_ROWS * wave;
  int rows[RP], pos0[RP], pos_row[RP], lo_row[RP];
  bool row_valid[RP];
  int64_t row[RP];
  RowBlock<KB> st[RP];
#pragma unroll
  for (int rt = 0; rt < RP; ++rt) {
    const int first = wave_first + 16 * rt;
    rows[rt] = max(0, min(16, q_len - first));
    row_valid[rt] = c < rows[rt];
    row[rt] = (int64_t)cu_rows[seq] + first + c;
    pos0[rt] = pos_wave + 16 * rt;
    pos_row[rt] = row_valid[rt] ? pos0[rt] + c : -1;
    lo_row[rt] = window > 0 ? max(0, pos_row[rt] - window + 1) : 0;
    if (projected.qkv != nullptr)
      init_rows_projected(st[rt], projected, row[rt], head, pos0[rt] + c, row_valid[rt]);
    else
      init_rows<KB>(st[rt], q + (row[rt] * n_heads + head) * head_dim, row_valid[rt], head_dim);
  }
  const int kvh = head / (n_heads / n_kv);
  const int lo_wave = window > 0 ? max(0, pos_wave - window + 1) : 0;
  const int hi_wave = pos_wave + wave_rows - 1;
  const int lo_tile = window > 0 ? max(0, pos_tile - window + 1) : 0;
  const int hi_tile = pos_tile + min(TILE_ROWS, q_len - tile_first) - 1;
  const float scale_log2 = scale * 1.44269504088896340736f;
  const int64_t page_elems = (int64_t)PAGE_TOKENS * head_dim;
  const int* table = page_table + (int64_t)slot * max_pages;
  const int pg_first = lo_tile / PAGE_TOKENS, pg_last = hi_tile / PAGE_TOKENS;
  // LDS: one or two pages of keys, then as many of values; these are the addresses of this wave's first piece
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_raw + 1024 * wave);
  const uint32_t v_lds0 = lds0 + (TWO ? 2 : 1) * DIRECT_PAGE_BYTES;
  const uint32_t k_from = direct_offset_k(wave, lane), v_from = direct_offset_v(wave, lane);
  // where this lane's operands sit within a page: keys (16 t + c, piece 4 kb + g), values (16 dt + c, piece 4 h + g)
  int k_at[KB], v_at[2];
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) k_at[kb] = c * (2 * DIRECT_D) + (((4 * kb + g) ^ c) << 4);
#pragma unroll
  for (int h = 0; h < 2; ++h) v_at[h] = c * (2 * PAGE_TOKENS) + (((4 * h + g) ^ (c >> 1)) << 4);
  int page = table[pg_first];
  if (page >= 0) {
    direct_page(k_pages + ((int64_t)page * n_kv + kvh) * page_elems, k_from, lds0);
    if (TWO) direct_page(v_pages + ((int64_t)page * n_kv + kvh) * page_elems, v_from, v_lds0);
  }
  for (int pg = pg_first; pg <= pg_last; ++pg) {
    const int buf = TWO ? (pg - pg_first) & 1 : 0;
    const unsigned char* k_lds = lds_raw + buf * DIRECT_PAGE_BYTES;
    const unsigned char* v_lds = lds_raw + ((TWO ? 2 : 1) + buf) * DIRECT_PAGE_BYTES;
    wait_direct_loads();
    __syncthreads();   // this page's keys are in LDS; every wave is done with the page before and the buffers it used
    const int page_now = page;
    page = pg < pg_last ? table[pg + 1] : -1;
    if (!TWO && page_now >= 0) direct_page(v_pages + ((int64_t)page_now * n_kv + kvh) * page_elems, v_from, v_lds0);
    if (TWO && page >= 0) {
      direct_page(k_pages + ((int64_t)page * n_kv + kvh) * page_elems, k_from, lds0 + (buf ^ 1) * DIRECT_PAGE_BYTES);
      direct_page(v_pages + ((int64_t)page * n_kv + kvh) * page_elems, v_from, v_lds0 + (buf ^ 1) * DIRECT_PAGE_BYTES);
    }
    const int key0 = pg * PAGE_TOKENS;
    const bool sees = page_now >= 0 && key0 <= hi_wave && key0 + PAGE_TOKENS > lo_wave;   // some row sees some key
    bf16x8 p[RP][2];
    if (sees) {
      float alpha[RP];
      bool moved[RP];
      f32x4 s[RP][4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int u = 0; u < RP; ++u) s[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          const bf16x8 a = *(const bf16x8*)(k_lds + 16 * t * (2 * DIRECT_D) + k_at[kb]);
#pragma unroll
          for (int u = 0; u < RP; ++u) s[u][t] = MFMA16(a, st[u].q[kb], s[u][t]);
        }
      }
#pragma unroll
      for (int u = 0; u < RP; ++u) {
        const bool masked = key0 + PAGE_TOKENS - 1 > pos0[u] || rows[u] < 16 ||
                            (window > 0 && key0 < pos0[u] + 15 - window + 1);
        alpha[u] = masked ? page_softmax<KB, true>(st[u], s[u], p[u], scale_log2, key0, lo_row[u], pos_row[u], moved[u])
                          : page_softmax<KB, false>(st[u], s[u], p[u], scale_log2, key0, lo_row[u], pos_row[u], moved[u]);
      }
#pragma unroll
      for (int u = 0; u < RP; ++u)
        if (moved[u]) {                                       // rare once the maxima have settled
#pragma unroll
          for (int dt = 0; dt < 2 * KB; ++dt) st[u].o[dt] *= alpha[u];
        }
    }
    if (!TWO) {
      wait_direct_loads();
      __syncthreads();                                       // the values are in LDS; every wave is done with the keys
      if (page >= 0) direct_page(k_pages + ((int64_t)page * n_kv + kvh) * page_elems, k_from, lds0);
    }
    if (sees) {
#pragma unroll
      for (int dt = 0; dt < 2 * KB; ++dt)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const bf16x8 a = *(const bf16x8*)(v_lds + 16 * dt * (2 * PAGE_TOKENS) + v_at[h]);
#pragma unroll
          for (int u = 0; u < RP; ++u) st[u].o[dt] = MFMA16(a, p[u][h], st[u].o[dt]);
        }
    }
  }
  float row_l[RP];
#pragma unroll
  for (int u = 0; u < RP; ++u) row_l[u] = row_sum<KB>(st[u]);
#pragma unroll
  for (int u = 0; u < RP; ++u) {
    if (!row_valid[u]) continue;
    const float inv = 1.f / row_l[u];
    bf16_t* o = out + (row[u] * n_heads + head) * head_dim;
#pragma unroll
    for (int dt = 0; dt < 2 * KB; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[16 * dt + 4 * g + i] = float_to_bf16(st[u].o[dt][i] * inv);
  }
}

// ---------------------------------------------------------------------------------------------------
// One row per sequence. Grid: (sequences, kv heads * head blocks, splits); four waves per workgroup.
// The 16 "rows" of a wave are up to 16 query heads that share the kv head. A split covers a run of
// pages; its waves take them in turn, each page's loads issued before the previous page's second
// product so that memory stays busy, and merge their results in LDS. Each split writes an
// unnormalised partial (o, m, l); the combine kernel merges splits in a fixed order, so results do
// not depend on timing.
// One q or k head of one row, as the fused projection left it: RMSNorm over the head (optional), then the
// rotation of pairs (j, j + rot/2), with the same roundings as the stand-alone kernel (rope_kv.hip). One wave, in
// two halves so that a caller can put other loads between them: `head_load` issues every load (head_dim <= 256:
// at most 4 values per lane), `head_finish` computes. `tmp` is the wave's own LDS scratch of head_dim floats. The
// result is written as bfloat16 to `dst` (in LDS) and, if given, to `dst2` (in global memory).
struct HeadRegs {
  float x[4], wt[4], cs[4], sn[4];
};

// Where a row of the fused projection's output lies: as bfloat16 values, or as `parts` float partial sums over K,
// `part_stride` values apart, which are added up in order here and rounded as the product's own epilogue would.
struct ProjectedRow {
  const bf16_t* values;
  const float* sums;
  int parts;
  int64_t part_stride;
  __device__ __forceinline__ float at(int64_t i) const {
    if (sums == nullptr) return bf16_to_float(values[i]);
    float v = sums[i];
    for (int s = 1; s < parts; ++s) v += sums[s * part_stride + i];
    return rounded_as<bf16_t>(v);
  }
};

__device__ __forceinline__ void head_load(HeadRegs& r, const ProjectedRow& src, int64_t first, const void* __restrict__ w,
                                          int w_f32, int has_norm, const bf16_t* __restrict__ cos_t,
                                          const bf16_t* __restrict__ sin_t, int rot, int pos, int head_dim) {
  const int lane = threadIdx.x % WAVE;
  const int half = rot / 2;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int i = lane + WAVE * u;
    const bool in = i < head_dim;
    r.x[u] = in ? src.at(first + i) : 0.f;
    r.wt[u] = (in && has_norm) ? load_vector(w, i, w_f32) : 1.f;
    const int j = i < half ? i : i - half;
    r.cs[u] = (in && i < rot) ? bf16_to_float(cos_t[(int64_t)pos * half + j]) : 1.f;
    r.sn[u] = (in && i < rot) ? bf16_to_float(sin_t[(int64_t)pos * half + j]) : 0.f;
  }
}

__device__ __forceinline__ void head_finish(HeadRegs& r, int has_norm, float eps, int rot, int head_dim, float* tmp,
                                            bf16_t* dst, bf16_t* dst2) {
  const int lane = threadIdx.x % WAVE;
  const int half = rot / 2;
  if (has_norm) {
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) ss += r.x[u] * r.x[u];
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / (float)head_dim + eps);
#pragma unroll
    for (int u = 0; u < 4; ++u) r.x[u] = rounded_as<bf16_t>(rounded_as<bf16_t>(r.x[u] * inv) * r.wt[u]);
  }
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (lane + WAVE * u < head_dim) tmp[lane + WAVE * u] = r.x[u];
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int i = lane + WAVE * u;
    if (i >= head_dim) continue;
    float o = r.x[u];
    if (i < rot) {
      const float other = tmp[i < half ? i + half : i - half];
      const float a = rounded_as<bf16_t>(o * r.cs[u]), b = rounded_as<bf16_t>(other * r.sn[u]);
      o = i < half ? a - b : a + b;
    }
    const bf16_t v = float_to_bf16(o);
    dst[i] = v;
    if (dst2 != nullptr) dst2[i] = v;
  }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");   // the next head of this wave reuses tmp
  __builtin_amdgcn_wave_barrier();
}

// What the fused form of the split kernel needs to do the work of the norm/rotation/append kernel itself.
struct FusedQKV {
  const bf16_t* qkv;       // [rows, stride]: q heads, k heads, v heads of each row; null: q is given ready
  int64_t stride;
  int parts;               // > 0: qkv points to float partial sums [parts, rows, stride] instead
  int64_t part_stride;     // values from one partial sum to the next
  const void* q_w;
  const void* k_w;
  int w_f32, has_norm;
  float eps;
  const bf16_t* cos_t;
  const bf16_t* sin_t;
  int rot;
  int write_kv;
};

#define SPLIT_WAVES 4
#define SPLIT_MAX_D 256

template <int KB, bool FULL>
// The fused form appends the row's key and value through k_pages_w / v_pages_w, which are the same buffers as
// k_pages / v_pages: none of the four is declared restrict.
__global__ __launch_bounds__(64 * SPLIT_WAVES, 2) void attn_split_kernel(
    const bf16_t* __restrict__ q, const bf16_t* k_pages, const bf16_t* v_pages,
    const int* __restrict__ page_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_rows, const int* __restrict__ kv_len, float* __restrict__ part_o,
    float* __restrict__ part_ml, int n_heads, int n_kv, int head_dim, float scale, int window, int n_splits,
    FusedQKV fused, bf16_t* k_pages_w, bf16_t* v_pages_w, bf16_t* __restrict__ out) {
  __shared__ float merge_o[SPLIT_WAVES][16][32 * KB + 1];
  __shared__ float merge_ml[SPLIT_WAVES][16][2];
  __shared__ __attribute__((aligned(16))) bf16_t q_lds[16][32 * KB];
  __shared__ __attribute__((aligned(16))) bf16_t kv_new[2][32 * KB];   // the row's own key (normed, rotated) and value
  const int seq = blockIdx.x, split = blockIdx.z;
  const int group = n_heads / n_kv, blocks = (group + 15) / 16;
  const int kvh = blockIdx.y / blocks, hb = blockIdx.y % blocks;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int slot = seq_slot[seq];
  const int head = kvh * group + hb * 16 + c;
  const bool row_valid = hb * 16 + c < group;
  const int64_t row = cu_rows[seq];
  // pages of this split, taken by its waves in turn
  int pos = 0, lo = 0, pg = 0, pg1 = -1, pg_hi = 0, pg_first = 0;
  const int* table = page_table + (int64_t)max(slot, 0) * max_pages;
  if (slot >= 0) {
    pos = kv_len[seq] - 1;                                     // the row's own position
    lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int pg_lo = lo / PAGE_TOKENS;
    pg_hi = pos / PAGE_TOKENS;
    const int per = (pg_hi - pg_lo + n_splits) / n_splits;     // ceil(pages / splits)
    pg1 = min(pg_hi, pg_lo + split * per + per - 1);
    pg_first = pg_lo + split * per;
    pg = pg_first + wave;
  }
  const float scale_log2 = scale * 1.44269504088896340736f;
  const int64_t page_elems = (int64_t)PAGE_TOKENS * head_dim;
  PageK<KB> kf;
  PageV<KB> vf;
  int page = pg <= pg1 ? table[pg] : -1;
  RowBlock<KB> st;
  bool values_asked = false;                      // the values of the wave's first page are on their way already
  const bool fused_on = fused.qkv != nullptr;
  // exactly one split has the row's own page among its pages (splits past the sequence's end have none)
  const bool owns_last = fused_on && slot >= 0 && pg_first <= pg_hi && pg1 == pg_hi;
  if (fused_on) {
    // The row's q, k and v come straight from the projection. The waves norm and rotate the query heads this
    // workgroup serves into LDS. The workgroup whose pages include the row's own position also norms and rotates
    // the new key, appends key and value to the cache, and keeps both in LDS: the wave that reads that page puts
    // them into its operands itself, so nothing has to wait for memory. The loads of a wave's first head are
    // issued before those of its first page of keys and waited for first, so the two latencies overlap.
    float* tmp = &merge_o[wave][0][0];                          // free until the merge
    ProjectedRow src_row;
    src_row.values = fused.parts > 0 ? nullptr : fused.qkv + row * fused.stride;
    src_row.sums = fused.parts > 0 ? (const float*)fused.qkv + row * fused.stride : nullptr;
    src_row.parts = fused.parts;
    src_row.part_stride = fused.part_stride;
    HeadRegs first;
    const bool has_first = slot >= 0 && wave < group;
    if (has_first)
      head_load(first, src_row, (int64_t)(kvh * group + wave) * head_dim, fused.q_w, fused.w_f32, fused.has_norm,
                fused.cos_t, fused.sin_t, fused.rot, pos, head_dim);
    if (page >= 0) {
      // the first page's values too: asked for behind the barrier below they would cost a trip to memory of their own
      load_page_k<KB, FULL>(kf, k_pages + ((int64_t)page * n_kv + kvh) * page_elems, head_dim);
      load_page_v<KB, FULL>(vf, v_pages + ((int64_t)page * n_kv + kvh) * page_elems, head_dim);
      values_asked = true;
    }
    if (has_first)
      head_finish(first, fused.has_norm, fused.eps, fused.rot, head_dim, tmp, &q_lds[wave][0], nullptr);
    if (slot >= 0) {
      for (int r = wave + SPLIT_WAVES; r < group; r += SPLIT_WAVES) {
        HeadRegs more;
        head_load(more, src_row, (int64_t)(kvh * group + r) * head_dim, fused.q_w, fused.w_f32, fused.has_norm,
                  fused.cos_t, fused.sin_t, fused.rot, pos, head_dim);
        head_finish(more, fused.has_norm, fused.eps, fused.rot, head_dim, tmp, &q_lds[r][0], nullptr);
      }
      if (owns_last) {
        const int page_last = table[pg_hi];
        const int64_t base = ((int64_t)max(page_last, 0) * n_kv + kvh) * page_elems;
        const int at = pos % PAGE_TOKENS;
        const bool store = fused.write_kv && page_last >= 0;
        if (wave == SPLIT_WAVES - 1) {
          HeadRegs key;
          head_load(key, src_row, (int64_t)(n_heads + kvh) * head_dim, fused.k_w, fused.w_f32, fused.has_norm,
                    fused.cos_t, fused.sin_t, fused.rot, pos, head_dim);
          head_finish(key, fused.has_norm, fused.eps, fused.rot, head_dim, tmp, &kv_new[0][0],
                      store ? k_pages_w + base + (int64_t)at * head_dim : nullptr);
        }
        if (wave == SPLIT_WAVES - 2) {
          const int64_t vs = (int64_t)(n_heads + n_kv + kvh) * head_dim;
          for (int i = lane; i < head_dim; i += WAVE) {
            const bf16_t v = float_to_bf16(src_row.at(vs + i));
            kv_new[1][i] = v;
            if (store) v_pages_w[base + (int64_t)i * PAGE_TOKENS + value_column(at)] = v;
          }
        }
      }
    }
    __syncthreads();
    init_rows<KB>(st, &q_lds[c][0], row_valid && slot >= 0, head_dim);
  } else {
    if (page >= 0) load_page_k<KB, FULL>(kf, k_pages + ((int64_t)page * n_kv + kvh) * page_elems, head_dim);
    init_rows<KB>(st, q + (row * n_heads + head) * head_dim, row_valid && slot >= 0, head_dim);
  }
  while (pg <= pg1) {
    const int pg_next = pg + SPLIT_WAVES;
    const int page_next = pg_next <= pg1 ? table[pg_next] : -1;
    if (page >= 0) {
      if (!values_asked) load_page_v<KB, FULL>(vf, v_pages + ((int64_t)page * n_kv + kvh) * page_elems, head_dim);
      values_asked = false;
      if (fused_on && fused.write_kv && pg == pg_hi) {
        // this page holds the row's own position, whose key and value may not have reached memory yet: take them
        // from LDS. Key `at` is row at%16 of key tile at/16; as a value it is one element of one lane group.
        const int at = pos % PAGE_TOKENS;
        if (c == at % 16) {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (t == at / 16) {
#pragma unroll
              for (int kb = 0; kb < KB; ++kb) {
                const int d = FULL ? 32 * kb + 8 * g : min(32 * kb + 8 * g, head_dim - 8);
                kf.k[t][kb] = load8(&kv_new[0][d]);
              }
            }
        }
        const int col = value_column(at), hsel = col / 32, gsel = (col % 32) / 8, esel = col % 8;
        if (g == gsel) {
#pragma unroll
          for (int dt = 0; dt < 2 * KB; ++dt) {
            const int d = FULL ? 16 * dt + c : min(16 * dt + c, head_dim - 1);
            const __bf16 nv = __builtin_bit_cast(__bf16, kv_new[1][d].bits);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (h == hsel && e == esel) vf.v[dt][h][e] = nv;
          }
        }
      }
      f32x4 s[4];
      page_scores<KB>(s, kf, st);
      if (page_next >= 0)
        load_page_k<KB, FULL>(kf, k_pages + ((int64_t)page_next * n_kv + kvh) * page_elems, head_dim);
      page_update<KB>(st, s, vf, head_dim, scale_log2, pg * PAGE_TOKENS, lo, pos);
    } else if (page_next >= 0) {
      load_page_k<KB, FULL>(kf, k_pages + ((int64_t)page_next * n_kv + kvh) * page_elems, head_dim);
    }
    pg = pg_next;
    page = page_next;
  }
  // merge the four waves' results: o = sum_w 2^(m_w - m) o_w, l likewise
  const float l_wave = row_sum<KB>(st);
  if (row_valid) {
#pragma unroll
    for (int dt = 0; dt < 2 * KB; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) merge_o[wave][c][16 * dt + 4 * g + i] = st.o[dt][i];
    if (g == 0) {
      merge_ml[wave][c][0] = st.m;
      merge_ml[wave][c][1] = l_wave;
    }
  }
  __syncthreads();
  const int rows = min(16, group - hb * 16);
  for (int idx = threadIdx.x; idx < rows * head_dim; idx += blockDim.x) {     // all heads of the block at once
    const int r = idx / head_dim, d = idx % head_dim;
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < SPLIT_WAVES; ++w) m = fmaxf(m, merge_ml[w][r][0]);
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < SPLIT_WAVES; ++w) {
      const float mw = merge_ml[w][r][0];
      const float wgt = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - m);
      l += wgt * merge_ml[w][r][1];
      o += wgt * merge_o[w][r][d];
    }
    if (n_splits == 1) {                                   // nothing to combine: this is the result
      out[(row * n_heads + kvh * group + hb * 16 + r) * head_dim + d] = float_to_bf16(l > 0.f ? o / l : 0.f);
      continue;
    }
    const int64_t at = ((int64_t)seq * n_heads + kvh * group + hb * 16 + r) * n_splits + split;
    part_o[at * head_dim + d] = o;
    if (d == 0) {
      part_ml[at * 2] = m;       // in units of log2(e)
      part_ml[at * 2 + 1] = l;
    }
  }
}

// out[seq_row, head, :] = sum_s w_s o_s / sum_s w_s l_s,  w_s = 2^(m_s - max m)  (attn_decode.py:102-118)
#define COMBINE_MAX_SPLITS 64
#define COMBINE_THREADS 128          // head sizes up to 256: two features a thread
template <int COMBINE_HELD>          // how many splits a thread asks for before it knows their weights
__global__ __launch_bounds__(COMBINE_THREADS) void attn_combine_kernel(const float* __restrict__ part_o,
                                                           const float* __restrict__ part_ml,
                                                           const int* __restrict__ seq_slot,
                                                           const int* __restrict__ cu_rows, bf16_t* __restrict__ out,
                                                           int n_heads, int head_dim, int n_splits) {
  __shared__ float wgt[COMBINE_MAX_SPLITS];
  __shared__ float inv_l;
  const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int64_t row = cu_rows[seq];
  bf16_t* o = out + (row * n_heads + head) * head_dim;
  const float* ml = part_ml + ((int64_t)seq * n_heads + head) * n_splits * 2;
  const float* po = part_o + ((int64_t)seq * n_heads + head) * n_splits * head_dim;
  const bool live = seq_slot[seq] >= 0;
  // The partial outputs are asked for before the weights are known, so that one trip to memory serves both (the
  // kernel moves almost nothing: what it costs is its trips to memory one after the other). A thread holds the first
  // COMBINE_HELD splits of its (at most two) features; further splits are read after the weights.
  float held[2][COMBINE_HELD];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int d = min(tid + k * COMBINE_THREADS, head_dim - 1);        // every load unconditional, from a valid place
#pragma unroll
    for (int s = 0; s < COMBINE_HELD; ++s) held[k][s] = po[min(s, n_splits - 1) * head_dim + d];
  }
  if (tid < WAVE) {                       // the first wave turns (m_s, l_s) into weights
    const float ms = (live && tid < n_splits) ? ml[2 * tid] : -INFINITY;
    const float ls = (live && tid < n_splits) ? ml[2 * tid + 1] : 0.f;
    const float m = wave_max(ms);
    const float w = (ms == -INFINITY) ? 0.f : exp2f(ms - m);
    const float l = wave_sum(w * ls);
    if (tid < n_splits) wgt[tid] = w;
    if (tid == 0) inv_l = l > 0.f ? 1.f / l : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int d = tid + k * COMBINE_THREADS;
    if (d >= head_dim) continue;
    float num = 0.f;
#pragma unroll
    for (int s = 0; s < COMBINE_HELD; ++s)
      if (s < n_splits) num += wgt[s] * held[k][s];      // a split without keys has weight 0 and holds finite values
    for (int s = COMBINE_HELD; s < n_splits; ++s) num += wgt[s] * po[s * head_dim + d];
    o[d] = float_to_bf16(num * inv_l);
  }
}

#define DISPATCH_KB(KBV, CALL)                                                      \
  switch (KBV) {                                                                    \
    case 1: { constexpr int KB = 1; CALL; } break;                                  \
    case 2: { constexpr int KB = 2; CALL; } break;                                  \
    case 3: { constexpr int KB = 3; CALL; } break;                                  \
    case 4: { constexpr int KB = 4; CALL; } break;                                  \
    case 5: { constexpr int KB = 5; CALL; } break;                                  \
    case 6: { constexpr int KB = 6; CALL; } break;                                  \
    case 7: { constexpr int KB = 7; CALL; } break;                                  \
    case 8: { constexpr int KB = 8; CALL; } break;                                  \
    default: return -1;                                                             \
  }

static int head_shape_ok(int n_heads, int n_kv, int head_dim) {
  return head_dim > 0 && head_dim % 16 == 0 && head_dim <= 256 && n_kv > 0 && n_heads % n_kv == 0;
}

template <int GP, int RP>
static int launch_causal(const void* q, const void* k_pages, const void* v_pages, const int* page_table, int max_pages,
                         const int* seq_slot, const int* cu_rows, const int* tile_cu, const int* seq_start, int n_seqs,
                         int max_tiles, void* out, int n_heads, int n_kv, int head_dim, float scale, int window,
                         hipStream_t stream) {
  dim3 grid((max_tiles + 1) / 2, n_heads / GP), block(256);
  // max_tiles bounds the 64-row tiles of the sequences that take part. Tiles of 128 rows: a sequence with t
  // 64-row tiles has (t + 1) / 2 of them, so all together at most (max_tiles + n_seqs) / 2.
  if (GP == 1) grid = dim3(n_heads, RP == 1 ? max_tiles : (max_tiles + n_seqs + 1) / 2);
  if (grid.y > 65535) return -1;
  // two pages of keys [64][D+8] and two of values [D][64+8] (one with one unit per wave)
  const size_t lds = (2 * (size_t)PAGE_TOKENS * (head_dim + K_PAD) + (GP * RP == 1 ? 1 : 2) * (size_t)head_dim * (PAGE_TOKENS + V_PAD)) * 2;
#define LAUNCH_CAUSAL(FULLV)                                                                                       \
  {                                                                                                                \
    auto kernel = attn_causal_kernel<KB, FULLV, GP, RP>;                                                           \
    if (lds > 64 * 1024 &&                                                                                          \
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
      return -1;                                                                                                   \
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, (const bf16_t*)q, (const bf16_t*)k_pages,                 \
                       (const bf16_t*)v_pages, page_table, max_pages, seq_slot, cu_rows, tile_cu, seq_start, n_seqs, \
                       (bf16_t*)out, n_heads, n_kv, head_dim, scale, window);                                      \
  }
  if (head_dim % 32 == 0) {
    DISPATCH_KB(head_dim / 32, LAUNCH_CAUSAL(true));
  } else {
    DISPATCH_KB((head_dim + 31) / 32, LAUNCH_CAUSAL(false));
  }
#undef LAUNCH_CAUSAL
  return DRYFT_LAUNCH_CHECK();
}

template <int RP>
static int launch_causal_direct(const void* q, const void* k_pages, const void* v_pages, const int* page_table,
                                int max_pages, const int* seq_slot, const int* cu_rows, const int* tile_cu,
                                const int* seq_start, int n_seqs, int max_tiles, void* out, int n_heads, int n_kv,
                                float scale, int window, ProjectedQ projected, hipStream_t stream) {
  // max_tiles bounds the 64-row tiles of the sequences that take part; a sequence with t of them has ceil(t / RP)
  dim3 grid(n_heads, (max_tiles + (RP - 1) * (n_seqs + 1)) / RP), block(256);
  if (grid.y > 65535) return -1;
  const size_t lds = (size_t)(RP == 1 ? 2 : 4) * DIRECT_PAGE_BYTES;
  hipLaunchKernelGGL(attn_causal_direct_kernel<RP>, grid, block, lds, stream, (const bf16_t*)q, (const bf16_t*)k_pages,
                     (const bf16_t*)v_pages, page_table, max_pages, seq_slot, cu_rows, tile_cu, seq_start, n_seqs,
                     (bf16_t*)out, n_heads, n_kv, scale, window, projected);
  return DRYFT_LAUNCH_CHECK();
}

// mode: 0 = chosen here; 1 = one head and 16 rows per wave; 2 = two heads of a kv group per wave (even groups,
// head_dim <= 128); 3 = one head and 32 rows per wave (head_dim <= 128). At head size 128, modes 1 and 3 bring
// the pages straight into LDS; 5 and 7 are 1 and 3 with the pages staged through registers, as at other sizes.
static int causal_entry(const void* q, const void* k_pages, const void* v_pages, const int* page_table, int max_pages,
                        const int* seq_slot, const int* cu_rows, const int* tile_cu, const int* seq_start, int n_seqs,
                        int max_tiles, void* out, int n_heads, int n_kv, int head_dim, float scale, int window, int mode,
                        ProjectedQ projected, hipStream_t stream) {
  if (n_seqs <= 0 || max_tiles <= 0) return 0;
  if (!head_shape_ok(n_heads, n_kv, head_dim)) return -1;
  const int group = n_heads / n_kv;
  const bool staged = mode == 5 || mode == 7;
  if (staged) mode -= 4;
  if (mode < 0 || mode > 3 || (mode == 2 && (group % 2 || head_dim > 128)) || (mode == 3 && head_dim > 128)) return -1;
  const bool direct_ok = head_dim == DIRECT_D && (((uintptr_t)k_pages | (uintptr_t)v_pages) & 15) == 0;
  if (mode == 0) {
    // Two units per wave (twice the rows of one head, or two heads of a kv group) use every piece of a page that
    // is read from LDS twice; they also halve the number of workgroups, so they need four of them for every
    // compute unit. Measured on Qwen3-4B's heads, PFLOP/s with 16 rows / 32 rows / two heads per wave, pages
    // staged through registers, one sequence: 0.46 / 0.40 / 0.34 at 2,048 positions, 0.55 / 0.53 / 0.45 at 3,000,
    // 0.59 / 0.72 / 0.62 at 4,096, 0.63 / 0.77 / 0.69 at 8,192, 0.71 / 0.92 / 0.78 at 30,000; eight sequences of 2,048:
    // 0.58 / 0.67. With the pages straight into LDS, 16 rows a wave put four workgroups on a compute unit and stay
    // ahead while sequences are short: 16 / 32 rows a wave 0.57 / 0.51 at 2,048 positions, 0.71 / 0.62 at 3,000,
    // 0.82 / 0.80 at 4,096, 0.84 / 0.88 at 8,192, 1.00 / 1.07 at 30,000; eight sequences of 2,048: 0.84 / 0.75, two of
    // 4,096: 0.93 / 0.98. (Two heads per wave stay available as mode 2; nothing chooses them.)
    const bool enough = (int64_t)((max_tiles + 1) / 2) * n_heads >= 1024;
    const bool long_ones = (int64_t)max_tiles >= 64 * (int64_t)n_seqs;          // 4,096 rows a sequence on average
    mode = head_dim <= 128 && enough && (!direct_ok || long_ones) ? 3 : 1;
  }
#define CAUSAL(GPV, RPV)                                                                                          \
  return launch_causal<GPV, RPV>(q, k_pages, v_pages, page_table, max_pages, seq_slot, cu_rows, tile_cu, seq_start, \
                                 n_seqs, max_tiles, out, n_heads, n_kv, head_dim, scale, window, stream)
  if (direct_ok && !staged && mode != 2) {
    if (mode == 3)
      return launch_causal_direct<2>(q, k_pages, v_pages, page_table, max_pages, seq_slot, cu_rows, tile_cu, seq_start,
                                     n_seqs, max_tiles, out, n_heads, n_kv, scale, window, projected, stream);
    return launch_causal_direct<1>(q, k_pages, v_pages, page_table, max_pages, seq_slot, cu_rows, tile_cu, seq_start,
                                   n_seqs, max_tiles, out, n_heads, n_kv, scale, window, projected, stream);
  }
  if (projected.qkv != nullptr) return -1;                   // only the kernel above takes the projection itself
  if (mode == 2) CAUSAL(2, 1);
  if (mode == 3) CAUSAL(1, 2);
  CAUSAL(1, 1);
#undef CAUSAL
}

DRYFT_API int dryft_attn_causal_bf16(const void* q, const void* k_pages, const void* v_pages, const int* page_table,
                                     int max_pages, const int* seq_slot, const int* cu_rows, const int* tile_cu,
                                     const int* seq_start, int n_seqs, int max_tiles, void* out, int n_heads,
                                     int n_kv, int head_dim, float scale, int window, int mode, hipStream_t stream) {
  ProjectedQ none = {};
  return causal_entry(q, k_pages, v_pages, page_table, max_pages, seq_slot, cu_rows, tile_cu, seq_start, n_seqs,
                      max_tiles, out, n_heads, n_kv, head_dim, scale, window, mode, none, stream);
}

// Can the causal kernel take the queries from the fused projection itself (norm, rotation over `rot` features)?
DRYFT_API int dryft_attn_causal_takes_projection(int head_dim, int rot) { return head_dim == DIRECT_D && rot == DIRECT_D; }

// The same with the queries taken from the projection output qkv[rows, stride] (query heads first): per-head
// RMSNorm with q_w (has_norm) and rotation by the tables cos_t / sin_t [positions, head_dim / 2] happen on the way
// into the kernel's registers. Only where dryft_attn_causal_takes_projection says so; mode 0, 1 or 3.
DRYFT_API int dryft_attn_causal_projected_bf16(const void* qkv, int64_t qkv_stride, const void* q_w, int w_f32,
                                               int has_norm, float eps, const void* cos_t, const void* sin_t,
                                               const void* k_pages, const void* v_pages, const int* page_table,
                                               int max_pages, const int* seq_slot, const int* cu_rows,
                                               const int* tile_cu, const int* seq_start, int n_seqs, int max_tiles,
                                               void* out, int n_heads, int n_kv, int head_dim, float scale, int window,
                                               int mode, hipStream_t stream) {
  if (qkv == nullptr || cos_t == nullptr || sin_t == nullptr || (has_norm && q_w == nullptr)) return -1;
  if (head_dim != DIRECT_D || (mode != 0 && mode != 1 && mode != 3) || qkv_stride % 8 || ((uintptr_t)qkv & 15)) return -1;
  ProjectedQ projected = {(const bf16_t*)qkv, qkv_stride, q_w, w_f32, has_norm, eps, (const bf16_t*)cos_t, (const bf16_t*)sin_t};
  return causal_entry(nullptr, k_pages, v_pages, page_table, max_pages, seq_slot, cu_rows, tile_cu, seq_start, n_seqs,
                      max_tiles, out, n_heads, n_kv, head_dim, scale, window, mode, projected, stream);
}

static int launch_split(const void* q, const void* k_pages, const void* v_pages, const int* page_table, int max_pages,
                        const int* seq_slot, const int* cu_rows, const int* kv_len, int n_seqs, float* part_o,
                        float* part_ml, int n_splits, void* out, int n_heads, int n_kv, int head_dim, float scale,
                        int window, FusedQKV fused, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (!head_shape_ok(n_heads, n_kv, head_dim) || n_splits < 1 || n_splits > COMBINE_MAX_SPLITS) return -1;
  const int group = n_heads / n_kv, blocks = (group + 15) / 16;
  if (fused.qkv != nullptr && (blocks != 1 || fused.rot > head_dim || (fused.rot & 1))) return -1;
  dim3 grid(n_seqs, n_kv * blocks, n_splits), block(64 * SPLIT_WAVES);
#define LAUNCH_SPLIT(FULLV)                                                                                        \
  hipLaunchKernelGGL((attn_split_kernel<KB, FULLV>), grid, block, 0, stream, (const bf16_t*)q, (const bf16_t*)k_pages, \
                     (const bf16_t*)v_pages, page_table, max_pages, seq_slot, cu_rows, kv_len, part_o, part_ml,    \
                     n_heads, n_kv, head_dim, scale, window, n_splits, fused, (bf16_t*)k_pages, (bf16_t*)v_pages,       \
                     (bf16_t*)out)
  if (head_dim % 32 == 0) {
    DISPATCH_KB(head_dim / 32, LAUNCH_SPLIT(true));
  } else {
    DISPATCH_KB((head_dim + 31) / 32, LAUNCH_SPLIT(false));
  }
#undef LAUNCH_SPLIT
  int rc = DRYFT_LAUNCH_CHECK();
  if (rc || n_splits == 1) return rc;
#define COMBINE(HELD)                                                                                              \
  hipLaunchKernelGGL(attn_combine_kernel<HELD>, dim3(n_seqs, n_heads), dim3(COMBINE_THREADS), 0, stream, part_o,   \
                     part_ml, seq_slot, cu_rows, (bf16_t*)out, n_heads, head_dim, n_splits)
  if (n_splits <= 4) COMBINE(4);
  else if (n_splits <= 8) COMBINE(8);
  else if (n_splits <= 16) COMBINE(16);
  else COMBINE(32);
#undef COMBINE
  return DRYFT_LAUNCH_CHECK();
}

DRYFT_API int dryft_attn_split_bf16(const void* q, const void* k_pages, const void* v_pages, const int* page_table,
                                    int max_pages, const int* seq_slot, const int* cu_rows, const int* kv_len,
                                    int n_seqs, float* part_o, float* part_ml, int n_splits, void* out, int n_heads,
                                    int n_kv, int head_dim, float scale, int window, hipStream_t stream) {
  FusedQKV none = {};
  return launch_split(q, k_pages, v_pages, page_table, max_pages, seq_slot, cu_rows, kv_len, n_seqs, part_o, part_ml,
                      n_splits, out, n_heads, n_kv, head_dim, scale, window, none, stream);
}

// The same with the work of the norm/rotation/append kernel folded in: `qkv` is the fused projection's output
// for one row per sequence, as bfloat16 [rows, qkv_stride] (qkv_parts 0) or as qkv_parts float partial sums over K,
// [qkv_parts, rows, qkv_stride] with qkv_part_stride values from one to the next, which the kernel adds up in order
// and rounds on its way in. Takes kv groups of at most 16 query heads.
DRYFT_API int dryft_attn_decode_fused_bf16(const void* qkv, int64_t qkv_stride, int qkv_parts, int64_t qkv_part_stride,
                                           const void* q_w, const void* k_w,
                                           int w_f32, int has_norm, float eps, const void* cos_t, const void* sin_t,
                                           int rot, int write_kv, void* k_pages, void* v_pages, const int* page_table,
                                           int max_pages, const int* seq_slot, const int* cu_rows, const int* kv_len,
                                           int n_seqs, float* part_o, float* part_ml, int n_splits, void* out,
                                           int n_heads, int n_kv, int head_dim, float scale, int window,
                                           hipStream_t stream) {
  if (qkv == nullptr || qkv_parts < 0) return -1;
  FusedQKV fused = {(const bf16_t*)qkv, qkv_stride, qkv_parts, qkv_part_stride, q_w, k_w, w_f32, has_norm, eps,
                    (const bf16_t*)cos_t, (const bf16_t*)sin_t, rot, write_kv};
  return launch_split(nullptr, k_pages, v_pages, page_table, max_pages, seq_slot, cu_rows, kv_len, n_seqs, part_o,
                      part_ml, n_splits, out, n_heads, n_kv, head_dim, scale, window, fused, stream);
}
