// Reductions over partial blocks: N-way online-softmax (out, lse) merge and
// N-way block sum, each fused with the scatter into its destination.
// Both are HBM-bound: every source element is read once with a 16-byte load,
// accumulated in fp32 registers and written once.
#include <math.h>

#include "common.h"

namespace dcp {

template <int DTYPE>
struct Vec16 {
  static constexpr int N = 16 / sizeof(typename Elem<DTYPE>::raw);
};

template <int DTYPE>
__device__ __forceinline__ void fma_vec16(float (&acc)[Vec16<DTYPE>::N], float w, u32x4 bits) {
  if constexpr (DTYPE == DCP_DTYPE_FP32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] += w * __uint_as_float(bits[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[2 * i] += w * Elem<DTYPE>::load((uint16_t)(bits[i] & 0xffffu));
      acc[2 * i + 1] += w * Elem<DTYPE>::load((uint16_t)(bits[i] >> 16));
    }
  }
}

template <int DTYPE>
__device__ __forceinline__ u32x4 pack_vec16(const float (&acc)[Vec16<DTYPE>::N]) {
  u32x4 bits;
  if constexpr (DTYPE == DCP_DTYPE_FP32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) bits[i] = __float_as_uint(acc[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      bits[i] = (uint32_t)Elem<DTYPE>::store(acc[2 * i]) |
                ((uint32_t)Elem<DTYPE>::store(acc[2 * i + 1]) << 16);
  }
  return bits;
}

// Only the two infinities mark an empty source (the reference tests lse != -inf and lse != inf):
// a NaN LSE takes part in the merge and makes the merged LSE and output of its (token, head) NaN.
// fmaxf drops a NaN operand, so the kernels note one and put it into the running maximum themselves.
__device__ __forceinline__ bool lse_is_finite(float l) {
  return l != INFINITY && l != -INFINITY;
}

// ---------------------------------------------------------------------------
// (out, lse) merge.
//
// A group of LPR lanes (a power of two that divides 64, so a group never
// straddles a wave) owns one (token, head) row; lane g of the group handles
// the 16-byte words g, g+LPR, ... of the row.  Every lane of the group reads
// the sources' LSEs itself (same address across the group: one broadcast
// transaction), so no cross-lane traffic is needed.  Because the group sits
// inside one wave and each lane only overwrites elements it has already read,
// the destination may alias a source of the same op.
// grid: ops x (token chunks x heads), one dimension with the chunks of an op side by side:
// workgroups that run at the same time then read neighbouring pieces of the same few blocks
// (with the op as the fastest index, as a two-dimensional grid has it, they are spread over
// all the blocks of the launch at once).
// ---------------------------------------------------------------------------
constexpr int kMergeThreads = 256;
constexpr int kMergeXcds = 8;  // L2 caches (XCDs) of the device; workgroups are dealt to them in turn

// U sources are folded per step and TPG tokens (rows_per_wg apart) are handled by a lane group
// at once: all their U * TPG 16-byte words and LSEs are requested before any arithmetic, which
// is what keeps enough bytes in flight when an op has few sources.
template <int DTYPE, bool VECTOR, int U, int TPG>
__global__ __launch_bounds__(kMergeThreads) void merge_out_lse_kernel(
    const typename Elem<DTYPE>::raw* src_out, typename Elem<DTYPE>::raw* dst_out,
    const float* src_lse, float* dst_lse, int n_head, const int32_t* __restrict__ src_block_table,
    const int32_t* __restrict__ dst_token_offsets, const int32_t* __restrict__ n_tokens_per_block,
    const int32_t* __restrict__ block_lengths, int64_t out_block_stride, int64_t out_token_stride,
    int64_t lse_block_stride, int64_t lse_token_stride, int64_t src_lse_head_stride,
    int64_t dst_lse_head_stride, int head_dim, int max_n_blocks_per_op, int lanes_per_row, int row_chunks) {
  typedef typename Elem<DTYPE>::raw raw;
  constexpr int VN = VECTOR ? Vec16<DTYPE>::N : 1;
  const int op = blockIdx.x / row_chunks;
  const int chunk = blockIdx.x - op * row_chunks;
  const int n_tok = n_tokens_per_block[op];

  // A workgroup takes consecutive tokens of ONE head: its LSE reads and its LSE store are
  // then contiguous floats ([head][token] layout) instead of one 4-byte access per cache
  // line, and every token's head_dim elements are still one contiguous piece.
  const int rows_per_wg = kMergeThreads / lanes_per_row;
  const int h = chunk % n_head;
  const int t0 = (chunk / n_head) * (rows_per_wg * TPG) + threadIdx.x / lanes_per_row;
  const int g = threadIdx.x % lanes_per_row;
  if (t0 >= n_tok) return;

  const int n_src = block_lengths[op];
  const int32_t* table = src_block_table + (int64_t)op * max_n_blocks_per_op;
  const float* lse_head = src_lse + h * src_lse_head_stride;
  const raw* out_head = src_out + (int64_t)h * head_dim;
  const int n_words = head_dim / VN;
  int t[TPG];
  bool live[TPG];
#pragma unroll
  for (int k = 0; k < TPG; ++k) {
    live[k] = t0 + k * rows_per_wg < n_tok;
    t[k] = live[k] ? t0 + k * rows_per_wg : t0;  // a token past the end repeats the first one; never stored
  }

  float row_lse[TPG];  // the same in every iteration over w: it only depends on the LSEs
#pragma unroll
  for (int k = 0; k < TPG; ++k) row_lse[k] = -1.0f;
  // An op with a single source is the scatter-back of a finished block: its finite rows are
  // copied bit for bit (the weighted sum 0 + 1 * x would turn -0.0 into +0.0).
  const bool copy_only = n_src == 1;
  for (int w = g; copy_only && w < n_words; w += lanes_per_row) {
    const int64_t blk = table[0];
#pragma unroll
    for (int k = 0; k < TPG; ++k) {
      const float l = lse_head[t[k] * lse_token_stride + blk * lse_block_stride];
      const raw* p = out_head + t[k] * out_token_stride + blk * out_block_stride + (int64_t)w * VN;
      const bool finite = lse_is_finite(l);
      row_lse[k] = finite ? l : -1.0f;
      if (!live[k]) continue;
      const int64_t dst_tok = (int64_t)dst_token_offsets[op] + t[k];
      raw* q = dst_out + dst_tok * out_token_stride + (int64_t)h * head_dim + (int64_t)w * VN;
      if constexpr (VECTOR) {
        u32x4 x = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        const u32x4 zero = {0, 0, 0, 0};
        __builtin_nontemporal_store(finite ? x : zero, reinterpret_cast<u32x4*>(q));
      } else {
        const raw x = *p;
        *q = finite ? x : Elem<DTYPE>::store(0.0f);
      }
    }
  }
  for (int w = g; !copy_only && w < n_words; w += lanes_per_row) {
    float m[TPG], ssum[TPG], acc[TPG][VN];
#pragma unroll
    for (int k = 0; k < TPG; ++k) {
      m[k] = -INFINITY;
      ssum[k] = 0.0f;
#pragma unroll
      for (int i = 0; i < VN; ++i) acc[k][i] = 0.0f;
    }
    for (int j0 = 0; j0 < n_src; j0 += U) {
      float l[TPG][U];
      u32x4 x[TPG][U];
      raw x1[TPG][U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int j = min(j0 + u, n_src - 1);  // tail: re-read the last source, ignored below
        const int64_t blk = table[j];
#pragma unroll
        for (int k = 0; k < TPG; ++k) {
          l[k][u] = lse_head[t[k] * lse_token_stride + blk * lse_block_stride];
          const raw* p = out_head + t[k] * out_token_stride + blk * out_block_stride + (int64_t)w * VN;
          if constexpr (VECTOR) x[k][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
          else x1[k][u] = *p;
        }
      }
#pragma unroll
      for (int k = 0; k < TPG; ++k) {
        float m_new = m[k];
        bool nan_seen = false;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (j0 + u >= n_src || !lse_is_finite(l[k][u])) l[k][u] = -INFINITY;
          m_new = fmaxf(m_new, l[k][u]);
          nan_seen |= l[k][u] != l[k][u];
        }
        if (nan_seen) m_new = NAN;  // sums and weights below turn NaN and stay so
        if (m_new == -INFINITY) continue;  // nothing finite so far
        const float rescale = expf(m[k] - m_new);  // m = -inf -> 0
        ssum[k] *= rescale;
#pragma unroll
        for (int i = 0; i < VN; ++i) acc[k][i] *= rescale;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const float wgt = expf(l[k][u] - m_new);  // ignored source: exp(-inf) = 0, but its data may be
          if (l[k][u] == -INFINITY) continue;       // anything, so it is skipped, not multiplied by 0
          ssum[k] += wgt;
          if constexpr (VECTOR) fma_vec16<DTYPE>(acc[k], wgt, x[k][u]);
          else acc[k][0] += wgt * Elem<DTYPE>::load(x1[k][u]);
        }
        m[k] = m_new;
      }
    }
#pragma unroll
    for (int k = 0; k < TPG; ++k) {
      float new_lse = -1.0f;
      if (m[k] != -INFINITY) {
        new_lse = m[k] + logf(ssum[k]);
        const float inv = 1.0f / ssum[k];
#pragma unroll
        for (int i = 0; i < VN; ++i) acc[k][i] *= inv;
      }
      row_lse[k] = new_lse;
      if (!live[k]) continue;
      const int64_t dst_tok = (int64_t)dst_token_offsets[op] + t[k];
      raw* q = dst_out + dst_tok * out_token_stride + (int64_t)h * head_dim + (int64_t)w * VN;
      if constexpr (VECTOR) {
        __builtin_nontemporal_store(pack_vec16<DTYPE>(acc[k]), reinterpret_cast<u32x4*>(q));
      } else {
        *q = Elem<DTYPE>::store(acc[k][0]);
      }
    }
  }
  // after every read of the sources' LSEs (the destination may be one of them)
  if (g == 0) {
#pragma unroll
    for (int k = 0; k < TPG; ++k)
      if (live[k]) dst_lse[h * dst_lse_head_stride + ((int64_t)dst_token_offsets[op] + t[k]) * lse_token_stride] = row_lse[k];
  }
}

// ---------------------------------------------------------------------------
// The same merge for token rows that are dense over the heads, any number of sources (ops of up to
// four sources, which is what plans have, take the one-wave kernel further down); rows dense means
// out_token_stride = n_head * head_dim, and the LSEs are contiguous over tokens.  A workgroup takes
// kRowTokens consecutive tokens of one op with ALL their heads, so that every global access of
// the out data is part of a run of whole token rows (4 KiB per wave instruction at 32 heads x
// 128 bf16) instead of one 256-byte piece per 8 KiB, and works in two phases:
//   A  the sources' LSEs of its (head, token) pairs -> the merged LSE (stored) and one weight
//      exp(l_j - lse*) per (source, head, token), kept in LDS (0 for an ignored source);
//   B  out* = sum_j w_j out_j, 16 bytes per lane and source, kRowUnroll words in flight.
// grid: ops x token chunks, each XCD taking a contiguous eighth of them
// ---------------------------------------------------------------------------
constexpr int kRowTokens = 2;   // measured on 262144 tokens x 32 heads x 128 bf16, four sources: 16 tokens per
constexpr int kRowUnroll = 2;   // workgroup 5.36 TB/s, 4: 5.53, 2: 5.98, 1: 5.69; four words per source in flight: 5.53
constexpr int kRowWeightFloats = 12288;  // LDS for the weights: n_src * n_head * kRowTokens floats at most

template <int DTYPE, int U, int THREADS, int TOKENS, int RU>
__global__ __launch_bounds__(THREADS) void merge_rows_kernel(
    const typename Elem<DTYPE>::raw* src_out, typename Elem<DTYPE>::raw* dst_out, const float* src_lse,
    float* dst_lse, int n_head, const int32_t* __restrict__ src_block_table,
    const int32_t* __restrict__ dst_token_offsets, const int32_t* __restrict__ n_tokens_per_block,
    const int32_t* __restrict__ block_lengths, int64_t out_block_stride, int64_t out_token_stride,
    int64_t lse_block_stride, int64_t src_lse_head_stride, int64_t dst_lse_head_stride, int head_dim,
    int max_n_blocks_per_op, int chunks_per_op, int n_items) {
  typedef typename Elem<DTYPE>::raw raw;
  constexpr int VN = Vec16<DTYPE>::N;
  extern __shared__ float weight[];  // [source][head][token of the chunk]: max_n_blocks_per_op * n_head * TOKENS
  // Workgroups are dealt to the device's eight XCDs in turn.  The ones that land on one XCD take a
  // contiguous eighth of the (op, token chunk) items: the 128-byte line that holds the LSEs of 32
  // consecutive tokens of a (source, head) is then fetched into one L2 instead of all eight, and the
  // merged LSEs of those tokens leave that L2 as one full line.
  const int item = (int)(blockIdx.x % kMergeXcds) * (int)(gridDim.x / kMergeXcds) + (int)(blockIdx.x / kMergeXcds);
  if (item >= n_items) return;
  const int op = item / chunks_per_op;
  const int n_tok = n_tokens_per_block[op];
  const int t0 = (item - op * chunks_per_op) * TOKENS;
  if (t0 >= n_tok) return;
  const int n_src = block_lengths[op];
  const int tid = threadIdx.x;
  const int32_t* slot = src_block_table + (int64_t)op * max_n_blocks_per_op;  // the same for the whole workgroup: scalar loads
  const int64_t dst_tok0 = (int64_t)dst_token_offsets[op] + t0;
  const int plane = n_head * TOKENS;
  const int words_per_head = head_dim / VN;
  const int row_words = n_head * words_per_head;
  const int n_rows = min(TOKENS, n_tok - t0);
  const int total = n_rows * row_words;

  // word i of the chunk: token i / row_words, 16-byte word i % row_words of its row
  auto load_words = [&](u32x4 (&x)[U][RU], const int (&t)[RU], const int (&wd)[RU], int j0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = min(j0 + u, n_src - 1);  // tail: re-read the last source, ignored by the caller
      const raw* base = src_out + (int64_t)slot[j] * out_block_stride + (int64_t)t0 * out_token_stride;
#pragma unroll
      for (int k = 0; k < RU; ++k)
        x[u][k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + (int64_t)t[k] * out_token_stride + (int64_t)wd[k] * VN));
    }
  };
  auto locate = [&](int i0, int (&t)[RU], int (&wd)[RU], bool (&live)[RU]) {
#pragma unroll
    for (int k = 0; k < RU; ++k) {
      const int i = i0 + k * THREADS;
      live[k] = i < total;
      const int ii = live[k] ? i : i0;
      t[k] = ii / row_words;
      wd[k] = ii - t[k] * row_words;
    }
  };

  // The first out words of every lane are requested before the LSEs are looked at: they do not
  // depend on them, and the loads of the two phases are then in flight together.
  int i0 = tid;
  int t[RU], wd[RU];
  bool live[RU];
  u32x4 x[U][RU];
  if (i0 < total) {
    locate(i0, t, wd, live);
    load_words(x, t, wd, 0);
  }

  // ---- phase A --------------------------------------------------------------------------
  for (int pair = tid; pair < plane; pair += THREADS) {
    const int h = pair / TOKENS, tk = pair - h * TOKENS;
    if (t0 + tk >= n_tok) continue;
    const float* lse_row = src_lse + (int64_t)h * src_lse_head_stride + t0 + tk;
    float m = -INFINITY;
    bool nan_seen = false;
    for (int j = 0; j < n_src; ++j) {
      float l = lse_row[(int64_t)slot[j] * lse_block_stride];
      if (!lse_is_finite(l)) l = -INFINITY;
      weight[j * plane + pair] = l;
      m = fmaxf(m, l);
      nan_seen |= l != l;
    }
    if (nan_seen) m = NAN;  // the sum, the merged LSE and every weight of a non-empty source turn NaN
    float new_lse = -1.0f;
    if (m != -INFINITY) {
      float ssum = 0.0f;
      for (int j = 0; j < n_src; ++j) ssum += expf(weight[j * plane + pair] - m);  // ignored source: exp(-inf) = 0
      new_lse = m + logf(ssum);
      // a single source keeps its LSE bit for bit (m + log(1) may round)
      if (n_src == 1) new_lse = weight[pair];
    }
    for (int j = 0; j < n_src; ++j) {
      const float l = weight[j * plane + pair];
      weight[j * plane + pair] = (m == -INFINITY || l == -INFINITY) ? 0.0f : expf(l - new_lse);
    }
    // (after this pair's reads: the destination may be one of its sources)
    dst_lse[(int64_t)h * dst_lse_head_stride + dst_tok0 + tk] = new_lse;
  }
  __syncthreads();

  // ---- phase B --------------------------------------------------------------------------
  const bool copy_only = n_src == 1;  // the scatter-back of a finished block: bits, not 0 + 1 * x
  while (i0 < total) {
    float acc[RU][VN];
#pragma unroll
    for (int k = 0; k < RU; ++k)
#pragma unroll
      for (int e = 0; e < VN; ++e) acc[k][e] = 0.0f;
    u32x4 only[RU];
    for (int j0 = 0; j0 < n_src; j0 += U) {
      if (j0 > 0) load_words(x, t, wd, j0);  // (the first U sources are on their way already)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (j0 + u >= n_src) break;
#pragma unroll
        for (int k = 0; k < RU; ++k) {
          const float w = weight[(j0 + u) * plane + (wd[k] / words_per_head) * TOKENS + t[k]];
          if (w != 0.0f) fma_vec16<DTYPE>(acc[k], w, x[u][k]);  // an ignored source's data may be anything: skipped
          if (u == 0) only[k] = w != 0.0f ? x[0][k] : u32x4{0, 0, 0, 0};
        }
      }
    }
    raw* q[RU];
    bool store[RU];
#pragma unroll
    for (int k = 0; k < RU; ++k) {
      store[k] = live[k];
      q[k] = dst_out + (dst_tok0 + t[k]) * out_token_stride + (int64_t)wd[k] * VN;
    }
    // the next positions' loads go out before this one's stores
    i0 += THREADS * RU;
    if (i0 < total) {
      locate(i0, t, wd, live);
      load_words(x, t, wd, 0);
    }
#pragma unroll
    for (int k = 0; k < RU; ++k)
      if (store[k]) __builtin_nontemporal_store(copy_only ? only[k] : pack_vec16<DTYPE>(acc[k]), reinterpret_cast<u32x4*>(q[k]));
  }
}

// ---------------------------------------------------------------------------
// The same merge, one wave per workgroup, for ops of at most four sources (what plans have): a
// wave takes 64 * RU consecutive 16-byte words of one token row, every lane requests its word of
// all the sources and its (head, token)'s LSEs at once and forms the weights itself (the lanes
// of a quad share the exponentials: with every lane working out all of them the kernel was bound
// by them, 5.89 TB/s).  No LDS, no barrier, nothing serial in front of the loads: 6.13 TB/s on
// 262144 tokens x 32 heads x 128 bf16 with four sources, against 5.6-5.8 for the workgroup kernel
// above and 6.57 with the arithmetic taken out.  A (head, token) must lie within one wave's words
// (the wave reads its LSEs before it stores the merged one, which may replace a source's).
// grid: ops x tokens x pieces of a row, each XCD taking a contiguous eighth (see above)
// ---------------------------------------------------------------------------
// lane j of the caller's aligned group of four lanes hands its value to all four
__device__ __forceinline__ float quad_broadcast(float v, int j) {
  switch (j) {
    case 0: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x00, 0xf, 0xf, true));
    case 1: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x55, 0xf, 0xf, true));
    case 2: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xaa, 0xf, 0xf, true));
    default: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xff, 0xf, 0xf, true));
  }
}

template <int DTYPE, int U, int RU>
__global__ __launch_bounds__(64) void merge_rows_wave_kernel(
    const typename Elem<DTYPE>::raw* src_out, typename Elem<DTYPE>::raw* dst_out, const float* src_lse,
    float* dst_lse, const int32_t* __restrict__ src_block_table, const int32_t* __restrict__ dst_token_offsets,
    const int32_t* __restrict__ n_tokens_per_block, const int32_t* __restrict__ block_lengths,
    int64_t out_block_stride, int64_t out_token_stride, int64_t lse_block_stride, int64_t src_lse_head_stride,
    int64_t dst_lse_head_stride, int words_per_head, int max_n_blocks_per_op, int pieces_per_row, int pieces_per_op,
    int64_t n_items) {
  typedef typename Elem<DTYPE>::raw raw;
  constexpr int VN = Vec16<DTYPE>::N;
  const int64_t item = (int64_t)(blockIdx.x % kMergeXcds) * (gridDim.x / kMergeXcds) + blockIdx.x / kMergeXcds;
  if (item >= n_items) return;
  const int op = (int)(item / pieces_per_op);
  const int r = (int)(item - (int64_t)op * pieces_per_op);
  const int tok = r / pieces_per_row;
  if (tok >= n_tokens_per_block[op]) return;
  const int n_src = block_lengths[op];
  const int32_t* slot = src_block_table + (int64_t)op * max_n_blocks_per_op;
  const int w0 = (r - tok * pieces_per_row) * (64 * RU) + threadIdx.x;
  const int64_t dst_tok = (int64_t)dst_token_offsets[op] + tok;
  if (n_src <= 0) {  // nothing to merge: zeros and the LSE of an empty row
#pragma unroll
    for (int k = 0; k < RU; ++k) {
      const int wd = w0 + 64 * k;
      __builtin_nontemporal_store(u32x4{0, 0, 0, 0}, reinterpret_cast<u32x4*>(dst_out + dst_tok * out_token_stride + (int64_t)wd * VN));
      if (wd % words_per_head == 0) dst_lse[(int64_t)(wd / words_per_head) * dst_lse_head_stride + dst_tok] = -1.0f;
    }
    return;
  }

  u32x4 x[U][RU];
  float l[U][RU];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t blk = slot[min(u, n_src - 1)];  // (past the op's sources: the last one again, ignored below)
    const raw* row = src_out + blk * out_block_stride + (int64_t)tok * out_token_stride;
    const float* lse_tok = src_lse + blk * lse_block_stride + tok;
#pragma unroll
    for (int k = 0; k < RU; ++k) {
      const int wd = w0 + 64 * k;
      x[u][k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + (int64_t)wd * VN));
      l[u][k] = lse_tok[(int64_t)(wd / words_per_head) * src_lse_head_stride];
    }
  }
  const int quad_lane = threadIdx.x & (U >= 4 ? 3 : 1);
#pragma unroll
  for (int k = 0; k < RU; ++k) {
    const int wd = w0 + 64 * k;
    float m = -INFINITY;
    bool nan_seen = false;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (u >= n_src || !lse_is_finite(l[u][k])) l[u][k] = -INFINITY;
      m = fmaxf(m, l[u][k]);
      nan_seen |= l[u][k] != l[u][k];
    }
    if (nan_seen) m = NAN;  // the sum, the merged LSE and every weight of a non-empty source turn NaN
    float new_lse = -1.0f, w[U];
    if constexpr (U == 1) {
      new_lse = m == -INFINITY ? -1.0f : l[0][k];
      w[0] = m == -INFINITY ? 0.0f : 1.0f;
    } else {
      // The four lanes of a quad hold words of one (head, token): lane q works out the
      // exponentials of source q alone and the quad exchanges them (sources past the op's count
      // are -inf and add exp(-inf) = 0).  The sum runs over the sources in order, as in the
      // workgroup kernel, and gives the same bits.
      float mine = l[0][k];
#pragma unroll
      for (int u = 1; u < U; ++u) mine = quad_lane == u ? l[u][k] : mine;
      const float e_mine = expf(mine - m);
      float ssum = 0.0f;
#pragma unroll
      for (int u = 0; u < U; ++u) ssum += quad_broadcast(e_mine, u);
      if (m != -INFINITY) {
        new_lse = m + logf(ssum);
        if (n_src == 1) new_lse = l[0][k];  // a single source keeps its LSE bit for bit (m + log(1) may round)
      }
      const float w_mine = (m == -INFINITY || mine == -INFINITY) ? 0.0f : expf(mine - new_lse);
#pragma unroll
      for (int u = 0; u < U; ++u) w[u] = quad_broadcast(w_mine, u);
    }
    float acc[VN];
#pragma unroll
    for (int e = 0; e < VN; ++e) acc[e] = 0.0f;
    u32x4 only = {0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (u >= n_src) break;
      if (w[u] != 0.0f) fma_vec16<DTYPE>(acc, w[u], x[u][k]);  // an ignored source's data may be anything: skipped
      if (u == 0 && w[u] != 0.0f) only = x[0][k];
    }
    // the scatter-back of a finished block (one source) moves bits, not 0 + 1 * x
    raw* q = dst_out + dst_tok * out_token_stride + (int64_t)wd * VN;
    __builtin_nontemporal_store(n_src == 1 ? only : pack_vec16<DTYPE>(acc), reinterpret_cast<u32x4*>(q));
    if (wd % words_per_head == 0) dst_lse[(int64_t)(wd / words_per_head) * dst_lse_head_stride + dst_tok] = new_lse;
  }
}

template <int DTYPE>
static int launch_merge(const void* src_out, void* dst_out, const float* src_lse, float* dst_lse,
                        int n_head, const int32_t* src_block_table,
                        const int32_t* dst_token_offsets, const int32_t* n_tokens_per_block,
                        const int32_t* block_lengths, int n_red_ops, int block_size,
                        int64_t out_block_stride, int64_t out_token_stride,
                        int64_t lse_block_stride, int64_t lse_token_stride,
                        int64_t src_lse_head_stride, int64_t dst_lse_head_stride, int head_dim,
                        int max_n_blocks_per_op, void* stream) {
  typedef typename Elem<DTYPE>::raw raw;
  constexpr int VN = Vec16<DTYPE>::N;
  const bool vec = head_dim % VN == 0 && out_block_stride % VN == 0 &&
                   out_token_stride % VN == 0 &&
                   ((reinterpret_cast<uintptr_t>(src_out) | reinterpret_cast<uintptr_t>(dst_out)) &
                    15) == 0;
  const bool dense_rows = vec && out_token_stride == (int64_t)n_head * head_dim && lse_token_stride == 1;
  const bool wide = (int64_t)n_head * head_dim / VN * kRowTokens >= kMergeThreads * kRowUnroll &&
                    (int64_t)max_n_blocks_per_op * n_head * kRowTokens <= kRowWeightFloats;
  // the row-streaming kernels, when rows are dense over the heads, wide enough to give every lane of
  // its workgroups work (a head block of 4 x 128 bf16 is not: the two-source merges of a 98304-token
  // plan with two partials per row take 1.12 ms per step with the one-wave kernel against 0.50 with
  // the lane-group kernel below) and the weights fit in LDS
  if (dense_rows && wide) {
    const int wph = head_dim / VN, row_words = n_head * wph;
    if (max_n_blocks_per_op <= 4 && wph <= 64 && 64 % wph == 0 && wph % 4 == 0 && row_words % 64 == 0) {
      const int pieces_per_row = row_words / 64;
      const int64_t pieces_per_op = (int64_t)pieces_per_row * block_size;
      const int64_t items = pieces_per_op * n_red_ops;
      const int64_t n_wg = (items + kMergeXcds - 1) / kMergeXcds * kMergeXcds;
      DCP_REQUIRE(n_wg < ((int64_t)1 << 31) && pieces_per_op < ((int64_t)1 << 31), "merge: too many (op, token, piece) items");
      KernelTimer timer("merge_out_lse_kernel", stream);
      auto launch_wave = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)n_wg), dim3(64), 0, (hipStream_t)stream, (const raw*)src_out, (raw*)dst_out,
                           src_lse, dst_lse, src_block_table, dst_token_offsets, n_tokens_per_block, block_lengths,
                           out_block_stride, out_token_stride, lse_block_stride, src_lse_head_stride, dst_lse_head_stride,
                           wph, max_n_blocks_per_op, pieces_per_row, (int)pieces_per_op, items);
      };
      if (max_n_blocks_per_op > 2) launch_wave(merge_rows_wave_kernel<DTYPE, 4, 1>);
      else if (max_n_blocks_per_op == 2) launch_wave(merge_rows_wave_kernel<DTYPE, 2, 1>);
      else launch_wave(merge_rows_wave_kernel<DTYPE, 1, 1>);
      return check_launch("merge_out_lse_kernel");
    }
    const int64_t chunks = (block_size + kRowTokens - 1) / kRowTokens;
    const int64_t items = chunks * n_red_ops;
    const int64_t n_wg = (items + kMergeXcds - 1) / kMergeXcds * kMergeXcds;
    DCP_REQUIRE(n_wg < ((int64_t)1 << 31), "merge: too many (op, token chunk) items");
    dim3 grid((unsigned)n_wg);
    KernelTimer timer("merge_out_lse_kernel", stream);
    auto launch_rows = [&](auto kernel) {
      const size_t lds_bytes = (size_t)max_n_blocks_per_op * n_head * kRowTokens * sizeof(float);
      hipLaunchKernelGGL(kernel, grid, dim3(kMergeThreads), lds_bytes, (hipStream_t)stream, (const raw*)src_out, (raw*)dst_out,
                         src_lse, dst_lse, n_head, src_block_table, dst_token_offsets, n_tokens_per_block, block_lengths,
                         out_block_stride, out_token_stride, lse_block_stride, src_lse_head_stride, dst_lse_head_stride,
                         head_dim, max_n_blocks_per_op, (int)chunks, (int)items);
    };
    if (max_n_blocks_per_op >= 4) launch_rows(merge_rows_kernel<DTYPE, 4, kMergeThreads, kRowTokens, kRowUnroll>);
    else if (max_n_blocks_per_op >= 2) launch_rows(merge_rows_kernel<DTYPE, 2, kMergeThreads, kRowTokens, kRowUnroll>);
    else launch_rows(merge_rows_kernel<DTYPE, 1, kMergeThreads, kRowTokens, kRowUnroll>);
    return check_launch("merge_out_lse_kernel");
  }
  const int n_words = vec ? head_dim / VN : head_dim;
  int lpr = 1;
  while (lpr < 64 && n_words % (lpr * 2) == 0) lpr *= 2;
  const int rows_per_wg = kMergeThreads / lpr;
  // sources folded per step x tokens per lane group: eight 16-byte words in flight per lane
  // (two for a single source, which measured fastest: the op is then a plain copy)
  const int u = max_n_blocks_per_op >= 4 ? 4 : max_n_blocks_per_op >= 2 ? 2 : 1;
  const int tpg = u == 4 ? 2 : u == 2 ? 4 : 2;
  const int64_t row_chunks = (int64_t)((block_size + rows_per_wg * tpg - 1) / (rows_per_wg * tpg)) * n_head;
  DCP_REQUIRE(row_chunks * n_red_ops < ((int64_t)1 << 31), "merge: %d ops of %lld (token, head) rows are too many for one launch",
              n_red_ops, (long long)block_size * n_head);
  dim3 grid((unsigned)(row_chunks * n_red_ops));
  KernelTimer timer("merge_out_lse_kernel", stream);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kMergeThreads), 0, (hipStream_t)stream, (const raw*)src_out,
                       (raw*)dst_out, src_lse, dst_lse, n_head, src_block_table,
                       dst_token_offsets, n_tokens_per_block, block_lengths, out_block_stride,
                       out_token_stride, lse_block_stride, lse_token_stride, src_lse_head_stride,
                       dst_lse_head_stride, head_dim, max_n_blocks_per_op, lpr, (int)row_chunks);
  };
#define DCP_MERGE_PICK(V)                                           \
  do {                                                              \
    if (u == 4) launch(merge_out_lse_kernel<DTYPE, V, 4, 2>);       \
    else if (u == 2) launch(merge_out_lse_kernel<DTYPE, V, 2, 4>);  \
    else launch(merge_out_lse_kernel<DTYPE, V, 1, 2>);              \
  } while (0)
  if (vec) DCP_MERGE_PICK(true);
  else DCP_MERGE_PICK(false);
#undef DCP_MERGE_PICK
  return check_launch("merge_out_lse_kernel");
}

// ---------------------------------------------------------------------------
// Block sum.  grid: sums x chunks of THREADS * 16 bytes * kSumUnroll, one dimension with a sum's chunks
// side by side.  One wave per workgroup and one word per lane and source (1 KiB chunks) measured
// fastest on four sources of 262144 tokens x 32 heads x 128 bf16: 6.55 TB/s against 5.91 with
// 256 lanes x 2 words, 6.19 with 128 or 256 lanes x 1 word, 5.94 with 64 lanes x 2 words.
// ---------------------------------------------------------------------------
constexpr int kSumThreads = 64;
constexpr int kSumUnroll = 1;

template <int DTYPE, int THREADS, int kSumUnroll>
__global__ __launch_bounds__(THREADS) void blockwise_sum_kernel(
    const int64_t* __restrict__ src_ptrs, const int32_t* __restrict__ src_offsets,
    const int32_t* __restrict__ src_strides, const int32_t* __restrict__ n_ops_per_block,
    const int64_t* __restrict__ dst_ptrs, const int32_t* __restrict__ dst_offsets,
    const int32_t* __restrict__ dst_strides, const int32_t* __restrict__ n_elements,
    int max_n_ops_per_block, int chunks_per_sum) {
  typedef typename Elem<DTYPE>::raw raw;
  constexpr int VN = Vec16<DTYPE>::N;
  const int s = blockIdx.x / chunks_per_sum;
  const int64_t n_elem = n_elements[s];
  const int64_t chunk_elems = (int64_t)THREADS * VN * kSumUnroll;
  const int64_t begin = (int64_t)(blockIdx.x - s * chunks_per_sum) * chunk_elems;
  if (begin >= n_elem) return;
  const int64_t end = min(begin + chunk_elems, n_elem);

  const int n_ops = n_ops_per_block[s];
  const int32_t* offs = src_offsets + (int64_t)s * max_n_ops_per_block;
  const raw* src = reinterpret_cast<const raw*>(src_ptrs[s]);
  const int64_t src_stride = src_strides[s];
  raw* dst = reinterpret_cast<raw*>(dst_ptrs[s]) + (int64_t)dst_offsets[s] * dst_strides[s];

  const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0 &&
                       (src_stride % VN) == 0;
  int64_t vec_end = begin;
  if (aligned) {
    vec_end = begin + ((end - begin) / VN) * VN;
    // kSumUnroll positions x four sources: all their 16-byte words are requested before any
    // arithmetic (a position past the end repeats the chunk's first word and is not stored)
    int64_t pos[kSumUnroll];
    bool live[kSumUnroll];
    float acc[kSumUnroll][VN];
#pragma unroll
    for (int u = 0; u < kSumUnroll; ++u) {
      const int64_t i = begin + ((int64_t)u * THREADS + threadIdx.x) * VN;
      live[u] = i < vec_end;
      pos[u] = live[u] ? i : begin;
#pragma unroll
      for (int k = 0; k < VN; ++k) acc[u][k] = 0.0f;
    }
    if (begin < vec_end && n_ops == 1) {  // a single source: the scatter-back, copied bit for bit
      const raw* row = src + offs[0] * src_stride;
      u32x4 bits[kSumUnroll];
#pragma unroll
      for (int u = 0; u < kSumUnroll; ++u) bits[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + pos[u]));
#pragma unroll
      for (int u = 0; u < kSumUnroll; ++u)
        if (live[u]) __builtin_nontemporal_store(bits[u], reinterpret_cast<u32x4*>(dst + pos[u]));
    } else if (begin < vec_end) {
      for (int j0 = 0; j0 < n_ops; j0 += 4) {
        u32x4 bits[4][kSumUnroll];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const raw* row = src + offs[min(j0 + q, n_ops - 1)] * src_stride;  // tail: re-read the last source
#pragma unroll
          for (int u = 0; u < kSumUnroll; ++u)
            bits[q][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + pos[u]));
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (j0 + q >= n_ops) break;
#pragma unroll
          for (int u = 0; u < kSumUnroll; ++u) fma_vec16<DTYPE>(acc[u], 1.0f, bits[q][u]);
        }
      }
#pragma unroll
      for (int u = 0; u < kSumUnroll; ++u)
        if (live[u]) __builtin_nontemporal_store(pack_vec16<DTYPE>(acc[u]), reinterpret_cast<u32x4*>(dst + pos[u]));
    }
  }
  for (int64_t i = vec_end + threadIdx.x; i < end; i += THREADS) {
    if (n_ops == 1) {
      dst[i] = src[offs[0] * src_stride + i];
      continue;
    }
    float acc = 0.0f;
    for (int j = 0; j < n_ops; ++j) acc += Elem<DTYPE>::load(src[offs[j] * src_stride + i]);
    dst[i] = Elem<DTYPE>::store(acc);
  }
}

}  // namespace dcp

using namespace dcp;

extern "C" int dcp_update_out_lse(const void* src_out, void* dst_out, const float* src_lse,
                                  float* dst_lse, int n_head, const int32_t* src_block_table,
                                  const int32_t* dst_token_offsets,
                                  const int32_t* n_tokens_per_block,
                                  const int32_t* block_lengths, int n_red_ops, int block_size,
                                  int64_t out_block_stride, int64_t out_token_stride,
                                  int64_t lse_block_stride, int64_t lse_token_stride,
                                  int64_t src_lse_head_stride, int64_t dst_lse_head_stride,
                                  int head_dim, int max_n_blocks_per_op, int dtype,
                                  void* stream) {
  DCP_REQUIRE(max_n_blocks_per_op <= 64, "Too many blocks for reduction (%d > 64)",
              max_n_blocks_per_op);
  DCP_REQUIRE(max_n_blocks_per_op >= 1, "merge: max_n_blocks_per_op must be positive");
  DCP_REQUIRE(n_red_ops >= 0 && n_head >= 0 && block_size >= 0 && head_dim >= 0,
              "merge: negative size");
  if (n_red_ops == 0 || n_head == 0 || block_size == 0 || head_dim == 0) return DCP_OK;
  DCP_REQUIRE(src_out && dst_out && src_lse && dst_lse && src_block_table && dst_token_offsets &&
                  n_tokens_per_block && block_lengths,
              "merge: null argument");
#define DCP_MERGE_ARGS                                                                       \
  src_out, dst_out, src_lse, dst_lse, n_head, src_block_table, dst_token_offsets,            \
      n_tokens_per_block, block_lengths, n_red_ops, block_size, out_block_stride,            \
      out_token_stride, lse_block_stride, lse_token_stride, src_lse_head_stride,             \
      dst_lse_head_stride, head_dim, max_n_blocks_per_op, stream
  switch (dtype) {
    case DCP_DTYPE_BF16:
      return launch_merge<DCP_DTYPE_BF16>(DCP_MERGE_ARGS);
    case DCP_DTYPE_FP16:
      return launch_merge<DCP_DTYPE_FP16>(DCP_MERGE_ARGS);
    case DCP_DTYPE_FP32:
      return launch_merge<DCP_DTYPE_FP32>(DCP_MERGE_ARGS);
    default:
      return fail(DCP_ERR_UNSUPPORTED, "merge: unsupported dtype %d", dtype);
  }
#undef DCP_MERGE_ARGS
}

extern "C" int dcp_blockwise_sum(const int64_t* src_ptrs, const int32_t* src_offsets,
                                 const int32_t* src_strides, const int32_t* n_ops_per_block,
                                 const int64_t* dst_ptrs, const int32_t* dst_offsets,
                                 const int32_t* dst_strides, const int32_t* n_elements,
                                 int n_sums, int max_n_ops_per_block, int64_t block_numel,
                                 int dtype, void* stream) {
  const int esize = dtype_size(dtype);
  if (esize == 0) return fail(DCP_ERR_UNSUPPORTED, "Unsupported dtype: %d", dtype);
  DCP_REQUIRE(n_sums >= 0 && block_numel >= 0 && max_n_ops_per_block >= 1, "sum: bad size");
  if (n_sums == 0 || block_numel == 0) return DCP_OK;
  DCP_REQUIRE(src_ptrs && src_offsets && src_strides && n_ops_per_block && dst_ptrs &&
                  dst_offsets && dst_strides && n_elements,
              "sum: null table");
  const int64_t chunk_elems = (int64_t)kSumThreads * (16 / esize) * kSumUnroll;
  const int64_t chunks = (block_numel + chunk_elems - 1) / chunk_elems;
  DCP_REQUIRE(chunks * n_sums < ((int64_t)1 << 31), "sum: %d sums of %lld elements are too many for one launch", n_sums,
              (long long)block_numel);
  dim3 grid((unsigned)(chunks * n_sums));
  KernelTimer timer("blockwise_sum_kernel", stream);
#define DCP_SUM_LAUNCH(DT)                                                                          \
  hipLaunchKernelGGL((blockwise_sum_kernel<DT, kSumThreads, kSumUnroll>), grid, dim3(kSumThreads), 0, \
                     (hipStream_t)stream, src_ptrs, src_offsets, src_strides, n_ops_per_block,      \
                     dst_ptrs, dst_offsets, dst_strides, n_elements, max_n_ops_per_block, (int)chunks)
  switch (dtype) {
    case DCP_DTYPE_BF16:
      DCP_SUM_LAUNCH(DCP_DTYPE_BF16);
      break;
    case DCP_DTYPE_FP16:
      DCP_SUM_LAUNCH(DCP_DTYPE_FP16);
      break;
    default:
      DCP_SUM_LAUNCH(DCP_DTYPE_FP32);
      break;
  }
#undef DCP_SUM_LAUNCH
  return check_launch("blockwise_sum_kernel");
}
