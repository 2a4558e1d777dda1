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
// grid: (ops, token chunks x heads)
// ---------------------------------------------------------------------------
constexpr int kMergeThreads = 256;

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
    int64_t dst_lse_head_stride, int head_dim, int max_n_blocks_per_op, int lanes_per_row) {
  typedef typename Elem<DTYPE>::raw raw;
  constexpr int VN = VECTOR ? Vec16<DTYPE>::N : 1;
  const int op = blockIdx.x;
  const int n_tok = n_tokens_per_block[op];

  // A workgroup takes consecutive tokens of ONE head: its LSE reads and its LSE store are
  // then contiguous floats ([head][token] layout) instead of one 4-byte access per cache
  // line, and every token's head_dim elements are still one contiguous piece.
  const int rows_per_wg = kMergeThreads / lanes_per_row;
  const int h = blockIdx.y % n_head;
  const int t0 = (blockIdx.y / n_head) * (rows_per_wg * TPG) + threadIdx.x / lanes_per_row;
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
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (j0 + u >= n_src || !lse_is_finite(l[k][u])) l[k][u] = -INFINITY;
          m_new = fmaxf(m_new, l[k][u]);
        }
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
  const int n_words = vec ? head_dim / VN : head_dim;
  int lpr = 1;
  while (lpr < 64 && n_words % (lpr * 2) == 0) lpr *= 2;
  const int rows_per_wg = kMergeThreads / lpr;
  // sources folded per step x tokens per lane group: eight 16-byte words in flight per lane
  // (two for a single source, which measured fastest: the op is then a plain copy)
  const int u = max_n_blocks_per_op >= 4 ? 4 : max_n_blocks_per_op >= 2 ? 2 : 1;
  const int tpg = u == 4 ? 2 : u == 2 ? 4 : 2;
  const int64_t row_chunks = (int64_t)((block_size + rows_per_wg * tpg - 1) / (rows_per_wg * tpg)) * n_head;
  DCP_REQUIRE(row_chunks <= 65535, "merge: block of %lld (token, head) rows is too large",
              (long long)block_size * n_head);
  dim3 grid(n_red_ops, (unsigned)row_chunks);
  KernelTimer timer("merge_out_lse_kernel", stream);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kMergeThreads), 0, (hipStream_t)stream, (const raw*)src_out,
                       (raw*)dst_out, src_lse, dst_lse, n_head, src_block_table,
                       dst_token_offsets, n_tokens_per_block, block_lengths, out_block_stride,
                       out_token_stride, lse_block_stride, lse_token_stride, src_lse_head_stride,
                       dst_lse_head_stride, head_dim, max_n_blocks_per_op, lpr);
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
// Block sum.  grid: (sums, chunks of 256*16 bytes*UNROLL)
// ---------------------------------------------------------------------------
constexpr int kSumUnroll = 2;

template <int DTYPE>
__global__ __launch_bounds__(256) void blockwise_sum_kernel(
    const int64_t* __restrict__ src_ptrs, const int32_t* __restrict__ src_offsets,
    const int32_t* __restrict__ src_strides, const int32_t* __restrict__ n_ops_per_block,
    const int64_t* __restrict__ dst_ptrs, const int32_t* __restrict__ dst_offsets,
    const int32_t* __restrict__ dst_strides, const int32_t* __restrict__ n_elements,
    int max_n_ops_per_block) {
  typedef typename Elem<DTYPE>::raw raw;
  constexpr int VN = Vec16<DTYPE>::N;
  const int s = blockIdx.x;
  const int64_t n_elem = n_elements[s];
  const int64_t chunk_elems = (int64_t)256 * VN * kSumUnroll;
  const int64_t begin = (int64_t)blockIdx.y * chunk_elems;
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
      const int64_t i = begin + ((int64_t)u * 256 + threadIdx.x) * VN;
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
  for (int64_t i = vec_end + threadIdx.x; i < end; i += 256) {
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
  const int64_t chunk_elems = (int64_t)256 * (16 / esize) * kSumUnroll;
  const int64_t chunks = (block_numel + chunk_elems - 1) / chunk_elems;
  DCP_REQUIRE(chunks <= 65535, "sum: block of %lld elements is too large", (long long)block_numel);
  dim3 grid(n_sums, (unsigned)chunks);
  KernelTimer timer("blockwise_sum_kernel", stream);
#define DCP_SUM_LAUNCH(DT)                                                                     \
  hipLaunchKernelGGL(blockwise_sum_kernel<DT>, grid, dim3(256), 0, (hipStream_t)stream,        \
                     src_ptrs, src_offsets, src_strides, n_ops_per_block, dst_ptrs,            \
                     dst_offsets, dst_strides, n_elements, max_n_ops_per_block)
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
