// Block gather/scatter kernels: pointer-table block copy, per-token dKV copy
// and head-strided LSE copy.  Pure byte movement, HBM-bound.
//
// One workgroup moves one chunk of one block with 16-byte non-temporal loads
// and stores; consecutive lanes touch consecutive 16-byte words.  The chunk is
// 1 KiB (a single wave, one load per lane) for blocks of 2 MiB and more and for
// blocks of at most 256 KiB, and 16 KiB (256 lanes, four independent loads per
// lane) in between: measured on a seeded permutation of a 2 GiB bf16 tensor,
// 4 MiB blocks move at 6.67 TB/s in 1 KiB chunks, 6.2 in 4 KiB chunks of 256
// lanes and 5.8 in 16 KiB chunks, while the 1 MiB / 0.5 MiB blocks of an
// executor gather (ragged, two sizes in one launch) take 0.31 ms per launch
// with 4 KiB chunks against 0.23 with 16 KiB.
#include "common.h"

namespace dcp {

// Chunk size by block size, measured on 2 GiB moved through a seeded block permutation: 4 MiB blocks
// 6.67 TB/s in 1 KiB chunks (6.2 in 4 KiB chunks); 128 KiB blocks 6.10 TB/s in 1 KiB chunks against 5.88
// in 4 KiB and 5.4 in 16 KiB chunks; the 0.5-1 MiB blocks of an attention plan, ragged and of two sizes
// in one launch, 6.1 TB/s in 16 KiB chunks against 4.3 in 4 KiB chunks (four times the workgroups
// that find nothing to move).
constexpr int64_t kSmallChunkBlockBytes = 2 << 20;   // blocks at least this large use 1 KiB chunks,
constexpr int64_t kTinyBlockBytes = 256 << 10;       // and so do blocks at most this large

// Tables are nullable where the dKV variant has no such column: a null
// offset/stride table means offset 0, and n_count[p] is multiplied by
// `elems_per_count` (1 for the element-count variant, per_token_size for the
// token-count variant).
template <int kCopyUnroll, int kCopyThreads>
__global__ __launch_bounds__(kCopyThreads) void copy_varlen_kernel(
    const int64_t* __restrict__ src_ptrs, const int32_t* __restrict__ src_offsets,
    const int32_t* __restrict__ src_strides, const int64_t* __restrict__ dst_ptrs,
    const int32_t* __restrict__ dst_offsets, const int32_t* __restrict__ dst_strides,
    const int32_t* __restrict__ n_count, int64_t elems_per_count,
    int chunks_per_block, int elem_size) {
  constexpr int kCopyChunkBytes = kCopyThreads * 16 * kCopyUnroll;
  const int p = blockIdx.x / chunks_per_block;
  const int c = blockIdx.x - p * chunks_per_block;
  const int64_t n_bytes = (int64_t)n_count[p] * elems_per_count * elem_size;
  const int64_t begin = (int64_t)c * kCopyChunkBytes;
  if (begin >= n_bytes) return;
  const int64_t end = min(begin + (int64_t)kCopyChunkBytes, n_bytes);

  int64_t src_off = 0, dst_off = 0;
  if (src_offsets) src_off = (int64_t)src_offsets[p] * src_strides[p] * elem_size;
  if (dst_offsets) dst_off = (int64_t)dst_offsets[p] * dst_strides[p] * elem_size;
  const char* src = reinterpret_cast<const char*>(src_ptrs[p]) + src_off;
  char* dst = reinterpret_cast<char*>(dst_ptrs[p]) + dst_off;

  const bool aligned =
      ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
  if (aligned) {
    const int64_t vec_end = begin + ((end - begin) & ~(int64_t)15);
    const u32x4* s = reinterpret_cast<const u32x4*>(src + begin);
    u32x4* d = reinterpret_cast<u32x4*>(dst + begin);
    const int n_vec = (int)((vec_end - begin) >> 4);
    if (n_vec == kCopyThreads * kCopyUnroll) {
      u32x4 r[kCopyUnroll];
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u)
        r[u] = __builtin_nontemporal_load(s + threadIdx.x + u * kCopyThreads);
#pragma unroll
      for (int u = 0; u < kCopyUnroll; ++u)
        __builtin_nontemporal_store(r[u], d + threadIdx.x + u * kCopyThreads);
    } else {
      for (int i = threadIdx.x; i < n_vec; i += kCopyThreads) d[i] = s[i];
    }
    // sub-16-byte tail of the block (only in its last chunk)
    for (int64_t b = vec_end + threadIdx.x * elem_size; b < end;
         b += (int64_t)kCopyThreads * elem_size) {
      if (elem_size == 2)
        *reinterpret_cast<uint16_t*>(dst + b) = *reinterpret_cast<const uint16_t*>(src + b);
      else
        *reinterpret_cast<uint32_t*>(dst + b) = *reinterpret_cast<const uint32_t*>(src + b);
    }
  } else {
    for (int64_t b = begin + (int64_t)threadIdx.x * elem_size; b < end;
         b += (int64_t)kCopyThreads * elem_size) {
      if (elem_size == 2)
        *reinterpret_cast<uint16_t*>(dst + b) = *reinterpret_cast<const uint16_t*>(src + b);
      else
        *reinterpret_cast<uint32_t*>(dst + b) = *reinterpret_cast<const uint32_t*>(src + b);
    }
  }
}

// grid: (blocks, heads, token chunks); LSE rows are short and arbitrarily
// aligned, so this is a plain coalesced element copy.
template <typename T>
__global__ __launch_bounds__(256) void copy_lse_kernel(
    const int64_t* __restrict__ src_ptrs, const int32_t* __restrict__ src_token_offsets,
    const int32_t* __restrict__ src_head_strides, const int64_t* __restrict__ dst_ptrs,
    const int32_t* __restrict__ dst_token_offsets,
    const int32_t* __restrict__ dst_head_strides, const int32_t* __restrict__ n_tokens) {
  const int p = blockIdx.x;
  const int h = blockIdx.y;
  const int t = blockIdx.z * 256 + threadIdx.x;
  if (t >= n_tokens[p]) return;
  const T* src = reinterpret_cast<const T*>(src_ptrs[p]) +
                 (int64_t)h * src_head_strides[p] + src_token_offsets[p];
  T* dst = reinterpret_cast<T*>(dst_ptrs[p]) + (int64_t)h * dst_head_strides[p] +
           dst_token_offsets[p];
  dst[t] = src[t];
}

static int launch_copy(const int64_t* src_ptrs, const int32_t* src_offsets,
                       const int32_t* src_strides, const int64_t* dst_ptrs,
                       const int32_t* dst_offsets, const int32_t* dst_strides,
                       const int32_t* n_count, int64_t elems_per_count, int n_ptrs,
                       int64_t block_numel, int elem_size, void* stream) {
  const int64_t block_bytes = block_numel * elem_size;
  const int unroll = block_bytes >= kSmallChunkBlockBytes || block_bytes <= kTinyBlockBytes ? 1 : 4;
  const int threads = unroll == 1 ? 64 : 256;
  const int64_t chunk_bytes = (int64_t)threads * 16 * unroll;
  const int64_t chunks = (block_bytes + chunk_bytes - 1) / chunk_bytes;
  DCP_REQUIRE(chunks * n_ptrs < (int64_t)1 << 31, "copy grid too large: %lld blocks x %lld chunks",
              (long long)n_ptrs, (long long)chunks);
  KernelTimer timer("copy_varlen_kernel", stream);
  if (unroll == 1)
    hipLaunchKernelGGL((copy_varlen_kernel<1, 64>), dim3((unsigned)(chunks * n_ptrs)), dim3(64), 0,
                       (hipStream_t)stream, src_ptrs, src_offsets, src_strides, dst_ptrs,
                       dst_offsets, dst_strides, n_count, elems_per_count, (int)chunks, elem_size);
  else
    hipLaunchKernelGGL((copy_varlen_kernel<4, 256>), dim3((unsigned)(chunks * n_ptrs)), dim3(256), 0,
                       (hipStream_t)stream, src_ptrs, src_offsets, src_strides, dst_ptrs,
                       dst_offsets, dst_strides, n_count, elems_per_count, (int)chunks, elem_size);
  return check_launch("copy_varlen_kernel");
}

}  // namespace dcp

using namespace dcp;

extern "C" int dcp_fused_copy_varlen(const int64_t* src_ptrs, const int32_t* src_offsets,
                                     const int32_t* src_strides, const int64_t* dst_ptrs,
                                     const int32_t* dst_offsets, const int32_t* dst_strides,
                                     const int32_t* n_elements, int n_ptrs, int64_t block_numel,
                                     int elem_size, void* stream) {
  DCP_REQUIRE(elem_size == 2 || elem_size == 4, "copy: unsupported element size %d", elem_size);
  DCP_REQUIRE(n_ptrs >= 0 && block_numel >= 0, "copy: negative size");
  if (n_ptrs == 0 || block_numel == 0) return DCP_OK;
  DCP_REQUIRE(src_ptrs && dst_ptrs && src_offsets && src_strides && dst_offsets && dst_strides &&
                  n_elements,
              "copy: null table");
  return launch_copy(src_ptrs, src_offsets, src_strides, dst_ptrs, dst_offsets, dst_strides,
                     n_elements, 1, n_ptrs, block_numel, elem_size, stream);
}

extern "C" int dcp_fused_copy_varlen_dkv(const int64_t* src_ptrs, const int64_t* dst_ptrs,
                                         const int32_t* n_tokens, int n_ptrs, int max_n_tokens,
                                         int per_token_size, int elem_size, void* stream) {
  DCP_REQUIRE(elem_size == 2 || elem_size == 4, "dkv copy: unsupported element size %d",
              elem_size);
  DCP_REQUIRE(n_ptrs >= 0 && max_n_tokens >= 0 && per_token_size >= 0, "dkv copy: negative size");
  if (n_ptrs == 0 || max_n_tokens == 0 || per_token_size == 0) return DCP_OK;
  DCP_REQUIRE(src_ptrs && dst_ptrs && n_tokens, "dkv copy: null table");
  return launch_copy(src_ptrs, nullptr, nullptr, dst_ptrs, nullptr, nullptr, n_tokens,
                     per_token_size, n_ptrs, (int64_t)max_n_tokens * per_token_size, elem_size,
                     stream);
}

extern "C" int dcp_fused_copy_varlen_lse(const int64_t* src_ptrs,
                                         const int32_t* src_token_offsets,
                                         const int32_t* src_head_strides, const int64_t* dst_ptrs,
                                         const int32_t* dst_token_offsets,
                                         const int32_t* dst_head_strides, const int32_t* n_tokens,
                                         int n_ptrs, int head_block_size, int max_n_tokens,
                                         int elem_size, void* stream) {
  DCP_REQUIRE(elem_size == 2 || elem_size == 4, "lse copy: unsupported element size %d",
              elem_size);
  DCP_REQUIRE(n_ptrs >= 0 && head_block_size >= 0 && max_n_tokens >= 0,
              "lse copy: negative size");
  if (n_ptrs == 0 || head_block_size == 0 || max_n_tokens == 0) return DCP_OK;
  DCP_REQUIRE(head_block_size <= 65535 && max_n_tokens <= 65535 * 256,
              "lse copy: head_block_size %d or max_n_tokens %d too large", head_block_size,
              max_n_tokens);
  DCP_REQUIRE(src_ptrs && dst_ptrs && src_token_offsets && src_head_strides &&
                  dst_token_offsets && dst_head_strides && n_tokens,
              "lse copy: null table");
  dim3 grid(n_ptrs, head_block_size, (max_n_tokens + 255) / 256);
  KernelTimer timer("copy_lse_kernel", stream);
  if (elem_size == 4)
    hipLaunchKernelGGL(copy_lse_kernel<uint32_t>, grid, dim3(256), 0, (hipStream_t)stream,
                       src_ptrs, src_token_offsets, src_head_strides, dst_ptrs, dst_token_offsets,
                       dst_head_strides, n_tokens);
  else
    hipLaunchKernelGGL(copy_lse_kernel<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream,
                       src_ptrs, src_token_offsets, src_head_strides, dst_ptrs, dst_token_offsets,
                       dst_head_strides, n_tokens);
  return check_launch("copy_lse_kernel");
}
