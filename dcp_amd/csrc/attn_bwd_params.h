// Arguments and constants shared by the backward kernels (gfx950).
#pragma once

#include "attn_common.h"

namespace dcp {

struct AttnBwdParams {
  const void* dout;
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const float* lse;
  void* dq;
  void* dk;
  void* dv;
  float* delta;      // [total_q, H]: MINUS rowsum(dO * O)
  float* lse2;       // [total_q, H]: lse * log2(e); both written by the dQ kernel, read by the dK/dV kernel
  int32_t* hull;     // [batch * q_tiles_per_row, 8]
  int* tickets;      // work-item counters of the persistent dQ kernel (kTicketInts); zeroed by the hull kernel
  // the one-pass backward only (attn_bwd_fused.hip):
  float* dq_part;    // [batch * n_heads_q * subs_per_row][4096]: partial dQ of a (row, head, 32-query) chunk, fp32
  int* chain;        // [batch * n_heads_q * subs_per_row][4]: links of the chunk's chain done so far, per wave
  int* fault;        // [0]: raised by a wave whose wait for a chain link ran into the spin limit; [1]: unused word
  int subs_per_row;  // ceil(block_size / 32)
  // the dS-through-memory backward only (attn_bwd_ds.hip):
  void* ds;          // [total_kv / 64][n_heads_q][subs_per_row] pieces of 4 KiB: dS of 64 keys x 32 queries
  int64_t ds_pieces;  // pieces in use; two spare ones follow
  int head_dim;
  const int32_t* cu_seqlens_q;
  const int32_t* cu_seqlens_kv;
  const int32_t* attn_range;
  const int32_t* q_block_table;
  const int32_t* kv_block_table;
  const int32_t* out_block_table;
  const int32_t* dq_block_table;
  const int32_t* dkv_block_table;
  const int32_t* row_order;
  int n_ranges;
  int batch;
  int max_kv_blocks;
  int total_q;
  int block_size;
  int n_heads_q;
  int n_heads_kv;
  int64_t kv_slot_stride;
  int64_t kv_token_stride;
  int64_t dkv_slot_stride;
  int64_t dkv_token_stride;
  int n_out_slots;
  // element strides of a table entry: a slot of block_size tokens, or a single token when the
  // tables address the caller's unpadded tensors directly (entries are then token offsets)
  int64_t q_slot_stride;
  int64_t out_slot_stride;   // out and dout
  int64_t dq_slot_stride;
  int64_t lse_head_stride;
  int64_t lse_slot_stride;
  int dkv_xcd_group;     // dK/dV work items sharing one Q/dO stream (the key tiles of a row)
  int dq_xcd_group;      // dQ work items sharing one K/V stream
  int64_t n_dkv_items;   // batch * n_heads_kv * kv_tiles_per_row
  int64_t n_dq_items;    // batch * n_heads_q * dq_tiles_per_row
  int q_tiles_per_row;   // ceil(block_size / 64): query tiles of the dK/dV kernel
  int dq_tiles_per_row;  // ceil(block_size / 128): query tiles of the dQ kernel
  int kv_tiles_per_row;  // ceil(max_kv_blocks * block_size / 128): key tiles of the dK/dV kernel
  float scale;
  float scale_log2;
};

// Wave priorities by phase in the dK/dV kernel: a wave in one of its two matrix phases outranks a
// wave doing vector work or step control on the same SIMD (-1.1 to -1.5 % on the kernel; measured
// with the matrix phases at 1, 2 or 3 and unequal: all within 0.5 % of each other, all faster than
// none; the same in the dQ kernel made it 1.2 % slower).
constexpr int kPrioMatrix = 2, kPrioVector = 0;
constexpr int kBwdBM = 64;
constexpr int kBwdBN = 64;
constexpr int kBwdThreads = 256;
constexpr int kTicketInts = 16;  // one counter per XCD (the rest unused)

// The backward through dS in memory: prepare (hulls, -delta, lse2), the dK/dV kernel writing dS, the
// dQ kernel that reads it back (attn_bwd_ds.hip); the pieces it is made of live in three files.
int launch_bwd_through_ds(const AttnBwdParams& p, int dtype, hipStream_t stream);
int launch_bwd_prepare(const AttnBwdParams& p, int dtype, hipStream_t stream);
int launch_bwd_dkv_writing_ds(const AttnBwdParams& p, int dtype, hipStream_t stream);
size_t bwd_ds_workspace_bytes(int64_t total_kv, int batch, int block_size, int n_heads_q);

// The one-pass backward (prepare + fused kernel) for head size 128; p.hull, p.delta, p.lse2,
// p.dq_part, p.chain and p.fault point into the workspace.
int launch_bwd_fused(const AttnBwdParams& p, int dtype, hipStream_t stream);
// Bytes of workspace the one-pass backward needs beyond the two-kernel one's.
size_t bwd_fused_extra_workspace_bytes(int batch, int block_size, int n_heads_q, int head_dim);
// Whether dcp_attn_bwd takes the one-pass backward: it has been selected (dcp_attn_bwd_select, or
// DCP_BWD_MODE in the environment) and the current device deals the workgroups of a grid to its 8
// XCDs in turn -- the chain relies on the key tiles of a row sharing an L2 (checked once per device
// by a small kernel).
bool bwd_fused_available();
// Sets the selection (a DCP_BWD_* value; anything else only asks) and returns what it was.
int bwd_select(int mode);

}  // namespace dcp
