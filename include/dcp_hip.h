/*
 * C ABI of libdcp_hip.so: the gfx950 kernels behind DCP's per-device blockwise
 * attention executor.
 *
 * Conventions
 *  - every pointer marked "device" is a HIP device address on the current
 *    device; "host" pointers are ordinary host memory read before return;
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream); all
 *    work is enqueued on it and nothing synchronises with the host;
 *  - the library borrows memory for the duration of a launch: it allocates
 *    nothing and keeps no pointer;
 *  - return value 0 = launched, nonzero = rejected before any launch (argument
 *    error); dcp_last_error() then returns a message for the calling thread;
 *  - dtype codes follow the reference's wire integers
 *    (dcp/core/serialization.py:410-437): 0 bf16, 1 fp16, 2 fp32.
 *
 * Each entry point names the reference interface it replaces.
 */
#ifndef DCP_HIP_H_
#define DCP_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DCP_DTYPE_BF16 0
#define DCP_DTYPE_FP16 1
#define DCP_DTYPE_FP32 2

#define DCP_OK 0
#define DCP_ERR_ARG 1
#define DCP_ERR_UNSUPPORTED 2
#define DCP_ERR_LAUNCH 3

/* Library / ABI version (major*100 + minor). */
int dcp_version(void);

/* Message of the last nonzero return on this thread ("" if none). */
const char* dcp_last_error(void);

/*
 * Per-kernel timing for benchmarks (no counterpart in the reference, which
 * relies on external profilers).  While enabled, each kernel launch of this
 * library is bracketed by two events recorded on its launch stream.
 * dcp_profile_report waits for the recorded events, writes one line per kernel
 * name, "<name> <launches> <total_ms>\n", into `buffer` (NUL-terminated) and
 * forgets them; it returns nonzero if `capacity` was too small.  Disabled (the
 * default), launches record nothing.
 */
void dcp_profile_enable(int on);
int dcp_profile_report(char* buffer, size_t capacity);

/*
 * Block gather / scatter through pointer tables.
 * Replaces dcp.ops.fused_ops.fused_copy_{bf16,fp16,fp32}_varlen
 * (dcp/ops/fused_ops.py:842-864, 916-938, 1013-1035; kernels :290-335,
 * :472-517, :654-699), called from _handle_memcpy
 * (dcp/runtime/flash_attention/executor.py:793-805).
 *
 * For p in [0, n_ptrs), i in [0, n_elements[p]):
 *   ((T*)dst_ptrs[p])[dst_offsets[p]*dst_strides[p] + i] =
 *   ((T*)src_ptrs[p])[src_offsets[p]*src_strides[p] + i]
 * T has `elem_size` bytes (2 or 4); offsets/strides are in elements.
 * All seven tables are device int64/int32 arrays of length n_ptrs.
 * `block_numel` is the padded block size in elements (upper bound of
 * n_elements[p]); it only sizes the grid.
 */
int dcp_fused_copy_varlen(const int64_t* src_ptrs, const int32_t* src_offsets,
                          const int32_t* src_strides, const int64_t* dst_ptrs,
                          const int32_t* dst_offsets,
                          const int32_t* dst_strides,
                          const int32_t* n_elements, int n_ptrs,
                          int64_t block_numel, int elem_size, void* stream);

/*
 * Copy the first n_tokens[p] tokens (per_token_size elements each) of block p.
 * Replaces fused_copy_{bf16,fp16,fp32}_varlen_dkv (fused_ops.py:867-885,
 * 941-959, 1038-1056; kernel :338-367), used after the GQA backward
 * (executor.py:1102-1114).  src_ptrs/dst_ptrs address the blocks themselves.
 */
int dcp_fused_copy_varlen_dkv(const int64_t* src_ptrs, const int64_t* dst_ptrs,
                              const int32_t* n_tokens, int n_ptrs,
                              int max_n_tokens, int per_token_size,
                              int elem_size, void* stream);

/*
 * Head-strided copy of log-sum-exp blocks.
 * Replaces fused_copy_{bf16,fp16,fp32}_varlen_lse (fused_ops.py:888-913,
 * 962-987, 1059-1084; kernel :370-429), called from _handle_memcpy
 * (executor.py:806-810).
 * For h < head_block_size, t < n_tokens[p]:
 *   dst[p][h*dst_head_strides[p] + dst_token_offsets[p] + t] =
 *   src[p][h*src_head_strides[p] + src_token_offsets[p] + t]
 * Unlike the reference kernel, head_block_size need not be a power of two.
 */
int dcp_fused_copy_varlen_lse(const int64_t* src_ptrs,
                              const int32_t* src_token_offsets,
                              const int32_t* src_head_strides,
                              const int64_t* dst_ptrs,
                              const int32_t* dst_token_offsets,
                              const int32_t* dst_head_strides,
                              const int32_t* n_tokens, int n_ptrs,
                              int head_block_size, int max_n_tokens,
                              int elem_size, void* stream);

/*
 * N-way online-softmax merge of partial (out, lse) blocks, fused with the
 * scatter into the destination.
 * Replaces flash_attn_update_out_lse (fused_ops.py:149-247, kernel :15-146),
 * called from _handle_reduction (executor.py:1299-1329).
 *
 * For op o, head h < n_head, token t < n_tokens_per_block[o], over the
 * sources j < block_lengths[o] with block b_j = src_block_table[o*max_n+j]:
 *   l_j   = src_lse[h*src_lse_head_stride + b_j*lse_block_stride + t*lse_token_stride]
 *   sources with l_j = +-inf are ignored;
 *   lse*  = m + log(sum_j exp(l_j - m)),  m = max_j l_j
 *   out*  = sum_j exp(l_j - lse*) * src_out[b_j*out_block_stride + t*out_token_stride + h*head_dim + :]
 *   no finite source: lse* = -1, out* = 0.
 * dst_out[(dst_token_offsets[o]+t)*out_token_stride + h*head_dim + :] = out*
 * dst_lse[h*dst_lse_head_stride + (dst_token_offsets[o]+t)*lse_token_stride] = lse*
 * Math in fp32; out is stored in `dtype`, lse is fp32.  dst may alias one of
 * the sources of the same op (in-place fold).  max_n_blocks_per_op <= 64.
 */
int dcp_update_out_lse(const void* src_out, void* dst_out,
                       const float* src_lse, float* dst_lse, int n_head,
                       const int32_t* src_block_table,
                       const int32_t* dst_token_offsets,
                       const int32_t* n_tokens_per_block,
                       const int32_t* block_lengths, int n_red_ops,
                       int block_size, int64_t out_block_stride,
                       int64_t out_token_stride, int64_t lse_block_stride,
                       int64_t lse_token_stride, int64_t src_lse_head_stride,
                       int64_t dst_lse_head_stride, int head_dim,
                       int max_n_blocks_per_op, int dtype, void* stream);

/*
 * N-way block sum (dQ / dK / dV accumulation) fused with the scatter.
 * Replaces fused_blockwise_sum (fused_ops.py:1288-1360, kernels :1087-1285),
 * called from _handle_sum (executor.py:1530-1545).
 *   dst[s][dst_offsets[s]*dst_strides[s] + i] =
 *       sum_{j < n_ops_per_block[s]} src[s][src_offsets[s*max_n+j]*src_strides[s] + i]
 * for i < n_elements[s].  Accumulates in fp32 and rounds once (the reference
 * kernel accumulates in the storage type; see its test tolerance 1e-2).
 * dst may alias one of the sources of the same sum.
 */
int dcp_blockwise_sum(const int64_t* src_ptrs, const int32_t* src_offsets,
                      const int32_t* src_strides,
                      const int32_t* n_ops_per_block, const int64_t* dst_ptrs,
                      const int32_t* dst_offsets, const int32_t* dst_strides,
                      const int32_t* n_elements, int n_sums,
                      int max_n_ops_per_block, int64_t block_numel, int dtype,
                      void* stream);

/*
 * Range-masked, paged, variable-length attention forward.
 * Replaces dcp_flash_attn._flash_attn_varlen_forward as called by
 * _wrapped_flash_attn_varlen_forward (executor.py:117-187) from _handle_attn
 * (:884-913): no causal flag, no window, no dropout, no softcap.
 *
 * Batch row b = one q block.  Its seqlen_q = cu_seqlens_q[b+1]-cu_seqlens_q[b]
 * (<= block_size) queries live in slot q_block_table[b] of `q`
 * ([n_q_slots, block_size, n_heads_q, head_dim]); keys/values are the
 * concatenation of slots kv_block_table[b*max_kv_blocks + j] of `k`/`v`
 * (slot stride kv_slot_stride, token stride kv_token_stride, head stride
 * head_dim, in elements) for kv positions [0, cu_seqlens_kv[b+1]-cu_seqlens_kv[b]).
 * attn_range is int32 [n_ranges, 2, total_q]: query token t (global index
 * cu_seqlens_q[b]+i) attends kv positions in the union of
 * [attn_range[r][0][t], attn_range[r][1][t]).
 * Writes out ([n_out_slots, block_size, n_heads_q, head_dim]) at slot
 * out_block_table[b] and lse (fp32 [n_heads_q, n_out_slots, block_size]) at the
 * same slot.  Rows with no visible key: out = 0, lse = +inf.
 * q head h reads kv head h / (n_heads_q / n_heads_kv).
 * row_order: optional device int32[batch], a permutation of the rows giving
 * the order in which they are scheduled (put the rows with most keys first);
 * NULL = as numbered.  It changes no result.
 * Supported: dtype bf16/fp16, head_dim 64 or 128, block_size % 64 == 0,
 * softmax_scale > 0.  (A caller with another head size up to 128 zero-pads its
 * buffers to the next of the two and keeps its own softmax_scale, as the
 * reference pads head sizes its kernels do not take; the Python operator layer
 * does so.)
 * Key/value tiles are loaded whole: what a slot holds past the row's keys (and,
 * for keys a range excludes, inside it) reaches the matrix instructions and is
 * masked there.  It must be finite, and small enough that its dot products with
 * q stay finite; the reference's kernels zero-fill such loads instead.  Query
 * rows past seqlen_q are not read.
 * `workspace`: caller-provided device scratch of at least
 * dcp_attn_fwd_workspace_bytes() bytes, 4-byte aligned, for the kernel's work
 * counters (the launch is persistent: its workgroups take (row, head, query
 * tile) items from per-XCD counters).  Its contents are overwritten (a small
 * kernel zeroes it on `stream` before the attention kernel); one workspace
 * serves any number of launches that follow each other on a stream or in a
 * captured graph, launches that may run at the same time need one each.
 */
size_t dcp_attn_fwd_workspace_bytes(void);
int dcp_attn_fwd(const void* q, const void* k, const void* v, void* out,
                 float* lse, const int32_t* cu_seqlens_q,
                 const int32_t* cu_seqlens_kv, const int32_t* attn_range,
                 int n_ranges, const int32_t* q_block_table,
                 const int32_t* kv_block_table,
                 const int32_t* out_block_table, const int32_t* row_order,
                 int batch, int max_kv_blocks, int total_q, int block_size,
                 int n_heads_q, int n_heads_kv, int head_dim,
                 int64_t kv_slot_stride, int64_t kv_token_stride,
                 int n_out_slots, float softmax_scale, int dtype,
                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * dcp_attn_fwd with the stride of a table entry spelled out per tensor, so that
 * the tables can address the caller's UNPADDED tensors directly instead of
 * padded slots: entry e of q_block_table places the row's first query at
 * q + e*q_slot_stride (elements), entry e of out_block_table its first output
 * at out + e*out_slot_stride and its first LSE at
 * lse + head*lse_head_stride + e*lse_slot_stride; queries of a row are
 * n_heads_q*head_dim elements apart, their LSEs 1.  With
 *   q_slot_stride = out_slot_stride = block_size*n_heads_q*head_dim,
 *   lse_head_stride = n_out_slots*block_size, lse_slot_stride = block_size
 * this is dcp_attn_fwd.  With q_slot_stride = out_slot_stride =
 * n_heads_q*head_dim, lse_head_stride = tokens of the LSE tensor,
 * lse_slot_stride = 1 and kv_slot_stride = kv_token_stride, every table entry
 * is a TOKEN offset into [tokens, heads, head_dim] tensors (LSE:
 * [n_heads_q, tokens]): what the reference's plans spell out as a gather into
 * slots before the kernel (MemcpyInstr, executor.py:793-811) and a
 * single-source scatter after it (executor.py:1269-1329) then needs no copy.
 * Only the row's seqlen_q queries are read and written; key/value tiles are
 * still loaded whole, block_size keys from every table entry on, so the k/v
 * tensors must be readable (and finite) for block_size tokens past their last
 * block's first token.  merged_form != 0: a query without a visible key gets
 * lse = -1 instead of +inf (out = 0 either way), which is what the reference's
 * merge kernel leaves for a row none of whose sources is finite
 * (fused_ops.py:118-143) -- for outputs written where that merge would have
 * put them.  No counterpart in the reference.
 */
int dcp_attn_fwd_strided(const void* q, const void* k, const void* v, void* out,
                         float* lse, const int32_t* cu_seqlens_q,
                         const int32_t* cu_seqlens_kv,
                         const int32_t* attn_range, int n_ranges,
                         const int32_t* q_block_table,
                         const int32_t* kv_block_table,
                         const int32_t* out_block_table,
                         const int32_t* row_order, int batch,
                         int max_kv_blocks, int total_q, int block_size,
                         int n_heads_q, int n_heads_kv, int head_dim,
                         int64_t kv_slot_stride, int64_t kv_token_stride,
                         int64_t q_slot_stride, int64_t out_slot_stride,
                         int64_t lse_head_stride, int64_t lse_slot_stride,
                         int merged_form, float softmax_scale, int dtype,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Range-masked, paged, variable-length attention backward.
 * Replaces dcp_flash_attn._flash_attn_varlen_backward as called by
 * _wrapped_flash_attn_varlen_backward (executor.py:256-337) from
 * _handle_attn_bw (:1058-1115).
 *
 * Inputs as dcp_attn_fwd plus dout/out (slots out_block_table[b]) and lse.
 * dq ([n_dq_slots, block_size, n_heads_q, head_dim]) slot dq_block_table[b]
 * receives the row's dQ.  dk/dv: slot dkv_block_table[b*max_kv_blocks + j]
 * receives the dK/dV of the row's j-th kv block, summed over the q heads of
 * each kv head's group.  The kv positions of the row below its key count
 * (cu_seqlens_kv[b+1]-cu_seqlens_kv[b]) rounded up to 32 are written, all heads
 * and dims, with 0 where no query of the row attends; positions past that keep
 * what the slot held.  A key count that is a multiple of block_size, as every
 * plan has it, therefore needs no pre-zeroing.  No atomics are used: results
 * are bit-reproducible from run to run.
 * `workspace` is caller-provided device scratch of at least
 * dcp_attn_bwd_workspace_bytes(...) bytes, 16-byte aligned; its contents are
 * overwritten.  Slot padding (q/dout/out rows past seqlen_q inside a 64-row
 * tile, k/v rows past the row's keys) is loaded and masked, not skipped: it
 * must be finite and small enough that its dot products with the data stay
 * finite.
 */
int dcp_attn_bwd(const void* dout, const void* q, const void* k, const void* v,
                 const void* out, const float* lse, void* dq, void* dk,
                 void* dv, void* workspace, size_t workspace_bytes,
                 const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_kv,
                 const int32_t* attn_range, int n_ranges,
                 const int32_t* q_block_table, const int32_t* kv_block_table,
                 const int32_t* out_block_table,
                 const int32_t* dq_block_table,
                 const int32_t* dkv_block_table, const int32_t* row_order,
                 int batch, int max_kv_blocks, int total_q, int block_size,
                 int n_heads_q, int n_heads_kv, int head_dim,
                 int64_t kv_slot_stride, int64_t kv_token_stride,
                 int64_t dkv_slot_stride, int64_t dkv_token_stride,
                 int n_out_slots, float softmax_scale, int dtype,
                 void* stream);

/*
 * dcp_attn_bwd with the stride of a table entry spelled out per tensor (see
 * dcp_attn_fwd_strided) and with total_kv, the sum of the rows' key counts
 * (cu_seqlens_kv[batch], which the host side of the call cannot read; 0 = not
 * known, which rules DCP_BWD_THROUGH_DS out): q_slot_stride for q, out_slot_stride for out AND dout
 * (they share out_block_table), dq_slot_stride for dq, lse_head_stride /
 * lse_slot_stride for lse.  With token strides the tables address the caller's
 * unpadded q, out, dout, lse, k and v directly and dQ is written straight into
 * the unpadded dq.  The dK/dV kernel loads whole 64-query tiles of q and dout:
 * those tensors must be readable (and finite) for 64 tokens past the last
 * row's queries.  dk/dv stay padded slots (a row writes whole 32-key groups).
 * No counterpart in the reference.
 */
int dcp_attn_bwd_strided(const void* dout, const void* q, const void* k,
                         const void* v, const void* out, const float* lse,
                         void* dq, void* dk, void* dv, void* workspace,
                         size_t workspace_bytes, const int32_t* cu_seqlens_q,
                         const int32_t* cu_seqlens_kv,
                         const int32_t* attn_range, int n_ranges,
                         const int32_t* q_block_table,
                         const int32_t* kv_block_table,
                         const int32_t* out_block_table,
                         const int32_t* dq_block_table,
                         const int32_t* dkv_block_table,
                         const int32_t* row_order, int batch, int max_kv_blocks,
                         int total_q, int block_size, int n_heads_q,
                         int n_heads_kv, int head_dim, int64_t kv_slot_stride,
                         int64_t kv_token_stride, int64_t dkv_slot_stride,
                         int64_t dkv_token_stride, int64_t q_slot_stride,
                         int64_t out_slot_stride, int64_t dq_slot_stride,
                         int64_t lse_head_stride, int64_t lse_slot_stride,
                         int64_t total_kv, float softmax_scale, int dtype,
                         void* stream);

/*
 * Bytes of scratch dcp_attn_bwd needs for these sizes: rowsum(dO*O) and the
 * base-2 log-sum-exp (total_q*n_heads_q floats each), the per-(row, 64-query
 * tile) range hulls and the dQ kernel's work counters.  No counterpart in the reference (its
 * flash-attention fork allocates these inside the call).
 */
size_t dcp_attn_bwd_workspace_bytes(int batch, int total_q, int block_size,
                                    int n_heads_q, int head_dim);

/*
 * Which of its implementations the backward takes from now on (a setting of the
 * process; DCP_BWD_MODE=0/1/2 in the environment presets it).  All three are
 * free of atomics and bit-reproducible.
 *  DCP_BWD_TWO_KERNELS  a query-outer kernel for dQ and a key-outer one for
 *      dK/dV, each recomputing S and dP: seven matrix products for the
 *      backward's five, nothing but the small workspace.
 *  DCP_BWD_ONE_PASS  one key-outer pass (head size 128 only) in which the key
 *      tiles of a row add their shares of dQ one after the other through an
 *      fp32 partial sum in the workspace: five products.  Measured SLOWER on
 *      MI355X (18 ms against 12.5 ms on 65536 causal tokens) and kept as the
 *      measured alternative; only taken on a device on which the workgroups of
 *      a row share an L2 (the library checks).
 *  DCP_BWD_THROUGH_DS  (the default) the key-outer kernel also stores dS, 2 bytes
 *      per (query, key) pair and head of every tile pair it visits, and the dQ
 *      kernel reads it back instead of recomputing it: five products, paid for
 *      with HBM traffic and workspace (4 KiB per 64 keys x 32 queries x head:
 *      21 GB on 65536 causal tokens with 32 heads).  Only
 *      dcp_attn_bwd_strided, which is told total_kv, can take it.
 * A mode whose workspace the caller did not provide (see
 * dcp_attn_bwd_workspace_bytes_kv) or whose conditions do not hold falls back
 * to DCP_BWD_TWO_KERNELS.  Returns the previous setting; any other argument
 * only asks.  No counterpart in the reference, whose backward is one
 * non-deterministic pass with atomic adds
 * (dcp/runtime/flash_attention/executor.py:292-334).
 */
#define DCP_BWD_TWO_KERNELS 0
#define DCP_BWD_ONE_PASS 1
#define DCP_BWD_THROUGH_DS 2
int dcp_attn_bwd_select(int mode);

/*
 * Bytes of workspace the SELECTED backward needs for these sizes, total_kv =
 * the sum of the rows' key counts (cu_seqlens_kv[batch]); what
 * dcp_attn_bwd_workspace_bytes reports plus, for DCP_BWD_THROUGH_DS, the dS
 * pieces, and for DCP_BWD_ONE_PASS the partial sums and chain counters.
 */
size_t dcp_attn_bwd_workspace_bytes_kv(int batch, int total_q, int64_t total_kv,
                                       int block_size, int n_heads_q,
                                       int head_dim);

/*
 * dcp_attn_bwd for callers that cannot allocate device memory or carry a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  Same arguments, results
 * and errors as dcp_attn_bwd without `workspace`/`workspace_bytes`: the scratch
 * is a static device array inside the library, DCP_ATTN_BWD_STATIC_SCRATCH_BYTES
 * long, which every GPU the library runs on holds until the process ends.  Its
 * address on a device is looked up once, by the first of
 * dcp_attn_bwd_static_scratch_bytes() or dcp_attn_bwd_static() called with that
 * device current: a caller that records dcp_attn_bwd_static into a HIP graph
 * calls dcp_attn_bwd_static_scratch_bytes() once per device beforehand, outside
 * the capture, and the recorded call then makes no runtime query.  The call
 * allocates and frees nothing.  Sizes for which dcp_attn_bwd_workspace_bytes(...) exceeds the
 * scratch are rejected with DCP_ERR_ARG.  All calls on one GPU share the one
 * array: calls that may overlap on that GPU (different streams, or graphs
 * replayed side by side) race; calls that follow each other on a stream do not.
 */
#define DCP_ATTN_BWD_STATIC_SCRATCH_BYTES (32u << 20)
size_t dcp_attn_bwd_static_scratch_bytes(void);
int dcp_attn_bwd_static(const void* dout, const void* q, const void* k,
                        const void* v, const void* out, const float* lse,
                        void* dq, void* dk, void* dv,
                        const int32_t* cu_seqlens_q,
                        const int32_t* cu_seqlens_kv,
                        const int32_t* attn_range, int n_ranges,
                        const int32_t* q_block_table,
                        const int32_t* kv_block_table,
                        const int32_t* out_block_table,
                        const int32_t* dq_block_table,
                        const int32_t* dkv_block_table,
                        const int32_t* row_order, int batch, int max_kv_blocks,
                        int total_q, int block_size, int n_heads_q,
                        int n_heads_kv, int head_dim, int64_t kv_slot_stride,
                        int64_t kv_token_stride, int64_t dkv_slot_stride,
                        int64_t dkv_token_stride, int n_out_slots,
                        float softmax_scale, int dtype, void* stream);

/*
 * Stage packer of the planner (host code, no GPU work, `stream`-less): decides
 * which attention blocks ("workloads") every device may run in pipeline stage
 * `stage_id` and which data blocks must be sent to it first, under a cap on the
 * bytes each device sends to other nodes in the stage.
 * Replaces dcp_cpp.greedy_selection_per_device
 * (csrc/pipeline_generator/pipeline_generator.cpp:19-323, bound in
 * csrc/interface.cpp:9-11, called from dcp/core/pipeline.py:651-666,703-716).
 * The reference's sets and dicts of (node, rank) tuples become dense tables;
 * all pointers are HOST memory:
 *   device_node[d]               node of device d (devices are 0..n_devices-1)
 *   workload_costs[w], workload_scheduled[w] (nonzero: already placed in an
 *                                earlier stage, i.e. the reference's
 *                                `scheduled_workloads` set)
 *   input_sizes[i], input_kind[i]  size and DCP_BLOCK_* kind of data block i
 *                                (the reference's input_block_type_map strings
 *                                "OUT" / "LSE" / "dOUT", anything else OTHER)
 *   workload_input_offsets/workload_inputs   CSR of workload_input_map
 *   device_workload_offsets/device_workloads CSR of device_workload_map
 *   held_since[d * n_inputs + i] in/out: the stage since which device d holds
 *                                block i (-1 = from the start), DCP_NOT_HELD if
 *                                it does not (device_local_inputs_map; updated
 *                                in place = the third element of the result)
 *   target_cross_node_load[d]    target_comm_load_per_node
 * Results: unlocked_by[w] = device that may now run workload w, or -1 (first
 * element of the reference's result); the transfers (comm_dst[k], comm_input[k],
 * comm_src[k]) for k < *n_comm in the order they were decided (second element;
 * n_devices * n_inputs entries always suffice -- on a nonzero return because
 * `comm_capacity` was too small, *n_comm holds the needed count and held_since
 * has been modified: call again from the original table); optionally each
 * device's outgoing cross-node and same-node bytes (what the reference logs).
 * Where the reference's choice depends on the iteration order of a hash table
 * (equal compute times, equal sender loads, equal costs) the lowest device
 * index / workload id wins.
 */
#define DCP_BLOCK_OTHER 0
#define DCP_BLOCK_OUT 1
#define DCP_BLOCK_LSE 2
#define DCP_BLOCK_DOUT 3
#define DCP_NOT_HELD INT32_MIN
int dcp_greedy_stage_selection(
    int n_devices, const int32_t* device_node, int n_workloads,
    const float* workload_costs, const uint8_t* workload_scheduled,
    int n_inputs, const float* input_sizes, const uint8_t* input_kind,
    const int32_t* workload_input_offsets, const int32_t* workload_inputs,
    const int32_t* device_workload_offsets, const int32_t* device_workloads,
    int32_t* held_since, const float* target_cross_node_load, int is_bw,
    int stage_id, int32_t* unlocked_by, int32_t* comm_dst, int32_t* comm_input,
    int32_t* comm_src, int64_t comm_capacity, int64_t* n_comm,
    float* cross_node_load_out, float* intra_node_load_out);

#ifdef __cplusplus
}
#endif
#endif /* DCP_HIP_H_ */
