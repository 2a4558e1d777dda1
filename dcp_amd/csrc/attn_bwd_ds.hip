// Backward through dS in memory (gfx950): five matrix products instead of seven, paid for with
// HBM traffic the attention kernels otherwise leave unused.
//
//   bwd_prepare_kernel       (attn_bwd_fused.hip) hulls, -delta, base-2 log-sum-exp
//   attn_bwd_dkv_kernel<.., true>  (attn_bwd.hip) the key-outer kernel as always -- S, dP, dV, dK --
//                            which also stores dS, rounded to the storage type as it feeds dK
//   attn_bwd_dq_ds_kernel    (here) query-outer: dQ^T[d, q] += K^T[d, kv] dS^T[kv, q], with dS^T read
//                            back from memory instead of being recomputed from Q, K, V and dO
//
// The two-kernel backward recomputes S and dP in its dQ kernel (three products); this dQ kernel
// runs one, has no softmax arithmetic, no masks (masked dS was stored as zero) and no per-query
// values, and is bound by the stream of dS out of HBM: 2 bytes per (query, key) pair and head of
// every (64-query tile, 128-key tile) pair the dK/dV kernel visits.
//
// dS travels in pieces of 64 keys x 32 queries of one head (4 KiB), written by a wave of the dK/dV
// kernel exactly as its lanes hold them (lane = key, four consecutive queries per register pair)
// in whole 1 KiB stores.  A wave here owns 32 queries (one piece per 64-key tile), brings its
// pieces into a region of LDS of its own with global_load_lds and reads them as the B operand
// through transposing loads, whose per-lane addresses undo the layout; no other wave touches the
// piece, so it needs no barrier, only the wave's own wait.  K tiles are shared by the workgroup's
// waves as in the other kernels.
//
// The kernel does nothing but wait for memory unless loads are in flight all the time (with the
// matrix instructions taken out it runs as long as with them), so a workgroup is eight waves (256
// queries, one workgroup per CU: half the K traffic of four-wave workgroups) with three stages of
// pieces in LDS: while step s is multiplied, the loads of steps s + 1 and s + 2 are under way, and a
// wave waits for step s alone by counting its own loads (vmcnt), not for everything.  Where the kv
// head has an even number of q heads a work item takes two of them, alternating between them tile
// by tile: a K tile in LDS serves both heads' pieces (half the K loads again), and the waves meet at
// a barrier only where the K tile changes, every other step.  On the 65536-token causal benchmark
// (16.8 GB of dS) the kernel takes 3.0 ms, 5.9 TB/s out of HBM; with one head per item 3.2 ms;
// with four-wave workgroups, two stages and a full wait per tile 3.4 ms.  A kernel that only
// streams 4 KiB pieces per wave into LDS the same way reads 7.0 TB/s (6.6 with a workgroup barrier
// per step, 6.0-6.2 with a K tile's loads beside it); the rest is the start of every work item (a
// chain of dependent table reads and an empty pipeline: with no tiles at all the kernel takes
// 0.21 ms, and every item waits once for its first tile).
#include <math.h>

#include <algorithm>

#include "attn_bwd_params.h"

namespace dcp {

constexpr int kDsWaves = 8;
constexpr int kDsThreads = 64 * kDsWaves;
constexpr int kDsBM = 32 * kDsWaves;  // queries per workgroup
constexpr int kDsBN = 64;             // keys per tile
constexpr int kDsStages = 3;

// HH: q heads per work item (1, or 2 of the same kv head).  With two, a K tile brought into LDS
// serves both heads' pieces: the sequence of steps is (tile 0, head 0), (tile 0, head 1), (tile 1,
// head 0), ... -- half the K loads, and a barrier only where the K tile changes (the pieces are
// private to their wave).
template <int DTYPE, int D, int HH>
__device__ __forceinline__ void attn_bwd_dq_ds_item(KernArgs<AttnBwdParams>& p, int item) {
  constexpr int BN = kDsBN;
  constexpr int DT = D / 32;
  constexpr int KSTAGES = HH == 1 ? kDsStages : 2;  // K tiles requested two steps ahead: two tiles, or one
  typedef KvTile<D, kDsWaves> Tile;
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[KSTAGES][Tile::SIZE];
  __shared__ __attribute__((aligned(16))) uint16_t ds_lds[kDsStages][kDsWaves][2048];  // [stage][wave]: one piece
  __shared__ int slot_lds[kSlotTableCap];

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int c = lane & 31;
  const int h = lane >> 5;

  int wg = item;
  const int qt = __builtin_amdgcn_readfirstlane(wg % p.dq_tiles_per_row);
  wg /= p.dq_tiles_per_row;
  const int head = __builtin_amdgcn_readfirstlane(wg % (p.n_heads_q / HH)) * HH;  // the item's first head
  const int bi = __builtin_amdgcn_readfirstlane(wg / (p.n_heads_q / HH));
  const int b = __builtin_amdgcn_readfirstlane(p.row_order ? p.row_order[bi] : bi);
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int kv_begin = p.cu_seqlens_kv[b];
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - kv_begin;
  if (qt * kDsBM >= seqlen_q) return;
  const int kv_head = __builtin_amdgcn_readfirstlane(head / (p.n_heads_q / p.n_heads_kv));
  const int64_t q_row_stride = (int64_t)p.n_heads_q * D;
  const int q_local = qt * kDsBM + w * 32 + c;
  const bool q_valid = q_local < seqlen_q;

  // ---- which key tiles: the 128-key tiles the dK/dV kernel visited for this wave's 64-query tile
  // (the same test on the same hulls: a piece that was never written is never read), and for the
  // workgroup the hull of its two 64-query tiles -----------------------------------------------
  constexpr int T64 = kDsBM / 64;  // 64-query tiles of a workgroup
  const int qt64 = T64 * qt + (w >> 1);
  const bool wave_has_tile = qt64 < p.q_tiles_per_row;
  const int32_t* hull_row = p.hull + (int64_t)b * p.q_tiles_per_row * 8;
  int hw[4] = {0x7fffffff, 0, 0x7fffffff, 0};
  if (wave_has_tile) {
#pragma unroll
    for (int i = 0; i < 4; ++i) hw[i] = __builtin_amdgcn_readfirstlane(hull_row[qt64 * 8 + i]);
  }
  const TileRuns mine(hw[0], hw[1], hw[2], hw[3], 128);  // in 128-key tiles
  int g[4] = {0x7fffffff, 0, 0x7fffffff, 0};
#pragma unroll
  for (int t = 0; t < T64; ++t) {
    if (T64 * qt + t >= p.q_tiles_per_row) continue;
    const int32_t* hu = hull_row + (T64 * qt + t) * 8;
    g[0] = min(g[0], __builtin_amdgcn_readfirstlane(hu[0]));
    g[1] = max(g[1], __builtin_amdgcn_readfirstlane(hu[1]));
    g[2] = min(g[2], __builtin_amdgcn_readfirstlane(hu[2]));
    g[3] = max(g[3], __builtin_amdgcn_readfirstlane(hu[3]));
  }
  TileRuns runs(g[0], g[1], g[2], g[3], 128);
  // as runs of 64-key tiles, none past the row's last key (its key count is a multiple of 64)
  const int last64 = (seqlen_kv + BN - 1) / BN;
  runs.a0 *= 2;
  runs.b0 = min(runs.b0 * 2, last64);
  runs.a1 *= 2;
  runs.b1 = min(runs.b1 * 2, last64);
  if (runs.b0 < runs.a0) runs.b0 = runs.a0;
  if (runs.b1 < runs.a1) runs.b1 = runs.a1;
  const int n_tiles = runs.count();

  const int32_t* kv_table = p.kv_block_table + (int64_t)b * p.max_kv_blocks;
  load_slot_table(slot_lds, kv_table, p.max_kv_blocks, tid, kDsThreads);
  __syncthreads();

  f32x16 dq_acc[HH][DT];
#pragma unroll
  for (int hh = 0; hh < HH; ++hh)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) dq_acc[hh][dt][i] = 0.0f;

  const uint16_t* kg = reinterpret_cast<const uint16_t*>(p.k) + (int64_t)kv_head * D;
  const uint32_t kv_goff0 = Tile::lane_offset0(p.kv_token_stride, w, lane);
  const int col_rd = Tile::col_base(lane, false);  // K^T, contraction index = key in plain order
  // this lane's 8 bytes inside a piece for k-step 0 (see the file comment and attn_bwd.hip):
  // 16-lane group L = lane >> 4: queries 16 (L & 1) + ..., keys 8 (L >> 1) + ...; lane j of the group
  // supplies key row j >> 2 and the four queries 4 (j & 3)..
  const int j = lane & 15, L = lane >> 4;
  const int ds_rd = (L & 1) * 1024 + (2 * (8 * (L >> 1) + (j >> 2)) + (j & 1)) * 16 + ((j & 3) >> 1) * 8;  // bytes

  const int tiles_per_block = p.block_size / BN;
  const int64_t tile_stride = (int64_t)BN * p.kv_token_stride;
  TileCursor cursor;
  // the wave's piece of key tile t (the layout is described in the dK/dV kernel): its pieces lie one
  // after another in key order
  const int sub = qt * kDsWaves + w;
  const uint64_t row_base = ((uint64_t)(kv_begin / 64) + b) * p.n_heads_q * p.subs_per_row;
  const uint64_t piece0 = reinterpret_cast<uint64_t>(p.ds) +
                          ((row_base + ((uint64_t)head * p.subs_per_row + sub) * (uint64_t)last64) << 12);
  const uint64_t piece_step = 4096;
  const uint64_t head_step = ((uint64_t)p.subs_per_row * (uint64_t)last64) << 12;  // to the next head's pieces
  auto wave_sees = [&](int t64) {
    const int t = t64 >> 1;
    return wave_has_tile && ((t >= mine.a0 && t < mine.b0) || (t >= mine.a1 && t < mine.b1));
  };
  constexpr int NL = Tile::LPW;
  uint32_t fill_k = 0, fill_ds = 0;
  // what a step needs: (for the item's first head) this wave's share of the K tile `cursor` points at,
  // and the wave's own piece of that tile and head if it sees the tile
  auto request = [&](int hh) {
    if (hh == 0) {
#pragma unroll
      for (int i = 0; i < NL; ++i) Tile::load_group(fill_k, kg + cursor.off, kv_goff0, p.kv_token_stride, w, i);
    }
    if (wave_sees(cursor.tile)) {
      const uint64_t src = uniform64(piece0 + hh * head_step + (uint64_t)cursor.tile * piece_step);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        Tile::load_group_at_streaming(__builtin_amdgcn_readfirstlane(fill_ds + i * 1024), uniform64(src + i * 1024), lane * 16);
    }
  };
  auto advance = [&]() {
    if (cursor.index + 1 < n_tiles)
      cursor.advance(runs, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
  };
  auto compute = [&](f32x16 (&acc)[DT], int t64, const uint16_t* k_lds, const uint16_t* piece) {
    if (!wave_sees(t64)) return;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const char* pb = reinterpret_cast<const char*>(piece) + ds_rd;
    auto ds_operand = [&](int ks) -> u32x4 {
      const char* p0 = pb + (ks >> 1) * 2048 + (ks & 1) * 512;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0 + 128));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      return u32x4{l2[0], l2[1], h2[0], h2[1]};
    };
    u32x4 kt_a[2][DT], dsb[2];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) kt_a[0][dt] = Tile::template read_col<false>(k_lds, col_rd, 0, dt);
    dsb[0] = ds_operand(0);
#pragma unroll
    for (int ks = 0; ks < BN / 16; ++ks) {
      if (ks + 1 < BN / 16) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) kt_a[(ks + 1) & 1][dt] = Tile::template read_col<false>(k_lds, col_rd, ks + 1, dt);
        dsb[(ks + 1) & 1] = ds_operand(ks + 1);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[dt] = mfma_32x32x16<DTYPE>(kt_a[ks & 1][dt], dsb[ks & 1], acc[dt]);
    }
  };

  // Step s = (tile s / HH, head s % HH).  The pieces go through three stages (step s in stage
  // s % 3), the K tiles through KSTAGES.  Before it multiplies step s, a wave waits until the loads it
  // issued for step s have landed -- the ones for step s + 1, issued after them, may still be under
  // way: vmcnt counts a wave's loads in order -- and, where the K tile changes, meets the others at a
  // barrier: everybody's share of the K tile is there, and everybody is done with the tile before,
  // whose stage (with three K stages: the stage of the tile before that) the loads of step s + 2
  // now refill.  The pieces are private to their wave and need no barrier.
  const uint32_t k_at0 = lds_address(&k_lds[0][0]), ds_at0 = lds_address(&ds_lds[0][w][0]);
  constexpr uint32_t kKStageBytes = Tile::SIZE * 2, kDsStageBytes = kDsWaves * 4096;
  const int total = HH * n_tiles;
  if (n_tiles > 0) {
    cursor.seek(runs, 0, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
    fill_k = k_at0;
    fill_ds = ds_at0;
    request(0);
    if (total > 1) {
      if (HH == 1) advance();
      fill_k = k_at0 + kKStageBytes;  // (only used when this step brings a K tile: HH == 1)
      fill_ds = ds_at0 + kDsStageBytes;
      request(1 % HH);
    }
  }
  int ds_stage = 0, k_stage = 0;
  for (int t = 0; t < n_tiles; ++t) {
#pragma unroll
    for (int hh = 0; hh < HH; ++hh) {
      const int s_idx = t * HH + hh;
      // the next step: its head, its tile, what it loads
      const bool next_new_tile = hh + 1 == HH;
      const int t_next = next_new_tile ? t + 1 : t;
      if (s_idx + 1 >= total) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      } else {
        const bool sees = wave_sees(runs.tile(t_next));
        if (next_new_tile) {
          if (sees) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL + 4) : "memory");
          else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
        } else {
          if (sees) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
          else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
      }
      if (hh == 0) phase_barrier();
      if (s_idx + 2 < total) {
        // step s + 2: head (hh + 2) % HH; it brings the next K tile along if that is the item's first head
        const int hh_req = (hh + 2) % HH;  // (a constant once the loop over hh is unrolled)
        if (hh_req == 0) advance();
        fill_ds = ds_at0 + (ds_stage == 0 ? 2 : ds_stage - 1) * kDsStageBytes;  // (s + 2) % 3
        if (hh_req == 0) fill_k = k_at0 + (HH == 1 ? (k_stage == 0 ? 2 : k_stage - 1) : (k_stage ^ 1)) * kKStageBytes;
        request(hh_req);
      }
      compute(dq_acc[hh], runs.tile(t), &k_lds[k_stage][0], &ds_lds[ds_stage][w][0]);
      ds_stage = ds_stage == kDsStages - 1 ? 0 : ds_stage + 1;
    }
    k_stage = k_stage == KSTAGES - 1 ? 0 : k_stage + 1;
  }

  if (!q_valid) return;
#pragma unroll
  for (int hh = 0; hh < HH; ++hh) {
    uint16_t* op = reinterpret_cast<uint16_t*>(p.dq) + (int64_t)p.dq_block_table[b] * p.dq_slot_stride +
                   (int64_t)q_local * q_row_stride + (int64_t)(head + hh) * D + 4 * h;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        u32x2 pk = {pack2<DTYPE>(dq_acc[hh][dt][4 * gq] * p.scale, dq_acc[hh][dt][4 * gq + 1] * p.scale),
                    pack2<DTYPE>(dq_acc[hh][dt][4 * gq + 2] * p.scale, dq_acc[hh][dt][4 * gq + 3] * p.scale)};
        *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * gq) = pk;
      }
  }
}

// persistent, like the recomputing dQ kernel: per-XCD tickets in the workspace (zeroed by the prepare kernel)
template <int DTYPE, int D, int HH>
__global__ __launch_bounds__(kDsThreads, 1) void attn_bwd_dq_ds_kernel(const AttnBwdParams p) {
  __shared__ int ticket_lds;
  const int x = blockIdx.x % kNumXcd;
  const int64_t n_streams = (p.n_dq_items + p.dq_xcd_group - 1) / p.dq_xcd_group;
  const int64_t n_x = n_streams > x ? (n_streams - x + kNumXcd - 1) / kNumXcd * p.dq_xcd_group : 0;
  while (true) {
    if (threadIdx.x == 0) ticket_lds = atomicAdd(&p.tickets[x], 1);
    __syncthreads();
    const int i = __builtin_amdgcn_readfirstlane(ticket_lds);
    if (i >= n_x) break;
    const int64_t item = (x + kNumXcd * (int64_t)(i / p.dq_xcd_group)) * p.dq_xcd_group + i % p.dq_xcd_group;
    if (item < p.n_dq_items) attn_bwd_dq_ds_item<DTYPE, D, HH>(fresh_kernel_args<AttnBwdParams>(), (int)item);
    __syncthreads();
  }
}

size_t bwd_ds_workspace_bytes(int64_t total_kv, int batch, int block_size, int n_heads_q) {
  if (total_kv <= 0) return 0;
  const size_t subs = (block_size + 31) / 32;
  // a 64-key tile more per row than total_kv / 64 (rows may end inside a tile), and two spare pieces (see the dK/dV kernel)
  return ((size_t)(total_kv / 64 + batch + 1) * n_heads_q * subs + 2) << 12;
}

int launch_bwd_through_ds(const AttnBwdParams& p, int dtype, hipStream_t stream) {
  if (const int e = launch_bwd_prepare(p, dtype, stream)) return e;  // (also zeroes the dQ kernel's tickets)
  if (const int e = launch_bwd_dkv_writing_ds(p, dtype, stream)) return e;
  // this dQ kernel's work items: (row, one or two q heads of a kv head, 256-query tile); the tiles and
  // heads that share a K stay on one XCD
  const int per_kv = p.n_heads_q / p.n_heads_kv;
  const int hh = per_kv % 2 == 0 ? 2 : 1;  // (four heads' accumulators do not fit the 256 registers of a wave)
  AttnBwdParams q = p;
  q.dq_tiles_per_row = (p.block_size + kDsBM - 1) / kDsBM;
  q.n_dq_items = (int64_t)p.batch * (p.n_heads_q / hh) * q.dq_tiles_per_row;
  q.dq_xcd_group = q.dq_tiles_per_row * (per_kv / hh);
  DCP_REQUIRE(q.n_dq_items < ((int64_t)1 << 31), "attn_bwd: grid too large");
  const int64_t n_dq = std::min<int64_t>(xcd_grid_size(q.n_dq_items, 1), xcd_grid_size((int64_t)device_cu_count(), 1));
  KernelTimer timer("attn_bwd_dq_ds_kernel", stream);
  const dim3 grid((unsigned)n_dq), block(kDsThreads);
#define DCP_DQ_DS_LAUNCH(DT, HD, HH) hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<DT, HD, HH>), grid, block, 0, stream, q)
  if (dtype == DCP_DTYPE_BF16) {
    if (p.head_dim == 128) { if (hh == 2) DCP_DQ_DS_LAUNCH(DCP_DTYPE_BF16, 128, 2); else DCP_DQ_DS_LAUNCH(DCP_DTYPE_BF16, 128, 1); }
    else { if (hh == 2) DCP_DQ_DS_LAUNCH(DCP_DTYPE_BF16, 64, 2); else DCP_DQ_DS_LAUNCH(DCP_DTYPE_BF16, 64, 1); }
  } else {
    if (p.head_dim == 128) { if (hh == 2) DCP_DQ_DS_LAUNCH(DCP_DTYPE_FP16, 128, 2); else DCP_DQ_DS_LAUNCH(DCP_DTYPE_FP16, 128, 1); }
    else { if (hh == 2) DCP_DQ_DS_LAUNCH(DCP_DTYPE_FP16, 64, 2); else DCP_DQ_DS_LAUNCH(DCP_DTYPE_FP16, 64, 1); }
  }
#undef DCP_DQ_DS_LAUNCH
  return check_launch("attn_bwd_dq_ds_kernel");
}

}  // namespace dcp
