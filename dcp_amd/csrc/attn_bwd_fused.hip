// Range-masked paged attention backward in ONE key-outer pass (head size 128, gfx950).
//
// The two-kernel backward (attn_bwd.hip) recomputes S and dP in a second, query-outer kernel in
// order to keep dQ in registers: seven matrix products for the five the backward consists of.
// Here the key-outer kernel forms dQ as well:
//
//   bwd_prepare_kernel     per (row, 64-query tile): the range hulls, -delta = -sum_d dO*O and the
//                          base-2 log-sum-exp of its queries, the chain counters zeroed, dQ zeroed
//                          where no key tile will ever visit the tile
//   attn_bwd_fused_kernel  one workgroup per (row, kv head, 128-key tile): dK^T, dV^T of its keys
//                          in registers as in the dK/dV kernel, and per step its contribution
//                          dS K (over its 128 keys) to dQ of the step's queries
//
// A step is 32 queries of one q head.  Wave w owns keys 32w..32w+31 for S, dP, dV and dK exactly
// as in the dK/dV kernel; dS of the four waves meets in LDS ([key][query], written in accumulator
// order, read back by transposing loads), and wave w then forms
//
//   dQ^T[32w..32w+31, q] += K^T[dims of the wave, 128 keys] dS^T[128 keys, q]
//
// i.e. the dQ contribution of ALL the workgroup's keys for its slice of the head dims: 8 matrix
// instructions per wave and step where the recomputing kernel needed 24 (S, dP, dQ).
//
// The contributions of a row's key tiles to one (head, 32-query) chunk of dQ are added in a
// CHAIN, in key order and without atomics: the tiles of a row that see a query tile are known to
// every workgroup from the tile's range hull, so each knows its rank among them.  Rank 0 starts
// from zero; rank r waits until the chunk's counter says r (rank r-1 has stored its partial sum,
// fp32, in the workspace), takes the partial sum as the initial value of its dQ^T accumulator,
// adds its own product, stores it back and passes the counter on; the last rank scales, rounds
// and writes dQ itself.  (fp32 atomic adds run at 1.4 TB/s on this device whatever the cache
// level they are asked for -- three times less than the 4 B per (query, key) pair and head that
// 128-key tiles produce -- and they would make dQ depend on the order of arrival.  The chain
// moves the same bytes as ordinary loads and stores, 16 bytes per lane, and the order is fixed:
// dQ is bit-reproducible.)
//
// Each wave passes its own slice on (one counter per chunk and wave), so no workgroup barrier is
// involved.  All key tiles of a row sit on one XCD (their workgroup ids are dealt that way, for
// the sake of the Q/dO tiles they share), so a partial sum travels through that XCD's L2: the
// stores are complete (acknowledged by the L2) before the counter is passed on, and the next
// rank reads counter and data past its CU's own cache (sc1).  Workgroups are dispatched in id
// order and a workgroup only ever waits for lower ids of its own row, so the chain cannot
// deadlock; a spin limit bounds every wait all the same (a wave that reaches it raises the fault
// flag in the workspace and goes on with what it finds).
//
// Steps run over the query tiles from the LAST to the first (heads innermost): with a causal mask
// every key tile of a row sees the last query tile, so all of them start there one behind the
// other, and a tile on the diagonal simply finishes early instead of idling until its
// predecessors reach its first tile.
#include <math.h>
#include <stdlib.h>

#include <algorithm>
#include <mutex>

#include "attn_bwd_params.h"

namespace dcp {

constexpr int kFusedBM = 32;              // queries per step
constexpr int kFusedBN = 128;             // keys per workgroup
constexpr int kDsStride = 36;             // elements per key row of the dS exchange (32 queries + 8 bytes)
constexpr int kChunkFloats = 4096;        // one chunk of partial dQ: 32 queries x 128 dims
constexpr int kSpinLimit = 1 << 20;       // polls of a chain counter before a wave gives up (and raises the fault flag)

// Key tiles (128 keys) that see a 64-query tile, from the tile's range hull: two runs of tile
// numbers.  Every workgroup of a row derives its rank in the chain of a query tile from this,
// and the prepare kernel the number of links, so both must be this one function.
__device__ __forceinline__ TileRuns chain_runs(const int32_t* hull) {
  return TileRuns(hull[0], hull[1], hull[2], hull[3], kFusedBN);
}

// ---------------------------------------------------------------------------
// prepare: hulls, -delta, lse2, counters
// ---------------------------------------------------------------------------
template <int DTYPE, int D>
__global__ __launch_bounds__(kBwdThreads) void bwd_prepare_kernel(const AttnBwdParams p) {
  __shared__ int hull_lds[8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x / p.q_tiles_per_row;
  const int qt = blockIdx.x - b * p.q_tiles_per_row;
  if (blockIdx.x == 0 && tid == 0 && p.fault != nullptr) *p.fault = 0;
  if (blockIdx.x == 0 && tid < kTicketInts) p.tickets[tid] = 0;  // for a persistent dQ kernel that follows
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - p.cu_seqlens_kv[b];
  if (wave == 0) {
    const int ql = qt * kBwdBM + lane;
    int s0 = 0, l0 = 0, s1 = 0, l1 = 0;
    if (ql < seqlen_q) {
      const int32_t* r = p.attn_range + q_begin + ql;
      s0 = r[0];
      l0 = max(min(r[p.total_q], seqlen_kv) - s0, 0);
      if (p.n_ranges == 2) {
        s1 = r[2 * (int64_t)p.total_q];
        l1 = max(min(r[3 * (int64_t)p.total_q], seqlen_kv) - s1, 0);
      }
    }
    const int big = 0x7fffffff;
    const int v0 = wave_min(l0 > 0 ? s0 : big), v1 = wave_max(l0 > 0 ? s0 + l0 : 0);
    const int v2 = wave_min(l1 > 0 ? s1 : big), v3 = wave_max(l1 > 0 ? s1 + l1 : 0);
    const int v4 = wave_max(l0 > 0 ? s0 : big), v5 = wave_min(l0 > 0 ? s0 + l0 : 0);
    const int v6 = wave_max(l1 > 0 ? s1 : big), v7 = wave_min(l1 > 0 ? s1 + l1 : 0);
    if (lane < 8) {
      const int vals[8] = {v0, v1, v2, v3, v4, v5, v6, v7};
      int mine = vals[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) mine = lane == i ? vals[i] : mine;
      p.hull[(int64_t)blockIdx.x * 8 + lane] = mine;
      hull_lds[lane] = mine;
    }
  }
  __syncthreads();
  // (dQ of a query tile no key tile visits is only zeroed here for the one-pass kernel, which
  // writes dQ tile by tile; a query-outer dQ kernel writes every valid query itself)
  const bool nobody_visits = p.chain != nullptr && chain_runs(hull_lds).count() == 0;

  // counters of the tile's chunks: [(row, head, 32-query sub-tile)][wave]
  const int H = p.n_heads_q;
  for (int i = tid; p.chain != nullptr && i < H * 2 * 4; i += kBwdThreads) {
    const int head = i / 8, rest = i - head * 8;
    const int sub = qt * 2 + rest / 4;
    if (sub < p.subs_per_row) p.chain[(((int64_t)b * H + head) * p.subs_per_row + sub) * 4 + (rest & 3)] = 0;
  }

  // -delta and lse2 of the tile's (query, head) pairs: 16 lanes per pair, 8 elements each
  // (head size 128; 8 lanes do for 64)
  constexpr int LPP = D / 8;               // lanes per pair
  constexpr int PPW = 64 / LPP;            // pairs per wave instruction
  const int n_q = min(kBwdBM, seqlen_q - qt * kBwdBM);
  const int o_slot = p.out_block_table[b];
  const int64_t row_stride = (int64_t)H * D;
  const int sub_lane = lane % LPP;
  // (four positions per round, all their words requested before anything is stored: the stores could
  // alias the loads as far as the compiler knows, so it would not move a load above one itself)
  constexpr int U = 4;
  constexpr int STEP = (kBwdThreads / 64) * PPW;
  for (int pair0 = wave * PPW; pair0 < n_q * H; pair0 += U * STEP) {
    u32x4 o[U], g[U];
    float l[U];
    bool live[U];
    int q_local[U], head[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int pair = pair0 + u * STEP + lane / LPP;
      live[u] = pair < n_q * H;
      const int ql = live[u] ? pair / H : 0;
      head[u] = live[u] ? pair - ql * H : 0;
      q_local[u] = qt * kBwdBM + ql;
      const int64_t off = (int64_t)o_slot * p.out_slot_stride + (int64_t)q_local[u] * row_stride + (int64_t)head[u] * D + sub_lane * 8;
      o[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.out) + off));  // read here only
      g[u] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.dout) + off);
      l[u] = p.lse[(int64_t)head[u] * p.lse_head_stride + (int64_t)o_slot * p.lse_slot_stride + q_local[u]];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float dot = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dot += Elem<DTYPE>::load((uint16_t)(o[u][i] & 0xffffu)) * Elem<DTYPE>::load((uint16_t)(g[u][i] & 0xffffu));
        dot += Elem<DTYPE>::load((uint16_t)(o[u][i] >> 16)) * Elem<DTYPE>::load((uint16_t)(g[u][i] >> 16));
      }
#pragma unroll
      for (int m = 1; m < LPP; m *= 2) dot += __shfl_xor(dot, m);
      if (live[u] && sub_lane == 0) {
        const int64_t qrow = (int64_t)(q_begin + q_local[u]) * H + head[u];
        p.delta[qrow] = -dot;
        p.lse2[qrow] = l[u] * kLog2e;
      }
      if (nobody_visits && live[u]) {  // no key tile sees these queries: their dQ is zero, and nobody else writes it
        const u32x4 zero = {0, 0, 0, 0};
        *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(p.dq) +
                                  (int64_t)p.dq_block_table[b] * p.dq_slot_stride + (int64_t)q_local[u] * row_stride +
                                  (int64_t)head[u] * D + sub_lane * 8) = zero;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// the fused kernel
// ---------------------------------------------------------------------------
// One 16-byte word per lane from global memory straight into LDS, lane l's word at lds_at + 16 l,
// every lane with an address of its own.
__device__ __forceinline__ void load_async_b128(uint32_t lds_at, const void* g) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_at)), "v"(g)
               : "memory");
}

template <int DTYPE>
__global__ __launch_bounds__(kBwdThreads, 2) void attn_bwd_fused_kernel(const AttnBwdParams p) {
  constexpr int D = 128, BM = kFusedBM, BN = kFusedBN;
  constexpr int KS = D / 16;  // k-steps over the head dim
  constexpr int DT = D / 32;  // 32-dim blocks of dK^T / dV^T
  typedef KvTile<D> Tile;     // 64 rows x D: a step's Q (rows 0..31) and dO (rows 32..63); half of the K tile

  __shared__ __attribute__((aligned(16))) uint16_t qdo[2][Tile::SIZE];  // two stages
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[2][Tile::SIZE];  // keys 0..63, 64..127
  __shared__ __attribute__((aligned(16))) uint16_t ds_lds[BN * kDsStride];
  __shared__ __attribute__((aligned(16))) int rng_lds[2][4][BM];  // planes: start0, end0, start1, end1
  __shared__ __attribute__((aligned(16))) float sc_lds[2][2][BM];  // lse2, -delta

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int c = lane & 31;
  const int h = lane >> 5;

  // ---- which (row, kv head, key tile) ------------------------------------------
  int wg = xcd_logical_id(blockIdx.x, p.dkv_xcd_group, p.n_dkv_items);
  if (wg < 0) return;
  const int kt = __builtin_amdgcn_readfirstlane(wg % p.kv_tiles_per_row);
  wg /= p.kv_tiles_per_row;
  const int kv_head = __builtin_amdgcn_readfirstlane(wg % p.n_heads_kv);
  const int bi = __builtin_amdgcn_readfirstlane(wg / p.n_heads_kv);
  const int b = __builtin_amdgcn_readfirstlane(p.row_order ? p.row_order[bi] : bi);
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - p.cu_seqlens_kv[b];
  const int k0 = kt * BN;
  if (k0 >= seqlen_kv) return;
  const int kw = k0 + w * 32;
  const bool has_keys = kw < seqlen_kv;
  const int kv_or_beyond = kw + c < seqlen_kv ? kw + c : 0x7fffffff;
  const int kw_safe = has_keys ? kw : k0;
  const int blk = __builtin_amdgcn_readfirstlane(kw_safe / p.block_size);
  const int tok0 = kw_safe - blk * p.block_size;
  const int group = p.n_heads_q / p.n_heads_kv;
  const int H = p.n_heads_q;
  const int64_t q_row_stride = (int64_t)H * D;
  const int q_slot = p.q_block_table[b];
  const int o_slot = p.out_block_table[b];
  const int n_q_tiles = (seqlen_q + kBwdBM - 1) / kBwdBM;
  const int32_t* kv_table = p.kv_block_table + (int64_t)b * p.max_kv_blocks;

  // ---- the K tile of the workgroup's 128 keys into LDS (rows past the row's last key repeat
  // the tile's first key: finite, and masked wherever they are used) ---------------------------
  {
    constexpr int CH = D / 8;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < Tile::LPW; ++i) {
        const int grp = w * Tile::LPW + i;
        const int r = t * 64 + Tile::row_of(grp, lane / CH);
        const int key = k0 + r < seqlen_kv ? k0 + r : k0;
        const int kb = key / p.block_size;
        const int64_t off = (int64_t)kv_table[kb] * p.kv_slot_stride + (int64_t)(key - kb * p.block_size) * p.kv_token_stride +
                            (int64_t)kv_head * D + (lane % CH) * 8;
        load_async_b128(lds_address(&k_lds[t][0]) + grp * (Tile::GROUP_STRIDE * 2),
                        reinterpret_cast<const uint16_t*>(p.k) + off);
      }
  }
  // ---- V of this wave's 32 keys as B operands (lane = key, slots = dims) -------------------
  u32x4 vreg[KS];
  {
    const int64_t off = (int64_t)kv_table[blk] * p.kv_slot_stride + (int64_t)(tok0 + c) * p.kv_token_stride +
                        (int64_t)kv_head * D + h * 8;
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.v) + off;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) vreg[ks] = *reinterpret_cast<const u32x4*>(vp + ks * 16);
  }

  f32x16 dk_acc[DT], dv_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dk_acc[dt][i] = 0.0f;
      dv_acc[dt][i] = 0.0f;
    }

  // ---- per 64-query tile (lane = tile): does the workgroup's key tile see it, its rank in the
  // tile's chain and the chain's length; does every query of it see all of this wave's keys ----
  unsigned long long act_mask, unm_w;
  int rank_v = 0, count_v = 0;
  {
    bool a = false, u = false;
    if (lane < n_q_tiles) {
      const int32_t* hu = p.hull + ((int64_t)b * p.q_tiles_per_row + lane) * 8;
      const TileRuns runs = chain_runs(hu);
      const bool in0 = kt >= runs.a0 && kt < runs.b0, in1 = kt >= runs.a1 && kt < runs.b1;
      a = in0 || in1;
      rank_v = in0 ? kt - runs.a0 : (runs.b0 - runs.a0) + (kt - runs.a1);
      count_v = runs.count();
      u = has_keys && ((hu[4] <= kw && kw + 32 <= hu[5]) || (hu[6] <= kw && kw + 32 <= hu[7]));
    }
    act_mask = __ballot(a);
    unm_w = __ballot(u);
  }
  const uint32_t act_lo = __builtin_amdgcn_readfirstlane((uint32_t)act_mask);
  const uint32_t act_hi = __builtin_amdgcn_readfirstlane((uint32_t)(act_mask >> 32));
  act_mask = ((unsigned long long)act_hi << 32) | act_lo;

  // loop-invariant per-lane pieces of the addresses used in the loop
  const int row_rd = Tile::row_base(c, h);
  const int col_rd = Tile::col_base(lane, true);    // Q^T / dO^T in accumulator row order
  const int col_rd_k = Tile::col_base(lane, false);  // K^T slices, contraction index = key in plain order
  const uint16_t* q_base = reinterpret_cast<const uint16_t*>(p.q) + (int64_t)q_slot * p.q_slot_stride;
  const uint16_t* do_base = reinterpret_cast<const uint16_t*>(p.dout) + (int64_t)o_slot * p.out_slot_stride;
  const uint32_t qdo_at = lds_address(&qdo[0][0]);
  // A step's tile is one 64-row tile: Q of its 32 queries in rows 0..31, dO in rows 32..63, so a
  // group load takes its lanes 0..31 from Q and 32..63 from dO.  Per lane: which array, which of
  // the 32 queries (group load i of the wave adds 4 i rows) and which 16 bytes of the row.
  const char* lane_src;
  {
    constexpr int CH = D / 8;
    const int r = Tile::row_of(w * Tile::LPW, lane / CH);  // 0..63
    lane_src = reinterpret_cast<const char*>((r < 32 ? q_base : do_base) + (int64_t)(r & 31) * q_row_stride + (lane % CH) * 8);
  }
  const int64_t group_step = Tile::group_global_step(q_row_stride);
  auto request_tile_group = [&](int i, int head, int sub, int st) {
    const int64_t off = ((int64_t)sub * BM * q_row_stride + (int64_t)head * D) * 2 + i * group_step;
    load_async_b128(Tile::group_lds_at(qdo_at + st * (Tile::SIZE * 2), w, i), lane_src + off);
  };
  // Per-query values of a step, one dword load per wave: wave 0 the first range's starts (lanes
  // 0..31) and ends (32..63), wave 1 the second range's (the first's again when there is one
  // range), waves 2 and 3 lse2 and -delta.
  const uint32_t rng_at = lds_address(&rng_lds[0][0][0]), sc_at = lds_address(&sc_lds[0][0][0]);
  auto request_scalars = [&](int head, int sub, int st) {
    const int ql = min(sub * BM + c, seqlen_q - 1);
    if (w < 2) {
      const int plane = (p.n_ranges == 2 ? 2 * w : 0) + h;
      load_async_dword(rng_at + (st * 4 + 2 * w) * BM * 4, p.attn_range + (int64_t)plane * p.total_q + q_begin + ql);
    } else {  // (wave 3 repeats wave 2's request: every wave makes one, which the waits count on)
      const float* src = (h ? p.delta : p.lse2) + (int64_t)(q_begin + ql) * H + head;
      load_async_dword(sc_at + st * 2 * BM * 4, src);
    }
  };

  // ---- steps: query tiles from the last to the first, their two halves, the group's heads ----
  unsigned long long rem = act_mask;
  int qt = rem ? 63 - __builtin_clzll(rem) : 0, half = 1, hg = 0;
  int st = 0;
  const bool any = act_mask != 0 && group > 0;
  if (any) {
    request_scalars(kv_head * group, qt * 2 + half, 0);
#pragma unroll
    for (int i = 0; i < Tile::LPW; ++i) request_tile_group(i, kv_head * group, qt * 2 + half, 0);
  }
  // the counter a wave has to pass on once its stores of the step before are complete
  int* pend_ctr = p.fault + 1;  // (a word nobody reads, while there is nothing to pass on)
  int pend_val = 0;
  bool going = any, gave_up = false;
  if (any) wait_loads();  // the K tile, V, the hulls and the first step's requests
  while (going) {
    const int head = kv_head * group + hg;
    const int sub = qt * 2 + half;
    const bool unmasked = (unm_w >> qt) & 1;
    const int rank = __builtin_amdgcn_readlane(rank_v, qt), count = __builtin_amdgcn_readlane(count_v, qt);
    const bool first = rank == 0, last = rank == count - 1;
    // next step
    int qt_n = qt, half_n = half, hg_n = hg + 1;
    unsigned long long rem_n = rem;
    if (hg_n == group) {
      hg_n = 0;
      if (half == 1) half_n = 0;
      else {
        half_n = 1;
        rem_n = rem & ~(1ull << qt);
        qt_n = rem_n ? 63 - __builtin_clzll(rem_n) : qt;
      }
    }
    const bool more = !(hg + 1 == group && half == 0 && rem_n == 0);
    const int head_n = more ? kv_head * group + hg_n : head;
    const int sub_n = more ? qt_n * 2 + half_n : sub;

    // The step's tile and per-query values were requested during the step before, ahead of that
    // step's four stores of dQ, which alone may still be under way.
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    phase_barrier();
    const int64_t chunk = ((int64_t)b * H + head) * p.subs_per_row + sub;
    int* ctr = p.chain + chunk * 4 + w;
    float* part = p.dq_part + chunk * kChunkFloats + w * 1024 + lane * 4;
    // the chain counter is asked for now and looked at after the first matrix phase
    int seen = first ? 0 : __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    const uint16_t* t_lds = qdo[st];
    // ---- S = Q K^T, dP = dO V^T on 32 queries x 32 keys ------------------------------------
    f32x16 s_acc, dp_acc;
    const int q_left = seqlen_q - (sub * BM + 4 * h);
    if (unmasked) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s_acc[i] = 0.0f;
    } else {
      typedef int i32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        i32x4 rs[4];
#pragma unroll
        for (int pl = 0; pl < 4; ++pl) rs[pl] = *reinterpret_cast<const i32x4*>(&rng_lds[st][pl][8 * g + 4 * h]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          bool ok = ((kv_or_beyond >= rs[0][r]) & (kv_or_beyond < rs[1][r])) |
                    ((kv_or_beyond >= rs[2][r]) & (kv_or_beyond < rs[3][r]));
          ok &= 8 * g + r < q_left;
          s_acc[4 * g + r] = ok ? 0.0f : -INFINITY;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sc_lds[st][1][8 * g + 4 * h]);
#pragma unroll
      for (int r = 0; r < 4; ++r) dp_acc[4 * g + r] = d4[r];
    }
    {
      // stream of LDS operands, two entries ahead: per k-step the Q rows, the K rows of the wave's
      // keys (B operand of S) and the dO rows
      constexpr int N1 = 3 * KS, AHEAD = 2, RING = 4;
      const uint16_t* kw_lds = k_lds[w >> 1];
      auto entry = [&](int o) -> u32x4 {
        const int ks = o / 3, kind = o % 3;
        if (kind == 1) return Tile::read_row(kw_lds, row_rd, w & 1, ks);
        return Tile::read_row(t_lds, row_rd, kind == 0 ? 0 : 1, ks);
      };
      u32x4 buf[RING];
#pragma unroll
      for (int o = 0; o < AHEAD; ++o) buf[o] = entry(o);
      __builtin_amdgcn_s_setprio(kPrioMatrix);
#pragma unroll
      for (int o = 0; o < N1; ++o) {
        const int ks = o / 3, kind = o % 3;
        if (kind == 1) s_acc = mfma_32x32x16<DTYPE>(buf[(o - 1) % RING], buf[o % RING], s_acc);
        else if (kind == 2) dp_acc = mfma_32x32x16<DTYPE>(buf[o % RING], vreg[ks], dp_acc);
        if (o + AHEAD < N1) buf[(o + AHEAD) % RING] = entry(o + AHEAD);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- the chain: wait for the ranks before this one, take their partial sum --------------
    // By now the stores of the step before are complete (they were issued before the first phase):
    // its counter is passed on.  Then this step's link.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __hip_atomic_store(pend_ctr, pend_val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    f32x4 dq0, dq1, dq2, dq3;  // dQ^T[32 w + 8 g + 4 h + r, query c] = dq<g>[r]
    if (!first) {
      // (bounded: a wave that has waited kSpinLimit polls raises the fault flag; every other wave
      // looks at the flag now and then and, once it is up, waits for nothing any more)
      int spins = 0;
      while (seen != rank && !gave_up) {
        seen = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((++spins & 1023) == 0) {
          if (spins >= kSpinLimit) __hip_atomic_store(p.fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          gave_up = spins >= kSpinLimit || __hip_atomic_load(p.fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
        }
      }
      asm volatile(
          "global_load_dwordx4 %0, %4, off sc1\n\t"
          "global_load_dwordx4 %1, %4, off offset:1024 sc1\n\t"
          "global_load_dwordx4 %2, %4, off offset:2048 sc1\n\t"
          "global_load_dwordx4 %3, %4, off offset:3072 sc1"
          : "=&v"(dq0), "=&v"(dq1), "=&v"(dq2), "=&v"(dq3)
          : "v"(part)
          : "memory");
    } else {
      dq0 = dq1 = dq2 = dq3 = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- P = exp2(S c - lse), dS = P (dP - delta) ----------------------------------------
    __builtin_amdgcn_s_setprio(kPrioVector);
    u32x4 pb[2], dsb[2];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sc_lds[st][0][8 * g + 4 * h]);
      float pv[4], dsv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pv[r] = fast_exp2(fmaf(s_acc[4 * g + r], p.scale_log2, -l4[r]));
        dsv[r] = pv[r] * dp_acc[4 * g + r];
      }
      pb[g >> 1][(g & 1) * 2] = pack2<DTYPE>(pv[0], pv[1]);
      pb[g >> 1][(g & 1) * 2 + 1] = pack2<DTYPE>(pv[2], pv[3]);
      dsb[g >> 1][(g & 1) * 2] = pack2<DTYPE>(dsv[0], dsv[1]);
      dsb[g >> 1][(g & 1) * 2 + 1] = pack2<DTYPE>(dsv[2], dsv[3]);
    }
    // dS of the wave's keys for the other waves: row = key, 4 consecutive queries per register pair
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 two = {dsb[g >> 1][(g & 1) * 2], dsb[g >> 1][(g & 1) * 2 + 1]};
      *reinterpret_cast<u32x2*>(&ds_lds[(32 * w + c) * kDsStride + 8 * g + 4 * h]) = two;
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(kPrioMatrix);
    // ---- dV^T += dO^T P, dK^T += Q^T dS over the step's 32 queries ---------------------------
    {
      constexpr int N2 = 4 * DT, AHEAD = 2, RING = 4;
      auto entry = [&](int i) -> u32x4 {
        const int s2 = i / (2 * DT), d = (i % (2 * DT)) / 2;
        return Tile::template read_col<true>(t_lds, col_rd + ((i & 1) ? 0 : Tile::ROW32), s2, d);
      };
      u32x4 buf[RING];
#pragma unroll
      for (int i = 0; i < AHEAD; ++i) buf[i] = entry(i);
      // The next step's tile and per-query values are requested here, AFTER the partial sum: the
      // wait for the partial sum below then leaves these five requests in flight (vmcnt counts
      // in order), and they have until the top of the next step to land.
      request_scalars(head_n, sub_n, st ^ 1);
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        const int s2 = i / (2 * DT), d = (i % (2 * DT)) / 2;
        if (i & 1) dk_acc[d] = mfma_32x32x16<DTYPE>(buf[i % RING], dsb[s2], dk_acc[d]);
        else dv_acc[d] = mfma_32x32x16<DTYPE>(buf[i % RING], pb[s2], dv_acc[d]);
        if (i + AHEAD < N2) buf[(i + AHEAD) % RING] = entry(i + AHEAD);
        if (i % 4 == 1) request_tile_group(i / 4, head_n, sub_n, st ^ 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // dS of all four waves is in LDS
    phase_barrier();
    // The partial sum has landed (the five requests made after it may still be in flight).
    asm volatile("s_waitcnt vmcnt(5)" : "+v"(dq0), "+v"(dq1), "+v"(dq2), "+v"(dq3)::"memory");
    // ---- dQ^T[dims of the wave, q] += K^T dS^T over the workgroup's 128 keys -------------------
    {
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        acc[r] = dq0[r];
        acc[4 + r] = dq1[r];
        acc[8 + r] = dq2[r];
        acc[12 + r] = dq3[r];
      }
      typedef short s16x4 __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
      const int j = lane & 15;
      const uint16_t* ds_rd = ds_lds + (8 * h + (j >> 2)) * kDsStride + ((lane >> 4) & 1) * 16 + 4 * (j & 3);
      auto ds_entry = [&](int s) -> u32x4 {
        const uint16_t* p0 = ds_rd + 16 * s * kDsStride;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0 + 4 * kDsStride));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        return u32x4{l2[0], l2[1], h2[0], h2[1]};
      };
      auto k_entry = [&](int s) -> u32x4 { return Tile::template read_col<false>(k_lds[s >> 2], col_rd_k, s & 3, w); };
      u32x4 ka[2], da[2];
      ka[0] = k_entry(0);
      da[0] = ds_entry(0);
#pragma unroll
      for (int s = 0; s < BN / 16; ++s) {
        if (s + 1 < BN / 16) {
          ka[(s + 1) & 1] = k_entry(s + 1);
          da[(s + 1) & 1] = ds_entry(s + 1);
        }
        acc = mfma_32x32x16<DTYPE>(ka[s & 1], da[s & 1], acc);
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_setprio(kPrioVector);
      if (last) {  // the chunk is complete: scale, round, write dQ
        if (sub * BM + c < seqlen_q) {
          uint16_t* op = reinterpret_cast<uint16_t*>(p.dq) +
                         (int64_t)p.dq_block_table[b] * p.dq_slot_stride + (int64_t)(sub * BM + c) * q_row_stride + (int64_t)head * D +
                         32 * w + 4 * h;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            u32x2 pk = {pack2<DTYPE>(acc[4 * g] * p.scale, acc[4 * g + 1] * p.scale),
                        pack2<DTYPE>(acc[4 * g + 2] * p.scale, acc[4 * g + 3] * p.scale)};
            *reinterpret_cast<u32x2*>(op + 8 * g) = pk;
          }
        } else {  // (every wave issues four stores per step: the wait at the top of a step counts them)
#pragma unroll
          for (int g = 0; g < 4; ++g) *reinterpret_cast<f32x4*>(part + g * 256) = f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
        }
      } else {
#pragma unroll
        for (int g = 0; g < 4; ++g) *reinterpret_cast<f32x4*>(part + g * 256) = f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
      }
      pend_ctr = ctr;
      pend_val = rank + 1;
    }
    st ^= 1;
    going = more;
    qt = qt_n;
    half = half_n;
    hg = hg_n;
    rem = rem_n;
  }
  // the last step's stores, then its counter
  __builtin_amdgcn_s_waitcnt(0);
  if (any) __hip_atomic_store(pend_ctr, pend_val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // ---- dK and dV of the wave's keys are complete: scale, round, store ---------------------
  if (!has_keys) return;
  const int64_t off = (int64_t)p.dkv_block_table[(int64_t)b * p.max_kv_blocks + blk] * p.dkv_slot_stride +
                      (int64_t)(tok0 + c) * p.dkv_token_stride + (int64_t)kv_head * D + 4 * h;
  uint16_t* dv_dst = reinterpret_cast<uint16_t*>(p.dv) + off;
  uint16_t* dk_dst = reinterpret_cast<uint16_t*>(p.dk) + off;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int i = 4 * g;
      u32x2 v4 = {pack2<DTYPE>(dv_acc[dt][i], dv_acc[dt][i + 1]), pack2<DTYPE>(dv_acc[dt][i + 2], dv_acc[dt][i + 3])};
      *reinterpret_cast<u32x2*>(dv_dst + dt * 32 + 8 * g) = v4;
      u32x2 k4 = {pack2<DTYPE>(dk_acc[dt][i] * p.scale, dk_acc[dt][i + 1] * p.scale),
                  pack2<DTYPE>(dk_acc[dt][i + 2] * p.scale, dk_acc[dt][i + 3] * p.scale)};
      *reinterpret_cast<u32x2*>(dk_dst + dt * 32 + 8 * g) = k4;
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
namespace {
size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

__global__ void xcd_probe_kernel(int* out) {
  if (threadIdx.x == 0) {
    int x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    out[blockIdx.x] = x & 15;
  }
}

// 1: the workgroups of a grid are dealt to the 8 XCDs in turn on this device (workgroups b and
// b + 8 share an XCD; which XCD the first one gets differs from launch to launch); 0: not so
// (or the probe failed)
int probe_xcd_dealing() {
  constexpr int N = 4 * kNumXcd * 8;
  int* dev = nullptr;
  if (hipMalloc(&dev, N * sizeof(int)) != hipSuccess) return 0;
  int host[N];
  bool ok = true;
  hipLaunchKernelGGL(xcd_probe_kernel, dim3(N), dim3(64), 0, 0, dev);
  ok = hipMemcpy(host, dev, sizeof(host), hipMemcpyDeviceToHost) == hipSuccess;
  (void)hipFree(dev);
  for (int i = 0; ok && i < N; ++i) ok = host[i] == (host[0] + i) % kNumXcd;
  return ok ? 1 : 0;
}
}  // namespace

namespace {
std::mutex g_select_mu;
int g_mode = -1;  // -1: not set yet (the environment decides); DCP_BWD_* values
}  // namespace

int bwd_select(int mode) {
  std::lock_guard<std::mutex> hold(g_select_mu);
  if (g_mode < 0) {
    const char* e = getenv("DCP_BWD_MODE");
    g_mode = e != nullptr && e[0] >= '0' && e[0] <= '2' ? e[0] - '0' : DCP_BWD_THROUGH_DS;
  }
  const int before = g_mode;
  if (mode >= 0 && mode <= 2) g_mode = mode;
  return before;
}

bool bwd_fused_available() {
  if (bwd_select(-1) != DCP_BWD_ONE_PASS) return false;
  static std::mutex mu;
  static int cached[64];  // 0: not asked yet, 1: yes, 2: no
  std::lock_guard<std::mutex> hold(mu);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
  if (cached[dev] == 0) cached[dev] = probe_xcd_dealing() ? 1 : 2;
  return cached[dev] == 1;
}

size_t bwd_fused_extra_workspace_bytes(int batch, int block_size, int n_heads_q, int head_dim) {
  if (head_dim != 128) return 0;
  const size_t chunks = (size_t)batch * n_heads_q * ((block_size + kFusedBM - 1) / kFusedBM);
  return align256(chunks * kChunkFloats * sizeof(float)) + align256(chunks * 4 * sizeof(int)) + 256;
}

int launch_bwd_prepare(const AttnBwdParams& p, int dtype, hipStream_t stream) {
  KernelTimer timer("bwd_prepare_kernel", stream);
  const dim3 grid(p.batch * p.q_tiles_per_row), block(kBwdThreads);
  if (dtype == DCP_DTYPE_BF16) {
    if (p.head_dim == 128) hipLaunchKernelGGL((bwd_prepare_kernel<DCP_DTYPE_BF16, 128>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((bwd_prepare_kernel<DCP_DTYPE_BF16, 64>), grid, block, 0, stream, p);
  } else {
    if (p.head_dim == 128) hipLaunchKernelGGL((bwd_prepare_kernel<DCP_DTYPE_FP16, 128>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((bwd_prepare_kernel<DCP_DTYPE_FP16, 64>), grid, block, 0, stream, p);
  }
  return check_launch("bwd_prepare_kernel");
}

int launch_bwd_fused(const AttnBwdParams& p, int dtype, hipStream_t stream) {
  const int64_t n_wg = xcd_grid_size(p.n_dkv_items, p.dkv_xcd_group);
  DCP_REQUIRE(n_wg < ((int64_t)1 << 31), "attn_bwd: grid too large");
  if (const int e = launch_bwd_prepare(p, dtype, stream)) return e;
  {
    KernelTimer timer("attn_bwd_fused_kernel", stream);
    if (dtype == DCP_DTYPE_BF16)
      hipLaunchKernelGGL((attn_bwd_fused_kernel<DCP_DTYPE_BF16>), dim3((unsigned)n_wg), dim3(kBwdThreads), 0, stream, p);
    else
      hipLaunchKernelGGL((attn_bwd_fused_kernel<DCP_DTYPE_FP16>), dim3((unsigned)n_wg), dim3(kBwdThreads), 0, stream, p);
  }
  return check_launch("attn_bwd fused kernels");
}

}  // namespace dcp
