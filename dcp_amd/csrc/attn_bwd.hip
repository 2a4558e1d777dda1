// Range-masked paged attention backward for gfx950.
//
// One small kernel and two big ones per call, in this order:
//
//   bwd_tile_hull_kernel per (row, 64-query tile): hull and core of the rows'
//                        key ranges, so the dK/dV kernel can skip / unmask tiles
//   attn_bwd_dq_kernel   query-outer: one workgroup per (row, head, 128-query
//                        tile) walks the key tiles and keeps dQ^T in registers.
//                        Its prologue also computes -delta[q, h] = -sum_d dO*O
//                        (negated: it is added, as an accumulator's initial
//                        value) and the base-2 log-sum-exp of its queries and
//                        leaves them in the workspace for the next kernel
//   attn_bwd_dkv_kernel  key-outer: one workgroup per (row, 128-key tile, kv
//                        head) loops over the q heads of the kv head's group
//                        and the 64-query tiles of the row and keeps dK^T and
//                        dV^T of its keys in registers
//
// dQ and dK/dV each get the loop order that keeps them in registers; S and dP
// are recomputed in the second kernel (7 matrix products instead of 5).  The
// alternative, one key-outer kernel that adds dQ contributions with fp32
// atomics, was measured at 57 ms against 26 ms with the atomics removed on the
// 64k-token causal schedule: device-scope float atomics from eight XCDs cost
// more than the two recomputed products.
//
// dK/dV kernel.  Wave w owns keys 32w..32w+31 of the workgroup's 128 from start
// to end.  A step is one (q head, 64-query tile); the wave takes its two halves
// of 32 queries one after the other (a sub-step):
//
//   S  = Q K^T          A = Q rows from LDS,   B = K held in registers
//   dP = dO V^T         A = dO rows from LDS,  B = V held in registers
//   P  = exp2(S*c - lse), dS = P * (dP - delta)   accumulator layout: lane =
//                                                 key, 4 consecutive queries
//                                                 per register group
//   dV^T[dim, key] += dO^T P   A = dO^T: transpose-load from the row-major dO
//                              tile in accumulator row order, B = P straight
//                              from the accumulators
//   dK^T[dim, key] += Q^T dS   A = Q^T: transpose-load from the Q tile, B = dS
//
// P and dS never leave the registers, so a step needs one workgroup barrier (the
// one that publishes its tiles) and LDS holds nothing but the Q and dO tiles, two
// stages of each: everything a step reads is requested one step ahead.  With four
// waves side by side along the keys, a Q/dO tile brought into LDS, a barrier and a
// step's scalar control serve 64 matrix instructions per wave (with two waves
// along the keys and two along the queries it was 32, and the two query halves
// had to be added through LDS at the end).  The range mask enters S as the
// accumulator's initial value (0 or -inf).  dK/dV of a key never leave the wave
// until the end, so the per-(row, kv block) private dKV blocks of the plan need
// no atomics and are written whole (zeros where no query of the row attends).
#include <math.h>

#include <algorithm>
#include <mutex>

#include "attn_bwd_params.h"

namespace dcp {

// One wave per (row, 64-query tile).  hull[0..3] = lo0, hi0, lo1, hi1 over
// rows with a non-empty range; hull[4..7] = the intersection (core) of the
// rows' ranges, empty as soon as one row has an empty range.
__global__ __launch_bounds__(64) void bwd_tile_hull_kernel(const AttnBwdParams p) {
  if (blockIdx.x == 0 && threadIdx.x < kTicketInts) p.tickets[threadIdx.x] = 0;  // for the dQ kernel that follows
  const int b = blockIdx.x / p.q_tiles_per_row;
  const int qt = blockIdx.x - b * p.q_tiles_per_row;
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - p.cu_seqlens_kv[b];
  const int ql = qt * kBwdBM + threadIdx.x;
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
  if (threadIdx.x < 8) {
    const int vals[8] = {v0, v1, v2, v3, v4, v5, v6, v7};
    int mine = vals[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) mine = threadIdx.x == i ? vals[i] : mine;
    p.hull[(int64_t)blockIdx.x * 8 + threadIdx.x] = mine;
  }
}

// ---------------------------------------------------------------------------
// dK/dV kernel
// ---------------------------------------------------------------------------
constexpr int kDkvBN = 128;  // keys per workgroup: four waves of 32 keys each

// WRITE_DS: the kernel also leaves dS (the storage type, zero where masked) in the workspace, for
// the dQ kernel that contracts it with K instead of recomputing S and dP (attn_bwd_ds.hip).  A
// piece is the dS of 64 keys x 32 queries of one head, 4 KiB, laid out as the lanes of this kernel
// hold it: [32-key half][16-query half][key][4-query group within the 16: 2 x 2][4 queries].
template <int DTYPE, int D, bool WRITE_DS>
__global__ __launch_bounds__(kBwdThreads, 2) void attn_bwd_dkv_kernel(const AttnBwdParams p) {
  constexpr int BM = kBwdBM, BN = kDkvBN;
  constexpr int KS = D / 16;  // k-steps over the head dim
  constexpr int DT = D / 32;  // 32-dim blocks of dK^T / dV^T
  typedef KvTile<D> Tile;     // the Q and dO tiles: 64 queries x D

  // two stages of everything a step reads: its Q and dO tiles and the per-query scalars
  __shared__ __attribute__((aligned(16))) uint16_t tiles[4][Tile::SIZE];  // [2 * stage + (0: Q, 1: dO)]
  __shared__ __attribute__((aligned(16))) int rng_lds[2][4][BM];  // planes: start0, end0, start1, end1
  __shared__ __attribute__((aligned(16))) float lse_lds[2][BM];
  __shared__ __attribute__((aligned(16))) float delta_lds[2][BM];
  __shared__ unsigned long long mask_lds[kBwdThreads / 64];
  // With D = 128 the accumulators (128 registers), K and V (64) and the products in flight do
  // not fit in 256 registers.  The compiler would spill to scratch memory, and a scratch
  // reload waits for every outstanding global load, i.e. for the tiles requested a step
  // ahead.  So the last VL k-steps of V are parked in LDS instead (per lane, read back with
  // the other operands).
  constexpr int VL = D == 128 ? 2 : 0;
  __shared__ u32x4 v_park[VL > 0 ? kBwdThreads / 64 : 1][VL > 0 ? VL : 1][64];

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // this wave's 32 keys of the tile
  const int lane = tid & 63;
  const int c = lane & 31;
  const int h = lane >> 5;

  // ---- which (row, kv head, key tile) ------------------------------------------
  // the key tiles of a row share its Q/dO tiles: keep them on one XCD
  int wg = xcd_logical_id(blockIdx.x, p.dkv_xcd_group, p.n_dkv_items);
  if (wg < 0) return;
  // Integer division runs on the vector unit, so its (uniform) results sit in vector registers
  // and drag every address derived from them there too: each tile load then costs three vector
  // instructions to rebuild a scalar base.  readfirstlane puts the indices back on the scalar unit.
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
  // A wave whose 32 keys lie past the row's keys (seqlen_kv need not be a multiple of 128) still
  // loads its share of every tile and meets every barrier; its arithmetic is switched off and it
  // stores nothing.  Its K/V addresses fall back to the tile's first keys so that they stay valid.
  const int kw = k0 + w * 32;
  const bool has_keys = kw < seqlen_kv;
  const int kv_or_beyond = kw + c < seqlen_kv ? kw + c : 0x7fffffff;  // this lane's key, for the range tests
  const int kw_safe = has_keys ? kw : k0;
  const int blk = __builtin_amdgcn_readfirstlane(kw_safe / p.block_size);
  const int tok0 = kw_safe - blk * p.block_size;
  const int group = p.n_heads_q / p.n_heads_kv;
  const int64_t q_row_stride = (int64_t)p.n_heads_q * D;
  const int q_slot = p.q_block_table[b];
  const int o_slot = p.out_block_table[b];
  const int n_q_tiles = (seqlen_q + BM - 1) / BM;  // rows past seqlen_q stay inside the padded block
  const int64_t kv_tile_off = (int64_t)p.kv_block_table[(int64_t)b * p.max_kv_blocks + blk] * p.kv_slot_stride +
                              (int64_t)tok0 * p.kv_token_stride + (int64_t)kv_head * D;

  // ---- K, V of this wave's 32 keys as B operands (lane = key, slots = dims) ------
  u32x4 kreg[KS], vreg[KS - VL];
  {
    const int64_t off = kv_tile_off + (int64_t)c * p.kv_token_stride + h * 8;
    const uint16_t* kp = reinterpret_cast<const uint16_t*>(p.k) + off;
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.v) + off;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kreg[ks] = *reinterpret_cast<const u32x4*>(kp + ks * 16);
#pragma unroll
    for (int ks = 0; ks < KS - VL; ++ks) vreg[ks] = *reinterpret_cast<const u32x4*>(vp + ks * 16);
#pragma unroll
    for (int j = 0; j < VL; ++j) v_park[w][j][lane] = *reinterpret_cast<const u32x4*>(vp + (KS - VL + j) * 16);
  }

  // dK^T and dV^T of this wave's keys: (all dims) x (32 keys), complete when the loop ends
  f32x16 dk_acc[DT], dv_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dk_acc[dt][i] = 0.0f;
      dv_acc[dt][i] = 0.0f;
    }

  const int32_t* hull_row = p.hull + (int64_t)b * p.q_tiles_per_row * 8;
  // loop-invariant per-lane pieces of the addresses used in the loop
  const int row_rd = Tile::row_base(c, h);
  const int col_rd = Tile::col_base(lane, true);
  const uint16_t* q_base = reinterpret_cast<const uint16_t*>(p.q) + (int64_t)q_slot * p.q_slot_stride;
  const uint16_t* do_base = reinterpret_cast<const uint16_t*>(p.dout) + (int64_t)o_slot * p.out_slot_stride;
  const uint32_t tiles_at = lds_address(&tiles[0][0]);

  // ---- which 64-query tiles of the row see this wave's keys (the same for every head) ------
  // bit qt of `act_w`: some row of tile qt sees some of the wave's keys; of `unm_w`: every row sees
  // all of them.  Taken once from the per-tile hulls, so the loop never waits for a table.  The
  // workgroup walks the tiles any of its waves needs (`act_mask`); a wave sits out the others.
  unsigned long long act_w, unm_w;
  {
    bool a = false, u = false;
    if (has_keys && lane < n_q_tiles) {
      const int32_t* hu = hull_row + lane * 8;
      a = (kw < hu[1] && kw + 32 > hu[0]) || (kw < hu[3] && kw + 32 > hu[2]);
      u = (hu[4] <= kw && kw + 32 <= hu[5]) || (hu[6] <= kw && kw + 32 <= hu[7]);
    }
    act_w = __ballot(a);
    unm_w = __ballot(u);
    if (lane == 0) mask_lds[w] = act_w;
  }
  __syncthreads();
  const unsigned long long act = mask_lds[0] | mask_lds[1] | mask_lds[2] | mask_lds[3];
  const uint32_t act_lo = __builtin_amdgcn_readfirstlane((uint32_t)act);
  const uint32_t act_hi = __builtin_amdgcn_readfirstlane((uint32_t)(act >> 32));
  const unsigned long long act_mask = ((unsigned long long)act_hi << 32) | act_lo;

  // Everything step (head, qt) reads is requested a step ahead, straight into LDS stage st
  // and with nothing held in registers meanwhile: the Q and dO tiles, and one value per
  // query of the range planes (waves 0 and 1), lse (wave 2) and delta (wave 3).  Queries
  // past seqlen_q read the last valid query's values; they are masked where they are used.
  const uint32_t rng_at = lds_address(&rng_lds[0][0][0]), lse_at = lds_address(&lse_lds[0][0]),
                 delta_at = lds_address(&delta_lds[0][0]);
  const uint32_t goff0 = Tile::lane_offset0(q_row_stride, w, lane);
  // tile load idx of a step: the wave's group loads of the Q tile, then of the dO tile
  constexpr int NL = 2 * Tile::LPW;
  const uint64_t group_step = uniform64(Tile::group_global_step(q_row_stride));
  static_assert(NL <= KS, "a sub-step carries half of the tile loads, one per two k-steps of its first phase");
  auto request_tile = [&](int idx, int head, int qt, int st) {
    const int64_t off = (int64_t)qt * BM * q_row_stride + (int64_t)head * D;
    const bool is_do = idx >= Tile::LPW;
    Tile::load_group(tiles_at + (2 * st + (is_do ? 1 : 0)) * (Tile::SIZE * 2), (is_do ? do_base : q_base) + off, goff0,
                     q_row_stride, w, is_do ? idx - Tile::LPW : idx);
  };
  // Per-query values of a step, two dword loads per wave and no branches: wave 0 requests the
  // first range's starts and ends, wave 1 the second range's (the first's again, into planes
  // nobody reads, when there is one range), wave 2 the LSEs and wave 3 the deltas (each twice,
  // to the same place).  What depends on the wave's role is fixed here, once.
  const bool role_rng = w < 2, role_lse = w == 2;
  const int sc_plane = p.n_ranges == 2 ? 2 * w : 0;
  const char* sc_base0 = role_rng   ? reinterpret_cast<const char*>(p.attn_range + (int64_t)sc_plane * p.total_q + q_begin)
                         : role_lse ? reinterpret_cast<const char*>(p.lse2 + (int64_t)q_begin * p.n_heads_q)
                                    : reinterpret_cast<const char*>(p.delta + (int64_t)q_begin * p.n_heads_q);
  const int64_t sc_head_bytes = role_rng ? 0 : 4;
  const int64_t sc_second_bytes = role_rng ? (int64_t)p.total_q * 4 : 0;
  const int sc_query_bytes = role_rng ? 4 : p.n_heads_q * 4;
  const uint32_t sc_at0 = role_rng ? rng_at + (2 * w * BM) * 4 : role_lse ? lse_at : delta_at;
  const uint32_t sc_at_stage = role_rng ? 4 * BM * 4 : BM * 4, sc_at_second = role_rng ? BM * 4 : 0;
  auto request_scalars = [&](int head, int qt, int st) {
    const int ql = min(qt * BM + lane, seqlen_q - 1);
    const char* base = sc_base0 + head * sc_head_bytes;
    const uint32_t at = sc_at0 + st * sc_at_stage, voff = (uint32_t)(ql * sc_query_bytes);
    load_async_dword(at, voff, base);
    load_async_dword(at + sc_at_second, voff, base + sc_second_bytes);
  };

  // dS pieces (WRITE_DS).  The workspace holds the rows one after another; row b starts at 64-key
  // tile cu_seqlens_kv[b] / 64 + b (room for a last, partial tile of every row before it) and is laid
  // out [head][32-query chunk][64-key tile]: the pieces that a wave of the dQ kernel reads one after
  // another lie one after another (ordered by key tile first, they were 4 MiB apart at 32 heads and
  // 1024-token blocks, every one in a memory page of its own).  ds_lane: the lane's 16 bytes within a
  // [key][query half] plane of a piece.
  const int ds_row_tiles = (seqlen_kv + 63) / 64;
  const uint64_t ds_row_base = ((uint64_t)(p.cu_seqlens_kv[b] / 64) + b) * p.n_heads_q * p.subs_per_row;
  const int ds_tile_local = 2 * kt + (w >> 1);
  const uint64_t ds_chunk_bytes = has_keys ? (uint64_t)ds_row_tiles << 12 : 4096;  // from a 32-query chunk to the next
  const int ds_lane = (w & 1) * 128 + 2 * c + h;

  // steps: (q head of the group) x (active 64-query tile)
  int hg = 0;
  unsigned long long rem = act_mask;  // tiles of head hg still to do
  int st = 0;
  if (act_mask != 0 && group > 0) {
    request_scalars(kv_head * group, __builtin_ctzll(rem), 0);
#pragma unroll
    for (int i = 0; i < NL; ++i) request_tile(i, kv_head * group, __builtin_ctzll(rem), 0);
  }
  if constexpr (WRITE_DS) wait_loads();  // (the wait at the top of a step counts on two stores behind the tile loads)
  while (act_mask != 0 && hg < group) {
    const int qt = __builtin_ctzll(rem);
    const bool unmasked = (unm_w >> qt) & 1;
    rem &= rem - 1;
    int hg_next = hg;
    if (rem == 0) {
      rem = act_mask;
      ++hg_next;
    }
    const bool more = hg_next < group;

    if constexpr (WRITE_DS) {
      // The tiles and scalars of this step were requested before the previous step's last two
      // stores of dS: those may stay in flight (a full wait would sit out their trip to memory
      // at every step; measured 9.3 ms against 7.3 ms for the kernel).
      asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
      phase_barrier();
    } else {
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();  // this step's tiles and scalars are in LDS; the previous step is fully consumed
    }
    // The next step's tiles are requested one load at a time between the matrix instructions of
    // the first phases below: a burst here would hold the wave at its last load until the memory
    // pipeline has taken them all.  They are issued unconditionally, so that the step has no
    // branches around them: the last step requests its own tiles once more, into the stage nobody
    // reads any more.
    const int head_next = more ? kv_head * group + hg_next : kv_head * group + hg;
    const int qt_next = more ? __builtin_ctzll(rem) : qt;
    const uint16_t* q_lds = tiles[2 * st];
    const uint16_t* do_lds = tiles[2 * st + 1];
    // where the next step's tiles come from and go to, as wave-uniform scalars worked out once a
    // step: a load in the matrix phases then costs two scalar additions
    const int64_t off_next = (int64_t)qt_next * BM * q_row_stride + (int64_t)head_next * D;
    const uint64_t next_q = uniform64(reinterpret_cast<uint64_t>(q_base + off_next));
    const uint64_t next_do = uniform64(reinterpret_cast<uint64_t>(do_base + off_next));
    const uint32_t next_at = __builtin_amdgcn_readfirstlane(Tile::group_lds_at(tiles_at + 2 * (st ^ 1) * (Tile::SIZE * 2), w, 0));
    // where this step's dS goes: the pieces of (this wave's 64-key half tile, head, the step's two 32-query sub-tiles)
    // (a wave whose 32 keys lie past the row's last key has no piece -- its 64-key half tile would be
    // the next row's first, or lie past the end of the workspace -- and writes its zeros into two
    // spare pieces behind the last one instead: no branch around the stores)
    const uint64_t ds_step =
        WRITE_DS ? uniform64(reinterpret_cast<uint64_t>(p.ds) +
                             (((has_keys ? ds_row_base + ((uint64_t)(kv_head * group + hg) * p.subs_per_row + 2 * qt) * ds_row_tiles + ds_tile_local
                                         : (uint64_t)p.ds_pieces))
                              << 12))
                 : 0;

    // One sub-step = this wave's 32 keys against 32 of the step's 64 queries (QI = 0, 1).
    // (A real loop, not unrolled: one copy of the body keeps the register allocation of a single
    // sub-step; unrolled twice the compiler spills the K/V operands.)
    auto sub_step = [&](const int QI) {
      const int row_rd_q = row_rd + QI * Tile::ROW32, col_rd_q = col_rd + QI * Tile::ROW32;
      // ---- S = Q K^T, dP = dO V^T on 32 queries x 32 keys ---------------------------------
      // (A = rows of the Q / dO tile, B = K / V in registers; lane = key, element i = query
      // 32 QI + acc_row(i, h)).  The range mask enters S as the accumulator's initial value.
      f32x16 s_acc, dp_acc;
      const int q_left = seqlen_q - (qt * BM + QI * 32 + 4 * h);  // valid queries from this lane's first one on
      if (unmasked) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s_acc[i] = 0.0f;
      } else {
        // the four queries of an accumulator register group are consecutive: their range planes
        // come in 16-byte reads, requested together before the comparisons.  With one range the
        // second range's planes hold the first's again (see request_scalars): the union is the same.
        typedef int i32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          i32x4 rs[4];
#pragma unroll
          for (int pl = 0; pl < 4; ++pl) rs[pl] = *reinterpret_cast<const i32x4*>(&rng_lds[st][pl][QI * 32 + 8 * g + 4 * h]);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            // five comparisons per element and nothing else on the vector unit: a key past the
            // row's last one counts as beyond every range (kv_or_beyond), a query past the
            // row's last one fails its own test
            bool ok = ((kv_or_beyond >= rs[0][r]) & (kv_or_beyond < rs[1][r])) |
                      ((kv_or_beyond >= rs[2][r]) & (kv_or_beyond < rs[3][r]));
            ok &= 8 * g + r < q_left;
            s_acc[4 * g + r] = ok ? 0.0f : -INFINITY;
          }
          __builtin_amdgcn_sched_barrier(0);  // one group's planes in registers at a time
        }
      }
      // dP starts from -delta of its query (dS = P (dP - delta)): the subtraction rides on the
      // accumulation instead of costing a vector instruction per element afterwards
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(&delta_lds[st][QI * 32 + 8 * g + 4 * h]);
#pragma unroll
        for (int r = 0; r < 4; ++r) dp_acc[4 * g + r] = d4[r];
      }
      // Everything the sub-step's 32 MFMAs read from LDS forms one stream, read AHEAD entries
      // ahead into four rotating registers, across both matrix phases (the first operand of the
      // second phase is on its way while the vector phase runs):
      //   phase 1, per k-step: Q rows (-> S), [the parked V k-step (B operand)], dO rows (-> dP)
      //   phase 2, per (16-query step s2, 32-dim block d): dO^T (-> dV), Q^T (-> dK)
      constexpr int N1 = 2 * KS + VL, N2 = 4 * DT, NS = N1 + N2, AHEAD = 2, RING = 4, PRE = 1;
      constexpr int FIRST_PARKED = 2 * (KS - VL);  // stream index of the first k-step with a parked V
      auto entry = [&](int o) -> u32x4 {
        if (o < N1) {
          const int ks = o < FIRST_PARKED ? o / 2 : (KS - VL) + (o - FIRST_PARKED) / 3;
          const int kind = o < FIRST_PARKED ? (o & 1) * 2 : (o - FIRST_PARKED) % 3;  // 0: Q, 1: parked V, 2: dO
          if (kind == 1) return v_park[w][VL > 0 ? ks - (KS - VL) : 0][lane];
          return Tile::read_row(kind == 0 ? q_lds : do_lds, row_rd_q, 0, ks);
        }
        const int i = o - N1, s2 = i / (2 * DT), d = (i % (2 * DT)) / 2;
        return Tile::template read_col<true>((i & 1) ? q_lds : do_lds, col_rd_q, s2, d);
      };
      // this sub-step's half of the next step's tile loads: the Q tile (QI = 0) or the dO tile
      static_assert(NL / 2 == Tile::LPW, "a sub-step loads one whole tile");
      uint64_t load_src = uniform64(QI ? next_do : next_q);
      const uint32_t load_at = next_at + QI * (Tile::SIZE * 2);
      u32x4 buf[RING];
#pragma unroll
      for (int o = 0; o < AHEAD; ++o) buf[o] = entry(o);
      __builtin_amdgcn_s_setprio(kPrioMatrix);
      // (after the step's first LDS reads are on their way: the requests are inline assembly that
      // the compiler moves no memory access across)
      if (QI == 0) request_scalars(head_next, qt_next, st ^ 1);
#pragma unroll
      for (int o = 0; o < N1; ++o) {
        const int ks = o < FIRST_PARKED ? o / 2 : (KS - VL) + (o - FIRST_PARKED) / 3;
        const int kind = o < FIRST_PARKED ? (o & 1) * 2 : (o - FIRST_PARKED) % 3;
        if (kind == 0) s_acc = mfma_32x32x16<DTYPE>(buf[o % RING], kreg[ks], s_acc);
        else if (kind == 2 && ks < KS - VL) dp_acc = mfma_32x32x16<DTYPE>(buf[o % RING], vreg[ks < KS - VL ? ks : 0], dp_acc);
        else if (kind == 2) dp_acc = mfma_32x32x16<DTYPE>(buf[o % RING], buf[(o - 1) % RING], dp_acc);
        // the entry just used (and the one before it) are free: the next read goes there.  Only the
        // first operand of the second phase is requested before the vector phase (registers)
        if (o + AHEAD < N1 + PRE) buf[(o + AHEAD) % RING] = entry(o + AHEAD);
        // this sub-step's half of the next step's tile loads, one per two k-steps
        if (kind == 2 && ks % 2 == 0 && ks / 2 < NL / 2) {
          Tile::load_group_at(load_at + (ks / 2) * (Tile::GROUP_STRIDE * 2), load_src, goff0);
          load_src = uniform64(load_src + group_step);
        }
        __builtin_amdgcn_sched_barrier(0);  // keeps the order: reads neither pile up in registers nor fall behind
      }
      // ---- P = exp2(S c - lse), dS = P (dP - delta), packed in accumulator order: as B operands
      // they feed the next products without leaving the registers -------------------------------
      __builtin_amdgcn_s_setprio(kPrioVector);
      u32x4 pb[2], dsb[2];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int qrow = QI * 32 + 8 * g + 4 * h;
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(&lse_lds[st][qrow]);
        float pv[4], dsv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          pv[r] = fast_exp2(fmaf(s_acc[4 * g + r], p.scale_log2, -l4[r]));  // l4: lse * log2(e); masked: exp2(-inf) = 0
          dsv[r] = pv[r] * dp_acc[4 * g + r];
        }
        pb[g >> 1][(g & 1) * 2] = pack2<DTYPE>(pv[0], pv[1]);
        pb[g >> 1][(g & 1) * 2 + 1] = pack2<DTYPE>(pv[2], pv[3]);
        dsb[g >> 1][(g & 1) * 2] = pack2<DTYPE>(dsv[0], dsv[1]);
        dsb[g >> 1][(g & 1) * 2 + 1] = pack2<DTYPE>(dsv[2], dsv[3]);
      }
      if constexpr (WRITE_DS) {
        // (non-temporal: the pieces are read once, by another kernel; they must not push the row's
        // Q and dO tiles, which its key tiles share, out of the L2)
        // (and through a pointer that says "global memory": built from an integer it would be a
        // generic one, whose stores also count as LDS accesses and make every wait for an LDS
        // operand a wait for these stores)
        // The two stores go out one at a time between the matrix instructions of the second phase
        // (below), like the tile loads of the first.
      }
      typedef __attribute__((address_space(1))) u32x4 global_u32x4;
      global_u32x4* piece = (global_u32x4*)(ds_step + (uint64_t)QI * ds_chunk_bytes) + ds_lane;
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(kPrioMatrix);
#pragma unroll
      for (int o = N1 + PRE; o < N1 + AHEAD; ++o) buf[o % RING] = entry(o);
      // ---- dV^T[dim, key] += dO^T[dim, q] P[q, key];  dK^T[dim, key] += Q^T[dim, q] dS[q, key]
      // over the sub-step's 32 queries (dO^T and Q^T come out of the row-major tiles by
      // transpose loads, in the accumulators' row order) ---------------------------------------
#pragma unroll
      for (int o = N1; o < NS; ++o) {
        const int i = o - N1, s2 = i / (2 * DT), d = (i % (2 * DT)) / 2;
        if (i & 1) dk_acc[d] = mfma_32x32x16<DTYPE>(buf[o % RING], dsb[s2], dk_acc[d]);
        else dv_acc[d] = mfma_32x32x16<DTYPE>(buf[o % RING], pb[s2], dv_acc[d]);
        if (o + AHEAD < NS) buf[(o + AHEAD) % RING] = entry(o + AHEAD);
        if constexpr (WRITE_DS) {
          if (i == 3) __builtin_nontemporal_store(dsb[0], piece);
          if (i == 2 * DT + 1) __builtin_nontemporal_store(dsb[1], piece + 64);  // (2 * 2 * DT iterations)
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
#pragma clang loop unroll(disable)
    for (int qi = 0; qi < 2; ++qi) sub_step(qi);
    __builtin_amdgcn_s_setprio(kPrioVector);
    st ^= 1;
    hg = hg_next;
  }

  // ---- dK and dV of the wave's keys are complete: scale, round, store ---------------------
  wait_loads();  // the last step's (unused) requests must land before the workgroup's LDS is released
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
// dQ kernel: query-outer, like the forward.  One workgroup owns 128 query rows
// of one (row, head), wave w rows 32w..32w+31 (lane = query row), and walks the
// key tiles its rows can see:
//
//   S^T [kv, q] = K Q^T       A = K tile rows from LDS,  B = Q in registers
//   dP^T[kv, q] = V dO^T      A = V tile rows from LDS,  B = dO in registers
//   dS^T = exp2(S^T c - lse[q]) * (dP^T - delta[q])      per-lane scalars
//   dQ^T[d, q] += K^T dS^T    A = K^T: transpose-load from the same K tile,
//                             B = dS^T straight from the accumulators
//
// dQ of a row is complete when the loop ends: no atomics, no fp32 scratch, and
// the result does not depend on scheduling.
// ---------------------------------------------------------------------------
constexpr int kDqBM = 128;
constexpr int kDqBN = 64;

template <int DTYPE, int D>
__device__ __forceinline__ void attn_bwd_dq_item(KernArgs<AttnBwdParams>& p, int item) {
  constexpr int BN = kDqBN;
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  typedef KvTile<D> Tile;
  // two stages of (K tile, V tile); separate arrays so the compiler can tell
  // the stage being filled from the stage being read
  __shared__ __attribute__((aligned(16))) uint16_t k_lds0[Tile::SIZE];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds0[Tile::SIZE];
  __shared__ __attribute__((aligned(16))) uint16_t k_lds1[Tile::SIZE];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds1[Tile::SIZE];
  __shared__ int hull_lds[4][4];
  __shared__ int slot_lds[kSlotTableCap];

  int tid = threadIdx.x;
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int c = lane & 31;
  const int h = lane >> 5;

  int wg = item;
  // (indices back on the scalar unit after the vector-unit divisions, as in the dK/dV kernel)
  const int qt = __builtin_amdgcn_readfirstlane(wg % p.dq_tiles_per_row);
  wg /= p.dq_tiles_per_row;
  const int head = __builtin_amdgcn_readfirstlane(wg % p.n_heads_q);
  const int bi = __builtin_amdgcn_readfirstlane(wg / p.n_heads_q);
  const int b = __builtin_amdgcn_readfirstlane(p.row_order ? p.row_order[bi] : bi);
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - p.cu_seqlens_kv[b];
  if (qt * kDqBM >= seqlen_q) return;
  const int kv_head = __builtin_amdgcn_readfirstlane(head / (p.n_heads_q / p.n_heads_kv));
  const int64_t q_row_stride = (int64_t)p.n_heads_q * D;
  const int q_local = qt * kDqBM + w * 32 + c;
  const bool q_valid = q_local < seqlen_q;
  const int o_slot = p.out_block_table[b];

  // Q and dO fragments of this lane's query row (B operands), and the row's two scalars: the
  // base-2 log-sum-exp and -delta = -sum_d dO * O.  The lane holds half of the row's dims (those
  // of its k-slots), so delta is the lane's partial dot product plus the other half-wave's.  Both
  // scalars are also stored for the dK/dV kernel, which runs after this one and reads them per
  // (query, head) from the workspace: every (row, head, valid query) is written exactly once.
  u32x4 qreg[KS], doreg[KS];
  float lse2 = INFINITY, delta = 0.0f;
  {
    const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) +
                         (int64_t)p.q_block_table[b] * p.q_slot_stride + (int64_t)q_local * q_row_stride +
                         (int64_t)head * D + h * 8;
    const int64_t o_off = (int64_t)o_slot * p.out_slot_stride + (int64_t)q_local * q_row_stride + (int64_t)head * D + h * 8;
    const uint16_t* dp = reinterpret_cast<const uint16_t*>(p.dout) + o_off;
    const uint16_t* op = reinterpret_cast<const uint16_t*>(p.out) + o_off;
    float dot = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 z = {0, 0, 0, 0};
      qreg[ks] = q_valid ? *reinterpret_cast<const u32x4*>(qp + ks * 16) : z;
      doreg[ks] = q_valid ? *reinterpret_cast<const u32x4*>(dp + ks * 16) : z;
      const u32x4 o = q_valid ? *reinterpret_cast<const u32x4*>(op + ks * 16) : z;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dot += Elem<DTYPE>::load((uint16_t)(o[i] & 0xffffu)) * Elem<DTYPE>::load((uint16_t)(doreg[ks][i] & 0xffffu));
        dot += Elem<DTYPE>::load((uint16_t)(o[i] >> 16)) * Elem<DTYPE>::load((uint16_t)(doreg[ks][i] >> 16));
      }
    }
    delta = -halves_sum(dot);
    if (q_valid) {
      lse2 = p.lse[(int64_t)head * p.lse_head_stride + (int64_t)o_slot * p.lse_slot_stride + q_local] * kLog2e;
      if (h == 0) {
        const int64_t qrow = (int64_t)(q_begin + q_local) * p.n_heads_q + head;
        p.delta[qrow] = delta;
        p.lse2[qrow] = lse2;
      }
    }
  }
  RangePair rng = {0, 0, 0, 0};
  if (q_valid) {
    const int32_t* r = p.attn_range + q_begin + q_local;
    const int s0 = r[0], e0 = min(r[p.total_q], seqlen_kv);
    rng.s0 = s0;
    rng.len0 = max(e0 - s0, 0);
    if (p.n_ranges == 2) {
      const int s1 = r[2 * (int64_t)p.total_q], e1 = min(r[3 * (int64_t)p.total_q], seqlen_kv);
      rng.s1 = s1;
      rng.len1 = max(e1 - s1, 0);
    }
  }
  const int big = 0x7fffffff;
  const int w_lo0 = wave_min(rng.len0 > 0 ? rng.s0 : big);
  const int w_hi0 = wave_max(rng.len0 > 0 ? rng.s0 + rng.len0 : 0);
  const int w_lo1 = wave_min(rng.len1 > 0 ? rng.s1 : big);
  const int w_hi1 = wave_max(rng.len1 > 0 ? rng.s1 + rng.len1 : 0);
  const int core_lo0 = wave_max(rng.len0 > 0 ? rng.s0 : big);
  const int core_hi0 = wave_min(rng.len0 > 0 ? rng.s0 + rng.len0 : 0);
  const int core_lo1 = wave_max(rng.len1 > 0 ? rng.s1 : big);
  const int core_hi1 = wave_min(rng.len1 > 0 ? rng.s1 + rng.len1 : 0);
  const int32_t* kv_table = p.kv_block_table + (int64_t)b * p.max_kv_blocks;
  load_slot_table(slot_lds, kv_table, p.max_kv_blocks, tid, kBwdThreads);
  if (lane == 0) {
    hull_lds[w][0] = w_lo0;
    hull_lds[w][1] = w_hi0;
    hull_lds[w][2] = w_lo1;
    hull_lds[w][3] = w_hi1;
  }
  __syncthreads();
  int g_lo0 = big, g_hi0 = 0, g_lo1 = big, g_hi1 = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    g_lo0 = min(g_lo0, hull_lds[i][0]);
    g_hi0 = max(g_hi0, hull_lds[i][1]);
    g_lo1 = min(g_lo1, hull_lds[i][2]);
    g_hi1 = max(g_hi1, hull_lds[i][3]);
  }
  // the same in every lane: say so, and the tile list, the cursor and the loop control that
  // derive from them live on the scalar unit
  g_lo0 = __builtin_amdgcn_readfirstlane(g_lo0);
  g_hi0 = __builtin_amdgcn_readfirstlane(g_hi0);
  g_lo1 = __builtin_amdgcn_readfirstlane(g_lo1);
  g_hi1 = __builtin_amdgcn_readfirstlane(g_hi1);
  const TileRuns runs(g_lo0, g_hi0, g_lo1, g_hi1, BN);
  const int n_tiles = runs.count();

  f32x16 dq_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq_acc[dt][i] = 0.0f;
  // dP^T starts from -delta of the lane's query (dS = P (dP - delta)): a register block that
  // holds it serves as the C operand of the first MFMA of every dP^T chain, so the subtraction
  // costs no vector instruction per element
  f32x16 dp_init;
#pragma unroll
  for (int i = 0; i < 16; ++i) dp_init[i] = delta;

  const uint16_t* kg = reinterpret_cast<const uint16_t*>(p.k) + (int64_t)kv_head * D;
  const uint16_t* vg = reinterpret_cast<const uint16_t*>(p.v) + (int64_t)kv_head * D;
  const uint32_t kv_goff0 = Tile::lane_offset0(p.kv_token_stride, w, lane);
  const int row_rd = Tile::row_base(c, h);
  const int col_rd = Tile::col_base(lane, true);

  // the cursor names the tile to request next (one ahead of the tile being multiplied)
  const int tiles_per_block = p.block_size / BN;
  const int64_t tile_stride = (int64_t)BN * p.kv_token_stride;
  TileCursor cursor;
  // This wave's share of a tile's loads (LPW groups of K, then LPW of V) is issued one load at a
  // time between the matrix instructions, and unconditionally, so that no branch surrounds a
  // load: past the end of the list the cursor stays on the last tile, which is then fetched
  // again into a stage nobody reads any more.
  constexpr int NL = 2 * Tile::LPW;
  uint32_t fill_k = 0, fill_v = 0;
  auto issue_load = [&](int idx) {
    if (idx < Tile::LPW) Tile::load_group(fill_k, kg + cursor.off, kv_goff0, p.kv_token_stride, w, idx);
    else if (idx < NL) Tile::load_group(fill_v, vg + cursor.off, kv_goff0, p.kv_token_stride, w, idx - Tile::LPW);
  };
  auto advance = [&]() {
    if (cursor.index + 1 < n_tiles)
      cursor.advance(runs, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
  };

  auto compute = [&](int kt, const uint16_t* k_lds, const uint16_t* v_lds) {
    const int k0 = kt * BN;
    const bool wave_active = (k0 < w_hi0 && k0 + BN > w_lo0) || (k0 < w_hi1 && k0 + BN > w_lo1);
    if (!wave_active) {  // its share of the next tile is still to be requested
#pragma unroll
      for (int i = 0; i < NL; ++i) issue_load(i);
      return;
    }
    const bool unmasked = (core_lo0 <= k0 && k0 + BN <= core_hi0) || (core_lo1 <= k0 && k0 + BN <= core_hi1);

    u32x4 dsb[4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      // the range mask enters S^T as the accumulator's initial value (0 / -inf)
      f32x16 s_acc, dp_acc;
      if (unmasked) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s_acc[i] = 0.0f;
      } else {
        const uint32_t closed = rng.closed_window(k0 + nt * 32) >> (4 * h);  // bit = key - first key of the half
#pragma unroll
        for (int i = 0; i < 16; ++i) s_acc[i] = masked_start(closed, 8 * (i / 4) + (i % 4));
      }
      // operands four k-steps at a time; the two accumulation chains interleave
#pragma unroll
      for (int half = 0; half < KS / 4; ++half) {
        u32x4 ka[4], va[4];
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) ka[k4] = Tile::read_row(k_lds, row_rd, nt, half * 4 + k4);
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) va[k4] = Tile::read_row(v_lds, row_rd, nt, half * 4 + k4);
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) {
          s_acc = mfma_32x32x16<DTYPE>(ka[k4], qreg[half * 4 + k4], s_acc);
          dp_acc = mfma_32x32x16<DTYPE>(va[k4], doreg[half * 4 + k4], half == 0 && k4 == 0 ? dp_init : dp_acc);
        }
        // All of the tile's loads go out here, in the first phase, NL / (2 KS / 4) per group of
        // eight MFMAs: the last one then has the whole dQ phase to land before the wait at the
        // top of the next tile.
        constexpr int PER = NL / (2 * (KS / 4));
#pragma unroll
        for (int l = 0; l < PER; ++l) issue_load((nt * (KS / 4) + half) * PER + l);
      }
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        float e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = g * 8 + j;
          const float pr = fast_exp2(fmaf(s_acc[i], p.scale_log2, -lse2));  // masked: exp2(-inf) = 0
          e[j] = pr * dp_acc[i];
        }
        u32x4 packed = {pack2<DTYPE>(e[0], e[1]), pack2<DTYPE>(e[2], e[3]), pack2<DTYPE>(e[4], e[5]),
                        pack2<DTYPE>(e[6], e[7])};
        dsb[nt * 2 + g] = packed;
      }
    }
    // dQ^T[d, q] += K^T[d, kv] dS^T[kv, q]: K^T comes out of the K tile by transpose loads, one
    // 16-key step ahead; consecutive MFMAs go to different accumulators
    u32x4 kt_a[2][DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) kt_a[0][dt] = Tile::template read_col<true>(k_lds, col_rd, 0, dt);
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
      if (s2 + 1 < 4) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) kt_a[(s2 + 1) & 1][dt] = Tile::template read_col<true>(k_lds, col_rd, s2 + 1, dt);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) dq_acc[dt] = mfma_32x32x16<DTYPE>(kt_a[s2 & 1][dt], dsb[s2], dq_acc[dt]);
    }
  };

  const uint32_t k_at0 = lds_address(k_lds0), k_at1 = lds_address(k_lds1);
  const uint32_t v_at0 = lds_address(v_lds0), v_at1 = lds_address(v_lds1);
  if (n_tiles > 0) {
    cursor.seek(runs, 0, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
    fill_k = k_at0;
    fill_v = v_at0;
#pragma unroll
    for (int i = 0; i < NL; ++i) issue_load(i);
    advance();
  }
  for (int i = 0; i < n_tiles; i += 2) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // stage 0 is filled; nobody reads stage 1 any more
    fill_k = k_at1;
    fill_v = v_at1;
    compute(runs.tile(i), k_lds0, v_lds0);  // requests list entry i + 1 (or the last tile again)
    advance();
    if (i + 1 >= n_tiles) break;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // stage 1 is filled; nobody reads stage 0 any more
    fill_k = k_at0;
    fill_v = v_at0;
    compute(runs.tile(i + 1), k_lds1, v_lds1);
    advance();
  }
  if (n_tiles > 0) wait_loads();  // the fetch past the end of the list must land before the LDS is released

  if (!q_valid) return;
  uint16_t* op = reinterpret_cast<uint16_t*>(p.dq) +
                 (int64_t)p.dq_block_table[b] * p.dq_slot_stride + (int64_t)q_local * q_row_stride + (int64_t)head * D + 4 * h;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 pk = {pack2<DTYPE>(dq_acc[dt][4 * g] * p.scale, dq_acc[dt][4 * g + 1] * p.scale),
                  pack2<DTYPE>(dq_acc[dt][4 * g + 2] * p.scale, dq_acc[dt][4 * g + 3] * p.scale)};
      *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * g) = pk;
    }
}

// Persistent, like the forward kernel: as many workgroups as the device holds, each taking the
// next item of its XCD (workgroup b sits on XCD b % 8; the query tiles and grouped heads of a row
// share its K/V and stay on one XCD) from a ticket counter in the workspace, which the hull
// kernel zeroes before every launch.  2.7 % on the causal benchmark, 0.8 % with a lambda mask
// (whose items are all alike, so there is little dispatch imbalance to recover).
template <int DTYPE, int D>
__global__ __launch_bounds__(kBwdThreads, 2) void attn_bwd_dq_kernel(const AttnBwdParams p) {
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
    if (item < p.n_dq_items) attn_bwd_dq_item<DTYPE, D>(fresh_kernel_args<AttnBwdParams>(), (int)item);
    __syncthreads();  // the next item reuses the LDS tables and tiles, and the ticket's place
  }
}

template <int DTYPE, int D>
static int launch_bwd(const AttnBwdParams& p, hipStream_t stream) {
  const int64_t n_dkv = xcd_grid_size(p.n_dkv_items, p.dkv_xcd_group);
  DCP_REQUIRE(n_dkv < ((int64_t)1 << 31) && p.n_dq_items < ((int64_t)1 << 31), "attn_bwd: grid too large");
  // as many workgroups as the device holds at once (two per CU), a multiple of the XCD count
  const int64_t n_dq = std::min<int64_t>(xcd_grid_size(p.n_dq_items, 1), xcd_grid_size(2 * (int64_t)device_cu_count(), 1));
  {
    KernelTimer timer("bwd_tile_hull_kernel", stream);
    hipLaunchKernelGGL(bwd_tile_hull_kernel, dim3(p.batch * p.q_tiles_per_row), dim3(64), 0, stream, p);
  }
  {  // first: it also leaves -delta and the base-2 LSE of every query in the workspace for the dK/dV kernel
    KernelTimer timer("attn_bwd_dq_kernel", stream);
    hipLaunchKernelGGL((attn_bwd_dq_kernel<DTYPE, D>), dim3((unsigned)n_dq), dim3(kBwdThreads), 0, stream, p);
  }
  {
    KernelTimer timer("attn_bwd_dkv_kernel", stream);
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<DTYPE, D, false>), dim3((unsigned)n_dkv), dim3(kBwdThreads), 0, stream, p);
  }
  return check_launch("attn_bwd kernels");
}

// The dK/dV kernel alone, leaving dS in the workspace (p.delta and p.lse2 come from the prepare kernel).
int launch_bwd_dkv_writing_ds(const AttnBwdParams& p, int dtype, hipStream_t stream) {
  const int64_t n_dkv = xcd_grid_size(p.n_dkv_items, p.dkv_xcd_group);
  DCP_REQUIRE(n_dkv < ((int64_t)1 << 31), "attn_bwd: grid too large");
  KernelTimer timer("attn_bwd_dkv_kernel", stream);
  const dim3 grid((unsigned)n_dkv), block(kBwdThreads);
  if (dtype == DCP_DTYPE_BF16) {
    if (p.head_dim == 128) hipLaunchKernelGGL((attn_bwd_dkv_kernel<DCP_DTYPE_BF16, 128, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_bwd_dkv_kernel<DCP_DTYPE_BF16, 64, true>), grid, block, 0, stream, p);
  } else {
    if (p.head_dim == 128) hipLaunchKernelGGL((attn_bwd_dkv_kernel<DCP_DTYPE_FP16, 128, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_bwd_dkv_kernel<DCP_DTYPE_FP16, 64, true>), grid, block, 0, stream, p);
  }
  return check_launch("attn_bwd_dkv_kernel");
}

}  // namespace dcp

using namespace dcp;

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// What the two-kernel backward needs: -delta and lse2 per (query, head), the hulls, the tickets.
static size_t bwd_base_workspace_bytes(int batch, int total_q, int block_size, int n_heads_q) {
  const size_t q_tiles = (size_t)batch * ((block_size + kBwdBM - 1) / kBwdBM);
  return 2 * align256((size_t)total_q * n_heads_q * sizeof(float)) + align256(q_tiles * 8 * sizeof(int32_t)) +
         align256(kTicketInts * sizeof(int32_t));
}

extern "C" size_t dcp_attn_bwd_workspace_bytes(int batch, int total_q, int block_size, int n_heads_q,
                                               int head_dim) {
  if (batch < 0 || total_q < 0 || block_size <= 0 || n_heads_q <= 0 || head_dim <= 0) return 0;
  return bwd_base_workspace_bytes(batch, total_q, block_size, n_heads_q) +
         (bwd_fused_available() ? bwd_fused_extra_workspace_bytes(batch, block_size, n_heads_q, head_dim) : 0);
}

// Both entry points: argument checks, workspace carving, the four launches.
static int attn_bwd_launch(const void* dout, const void* q, const void* k, const void* v,
                           const void* out, const float* lse, void* dq, void* dk, void* dv,
                           void* workspace, size_t workspace_bytes, const int32_t* cu_seqlens_q,
                           const int32_t* cu_seqlens_kv, const int32_t* attn_range, int n_ranges,
                           const int32_t* q_block_table, const int32_t* kv_block_table,
                           const int32_t* out_block_table, const int32_t* dq_block_table,
                           const int32_t* dkv_block_table, const int32_t* row_order, int batch,
                           int max_kv_blocks, int total_q, int block_size, int n_heads_q,
                           int n_heads_kv, int head_dim, int64_t kv_slot_stride,
                           int64_t kv_token_stride, int64_t dkv_slot_stride,
                           int64_t dkv_token_stride, int64_t q_slot_stride, int64_t out_slot_stride,
                           int64_t dq_slot_stride, int64_t lse_head_stride, int64_t lse_slot_stride,
                           int64_t total_kv, float softmax_scale, int dtype, void* stream, bool allow_fused) {
  if (dtype != DCP_DTYPE_BF16 && dtype != DCP_DTYPE_FP16)
    return fail(DCP_ERR_UNSUPPORTED, "attn_bwd: dtype %d unsupported (bf16 and fp16 only)", dtype);
  if (head_dim != 64 && head_dim != 128)
    return fail(DCP_ERR_UNSUPPORTED, "attn_bwd: head_dim %d unsupported (64 or 128)", head_dim);
  DCP_REQUIRE(n_ranges == 1 || n_ranges == 2, "attn_bwd: n_ranges must be 1 or 2, got %d", n_ranges);
  DCP_REQUIRE(batch >= 0 && total_q >= 0, "attn_bwd: negative size");
  DCP_REQUIRE(softmax_scale > 0.0f, "attn_bwd: softmax_scale must be positive");
  if (batch == 0) return DCP_OK;
  DCP_REQUIRE(block_size > 0 && block_size % kBwdBN == 0,
              "attn_bwd: block_size %d must be a positive multiple of %d", block_size, kBwdBN);
  if (block_size > 64 * kBwdBM)
    return fail(DCP_ERR_UNSUPPORTED, "attn_bwd: block_size %d unsupported (at most %d)", block_size, 64 * kBwdBM);
  DCP_REQUIRE(n_heads_q > 0 && n_heads_kv > 0 && n_heads_q % n_heads_kv == 0,
              "attn_bwd: n_heads_q %d must be a multiple of n_heads_kv %d", n_heads_q, n_heads_kv);
  DCP_REQUIRE(max_kv_blocks > 0, "attn_bwd: empty block tables");
  DCP_REQUIRE(kv_token_stride % 8 == 0 && kv_slot_stride % 8 == 0 && dkv_token_stride % 4 == 0 &&
                  dkv_slot_stride % 4 == 0 && q_slot_stride % 8 == 0 && out_slot_stride % 8 == 0 && dq_slot_stride % 8 == 0,
              "attn_bwd: q, out, dout, dq, k, v strides must be multiples of 8 elements (dk/dv: 4)");
  DCP_REQUIRE(q_slot_stride > 0 && out_slot_stride > 0 && dq_slot_stride > 0 && lse_head_stride > 0 && lse_slot_stride > 0,
              "attn_bwd: table strides must be positive");
  DCP_REQUIRE(dout && q && k && v && out && lse && dq && dk && dv && workspace && cu_seqlens_q &&
                  cu_seqlens_kv && attn_range && q_block_table && kv_block_table && out_block_table &&
                  dq_block_table && dkv_block_table,
              "attn_bwd: null argument");
  DCP_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
                reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out) |
                reinterpret_cast<uintptr_t>(dout) | reinterpret_cast<uintptr_t>(dq) |
                reinterpret_cast<uintptr_t>(workspace)) & 15) == 0 &&
                  ((reinterpret_cast<uintptr_t>(dk) | reinterpret_cast<uintptr_t>(dv)) & 7) == 0,
              "attn_bwd: tensors must be 16-byte aligned (dk/dv: 8)");
  // The one-pass backward (head size 128) where the device allows it and the workspace holds its
  // partial sums; otherwise the two-kernel one, which needs the base workspace only.
  const size_t base = bwd_base_workspace_bytes(batch, total_q, block_size, n_heads_q);
  const size_t extra = bwd_fused_extra_workspace_bytes(batch, block_size, n_heads_q, head_dim);
  const bool fused = allow_fused && head_dim == 128 && bwd_fused_available() && workspace_bytes >= base + extra;
  // The backward through dS in memory where it is selected, the caller said how many keys the rows
  // have in all and the workspace holds the dS pieces.
  const size_t ds_bytes = bwd_ds_workspace_bytes(total_kv, batch, block_size, n_heads_q);
  const bool through_ds = allow_fused && !fused && bwd_select(-1) == DCP_BWD_THROUGH_DS && total_kv > 0 &&
                          workspace_bytes >= base + ds_bytes;
  DCP_REQUIRE(workspace_bytes >= base, "attn_bwd: workspace of %zu bytes is smaller than the %zu needed",
              workspace_bytes, base);
  AttnBwdParams p;
  p.dout = dout;
  p.q = q;
  p.k = k;
  p.v = v;
  p.out = out;
  p.lse = lse;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  char* ws = reinterpret_cast<char*>(workspace);
  p.delta = reinterpret_cast<float*>(ws);
  ws += align256((size_t)total_q * n_heads_q * sizeof(float));
  p.lse2 = reinterpret_cast<float*>(ws);
  ws += align256((size_t)total_q * n_heads_q * sizeof(float));
  p.hull = reinterpret_cast<int32_t*>(ws);
  ws += align256((size_t)batch * ((block_size + kBwdBM - 1) / kBwdBM) * 8 * sizeof(int32_t));
  p.tickets = reinterpret_cast<int*>(ws);
  ws += align256(kTicketInts * sizeof(int32_t));
  p.subs_per_row = (block_size + 31) / 32;
  p.head_dim = head_dim;
  p.dq_part = nullptr;
  p.chain = nullptr;
  p.fault = nullptr;
  p.ds = through_ds ? ws : nullptr;
  p.ds_pieces = (int64_t)(ds_bytes >> 12) - 2;  // the last two pieces are spare (waves without keys write there)
  if (fused) {
    const size_t chunks = (size_t)batch * n_heads_q * p.subs_per_row;
    p.dq_part = reinterpret_cast<float*>(ws);
    ws += align256(chunks * 4096 * sizeof(float));
    p.chain = reinterpret_cast<int*>(ws);
    ws += align256(chunks * 4 * sizeof(int));
    p.fault = reinterpret_cast<int*>(ws);
  }
  p.cu_seqlens_q = cu_seqlens_q;
  p.cu_seqlens_kv = cu_seqlens_kv;
  p.attn_range = attn_range;
  p.q_block_table = q_block_table;
  p.kv_block_table = kv_block_table;
  p.out_block_table = out_block_table;
  p.dq_block_table = dq_block_table;
  p.dkv_block_table = dkv_block_table;
  p.row_order = row_order;
  p.n_ranges = n_ranges;
  p.batch = batch;
  p.max_kv_blocks = max_kv_blocks;
  p.total_q = total_q;
  p.block_size = block_size;
  p.n_heads_q = n_heads_q;
  p.n_heads_kv = n_heads_kv;
  p.kv_slot_stride = kv_slot_stride;
  p.kv_token_stride = kv_token_stride;
  p.dkv_slot_stride = dkv_slot_stride;
  p.dkv_token_stride = dkv_token_stride;
  p.n_out_slots = 0;
  p.q_slot_stride = q_slot_stride;
  p.out_slot_stride = out_slot_stride;
  p.dq_slot_stride = dq_slot_stride;
  p.lse_head_stride = lse_head_stride;
  p.lse_slot_stride = lse_slot_stride;
  p.q_tiles_per_row = (block_size + kBwdBM - 1) / kBwdBM;
  p.dq_tiles_per_row = (block_size + kDqBM - 1) / kDqBM;
  p.kv_tiles_per_row = (int)(((int64_t)max_kv_blocks * block_size + kDkvBN - 1) / kDkvBN);
  p.n_dkv_items = (int64_t)batch * n_heads_kv * p.kv_tiles_per_row;
  p.n_dq_items = (int64_t)batch * n_heads_q * p.dq_tiles_per_row;
  p.dkv_xcd_group = p.kv_tiles_per_row;
  p.dq_xcd_group = p.dq_tiles_per_row * (n_heads_q / n_heads_kv);
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * kLog2e;
  if (fused) return launch_bwd_fused(p, dtype, (hipStream_t)stream);
  if (through_ds) return launch_bwd_through_ds(p, dtype, (hipStream_t)stream);
  if (dtype == DCP_DTYPE_BF16)
    return head_dim == 128 ? launch_bwd<DCP_DTYPE_BF16, 128>(p, (hipStream_t)stream)
                           : launch_bwd<DCP_DTYPE_BF16, 64>(p, (hipStream_t)stream);
  return head_dim == 128 ? launch_bwd<DCP_DTYPE_FP16, 128>(p, (hipStream_t)stream)
                         : launch_bwd<DCP_DTYPE_FP16, 64>(p, (hipStream_t)stream);
}

extern "C" int dcp_attn_bwd(const void* dout, const void* q, const void* k, const void* v,
                            const void* out, const float* lse, void* dq, void* dk, void* dv,
                            void* workspace, size_t workspace_bytes, const int32_t* cu_seqlens_q,
                            const int32_t* cu_seqlens_kv, const int32_t* attn_range, int n_ranges,
                            const int32_t* q_block_table, const int32_t* kv_block_table,
                            const int32_t* out_block_table, const int32_t* dq_block_table,
                            const int32_t* dkv_block_table, const int32_t* row_order, int batch,
                            int max_kv_blocks, int total_q, int block_size, int n_heads_q,
                            int n_heads_kv, int head_dim, int64_t kv_slot_stride,
                            int64_t kv_token_stride, int64_t dkv_slot_stride,
                            int64_t dkv_token_stride, int n_out_slots, float softmax_scale,
                            int dtype, void* stream) {
  DCP_REQUIRE(batch == 0 || n_out_slots > 0, "attn_bwd: empty block tables");
  const int64_t slot = (int64_t)block_size * n_heads_q * head_dim;
  return attn_bwd_launch(dout, q, k, v, out, lse, dq, dk, dv, workspace, workspace_bytes, cu_seqlens_q,
                         cu_seqlens_kv, attn_range, n_ranges, q_block_table, kv_block_table, out_block_table,
                         dq_block_table, dkv_block_table, row_order, batch, max_kv_blocks, total_q, block_size,
                         n_heads_q, n_heads_kv, head_dim, kv_slot_stride, kv_token_stride, dkv_slot_stride,
                         dkv_token_stride, slot, slot, slot, (int64_t)n_out_slots * block_size, block_size, 0,
                         softmax_scale, dtype, stream, true);
}

extern "C" int dcp_attn_bwd_strided(const void* dout, const void* q, const void* k, const void* v,
                                    const void* out, const float* lse, void* dq, void* dk, void* dv,
                                    void* workspace, size_t workspace_bytes, const int32_t* cu_seqlens_q,
                                    const int32_t* cu_seqlens_kv, const int32_t* attn_range, int n_ranges,
                                    const int32_t* q_block_table, const int32_t* kv_block_table,
                                    const int32_t* out_block_table, const int32_t* dq_block_table,
                                    const int32_t* dkv_block_table, const int32_t* row_order, int batch,
                                    int max_kv_blocks, int total_q, int block_size, int n_heads_q,
                                    int n_heads_kv, int head_dim, int64_t kv_slot_stride,
                                    int64_t kv_token_stride, int64_t dkv_slot_stride,
                                    int64_t dkv_token_stride, int64_t q_slot_stride, int64_t out_slot_stride,
                                    int64_t dq_slot_stride, int64_t lse_head_stride, int64_t lse_slot_stride,
                                    int64_t total_kv, float softmax_scale, int dtype, void* stream) {
  return attn_bwd_launch(dout, q, k, v, out, lse, dq, dk, dv, workspace, workspace_bytes, cu_seqlens_q,
                         cu_seqlens_kv, attn_range, n_ranges, q_block_table, kv_block_table, out_block_table,
                         dq_block_table, dkv_block_table, row_order, batch, max_kv_blocks, total_q, block_size,
                         n_heads_q, n_heads_kv, head_dim, kv_slot_stride, kv_token_stride, dkv_slot_stride,
                         dkv_token_stride, q_slot_stride, out_slot_stride, dq_slot_stride, lse_head_stride,
                         lse_slot_stride, total_kv, softmax_scale, dtype, stream, true);
}

extern "C" int dcp_attn_bwd_select(int mode) { return bwd_select(mode); }

extern "C" size_t dcp_attn_bwd_workspace_bytes_kv(int batch, int total_q, int64_t total_kv, int block_size,
                                                  int n_heads_q, int head_dim) {
  const size_t base = dcp_attn_bwd_workspace_bytes(batch, total_q, block_size, n_heads_q, head_dim);
  if (base == 0 || bwd_select(-1) != DCP_BWD_THROUGH_DS) return base;
  return base + bwd_ds_workspace_bytes(total_kv, batch, block_size, n_heads_q);
}

// ---------------------------------------------------------------------------
// The backward with its scratch inside the library, for callers that can neither allocate
// nor pass a workspace.  Every device the library runs on holds its own copy of `scratch`
// until the process ends.  In host code the array's name is only a handle: its device address
// is asked for once per device (with that device current) and kept.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[DCP_ATTN_BWD_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device, or nullptr (message set).
void* scratch_on_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(DCP_ERR_LAUNCH, "attn_bwd_static: no current device (or device index above %d)", kMaxDevices - 1);
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      fail(DCP_ERR_LAUNCH, "attn_bwd_static: hipGetSymbolAddress(scratch) on device %d: %s", dev,
           hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

// Also the set-up call of dcp_attn_bwd_static: it looks up (and keeps) the scratch array's address
// on the current device, so that the entry point itself makes no runtime query -- a caller that
// records it into a HIP graph calls this once per device beforehand, outside the capture.
extern "C" size_t dcp_attn_bwd_static_scratch_bytes(void) {
  (void)scratch_on_current_device();
  return DCP_ATTN_BWD_STATIC_SCRATCH_BYTES;
}

extern "C" int dcp_attn_bwd_static(const void* dout, const void* q, const void* k, const void* v,
                                   const void* out, const float* lse, void* dq, void* dk, void* dv,
                                   const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_kv,
                                   const int32_t* attn_range, int n_ranges, const int32_t* q_block_table,
                                   const int32_t* kv_block_table, const int32_t* out_block_table,
                                   const int32_t* dq_block_table, const int32_t* dkv_block_table,
                                   const int32_t* row_order, int batch, int max_kv_blocks, int total_q,
                                   int block_size, int n_heads_q, int n_heads_kv, int head_dim,
                                   int64_t kv_slot_stride, int64_t kv_token_stride, int64_t dkv_slot_stride,
                                   int64_t dkv_token_stride, int n_out_slots, float softmax_scale, int dtype,
                                   void* stream) {
  (void)head_dim;
  const size_t need = bwd_base_workspace_bytes(batch, total_q, block_size, n_heads_q);  // the two-kernel backward's
  DCP_REQUIRE(need <= (size_t)DCP_ATTN_BWD_STATIC_SCRATCH_BYTES,
              "attn_bwd_static: these sizes need %zu bytes of scratch, the built-in scratch holds %zu; "
              "use dcp_attn_bwd with a caller workspace",
              need, (size_t)DCP_ATTN_BWD_STATIC_SCRATCH_BYTES);
  void* ptr = scratch_on_current_device();
  if (ptr == nullptr) return DCP_ERR_LAUNCH;
  // Nothing in the scratch has to start at zero: delta, lse2 and the hulls are written for every
  // valid (token, head) / query tile before the kernels that read them run (and only those are
  // read), and the hull kernel zeroes the work counters on the stream.
  DCP_REQUIRE(batch == 0 || n_out_slots > 0, "attn_bwd_static: empty block tables");
  const int64_t slot = (int64_t)block_size * n_heads_q * head_dim;
  return attn_bwd_launch(dout, q, k, v, out, lse, dq, dk, dv, ptr, DCP_ATTN_BWD_STATIC_SCRATCH_BYTES, cu_seqlens_q,
                         cu_seqlens_kv, attn_range, n_ranges, q_block_table, kv_block_table, out_block_table,
                         dq_block_table, dkv_block_table, row_order, batch, max_kv_blocks, total_q, block_size,
                         n_heads_q, n_heads_kv, head_dim, kv_slot_stride, kv_token_stride, dkv_slot_stride,
                         dkv_token_stride, slot, slot, slot, (int64_t)n_out_slots * block_size, block_size, 0,
                         softmax_scale, dtype, stream, false);
}

