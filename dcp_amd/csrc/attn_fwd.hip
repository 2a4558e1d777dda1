// Range-masked paged attention forward for gfx950.
//
// One workgroup (4 waves) owns 128 query rows of one (row, head); wave w owns
// rows 32w..32w+31.  It walks the key tiles (64 keys) its rows can see and
// keeps a running softmax per query row.  Everything is computed transposed:
//
//   S^T[kv, q] = K Q^T      A = K tile from LDS, B = Q held in registers
//   O^T[d,  q] = V^T P^T    A = V^T tile from LDS, B = P^T straight from the
//                           S^T accumulators
//
// With the 32x32x16 MFMA a lane holds one column of the accumulator, so in
// this orientation a lane owns one query row: the row max / row sum need no
// cross-lane reduction beyond one exchange between the two half-waves, the
// rescale factor is a per-lane scalar, and the masked range of the row lives
// in four registers.
//
// Software pipeline inside a wave: S^T of tile j+1 is multiplied while tile j is
// exponentiated, MFMA by MFMA in one instruction stream, so the matrix pipe and the
// vector ALU work at the same time instead of taking turns; O^T += V^T P^T of tile
// j follows as a dense run of MFMAs that the other wave of the SIMD can fill with
// its own arithmetic.
//
// K and V tiles go from global memory straight into LDS (global_load_lds, no
// register staging), in two stages: the next tile streams in while the current
// one is multiplied.  The row order and padding of each tile are chosen so that
// operand reads are conflict-free and every LDS address in the key loop is a
// per-lane base plus an immediate.  V^T is never materialised: the transposing
// LDS load delivers it from the V tile.
//
// Key tiles are chosen per workgroup from the hull of its rows' ranges (tiles
// no row can see are never loaded), each wave skips tiles outside its own
// rows' hull, and a tile that lies inside every row's range of the wave skips
// the per-element range test.
#include <math.h>

#include <algorithm>

#include "attn_common.h"

namespace dcp {

struct AttnFwdParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  const int32_t* cu_seqlens_q;
  const int32_t* cu_seqlens_kv;
  const int32_t* attn_range;
  const int32_t* q_block_table;
  const int32_t* kv_block_table;
  const int32_t* out_block_table;
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
  int n_out_slots;
  // element strides of a table entry: a slot of block_size tokens, or a single token when the
  // tables address the caller's unpadded tensors directly (entries are then token offsets)
  int64_t q_slot_stride;
  int64_t out_slot_stride;
  int64_t lse_head_stride;
  int64_t lse_slot_stride;
  float empty_lse;   // what the LSE of a query without a visible key reads: +inf, or the merged form -1
  int q_tiles_per_row;
  int xcd_group;     // work items per shared K/V stream
  int64_t n_items;   // batch * n_heads_q * q_tiles_per_row
  float scale_log2;  // softmax_scale * log2(e)
  int* tickets;      // kNumXcd item counters, zeroed before the launch
};

// Wave priority by phase: the two waves of a SIMD come from different workgroups and drift
// through the loop independently.  Both matrix phases outrank the control code between them
// (2-3 % on the kernel), and the fused phase, whose vector work is the longer chain, outranks
// the dense one (another 1.5 %; the other way round it was 1.5 % slower).
constexpr int kPrioControl = 0, kPrioFused = 2, kPrioDense = 1;
constexpr int kFwdBN = 64;
constexpr int kFwdThreads = 256;
// The running maximum of a row is only raised (and O^T rescaled) when the tile's maximum
// exceeds it by more than this many powers of two; until then the weights of the tile are
// taken relative to the old maximum and are at most 2^kLazyMax.  With fp32 sums and
// accumulators that costs no accuracy, and it takes the rescale (64 multiplies per query
// block) out of almost every tile after a row's first few.
constexpr float kLazyMax = 8.0f;
// On the fast path a tile is exponentiated against the row's current reference without taking
// its maximum first; it is redone against a raised reference only if one lane's partial row sum
// of the tile (32 weights) reaches kMaxTileSum, i.e. if some weight might exceed it.  2^14 keeps
// every accepted weight representable in fp16 and far from overflowing the fp32 accumulators.
constexpr float kMaxTileSum = 16384.0f;

// QB = 32-row query blocks per wave: the workgroup owns 128*QB query rows.  With QB = 2 every
// K / V^T operand read from LDS feeds two matrix instructions and every tile brought into LDS
// serves twice the arithmetic; the wave then needs the whole register file (one workgroup
// per CU, accumulators in the AGPR half).
template <int DTYPE, int D, int QB>
__device__ __forceinline__ void attn_fwd_item(const AttnFwdParams& p, int item) {
  constexpr int BN = kFwdBN;
  constexpr int BM = 128 * QB;
  constexpr int KS = D / 16;  // k-steps of S^T = K Q^T
  constexpr int DT = D / 32;  // 32-row tiles of O^T
  typedef KvTile<D> KTile;  // read as rows (A operand of S^T)
  typedef KvTile<D> VTile;  // read as columns (A operand of O^T = V^T P^T)
  // two stages of (K tile, V tile); separate arrays so the compiler can tell
  // the stage being filled from the stage being read
  __shared__ __attribute__((aligned(16))) uint16_t k_lds0[KTile::SIZE];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds0[VTile::SIZE];
  __shared__ __attribute__((aligned(16))) uint16_t k_lds1[KTile::SIZE];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds1[VTile::SIZE];
  __shared__ int hull_lds[4][4];
  __shared__ int slot_lds[kSlotTableCap];

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int c = lane & 31;
  const int h = lane >> 5;

  // ---- which (row, head, q tile) ----------------------------------------
  // the query tiles and grouped heads of a row share its K/V: keep them on one XCD
  // Integer division runs on the vector unit, so its (uniform) results sit in vector registers
  // and drag every address derived from them there too: each tile load then costs three vector
  // instructions to rebuild a scalar base.  readfirstlane puts the indices back on the scalar unit.
  int wg = item;
  const int qt = __builtin_amdgcn_readfirstlane(wg % p.q_tiles_per_row);
  wg /= p.q_tiles_per_row;
  const int head = __builtin_amdgcn_readfirstlane(wg % p.n_heads_q);
  const int bi = __builtin_amdgcn_readfirstlane(wg / p.n_heads_q);
  const int b = __builtin_amdgcn_readfirstlane(p.row_order ? p.row_order[bi] : bi);
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - p.cu_seqlens_kv[b];
  if (qt * BM >= seqlen_q) return;
  const int kv_head = __builtin_amdgcn_readfirstlane(head / (p.n_heads_q / p.n_heads_kv));
  const int64_t q_row_stride = (int64_t)p.n_heads_q * D;

  int q_local[QB];
  bool q_valid[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    q_local[qb] = qt * BM + (w * QB + qb) * 32 + c;
    q_valid[qb] = q_local[qb] < seqlen_q;
  }

  // ---- Q fragments (B operands of S^T) -------------------------------------
  u32x4 qreg[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) +
                         (int64_t)p.q_block_table[b] * p.q_slot_stride + (int64_t)q_local[qb] * q_row_stride +
                         (int64_t)head * D + h * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 z = {0, 0, 0, 0};
      qreg[qb][ks] = q_valid[qb] ? *reinterpret_cast<const u32x4*>(qp + ks * 16) : z;
    }
  }

  // ---- this lane's query rows: ranges --------------------------------------
  RangePair rng[QB];
  const int big = 0x7fffffff;
  int w_lo0 = big, w_hi0 = 0, w_lo1 = big, w_hi1 = 0;            // hull: what any row of the wave can see
  int core_lo0 = 0, core_hi0 = big, core_lo1 = 0, core_hi1 = big;  // core: what every row sees
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    RangePair r4 = {0, 0, 0, 0};
    if (q_valid[qb]) {
      const int32_t* r = p.attn_range + q_begin + q_local[qb];
      const int s0 = r[0], e0 = min(r[p.total_q], seqlen_kv);
      r4.s0 = s0;
      r4.len0 = max(e0 - s0, 0);
      if (p.n_ranges == 2) {
        const int s1 = r[2 * (int64_t)p.total_q], e1 = min(r[3 * (int64_t)p.total_q], seqlen_kv);
        r4.s1 = s1;
        r4.len1 = max(e1 - s1, 0);
      }
    }
    rng[qb] = r4;
    w_lo0 = min(w_lo0, wave_min(r4.len0 > 0 ? r4.s0 : big));
    w_hi0 = max(w_hi0, wave_max(r4.len0 > 0 ? r4.s0 + r4.len0 : 0));
    w_lo1 = min(w_lo1, wave_min(r4.len1 > 0 ? r4.s1 : big));
    w_hi1 = max(w_hi1, wave_max(r4.len1 > 0 ? r4.s1 + r4.len1 : 0));
    core_lo0 = max(core_lo0, wave_max(r4.len0 > 0 ? r4.s0 : big));
    core_hi0 = min(core_hi0, wave_min(r4.len0 > 0 ? r4.s0 + r4.len0 : 0));
    core_lo1 = max(core_lo1, wave_max(r4.len1 > 0 ? r4.s1 : big));
    core_hi1 = min(core_hi1, wave_min(r4.len1 > 0 ? r4.s1 + r4.len1 : 0));
  }
  const int32_t* kv_table = p.kv_block_table + (int64_t)b * p.max_kv_blocks;
  load_slot_table(slot_lds, kv_table, p.max_kv_blocks, tid, kFwdThreads);
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

  // ---- running state ---------------------------------------------------------
  f32x16 o_acc[QB][DT];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[qb][dt][i] = 0.0f;
  float m_run[QB], l_run[QB];  // reference maximum (log2 domain); this half-wave's partial row sum
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.0f;
  }

  const uint16_t* kg = reinterpret_cast<const uint16_t*>(p.k) + (int64_t)kv_head * D;
  const uint16_t* vg = reinterpret_cast<const uint16_t*>(p.v) + (int64_t)kv_head * D;

  // loop-invariant per-lane pieces of every address used in the key loop
  const uint32_t kv_goff0 = KTile::lane_offset0(p.kv_token_stride, w, lane);
  const int k_rd = KTile::row_base(c, h);
  const int v_rd = VTile::col_base(lane, true);

  // The cursor runs two tiles ahead of the tile being exponentiated: it names the K
  // tile to request next.  V of a tile is requested one iteration after its K, from the
  // offset remembered then.
  const int tiles_per_block = p.block_size / BN;
  const int64_t tile_stride = (int64_t)BN * p.kv_token_stride;
  TileCursor cursor;
  auto cursor_next = [&]() {
    if (__builtin_expect(cursor.index + 1 < n_tiles, 1)) cursor.advance(runs, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
    else ++cursor.index;  // past the end: nothing left to request
  };
  const uint32_t k_at0 = lds_address(k_lds0), k_at1 = lds_address(k_lds1);
  const uint32_t v_at0 = lds_address(v_lds0), v_at1 = lds_address(v_lds1);
  // does any row of this wave see key tile `tile` / does every row see all of it
  auto wave_sees = [&](int tile) -> bool {
    const int k0 = tile * BN;
    return (k0 < w_hi0 && k0 + BN > w_lo0) || (k0 < w_hi1 && k0 + BN > w_lo1);
  };
  auto wave_sees_all = [&](int tile) -> bool {
    const int k0 = tile * BN;
    return (core_lo0 <= k0 && k0 + BN <= core_hi0) || (core_lo1 <= k0 && k0 + BN <= core_hi1);
  };
  // the same test in tile numbers, for the loop's fast path: tiles [full0, full0 + n_full0) and
  // [full1, full1 + n_full1) lie inside every row's range
  const int full0 = (core_lo0 > big - BN ? big / BN : (core_lo0 + BN - 1) / BN), n_full0 = max(core_hi0 / BN - full0, 0);
  const int full1 = (core_lo1 > big - BN ? big / BN : (core_lo1 + BN - 1) / BN), n_full1 = max(core_hi1 / BN - full1, 0);
  auto tile_is_full = [&](int tile) -> bool {
    return ((unsigned)(tile - full0) < (unsigned)n_full0) | ((unsigned)(tile - full1) < (unsigned)n_full1);
  };

  // The tile loads of an iteration (this wave's share: LPW groups of K, LPW of V) are issued
  // one at a time between the matrix instructions of the S^T product: as a burst after the
  // barrier they fill the memory pipeline's queue and the wave sits at its last load until the
  // queue has drained, and issued later (spread over the O^T product too) the last one is still
  // on its way at the wait that opens the next iteration.  Both stages they fill are free from
  // the iteration's first barrier on.  They are issued unconditionally, so that the loop has no
  // branches around them: past the end of the tile list the cursor stays on the last tile,
  // which is then fetched again into a stage nobody reads any more.
  constexpr int NL = 2 * KTile::LPW;
  uint32_t fill_k = 0, fill_v = 0;
  int64_t fill_k_off = 0, fill_v_off = 0;
  auto issue_load = [&](int idx) {
    if (idx < KTile::LPW) KTile::load_group(fill_k, kg + fill_k_off, kv_goff0, p.kv_token_stride, w, idx);
    else if (idx < NL) VTile::load_group(fill_v, vg + fill_v_off, kv_goff0, p.kv_token_stride, w, idx - KTile::LPW);
  };

  // Operand i of S^T = K Q^T: key half i & 1, k-step i >> 1 (the two halves alternate so
  // that consecutive MFMAs are independent); each operand feeds QB MFMAs.
  auto k_operand = [&](const uint16_t* k_lds, int i) { return KTile::read_row(k_lds, k_rd, i & 1, i >> 1); };

  // S^T of a tile on its own.  The range mask enters as the accumulator's initial
  // value: 0 where the row may look, -inf where it may not.
  auto multiply_qk = [&](int tile, const uint16_t* k_lds, f32x16 (&s_out)[2][QB]) {
    if (wave_sees_all(tile)) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
          for (int e = 0; e < 16; ++e) s_out[nt][qb][e] = 0.0f;
    } else {
      // the keys a row may not see, as a bit mask per 32-key half (bit = key - first key of the
      // half), shifted so that element e of this lane's half h is bit 8 (e / 4) + e % 4
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const uint32_t closed = rng[qb].closed_window(tile * BN + nt * 32) >> (4 * h);
#pragma unroll
          for (int e = 0; e < 16; ++e) s_out[nt][qb][e] = masked_start(closed, 8 * (e / 4) + (e % 4));
        }
    }
    constexpr int N = 2 * KS, AHEAD = 3;
    u32x4 ka[4];
#pragma unroll
    for (int i2 = 0; i2 < AHEAD; ++i2) ka[i2] = k_operand(k_lds, i2);
#pragma unroll
    for (int i2 = 0; i2 < N; ++i2) {
      if (i2 + AHEAD < N) ka[(i2 + AHEAD) & 3] = k_operand(k_lds, i2 + AHEAD);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
        s_out[i2 & 1][qb] = mfma_32x32x16<DTYPE>(ka[i2 & 3], qreg[qb][i2 >> 1], s_out[i2 & 1][qb]);
      if ((i2 + 1) % (N / NL) == 0) issue_load(i2 / (N / NL));
      __builtin_amdgcn_sched_barrier(0);  // keeps the operand reads from being hoisted into more registers
    }
  };

  // ---- online softmax (log2 domain), in pieces so that it can be interleaved ----
  u32x4 pb[QB][4];       // P^T of the current tile, packed: the B operands of O^T += V^T P^T
  float alpha[QB];       // pending rescale of O^T (applied before the tile's P^T is multiplied in)
  bool rescale[QB];
  float m_use[QB], lsum[QB];
  // The maximum step of a tile: the row maximum, and the row's reference raised to it if needed.
  auto softmax_max = [&](const f32x16 (&sc)[2][QB]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[nt][qb][e]);
      mx = halves_max(mx * p.scale_log2);  // -inf stays -inf (scale > 0)
      // raise the reference maximum only when the tile exceeds it by more than kLazyMax (always
      // for a row that had none yet: -inf + kLazyMax = -inf), then for every row of the wave
      rescale[qb] = __any(mx > m_run[qb] + kLazyMax);
      const float m_new = rescale[qb] ? fmaxf(m_run[qb], mx) : m_run[qb];
      m_use[qb] = (m_new == -INFINITY) ? 0.0f : m_new;
      alpha[qb] = fast_exp2(m_run[qb] - m_use[qb]);  // m_run = -inf -> 0; 1 where the maximum stays
      l_run[qb] *= alpha[qb];
      m_run[qb] = m_new;
      lsum[qb] = 0.0f;
    }
  };
  // elements 2*c2, 2*c2+1 of the 32 this lane holds for query block qb
  auto softmax_pair = [&](const f32x16 (&sc)[2][QB], int qb, int c2) {
    const int nt = c2 >> 3, e = (c2 & 7) * 2;
    const float e0 = fast_exp2(fmaf(sc[nt][qb][e], p.scale_log2, -m_use[qb]));
    const float e1 = fast_exp2(fmaf(sc[nt][qb][e + 1], p.scale_log2, -m_use[qb]));
    lsum[qb] += e0 + e1;
    pb[qb][nt * 2 + (e >> 3)][(e & 7) >> 1] = pack2<DTYPE>(e0, e1);
  };
  auto apply_rescale = [&]() {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
      if (__builtin_expect(rescale[qb], 0)) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int e = 0; e < 16; ++e) o_acc[qb][dt][e] *= alpha[qb];
      }
  };
  auto softmax = [&](const f32x16 (&sc)[2][QB]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
      for (int c2 = 0; c2 < 16; ++c2) softmax_pair(sc, qb, c2);
      l_run[qb] += lsum[qb];
    }
  };

  // S^T of the next tile and the softmax of the current one in one instruction stream:
  // every MFMA is followed by its share of the softmax arithmetic, so that the matrix
  // pipe and the vector ALU of the SIMD are busy at the same time.  Operands are read
  // three ahead.
  auto multiply_qk_with_softmax = [&](const uint16_t* k_lds, f32x16 (&s_out)[2][QB], const f32x16 (&sc)[2][QB]) {
    constexpr int N = 2 * KS;     // operands, QB MFMAs each
    constexpr int AHEAD = 3;
    constexpr int FIRST = 0;
    constexpr int PAIRS = 16 * QB;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int e = 0; e < 16; ++e) s_out[nt][qb][e] = 0.0f;
    u32x4 ka[4];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ka[i] = k_operand(k_lds, i);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (i + AHEAD < N) ka[(i + AHEAD) & 3] = k_operand(k_lds, i + AHEAD);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        s_out[i & 1][qb] = mfma_32x32x16<DTYPE>(ka[i & 3], qreg[qb][i >> 1], s_out[i & 1][qb]);
        if (i >= FIRST) {
          // pairs [lo, hi) of the PAIRS this wave owes, query block 0 first
          const int lo = ((i - FIRST) * QB + qb) * PAIRS / ((N - FIRST) * QB);
          const int hi = ((i - FIRST) * QB + qb + 1) * PAIRS / ((N - FIRST) * QB);
#pragma unroll
          for (int c2 = lo; c2 < hi; ++c2) softmax_pair(sc, c2 / 16, c2 % 16);
        }
      }
      if ((i + 1) % (N / NL) == 0) issue_load(i / (N / NL));
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // O^T += V^T P^T: V^T comes out of the row-major V tile by transpose loads, read
  // two operands ahead; consecutive MFMAs go to different accumulators
  auto multiply_pv = [&](const uint16_t* v_lds) {
    constexpr int N = 4 * DT;
    constexpr int AHEAD = 2;
    auto v_operand = [&](int i) { return VTile::template read_col<true>(v_lds, v_rd, i / DT, i % DT); };
    u32x4 va[4];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) va[i] = v_operand(i);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (i + AHEAD < N) va[(i + AHEAD) & 3] = v_operand(i + AHEAD);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
        o_acc[qb][i % DT] = mfma_32x32x16<DTYPE>(va[i & 3], pb[qb][i / DT], o_acc[qb][i % DT]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- key loop --------------------------------------------------------------------
  // Iteration j multiplies S^T of tile j+1 while it exponentiates tile j, then adds
  // tile j to O^T.  K tile j+1 and V tile j are in LDS by then; K tile j+2 and V tile
  // j+1 stream into the stages that K tile j and V tile j-1 have left.
  f32x16 s_a[2][QB], s_b[2][QB];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_a[nt][qb][e] = s_b[nt][qb][e] = 0.0f;
  int tile_cur = 0, tile_nxt = 0;  // key tile numbers of list entries j and j+1
  int64_t v_off = 0;               // offset of list entry j+1 (its V is requested in iteration j)
  bool cur_full = false;           // list entry j lies inside every row's range
  bool pending = false;            // the maximum step of list entry j has been done already
  bool anchored = false;           // every row of the wave has a (finite) reference maximum
  auto iteration = [&](int j, f32x16 (&s_cur)[2][QB], f32x16 (&s_nxt)[2][QB], const uint16_t* k_nxt, uint32_t k_fill,
                       const uint16_t* v_cur, uint32_t v_fill) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // K tile j+1 and V tile j are filled; nobody reads K tile j or V tile j-1 any more
    fill_k = k_fill;
    fill_v = v_fill;
    fill_k_off = cursor.off;
    fill_v_off = v_off;
    // the S^T product carries the tile loads; a wave that skips it still has its share to request
    const bool nxt_full = j + 1 < n_tiles && tile_is_full(tile_nxt);
    bool cur = true;
    if (__builtin_expect(cur_full && nxt_full && anchored, 1)) {
      // The common case, decided by one test per iteration: this tile and the next are inside
      // every row's range and every row has a reference maximum.  The weights are taken relative
      // to that reference WITHOUT looking at the tile's own maximum first ...
      if (!pending) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          lsum[qb] = 0.0f;
          rescale[qb] = false;
        }
      }
      __builtin_amdgcn_s_setprio(kPrioFused);
      multiply_qk_with_softmax(k_nxt, s_nxt, s_cur);
      // ... and the tile's partial row sums tell afterwards whether that was safe: every weight is
      // at most its lane's sum.  Only if a sum is out of bounds (or not a number) is the tile's
      // maximum taken, the reference raised and the tile exponentiated again.
      bool redo = false;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) redo |= __any(!(lsum[qb] < kMaxTileSum));
      if (__builtin_expect(redo, 0)) {
        softmax_max(s_cur);
        softmax(s_cur);
      } else {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) l_run[qb] += lsum[qb];
      }
    } else {
      cur = cur_full || wave_sees(tile_cur);
      const bool nxt = j + 1 < n_tiles && (nxt_full || wave_sees(tile_nxt));
      if (nxt) {
        multiply_qk(tile_nxt, k_nxt, s_nxt);
      } else {
#pragma unroll
        for (int i = 0; i < NL; ++i) issue_load(i);
      }
      if (cur) {
        if (!pending) softmax_max(s_cur);
        softmax(s_cur);
        anchored |= cur_full;  // a tile every row sees gives every row a reference
      }
    }
    pending = false;
    if (__builtin_expect(cur, 1)) {
      apply_rescale();
      __builtin_amdgcn_s_setprio(kPrioDense);
      multiply_pv(v_cur);
      __builtin_amdgcn_s_setprio(kPrioControl);
    }
    cur_full = nxt_full;
    tile_cur = tile_nxt;
    tile_nxt = cursor.tile;
    v_off = cursor.off;
    cursor_next();
  };
  if (n_tiles > 0) {
    cursor.seek(runs, 0, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
    tile_cur = cursor.tile;
    fill_k = k_at0;
    fill_v = v_at0;
    fill_k_off = fill_v_off = cursor.off;
#pragma unroll
    for (int i = 0; i < NL; ++i) issue_load(i);
    cursor_next();
    tile_nxt = cursor.tile;
    v_off = cursor.off;
    fill_k = k_at1;
    fill_k_off = cursor.off;
#pragma unroll
    for (int i = 0; i < KTile::LPW; ++i) issue_load(i);
    cursor_next();
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    cur_full = tile_is_full(tile_cur);
    if (wave_sees(tile_cur)) {
      multiply_qk(tile_cur, k_lds0, s_a);
      softmax_max(s_a);
      pending = true;
      anchored = cur_full;
    }
    for (int j = 0; j < n_tiles; j += 2) {
      iteration(j, s_a, s_b, k_lds1, k_at0, v_lds0, v_at1);
      if (__builtin_expect(j + 1 >= n_tiles, 0)) break;
      iteration(j + 1, s_b, s_a, k_lds0, k_at1, v_lds1, v_at0);
    }
    wait_loads();  // the fetches past the end of the list must land before the workgroup's LDS is released
  }

  // ---- epilogue ------------------------------------------------------------------
  const int o_slot = p.out_block_table[b];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l_tot = halves_sum(l_run[qb]);
    if (!q_valid[qb]) continue;
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    uint16_t* op = reinterpret_cast<uint16_t*>(p.out) +
                   (int64_t)o_slot * p.out_slot_stride + (int64_t)q_local[qb] * q_row_stride + (int64_t)head * D + 4 * h;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 pk = {pack2<DTYPE>(o_acc[qb][dt][4 * g] * inv, o_acc[qb][dt][4 * g + 1] * inv),
                    pack2<DTYPE>(o_acc[qb][dt][4 * g + 2] * inv, o_acc[qb][dt][4 * g + 3] * inv)};
        *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * g) = pk;
      }
    if (h == 0) {
      const float lse = l_tot > 0.0f ? (m_run[qb] + log2f(l_tot)) * kLn2 : p.empty_lse;
      p.lse[(int64_t)head * p.lse_head_stride + (int64_t)o_slot * p.lse_slot_stride + q_local[qb]] = lse;
    }
  }
}

// The kernel is persistent: the launch has (at most) as many workgroups as the device holds at
// once and each keeps taking the next work item of its XCD until none is left.  A grid of one
// workgroup per item loses a tenth of the device to dispatch: workgroup ids are dealt to the 8
// XCDs strictly in turn, so an XCD with a free slot waits until every XCD before it in the turn
// has taken its workgroup (13 us between two workgroups of a CU slot on average, against 100 us
// of work), and the last, unevenly long items leave slots empty at the end.
//
// Workgroup b sits on XCD b % 8.  The items that stream the same K/V (the query tiles and grouped
// heads of a row, `xcd_group` of them with consecutive ids) stay on one XCD: stream s belongs to
// XCD s % 8, and an XCD's items are handed out in id order (rows come longest first) through one
// ticket counter per XCD in `p.tickets`, which a one-wave kernel zeroes on the stream just before.
template <int DTYPE, int D, int QB>
__global__ __launch_bounds__(kFwdThreads, QB == 1 ? 2 : 1) void attn_fwd_kernel(const AttnFwdParams p) {
  __shared__ int ticket_lds;
  const int x = blockIdx.x % kNumXcd;
  const int64_t n_streams = (p.n_items + p.xcd_group - 1) / p.xcd_group;
  const int64_t n_x = n_streams > x ? (n_streams - x + kNumXcd - 1) / kNumXcd * p.xcd_group : 0;  // items of this XCD
  while (true) {
    if (threadIdx.x == 0) ticket_lds = atomicAdd(&p.tickets[x], 1);
    __syncthreads();
    const int i = __builtin_amdgcn_readfirstlane(ticket_lds);
    if (i >= n_x) break;
    const int64_t item = (x + kNumXcd * (int64_t)(i / p.xcd_group)) * p.xcd_group + i % p.xcd_group;
    if (item < p.n_items) attn_fwd_item<DTYPE, D, QB>(p, (int)item);
    __syncthreads();  // the next item reuses the LDS tables and tiles, and the ticket's place
  }
}

__global__ void attn_fwd_reset_tickets_kernel(int* tickets) {
  if (threadIdx.x < kNumXcd) tickets[threadIdx.x] = 0;
}

}  // namespace dcp

using namespace dcp;

extern "C" size_t dcp_attn_fwd_workspace_bytes(void) { return 16 * sizeof(int32_t); }

extern "C" int dcp_attn_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                            const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_kv,
                            const int32_t* attn_range, int n_ranges, const int32_t* q_block_table,
                            const int32_t* kv_block_table, const int32_t* out_block_table,
                            const int32_t* row_order, int batch, int max_kv_blocks, int total_q,
                            int block_size, int n_heads_q, int n_heads_kv, int head_dim,
                            int64_t kv_slot_stride, int64_t kv_token_stride, int n_out_slots,
                            float softmax_scale, int dtype, void* workspace, size_t workspace_bytes,
                            void* stream) {
  DCP_REQUIRE(batch == 0 || n_out_slots > 0, "attn_fwd: empty block tables");
  const int64_t slot = (int64_t)block_size * n_heads_q * head_dim;
  return dcp_attn_fwd_strided(q, k, v, out, lse, cu_seqlens_q, cu_seqlens_kv, attn_range, n_ranges, q_block_table,
                              kv_block_table, out_block_table, row_order, batch, max_kv_blocks, total_q, block_size,
                              n_heads_q, n_heads_kv, head_dim, kv_slot_stride, kv_token_stride, slot, slot,
                              (int64_t)n_out_slots * block_size, block_size, 0, softmax_scale, dtype, workspace,
                              workspace_bytes, stream);
}

extern "C" int dcp_attn_fwd_strided(const void* q, const void* k, const void* v, void* out, float* lse,
                                    const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_kv,
                                    const int32_t* attn_range, int n_ranges, const int32_t* q_block_table,
                                    const int32_t* kv_block_table, const int32_t* out_block_table,
                                    const int32_t* row_order, int batch, int max_kv_blocks, int total_q,
                                    int block_size, int n_heads_q, int n_heads_kv, int head_dim,
                                    int64_t kv_slot_stride, int64_t kv_token_stride, int64_t q_slot_stride,
                                    int64_t out_slot_stride, int64_t lse_head_stride, int64_t lse_slot_stride,
                                    int merged_form, float softmax_scale, int dtype, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  if (dtype != DCP_DTYPE_BF16 && dtype != DCP_DTYPE_FP16)
    return fail(DCP_ERR_UNSUPPORTED, "attn_fwd: dtype %d unsupported (bf16 and fp16 only)", dtype);
  if (head_dim != 64 && head_dim != 128)
    return fail(DCP_ERR_UNSUPPORTED, "attn_fwd: head_dim %d unsupported (64 or 128)", head_dim);
  DCP_REQUIRE(n_ranges == 1 || n_ranges == 2, "attn_fwd: n_ranges must be 1 or 2, got %d", n_ranges);
  DCP_REQUIRE(batch >= 0 && total_q >= 0, "attn_fwd: negative size");
  DCP_REQUIRE(softmax_scale > 0.0f, "attn_fwd: softmax_scale must be positive");
  if (batch == 0) return DCP_OK;
  DCP_REQUIRE(block_size > 0 && block_size % kFwdBN == 0,
              "attn_fwd: block_size %d must be a positive multiple of %d", block_size, kFwdBN);
  DCP_REQUIRE(n_heads_q > 0 && n_heads_kv > 0 && n_heads_q % n_heads_kv == 0,
              "attn_fwd: n_heads_q %d must be a multiple of n_heads_kv %d", n_heads_q, n_heads_kv);
  DCP_REQUIRE(max_kv_blocks > 0, "attn_fwd: empty block tables");
  DCP_REQUIRE(kv_token_stride % 8 == 0 && kv_slot_stride % 8 == 0 && q_slot_stride % 8 == 0 && out_slot_stride % 4 == 0,
              "attn_fwd: q, k, v strides must be multiples of 8 elements (out: 4)");
  DCP_REQUIRE(q_slot_stride > 0 && out_slot_stride > 0 && lse_head_stride > 0 && lse_slot_stride > 0,
              "attn_fwd: table strides must be positive");
  DCP_REQUIRE(q && k && v && out && lse && cu_seqlens_q && cu_seqlens_kv && attn_range &&
                  q_block_table && kv_block_table && out_block_table,
              "attn_fwd: null argument");
  DCP_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
                reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out)) & 15) == 0,
              "attn_fwd: q/k/v/out must be 16-byte aligned");
  DCP_REQUIRE(workspace && (reinterpret_cast<uintptr_t>(workspace) & 3) == 0 &&
                  workspace_bytes >= dcp_attn_fwd_workspace_bytes(),
              "attn_fwd: workspace of %zu bytes is missing or smaller than the %zu needed", workspace_bytes,
              dcp_attn_fwd_workspace_bytes());
  AttnFwdParams p;
  p.q = q;
  p.k = k;
  p.v = v;
  p.out = out;
  p.lse = lse;
  p.cu_seqlens_q = cu_seqlens_q;
  p.cu_seqlens_kv = cu_seqlens_kv;
  p.attn_range = attn_range;
  p.q_block_table = q_block_table;
  p.kv_block_table = kv_block_table;
  p.out_block_table = out_block_table;
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
  p.n_out_slots = 0;
  p.q_slot_stride = q_slot_stride;
  p.out_slot_stride = out_slot_stride;
  p.lse_head_stride = lse_head_stride;
  p.lse_slot_stride = lse_slot_stride;
  p.empty_lse = merged_form ? -1.0f : INFINITY;
  // One 32-row query block per wave.  (Two per wave do not pay with this compiler: it cannot
  // keep the O^T accumulators in the AGPR half of the register file without copies and spills.)
  const int bm = 128;
  p.q_tiles_per_row = (block_size + bm - 1) / bm;
  p.scale_log2 = softmax_scale * kLog2e;
  p.n_items = (int64_t)batch * n_heads_q * p.q_tiles_per_row;
  p.xcd_group = p.q_tiles_per_row * (n_heads_q / n_heads_kv);
  DCP_REQUIRE(p.n_items < ((int64_t)1 << 31), "attn_fwd: too many work items");
  // as many workgroups as the device holds at once (two per CU), a multiple of the XCD count
  const int64_t n_wg = std::min<int64_t>(xcd_grid_size(p.n_items, 1), xcd_grid_size(2 * (int64_t)device_cu_count(), 1));
  p.tickets = reinterpret_cast<int*>(workspace);
  dim3 grid((unsigned)n_wg), block(kFwdThreads);
  hipLaunchKernelGGL(attn_fwd_reset_tickets_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, p.tickets);
  KernelTimer timer("attn_fwd_kernel", stream);
#define DCP_FWD(DT, HD) \
  hipLaunchKernelGGL((attn_fwd_kernel<DT, HD, 1>), grid, block, 0, (hipStream_t)stream, p)
  if (dtype == DCP_DTYPE_BF16) {
    if (head_dim == 128) DCP_FWD(DCP_DTYPE_BF16, 128);
    else DCP_FWD(DCP_DTYPE_BF16, 64);
  } else {
    if (head_dim == 128) DCP_FWD(DCP_DTYPE_FP16, 128);
    else DCP_FWD(DCP_DTYPE_FP16, 64);
  }
#undef DCP_FWD
  return check_launch("attn_fwd_kernel");
}
