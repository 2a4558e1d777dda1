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
  int q_tiles_per_row;
  int xcd_group;     // work items per shared K/V stream
  int64_t n_items;   // batch * n_heads_q * q_tiles_per_row
  float scale_log2;  // softmax_scale * log2(e)
};

constexpr int kFwdBM = 128;
constexpr int kFwdBN = 64;
constexpr int kFwdThreads = 256;

template <int DTYPE, int D>
__global__ __launch_bounds__(kFwdThreads, 2) void attn_fwd_kernel(const AttnFwdParams p) {
  constexpr int BN = kFwdBN;
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
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int c = lane & 31;
  const int h = lane >> 5;

  // ---- which (row, head, q tile) ----------------------------------------
  // the query tiles and grouped heads of a row share its K/V: keep them on one XCD
  int wg = xcd_logical_id(blockIdx.x, p.xcd_group, p.n_items);
  if (wg < 0) return;
  const int qt = wg % p.q_tiles_per_row;
  wg /= p.q_tiles_per_row;
  const int head = wg % p.n_heads_q;
  const int bi = wg / p.n_heads_q;
  const int b = p.row_order ? p.row_order[bi] : bi;
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - p.cu_seqlens_kv[b];
  if (qt * kFwdBM >= seqlen_q) return;
  const int kv_head = head / (p.n_heads_q / p.n_heads_kv);
  const int64_t q_row_stride = (int64_t)p.n_heads_q * D;

  const int q_local = qt * kFwdBM + w * 32 + c;
  const bool q_valid = q_local < seqlen_q;

  // ---- Q fragment (B operand of S^T) ---------------------------------------
  u32x4 qreg[KS];
  {
    const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) +
                         ((int64_t)p.q_block_table[b] * p.block_size + q_local) * q_row_stride +
                         (int64_t)head * D + h * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 z = {0, 0, 0, 0};
      qreg[ks] = q_valid ? *reinterpret_cast<const u32x4*>(qp + ks * 16) : z;
    }
  }

  // ---- this lane's query row: ranges ---------------------------------------
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
  // hull (what any row of the wave can see) and core (what every row sees)
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
  const TileRuns runs(g_lo0, g_hi0, g_lo1, g_hi1, BN);
  const int n_tiles = runs.count();

  // ---- running state ---------------------------------------------------------
  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o_acc[dt][i] = 0.0f;
  float m_run = -INFINITY;  // running max, log2 domain
  float l_run = 0.0f;       // this half-wave's partial row sum

  const uint16_t* kg = reinterpret_cast<const uint16_t*>(p.k) + (int64_t)kv_head * D;
  const uint16_t* vg = reinterpret_cast<const uint16_t*>(p.v) + (int64_t)kv_head * D;

  // loop-invariant per-lane pieces of every address used in the key loop
  uint32_t k_goff[KTile::LPW], v_goff[VTile::LPW];
  KTile::lane_offsets(k_goff, p.kv_token_stride, w, lane);
  VTile::lane_offsets(v_goff, p.kv_token_stride, w, lane);
  const int k_rd = KTile::row_base(c, h);
  const int v_rd = VTile::col_base(lane, true);

  // The cursor runs two tiles ahead of the tile being exponentiated: it names the K
  // tile to request next.  V of a tile is requested one iteration after its K, from the
  // offset remembered then.
  const int tiles_per_block = p.block_size / BN;
  const int64_t tile_stride = (int64_t)BN * p.kv_token_stride;
  TileCursor cursor;
  auto cursor_next = [&]() {
    if (cursor.index + 1 < n_tiles) cursor.advance(runs, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
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

  // MFMA i of S^T = K Q^T: key half i & 1, k-step i >> 1 (the two halves alternate so
  // that consecutive MFMAs are independent)
  auto k_operand = [&](const uint16_t* k_lds, int i) { return KTile::read_row(k_lds, k_rd, i & 1, i >> 1); };

  // S^T of tile i on its own.  The range mask enters as the accumulator's initial
  // value: 0 where the row may look, -inf where it may not.
  auto multiply_qk = [&](int tile, const uint16_t* k_lds, f32x16 (&s_out)[2]) {
    if (wave_sees_all(tile)) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int e = 0; e < 16; ++e) s_out[nt][e] = 0.0f;
    } else {
      const int kb = tile * BN + 4 * h;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          s_out[nt][e] = rng.contains(kb + nt * 32 + 8 * (e / 4) + (e % 4)) ? 0.0f : -INFINITY;
    }
    constexpr int N = 2 * KS, AHEAD = 3;
    u32x4 ka[4];
#pragma unroll
    for (int i2 = 0; i2 < AHEAD; ++i2) ka[i2] = k_operand(k_lds, i2);
#pragma unroll
    for (int i2 = 0; i2 < N; ++i2) {
      if (i2 + AHEAD < N) ka[(i2 + AHEAD) & 3] = k_operand(k_lds, i2 + AHEAD);
      s_out[i2 & 1] = mfma_32x32x16<DTYPE>(ka[i2 & 3], qreg[i2 >> 1], s_out[i2 & 1]);
      __builtin_amdgcn_sched_barrier(0);  // keeps the operand reads from being hoisted into more registers
    }
  };

  // ---- online softmax (log2 domain), in pieces so that it can be interleaved ----
  u32x4 pb[4];          // P^T of the current tile, packed: the B operand of O^T += V^T P^T
  float alpha = 1.0f;   // pending rescale of O^T (applied before the tile's P^T is multiplied in)
  bool rescale = false;
  float m_use = 0.0f, lsum = 0.0f;
  auto softmax_max = [&](const f32x16 (&sc)[2]) {
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[nt][e]);
    mx *= p.scale_log2;  // -inf stays -inf (scale > 0)
    mx = fmaxf(mx, xor32(mx));
    const float m_new = fmaxf(m_run, mx);
    m_use = (m_new == -INFINITY) ? 0.0f : m_new;
    rescale = __any(m_new > m_run);
    alpha = fast_exp2(m_run - m_use);  // m_run = -inf -> 0; 1 where the max did not move
    l_run *= alpha;
    m_run = m_new;
    lsum = 0.0f;
  };
  // elements 2c, 2c+1 of the 32 this lane holds
  auto softmax_pair = [&](const f32x16 (&sc)[2], int c2) {
    const int nt = c2 >> 3, e = (c2 & 7) * 2;
    const float e0 = fast_exp2(fmaf(sc[nt][e], p.scale_log2, -m_use));
    const float e1 = fast_exp2(fmaf(sc[nt][e + 1], p.scale_log2, -m_use));
    lsum += e0 + e1;
    pb[nt * 2 + (e >> 3)][(e & 7) >> 1] = pack2<DTYPE>(e0, e1);
  };
  auto apply_rescale = [&]() {
    if (rescale) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[dt][e] *= alpha;
    }
  };
  auto softmax = [&](const f32x16 (&sc)[2]) {
    softmax_max(sc);
#pragma unroll
    for (int c2 = 0; c2 < 16; ++c2) softmax_pair(sc, c2);
    l_run += lsum;
  };

  // S^T of the next tile and the softmax of the current one in one instruction stream:
  // every MFMA is followed by its share of the softmax arithmetic, so that the matrix
  // pipe and the vector ALU of the SIMD are busy at the same time.  Operands are read
  // three MFMAs ahead.
  auto multiply_qk_with_softmax = [&](const uint16_t* k_lds, f32x16 (&s_out)[2], const f32x16 (&sc)[2]) {
    constexpr int N = 2 * KS;     // MFMAs
    constexpr int AHEAD = 3;
    constexpr int FIRST = N >= 8 ? 3 : 1;  // MFMAs that carry the max; the pairs follow
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_out[nt][e] = 0.0f;
    u32x4 ka[4];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ka[i] = k_operand(k_lds, i);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (i + AHEAD < N) ka[(i + AHEAD) & 3] = k_operand(k_lds, i + AHEAD);
      s_out[i & 1] = mfma_32x32x16<DTYPE>(ka[i & 3], qreg[i >> 1], s_out[i & 1]);
      if (i == 0) softmax_max(sc);
      if (i >= FIRST) {
        const int lo = (i - FIRST) * 16 / (N - FIRST), hi = (i + 1 - FIRST) * 16 / (N - FIRST);
#pragma unroll
        for (int c2 = lo; c2 < hi; ++c2) softmax_pair(sc, c2);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    l_run += lsum;
  };

  // O^T += V^T P^T: V^T comes out of the row-major V tile by transpose loads, read
  // two MFMAs ahead; consecutive MFMAs go to different 32-row tiles of O^T
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
      o_acc[i % DT] = mfma_32x32x16<DTYPE>(va[i & 3], pb[i / DT], o_acc[i % DT]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- key loop --------------------------------------------------------------------
  // Iteration j multiplies S^T of tile j+1 while it exponentiates tile j, then adds
  // tile j to O^T.  K tile j+1 and V tile j are in LDS by then; K tile j+2 and V tile
  // j+1 stream into the stages that K tile j and V tile j-1 have left.
  f32x16 s_a[2], s_b[2];
  int tile_cur = 0, tile_nxt = 0;  // key tile numbers of list entries j and j+1
  int64_t v_off = 0;               // offset of list entry j+1 (its V is requested in iteration j)
  auto iteration = [&](int j, f32x16 (&s_cur)[2], f32x16 (&s_nxt)[2], const uint16_t* k_nxt, uint32_t k_fill,
                       const uint16_t* v_cur, uint32_t v_fill) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // K tile j+1 and V tile j are filled; nobody reads K tile j or V tile j-1 any more
    if (j + 2 < n_tiles) KTile::load_async(k_fill, kg + cursor.off, k_goff, w);
    if (j + 1 < n_tiles) VTile::load_async(v_fill, vg + v_off, v_goff, w);
    const bool cur = wave_sees(tile_cur), nxt = j + 1 < n_tiles && wave_sees(tile_nxt);
    if (cur && nxt && wave_sees_all(tile_nxt)) {
      multiply_qk_with_softmax(k_nxt, s_nxt, s_cur);
    } else {
      if (nxt) multiply_qk(tile_nxt, k_nxt, s_nxt);
      if (cur) softmax(s_cur);
    }
    if (cur) {
      apply_rescale();
      multiply_pv(v_cur);
    }
    tile_cur = tile_nxt;
    tile_nxt = cursor.tile;
    v_off = cursor.off;
    cursor_next();
  };
  if (n_tiles > 0) {
    cursor.seek(runs, 0, tiles_per_block, slot_lds, kv_table, p.kv_slot_stride, tile_stride);
    tile_cur = cursor.tile;
    KTile::load_async(k_at0, kg + cursor.off, k_goff, w);
    VTile::load_async(v_at0, vg + cursor.off, v_goff, w);
    cursor_next();
    tile_nxt = cursor.tile;
    v_off = cursor.off;
    if (n_tiles > 1) KTile::load_async(k_at1, kg + cursor.off, k_goff, w);
    cursor_next();
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (wave_sees(tile_cur)) multiply_qk(tile_cur, k_lds0, s_a);
    for (int j = 0; j < n_tiles; j += 2) {
      iteration(j, s_a, s_b, k_lds1, k_at0, v_lds0, v_at1);
      if (j + 1 >= n_tiles) break;
      iteration(j + 1, s_b, s_a, k_lds0, k_at1, v_lds1, v_at0);
    }
  }

  // ---- epilogue ------------------------------------------------------------------
  const float l_tot = l_run + xor32(l_run);
  if (!q_valid) return;
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  const int o_slot = p.out_block_table[b];
  uint16_t* op = reinterpret_cast<uint16_t*>(p.out) +
                 ((int64_t)o_slot * p.block_size + q_local) * q_row_stride + (int64_t)head * D + 4 * h;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 pk = {pack2<DTYPE>(o_acc[dt][4 * g] * inv, o_acc[dt][4 * g + 1] * inv),
                  pack2<DTYPE>(o_acc[dt][4 * g + 2] * inv, o_acc[dt][4 * g + 3] * inv)};
      *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * g) = pk;
    }
  if (h == 0) {
    const float lse = l_tot > 0.0f ? (m_run + log2f(l_tot)) * kLn2 : INFINITY;
    p.lse[((int64_t)head * p.n_out_slots + o_slot) * p.block_size + q_local] = lse;
  }
}

}  // namespace dcp

using namespace dcp;

extern "C" int dcp_attn_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                            const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_kv,
                            const int32_t* attn_range, int n_ranges, const int32_t* q_block_table,
                            const int32_t* kv_block_table, const int32_t* out_block_table,
                            const int32_t* row_order, int batch, int max_kv_blocks, int total_q,
                            int block_size, int n_heads_q, int n_heads_kv, int head_dim,
                            int64_t kv_slot_stride, int64_t kv_token_stride, int n_out_slots,
                            float softmax_scale, int dtype, void* stream) {
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
  DCP_REQUIRE(max_kv_blocks > 0 && n_out_slots > 0, "attn_fwd: empty block tables");
  DCP_REQUIRE(kv_token_stride % 8 == 0 && kv_slot_stride % 8 == 0,
              "attn_fwd: kv strides must be multiples of 8 elements");
  DCP_REQUIRE(q && k && v && out && lse && cu_seqlens_q && cu_seqlens_kv && attn_range &&
                  q_block_table && kv_block_table && out_block_table,
              "attn_fwd: null argument");
  DCP_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
                reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out)) & 15) == 0,
              "attn_fwd: q/k/v/out must be 16-byte aligned");
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
  p.n_out_slots = n_out_slots;
  p.q_tiles_per_row = (block_size + kFwdBM - 1) / kFwdBM;
  p.scale_log2 = softmax_scale * kLog2e;
  p.n_items = (int64_t)batch * n_heads_q * p.q_tiles_per_row;
  p.xcd_group = p.q_tiles_per_row * (n_heads_q / n_heads_kv);
  const int64_t n_wg = xcd_grid_size(p.n_items, p.xcd_group);
  DCP_REQUIRE(n_wg < ((int64_t)1 << 31), "attn_fwd: grid too large");
  dim3 grid((unsigned)n_wg), block(kFwdThreads);
  KernelTimer timer("attn_fwd_kernel", stream);
#define DCP_FWD(DT, HD) \
  hipLaunchKernelGGL((attn_fwd_kernel<DT, HD>), grid, block, 0, (hipStream_t)stream, p)
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
