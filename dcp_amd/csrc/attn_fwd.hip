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
  const int32_t* kv_table = p.kv_block_table + (int64_t)b * p.max_kv_blocks;

  // loop-invariant per-lane pieces of every address used in the key loop
  uint32_t k_goff[KTile::LPW], v_goff[VTile::LPW];
  KTile::lane_offsets(k_goff, p.kv_token_stride, w, lane);
  VTile::lane_offsets(v_goff, p.kv_token_stride, w, lane);
  const int k_rd = KTile::row_base(c, h);
  const int v_rd = VTile::col_base(lane, true);

  // fill one stage with key tile `kt`
  auto fetch = [&](int kt, uint16_t* k_dst, uint16_t* v_dst) {
    const int k0 = kt * BN;
    const int blk = k0 / p.block_size;
    const int64_t off = (int64_t)kv_table[blk] * p.kv_slot_stride +
                        (int64_t)(k0 - blk * p.block_size) * p.kv_token_stride;
    KTile::load_async(k_dst, kg + off, k_goff, w);
    VTile::load_async(v_dst, vg + off, v_goff, w);
  };

  // one key tile out of a filled stage
  auto compute = [&](int kt, const uint16_t* k_lds, const uint16_t* v_lds) {
    const int k0 = kt * BN;
    const bool wave_active = (k0 < w_hi0 && k0 + BN > w_lo0) || (k0 < w_hi1 && k0 + BN > w_lo1);
    if (!wave_active) return;

    // ---- S^T = K Q^T -------------------------------------------------------------
    // The range mask enters as the accumulator's initial value: 0 where the row may
    // look, -inf where it may not.  A tile inside every row's range of the wave (the
    // common case) starts from the constant 0; everything after the first product is
    // the same code for both cases.
    const bool unmasked = (core_lo0 <= k0 && k0 + BN <= core_hi0) || (core_lo1 <= k0 && k0 + BN <= core_hi1);
    f32x16 s_acc[2];
    u32x4 ka[2][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      ka[0][ks] = KTile::read_row(k_lds, k_rd, 0, ks);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      ka[1][ks] = KTile::read_row(k_lds, k_rd, 1, ks);
    if (unmasked) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s_acc[nt][i] = 0.0f;
        s_acc[nt] = mfma_32x32x16<DTYPE>(ka[nt][0], qreg[0], s_acc[nt]);
      }
    } else {
      const int kb = k0 + 4 * h;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
          s_acc[nt][i] = rng.contains(kb + nt * 32 + 8 * (i / 4) + (i % 4)) ? 0.0f : -INFINITY;
        s_acc[nt] = mfma_32x32x16<DTYPE>(ka[nt][0], qreg[0], s_acc[nt]);
      }
    }
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int ks = 1; ks < KS; ++ks) s_acc[nt] = mfma_32x32x16<DTYPE>(ka[nt][ks], qreg[ks], s_acc[nt]);
    // first V^T operands: their latency hides under the softmax arithmetic
    u32x4 va[2][4];
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) va[0][s2] = VTile::template read_col<true>(v_lds, v_rd, s2, 0);

    // ---- online softmax (log2 domain) -----------------------------------------
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s_acc[nt][i]);
    mx *= p.scale_log2;  // -inf stays -inf (scale > 0)
    mx = fmaxf(mx, xor32(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
    if (__any(m_new > m_run)) {
      const float alpha = fast_exp2(m_run - m_use);  // m_run = -inf -> 0
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[dt][i] *= alpha;
    }
    m_run = m_new;
    u32x4 pb[4];
    float lsum = 0.0f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        float e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          e[j] = fast_exp2(fmaf(s_acc[nt][g * 8 + j], p.scale_log2, -m_use));
          lsum += e[j];
        }
        u32x4 packed = {pack2<DTYPE>(e[0], e[1]), pack2<DTYPE>(e[2], e[3]), pack2<DTYPE>(e[4], e[5]),
                        pack2<DTYPE>(e[6], e[7])};
        pb[nt * 2 + g] = packed;
      }
    l_run += lsum;

    // ---- O^T += V^T P^T: V^T comes out of the row-major V tile by transpose loads -----
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (dt + 1 < DT) {
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2)
          va[(dt + 1) & 1][s2] = VTile::template read_col<true>(v_lds, v_rd, s2, dt + 1);
      }
#pragma unroll
      for (int s2 = 0; s2 < 4; ++s2) o_acc[dt] = mfma_32x32x16<DTYPE>(va[dt & 1][s2], pb[s2], o_acc[dt]);
    }
  };

  // ---- key loop: tile i+1 streams into the other stage while tile i is used ----------
  if (n_tiles > 0) fetch(runs.tile(0), k_lds0, v_lds0);
  for (int i = 0; i < n_tiles; i += 2) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // stage 0 is filled; nobody reads stage 1 any more
    if (i + 1 < n_tiles) fetch(runs.tile(i + 1), k_lds1, v_lds1);
    compute(runs.tile(i), k_lds0, v_lds0);
    if (i + 1 >= n_tiles) break;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // stage 1 is filled; nobody reads stage 0 any more
    if (i + 2 < n_tiles) fetch(runs.tile(i + 2), k_lds0, v_lds0);
    compute(runs.tile(i + 1), k_lds1, v_lds1);
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
