// Range-masked paged attention backward for gfx950.
//
// Three small kernels and one big one per call:
//
//   bwd_prep_kernel      delta[q, h] = sum_d dO*O; zero the fp32 dQ accumulator
//   bwd_tile_hull_kernel per (row, 64-query tile): hull and core of the rows'
//                        key ranges, so the main kernel can skip / unmask tiles
//   attn_bwd_kernel      one workgroup per (row, 64-key tile, kv head): loops
//                        over the q heads of the kv head's group and the
//                        64-query tiles of the row, keeps dK^T and dV^T of its
//                        keys in registers, adds its dQ contribution to the
//                        fp32 accumulator with atomics
//   bwd_dq_store_kernel  dQ = scale * accumulator -> storage type, paged
//
// Main kernel, per (64 q) x (64 kv) tile, wave w = (qi, ki) owns the 32x32
// sub-tile (queries 32qi.., keys 32ki..):
//
//   S  = Q K^T          A = Q rows from LDS,   B = K held in registers
//   dP = dO V^T         A = dO rows from LDS,  B = V held in registers
//   P  = exp2(S*c - lse), dS = P * (dP - delta)      (accumulator layout:
//                                                     lane = key, regs = queries)
//   dV^T += dO^T P      A = dO^T from LDS, B = P straight from registers
//   dK^T += Q^T dS      A = Q^T from LDS,  B = dS straight from registers
//   dS -> LDS, then wave w computes the 32-column slice w of
//   dQ = dS K           A = dS rows from LDS,  B = K^T slice held in registers
//
// dK/dV of a key never leave the workgroup's registers until the end, so the
// per-(row, kv block) private dKV blocks of the plan need no atomics and are
// written whole (zeros where no query of the row attends).
#include <hip/amd_detail/amd_hip_unsafe_atomics.h>
#include <math.h>

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
  float* dq_accum;   // [total_q, H, D]
  float* delta;      // [total_q, H]
  int32_t* hull;     // [batch * q_tiles_per_row, 8]
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
  int q_tiles_per_row;   // ceil(block_size / 64)
  int kv_tiles_per_row;  // max_kv_blocks * block_size / 64
  float scale;
  float scale_log2;
};

constexpr int kBwdBM = 64;
constexpr int kBwdBN = 64;
constexpr int kBwdThreads = 256;

// ---------------------------------------------------------------------------
// delta and accumulator clear.  LPR lanes per (token, head) row, 8 elements
// each.  grid: (batch, row chunks)
// ---------------------------------------------------------------------------
template <int DTYPE, int D>
__global__ __launch_bounds__(256) void bwd_prep_kernel(const AttnBwdParams p) {
  constexpr int LPR = D / 8;
  constexpr int ROWS = 256 / LPR;
  const int b = blockIdx.x;
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int row = blockIdx.y * ROWS + threadIdx.x / LPR;
  const int g = threadIdx.x % LPR;
  const int t = row / p.n_heads_q;
  const int hd = row - t * p.n_heads_q;
  if (t >= seqlen_q) return;  // whole LPR-lane group leaves together
  const int64_t off = (((int64_t)p.out_block_table[b] * p.block_size + t) * p.n_heads_q + hd) * D + g * 8;
  const u32x4 o = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.out) + off);
  const u32x4 d = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.dout) + off);
  float acc = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    acc += Elem<DTYPE>::load((uint16_t)(o[i] & 0xffffu)) * Elem<DTYPE>::load((uint16_t)(d[i] & 0xffffu));
    acc += Elem<DTYPE>::load((uint16_t)(o[i] >> 16)) * Elem<DTYPE>::load((uint16_t)(d[i] >> 16));
  }
#pragma unroll
  for (int o2 = LPR / 2; o2 > 0; o2 >>= 1) acc += __shfl_xor(acc, o2);
  const int64_t qrow = ((int64_t)(q_begin + t) * p.n_heads_q + hd);
  if (g == 0) p.delta[qrow] = acc;
  f32x4 z = {0.f, 0.f, 0.f, 0.f};
  f32x4* acc_row_ptr = reinterpret_cast<f32x4*>(p.dq_accum + qrow * D + g * 8);
  acc_row_ptr[0] = z;
  acc_row_ptr[1] = z;
}

// One wave per (row, 64-query tile).  hull[0..3] = lo0, hi0, lo1, hi1 over
// rows with a non-empty range; hull[4..7] = the intersection (core) of the
// rows' ranges, empty as soon as one row has an empty range.
__global__ __launch_bounds__(64) void bwd_tile_hull_kernel(const AttnBwdParams p) {
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
// main kernel
// ---------------------------------------------------------------------------
template <int DTYPE, int D>
__global__ __launch_bounds__(kBwdThreads) void attn_bwd_kernel(const AttnBwdParams p) {
  constexpr int BM = kBwdBM, BN = kBwdBN;
  constexpr int KS = D / 16;          // k-steps over the head dim
  constexpr int DT = D / 32;          // 32-row tiles of dK^T / dV^T
  constexpr int ROW_STRIDE = D + 8;   // q_lds / do_lds rows (elements)
  constexpr int T_STRIDE = BM + 8;    // qt_lds / dot_lds / ds_lds rows (elements)
  constexpr int CH = D / 8;
  constexpr int UNITS = (BM / 4) * CH;  // (4 queries) x (8 dims) staging units
  constexpr int PASSES = (UNITS + kBwdThreads - 1) / kBwdThreads;
  static_assert(UNITS % kBwdThreads == 0 || UNITS < kBwdThreads, "staging map");

  __shared__ __attribute__((aligned(16))) uint16_t q_lds[BM * ROW_STRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t do_lds[BM * ROW_STRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t qt_lds[D * T_STRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t dot_lds[D * T_STRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t ds_lds[BM * T_STRIDE];
  __shared__ __attribute__((aligned(16))) int rng_lds[BM * 4];
  __shared__ __attribute__((aligned(16))) float lse_lds[BM];
  __shared__ __attribute__((aligned(16))) float delta_lds[BM];

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int c = lane & 31;
  const int h = lane >> 5;
  const int qi = w >> 1;  // query sub-tile of this wave
  const int ki = w & 1;   // key sub-tile of this wave

  // ---- which (row, kv head, key tile) ------------------------------------------
  int wg = blockIdx.x;
  const int kt = wg % p.kv_tiles_per_row;
  wg /= p.kv_tiles_per_row;
  const int kv_head = wg % p.n_heads_kv;
  const int bi = wg / p.n_heads_kv;
  const int b = p.row_order ? p.row_order[bi] : bi;
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int seqlen_kv = p.cu_seqlens_kv[b + 1] - p.cu_seqlens_kv[b];
  const int k0 = kt * BN;
  if (k0 >= seqlen_kv) return;
  const int blk = k0 / p.block_size;
  const int tok0 = k0 - blk * p.block_size;
  const int group = p.n_heads_q / p.n_heads_kv;
  const int64_t q_row_stride = (int64_t)p.n_heads_q * D;
  const int q_slot = p.q_block_table[b];
  const int o_slot = p.out_block_table[b];
  const int n_q_tiles = (seqlen_q + BM - 1) / BM;

  // ---- K, V of this wave's 32 keys as B operands (lane = key, slots = dims) ------
  u32x4 kreg[KS], vreg[KS];
  {
    const int64_t off = (int64_t)p.kv_block_table[(int64_t)b * p.max_kv_blocks + blk] * p.kv_slot_stride +
                        (int64_t)(tok0 + ki * 32 + c) * p.kv_token_stride + (int64_t)kv_head * D + h * 8;
    const uint16_t* kp = reinterpret_cast<const uint16_t*>(p.k) + off;
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.v) + off;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kreg[ks] = *reinterpret_cast<const u32x4*>(kp + ks * 16);
      vreg[ks] = *reinterpret_cast<const u32x4*>(vp + ks * 16);
    }
  }
  // ---- K^T slice for dQ: lane = dim (32w + c) of the slice, slots = keys ---------
  constexpr int DQ_SLICES = D / 32;      // 32-wide dQ column slices
  constexpr int DQ_PER_WAVE = DQ_SLICES / 4 > 0 ? DQ_SLICES / 4 : 1;
  const bool dq_wave = w < DQ_SLICES;    // D = 64: only waves 0,1 own a slice
  u32x4 ktreg[DQ_PER_WAVE][BN / 16];
  if (dq_wave) {
#pragma unroll
    for (int sl = 0; sl < DQ_PER_WAVE; ++sl) {
      const int dim = (w * DQ_PER_WAVE + sl) * 32 + c;
      const uint16_t* kp = reinterpret_cast<const uint16_t*>(p.k) +
                           (int64_t)p.kv_block_table[(int64_t)b * p.max_kv_blocks + blk] * p.kv_slot_stride +
                           (int64_t)tok0 * p.kv_token_stride + (int64_t)kv_head * D + dim;
#pragma unroll
      for (int s = 0; s < BN / 16; ++s) {
        uint32_t pk[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t lo = kp[(int64_t)(s * 16 + h * 8 + 2 * j) * p.kv_token_stride];
          const uint32_t hi = kp[(int64_t)(s * 16 + h * 8 + 2 * j + 1) * p.kv_token_stride];
          pk[j] = lo | (hi << 16);
        }
        u32x4 t = {pk[0], pk[1], pk[2], pk[3]};
        ktreg[sl][s] = t;
      }
    }
  }

  f32x16 dk_acc[DT], dv_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dk_acc[dt][i] = 0.0f;
      dv_acc[dt][i] = 0.0f;
    }

  const int32_t* hull_row = p.hull + (int64_t)b * p.q_tiles_per_row * 8;

  for (int hg = 0; hg < group; ++hg) {
    const int head = kv_head * group + hg;
    for (int qt = 0; qt < n_q_tiles; ++qt) {
      const int32_t* hu = hull_row + qt * 8;
      const int lo0 = hu[0], hi0 = hu[1], lo1 = hu[2], hi1 = hu[3];
      const bool active = (k0 < hi0 && k0 + BN > lo0) || (k0 < hi1 && k0 + BN > lo1);
      if (!active) continue;
      const bool unmasked = (hu[4] <= k0 && k0 + BN <= hu[5]) || (hu[6] <= k0 && k0 + BN <= hu[7]);

      // ---- stage Q and dO (row-major and transposed) ---------------------------------
      u32x4 qst[PASSES][4], dst[PASSES][4];
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) {
        const int u = ps * kBwdThreads + tid;
        if (u < UNITS) {
          const int qg = u % (BM / 4), dg = u / (BM / 4);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int ql = qt * BM + qg * 4 + r;
            u32x4 z = {0, 0, 0, 0};
            const bool ok = ql < seqlen_q;
            const int64_t qoff = ((int64_t)q_slot * p.block_size + ql) * q_row_stride + (int64_t)head * D + dg * 8;
            const int64_t ooff = ((int64_t)o_slot * p.block_size + ql) * q_row_stride + (int64_t)head * D + dg * 8;
            qst[ps][r] = ok ? *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.q) + qoff) : z;
            dst[ps][r] = ok ? *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.dout) + ooff) : z;
          }
        }
      }
      int4 my_rng = {0, 0, 0, 0};
      float my_lse = INFINITY, my_delta = 0.0f;
      if (tid < BM) {
        const int ql = qt * BM + tid;
        if (ql < seqlen_q) {
          const int32_t* r = p.attn_range + q_begin + ql;
          my_rng.x = r[0];
          my_rng.y = max(min(r[p.total_q], seqlen_kv) - my_rng.x, 0);
          if (p.n_ranges == 2) {
            my_rng.z = r[2 * (int64_t)p.total_q];
            my_rng.w = max(min(r[3 * (int64_t)p.total_q], seqlen_kv) - my_rng.z, 0);
          }
          my_lse = p.lse[((int64_t)head * p.n_out_slots + o_slot) * p.block_size + ql] * kLog2e;
          my_delta = p.delta[(int64_t)(q_begin + ql) * p.n_heads_q + head];
        }
      }
      __syncthreads();  // previous tile fully consumed
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) {
        const int u = ps * kBwdThreads + tid;
        if (u < UNITS) {
          const int qg = u % (BM / 4), dg = u / (BM / 4);
          const int pos = (qg / 4) * 16 + kslot_pos(qg % 4);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            *reinterpret_cast<u32x4*>(&q_lds[(qg * 4 + r) * ROW_STRIDE + dg * 8]) = qst[ps][r];
            *reinterpret_cast<u32x4*>(&do_lds[(qg * 4 + r) * ROW_STRIDE + dg * 8]) = dst[ps][r];
          }
#pragma unroll
          for (int m = 0; m < 4; ++m) {
            {
              const uint32_t a0 = qst[ps][0][m], a1 = qst[ps][1][m], a2 = qst[ps][2][m], a3 = qst[ps][3][m];
              u32x2 even = {(a0 & 0xffffu) | (a1 << 16), (a2 & 0xffffu) | (a3 << 16)};
              u32x2 odd = {(a0 >> 16) | (a1 & 0xffff0000u), (a2 >> 16) | (a3 & 0xffff0000u)};
              *reinterpret_cast<u32x2*>(&qt_lds[(dg * 8 + 2 * m) * T_STRIDE + pos]) = even;
              *reinterpret_cast<u32x2*>(&qt_lds[(dg * 8 + 2 * m + 1) * T_STRIDE + pos]) = odd;
            }
            {
              const uint32_t a0 = dst[ps][0][m], a1 = dst[ps][1][m], a2 = dst[ps][2][m], a3 = dst[ps][3][m];
              u32x2 even = {(a0 & 0xffffu) | (a1 << 16), (a2 & 0xffffu) | (a3 << 16)};
              u32x2 odd = {(a0 >> 16) | (a1 & 0xffff0000u), (a2 >> 16) | (a3 & 0xffff0000u)};
              *reinterpret_cast<u32x2*>(&dot_lds[(dg * 8 + 2 * m) * T_STRIDE + pos]) = even;
              *reinterpret_cast<u32x2*>(&dot_lds[(dg * 8 + 2 * m + 1) * T_STRIDE + pos]) = odd;
            }
          }
        }
      }
      if (tid < BM) {
        *reinterpret_cast<int4*>(&rng_lds[tid * 4]) = my_rng;
        lse_lds[tid] = my_lse;
        delta_lds[tid] = my_delta;
      }
      __syncthreads();

      // ---- S = Q K^T, dP = dO V^T ------------------------------------------------------
      f32x16 s_acc, dp_acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s_acc[i] = 0.0f;
        dp_acc[i] = 0.0f;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4 aq = *reinterpret_cast<const u32x4*>(&q_lds[(qi * 32 + c) * ROW_STRIDE + ks * 16 + h * 8]);
        s_acc = mfma_32x32x16<DTYPE>(aq, kreg[ks], s_acc);
        const u32x4 ad = *reinterpret_cast<const u32x4*>(&do_lds[(qi * 32 + c) * ROW_STRIDE + ks * 16 + h * 8]);
        dp_acc = mfma_32x32x16<DTYPE>(ad, vreg[ks], dp_acc);
      }

      // ---- P and dS (lane = key k0 + 32ki + c; element i = query 32qi + acc_row(i,h)) ----
      u32x4 pb[2], dsb[2];
      const int kv = k0 + ki * 32 + c;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int qrow = qi * 32 + 8 * g + 4 * h;
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(&lse_lds[qrow]);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(&delta_lds[qrow]);
        float pv[4], dsv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float e = exp2f(fmaf(s_acc[4 * g + r], p.scale_log2, -l4[r]));
          float ds = e * (dp_acc[4 * g + r] - d4[r]);
          if (!unmasked) {
            const int4 rg = *reinterpret_cast<const int4*>(&rng_lds[(qrow + r) * 4]);
            const bool ok = ((unsigned)(kv - rg.x) < (unsigned)rg.y) | ((unsigned)(kv - rg.z) < (unsigned)rg.w);
            e = ok ? e : 0.0f;
            ds = ok ? ds : 0.0f;
          }
          pv[r] = e;
          dsv[r] = ds;
        }
        const uint32_t p01 = pack2<DTYPE>(pv[0], pv[1]), p23 = pack2<DTYPE>(pv[2], pv[3]);
        const uint32_t s01 = pack2<DTYPE>(dsv[0], dsv[1]), s23 = pack2<DTYPE>(dsv[2], dsv[3]);
        pb[g / 2][(g % 2) * 2] = p01;
        pb[g / 2][(g % 2) * 2 + 1] = p23;
        dsb[g / 2][(g % 2) * 2] = s01;
        dsb[g / 2][(g % 2) * 2 + 1] = s23;
        // dS row-major [q][kv] for the dQ product
        uint16_t* dsp = &ds_lds[qrow * T_STRIDE + ki * 32 + c];
        dsp[0] = (uint16_t)(s01 & 0xffffu);
        dsp[T_STRIDE] = (uint16_t)(s01 >> 16);
        dsp[2 * T_STRIDE] = (uint16_t)(s23 & 0xffffu);
        dsp[3 * T_STRIDE] = (uint16_t)(s23 >> 16);
      }

      // ---- dV^T += dO^T P, dK^T += Q^T dS (contraction over this wave's 32 queries) -------
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const int col = (qi * 2 + s) * 16 + h * 8;
          const u32x4 ad = *reinterpret_cast<const u32x4*>(&dot_lds[(dt * 32 + c) * T_STRIDE + col]);
          dv_acc[dt] = mfma_32x32x16<DTYPE>(ad, pb[s], dv_acc[dt]);
          const u32x4 aq = *reinterpret_cast<const u32x4*>(&qt_lds[(dt * 32 + c) * T_STRIDE + col]);
          dk_acc[dt] = mfma_32x32x16<DTYPE>(aq, dsb[s], dk_acc[dt]);
        }

      __syncthreads();  // dS of all four waves is in LDS

      // ---- dQ[:, slice] = dS K[:, slice] -----------------------------------------------------
      if (dq_wave) {
#pragma unroll
        for (int sl = 0; sl < DQ_PER_WAVE; ++sl) {
          const int dim = (w * DQ_PER_WAVE + sl) * 32 + c;
#pragma unroll
          for (int q2 = 0; q2 < 2; ++q2) {
            f32x16 dq_acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) dq_acc[i] = 0.0f;
#pragma unroll
            for (int s = 0; s < BN / 16; ++s) {
              const u32x4 a = *reinterpret_cast<const u32x4*>(&ds_lds[(q2 * 32 + c) * T_STRIDE + s * 16 + h * 8]);
              dq_acc = mfma_32x32x16<DTYPE>(a, ktreg[sl][s], dq_acc);
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int ql = qt * BM + q2 * 32 + acc_row(i, h);
              if (ql < seqlen_q)
                unsafeAtomicAdd(p.dq_accum + ((int64_t)(q_begin + ql) * p.n_heads_q + head) * D + dim, dq_acc[i]);
            }
          }
        }
      }
    }
  }

  // ---- combine the two query halves and store dK, dV -------------------------------------
  // wave (0, ki) finishes dK of keys 32ki.., wave (1, ki) finishes dV; each parks
  // the accumulator the other one needs in LDS (the staging arrays are free now).
  __syncthreads();
  auto park_region = [&](int wave) -> float* {
    // each staging array is at least DT*16*64 floats
    uint16_t* r = wave == 0 ? q_lds : wave == 1 ? do_lds : wave == 2 ? qt_lds : dot_lds;
    return reinterpret_cast<float*>(r);
  };
  {
    float* mine = park_region(w);
    if (qi == 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mine[(dt * 16 + i) * 64 + lane] = dv_acc[dt][i];
    } else {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mine[(dt * 16 + i) * 64 + lane] = dk_acc[dt][i];
    }
  }
  __syncthreads();
  {
    const float* take = park_region(w ^ 2);  // partner: same keys, other query half
    const int64_t off = (int64_t)p.dkv_block_table[(int64_t)b * p.max_kv_blocks + blk] * p.dkv_slot_stride +
                        (int64_t)(tok0 + ki * 32 + c) * p.dkv_token_stride + (int64_t)kv_head * D + 4 * h;
    uint16_t* dst_ptr = reinterpret_cast<uint16_t*>(qi == 0 ? p.dk : p.dv) + off;
    const float mul = (qi == 0) ? p.scale : 1.0f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float v4[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = 4 * g + r;
          const float own = (qi == 0) ? dk_acc[dt][i] : dv_acc[dt][i];
          v4[r] = (own + take[(dt * 16 + i) * 64 + lane]) * mul;
        }
        u32x2 pk = {pack2<DTYPE>(v4[0], v4[1]), pack2<DTYPE>(v4[2], v4[3])};
        *reinterpret_cast<u32x2*>(dst_ptr + dt * 32 + 8 * g) = pk;
      }
  }
}

// dQ = scale * accumulator, stored paged.  grid: (batch, row chunks)
template <int DTYPE, int D>
__global__ __launch_bounds__(256) void bwd_dq_store_kernel(const AttnBwdParams p) {
  constexpr int LPR = D / 8;
  constexpr int ROWS = 256 / LPR;
  const int b = blockIdx.x;
  const int q_begin = p.cu_seqlens_q[b];
  const int seqlen_q = p.cu_seqlens_q[b + 1] - q_begin;
  const int row = blockIdx.y * ROWS + threadIdx.x / LPR;
  const int g = threadIdx.x % LPR;
  const int t = row / p.n_heads_q;
  const int hd = row - t * p.n_heads_q;
  if (t >= seqlen_q) return;
  const f32x4* src = reinterpret_cast<const f32x4*>(p.dq_accum + ((int64_t)(q_begin + t) * p.n_heads_q + hd) * D + g * 8);
  const f32x4 a = src[0], c4 = src[1];
  u32x4 pk = {pack2<DTYPE>(a[0] * p.scale, a[1] * p.scale), pack2<DTYPE>(a[2] * p.scale, a[3] * p.scale),
              pack2<DTYPE>(c4[0] * p.scale, c4[1] * p.scale), pack2<DTYPE>(c4[2] * p.scale, c4[3] * p.scale)};
  uint16_t* dst = reinterpret_cast<uint16_t*>(p.dq) +
                  (((int64_t)p.dq_block_table[b] * p.block_size + t) * p.n_heads_q + hd) * D + g * 8;
  *reinterpret_cast<u32x4*>(dst) = pk;
}

template <int DTYPE, int D>
static int launch_bwd(const AttnBwdParams& p, hipStream_t stream) {
  constexpr int ROWS = 256 / (D / 8);
  const int64_t rows = (int64_t)p.block_size * p.n_heads_q;
  const int64_t chunks = (rows + ROWS - 1) / ROWS;
  DCP_REQUIRE(chunks <= 65535, "attn_bwd: block of %lld (token, head) rows is too large", (long long)rows);
  dim3 prep_grid(p.batch, (unsigned)chunks);
  {
    KernelTimer timer("bwd_prep_kernel", stream);
    hipLaunchKernelGGL((bwd_prep_kernel<DTYPE, D>), prep_grid, dim3(256), 0, stream, p);
  }
  {
    KernelTimer timer("bwd_tile_hull_kernel", stream);
    hipLaunchKernelGGL(bwd_tile_hull_kernel, dim3(p.batch * p.q_tiles_per_row), dim3(64), 0, stream, p);
  }
  const int64_t n_wg = (int64_t)p.batch * p.n_heads_kv * p.kv_tiles_per_row;
  DCP_REQUIRE(n_wg < ((int64_t)1 << 31), "attn_bwd: grid too large");
  {
    KernelTimer timer("attn_bwd_kernel", stream);
    hipLaunchKernelGGL((attn_bwd_kernel<DTYPE, D>), dim3((unsigned)n_wg), dim3(kBwdThreads), 0, stream, p);
  }
  {
    KernelTimer timer("bwd_dq_store_kernel", stream);
    hipLaunchKernelGGL((bwd_dq_store_kernel<DTYPE, D>), prep_grid, dim3(256), 0, stream, p);
  }
  return check_launch("attn_bwd kernels");
}

}  // namespace dcp

using namespace dcp;

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

extern "C" size_t dcp_attn_bwd_workspace_bytes(int batch, int total_q, int block_size, int n_heads_q,
                                               int head_dim) {
  if (batch < 0 || total_q < 0 || block_size <= 0 || n_heads_q <= 0 || head_dim <= 0) return 0;
  const size_t q_tiles = (size_t)batch * ((block_size + kBwdBM - 1) / kBwdBM);
  return align256((size_t)total_q * n_heads_q * head_dim * sizeof(float)) +
         align256((size_t)total_q * n_heads_q * sizeof(float)) + align256(q_tiles * 8 * sizeof(int32_t));
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
  DCP_REQUIRE(n_heads_q > 0 && n_heads_kv > 0 && n_heads_q % n_heads_kv == 0,
              "attn_bwd: n_heads_q %d must be a multiple of n_heads_kv %d", n_heads_q, n_heads_kv);
  DCP_REQUIRE(max_kv_blocks > 0 && n_out_slots > 0, "attn_bwd: empty block tables");
  DCP_REQUIRE(kv_token_stride % 8 == 0 && kv_slot_stride % 8 == 0 && dkv_token_stride % 4 == 0 &&
                  dkv_slot_stride % 4 == 0,
              "attn_bwd: kv strides must be multiples of 8 elements (dkv: 4)");
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
  const size_t need = dcp_attn_bwd_workspace_bytes(batch, total_q, block_size, n_heads_q, head_dim);
  DCP_REQUIRE(workspace_bytes >= need, "attn_bwd: workspace of %zu bytes is smaller than the %zu needed",
              workspace_bytes, need);
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
  p.dq_accum = reinterpret_cast<float*>(ws);
  ws += align256((size_t)total_q * n_heads_q * head_dim * sizeof(float));
  p.delta = reinterpret_cast<float*>(ws);
  ws += align256((size_t)total_q * n_heads_q * sizeof(float));
  p.hull = reinterpret_cast<int32_t*>(ws);
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
  p.n_out_slots = n_out_slots;
  p.q_tiles_per_row = (block_size + kBwdBM - 1) / kBwdBM;
  p.kv_tiles_per_row = max_kv_blocks * (block_size / kBwdBN);
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * kLog2e;
  if (dtype == DCP_DTYPE_BF16)
    return head_dim == 128 ? launch_bwd<DCP_DTYPE_BF16, 128>(p, (hipStream_t)stream)
                           : launch_bwd<DCP_DTYPE_BF16, 64>(p, (hipStream_t)stream);
  return head_dim == 128 ? launch_bwd<DCP_DTYPE_FP16, 128>(p, (hipStream_t)stream)
                         : launch_bwd<DCP_DTYPE_FP16, 64>(p, (hipStream_t)stream);
}
