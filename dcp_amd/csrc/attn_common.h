// MFMA and wave-level helpers shared by the attention kernels (gfx950).
#pragma once

#include "common.h"

namespace dcp {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// D(32x32, f32) += A(32x16) * B(16x32), 16-bit inputs.
// Lane l = 32*h + c holds: A row c, k-slots 8h..8h+7; B column c, the same
// k-slots; D column c, rows 8*(i/4) + 4h + i%4 for i in [0,16).
template <int DTYPE>
__device__ __forceinline__ f32x16 mfma_32x32x16(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (DTYPE == DCP_DTYPE_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
}

// Two fp32 -> one dword of two 16-bit values (round to nearest even).
template <int DTYPE>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (DTYPE == DCP_DTYPE_BF16) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  } else {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  }
}

// 2^x as the single hardware instruction: no denormal-range fix-up (results
// below 2^-126 flush to zero, which is what a softmax weight that small is).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32); }

__device__ __forceinline__ int wave_min(int x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = min(x, __shfl_xor(x, o));
  return x;
}
__device__ __forceinline__ int wave_max(int x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = max(x, __shfl_xor(x, o));
  return x;
}

// Row index (within a 32-row MFMA tile) of accumulator element i for a lane
// in half h.
__device__ __forceinline__ constexpr int acc_row(int i, int h) {
  return 8 * (i / 4) + 4 * h + (i % 4);
}

// Position, inside a group of 16 contraction indices stored contiguously in
// LDS, of the 4-index subgroup r (indices 4r..4r+3), chosen so that a lane in
// half h reads its 8 k-slots {4h..4h+3, 8+4h..8+4h+3} with one 16-byte load at
// position 8h.  These are exactly the rows a lane holds in accumulator
// elements 0..7 of a 32x32 tile, so an accumulator feeds the next MFMA as its
// B operand without any cross-lane movement.
__device__ __forceinline__ constexpr int kslot_pos(int r) {
  return r == 0 ? 0 : r == 1 ? 8 : r == 2 ? 4 : 12;
}

// ---------------------------------------------------------------------------
// Dense LDS tile [rows][D] of 16-bit elements, filled straight from global
// memory (no register staging) and read as MFMA operands in both orientations
// without bank conflicts.
//
// A row is D/8 16-byte chunks; the chunk at position p of row r holds logical
// chunk p ^ swz(r).  With swz(r) = (r&3)<<2 | (r>>2)&3 (D = 128; the D = 64
// variant plays the same game with 128-byte rows):
//  - 16 lanes reading the same logical chunk of 16 consecutive rows touch 16
//    different chunk positions (all 64 banks once);
//  - a transpose load, whose 32 lanes touch 4 consecutive rows x 4 consecutive
//    chunks, also touches 16 different chunk positions.
// global_load_lds writes lane l's 16 bytes at (instruction base) + 16*l, so one
// wave instruction fills 1024 contiguous bytes = 512/D rows, each lane
// fetching the logical chunk that belongs at its position.
// ---------------------------------------------------------------------------
template <int D>
struct SwzTile {
  static constexpr int CH = D / 8;                 // chunks per row
  static constexpr int RPI = 512 / D;              // rows per wave instruction
  __device__ static __forceinline__ int swz(int r) {
    return D == 128 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
  }
  // element offset of logical chunk `chunk` of row r
  __device__ static __forceinline__ int at(int r, int chunk) { return r * D + ((chunk ^ swz(r)) << 3); }

  // Asynchronously copy `rows` rows (multiple of 4*RPI... 64 here) of a global
  // tile whose rows are `row_stride` elements apart into `tile`; 4 waves.
  template <int ROWS>
  __device__ static __forceinline__ void load_async(uint16_t* tile, const uint16_t* g, int64_t row_stride,
                                                    int wave, int lane) {
    constexpr int PER_WAVE = ROWS / (4 * RPI);
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
      const int r0 = (wave * PER_WAVE + i) * RPI;
      const int r = r0 + lane / CH;
      const int chunk = (lane % CH) ^ swz(r);
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(g + (int64_t)r * row_stride + chunk * 8),
          (__attribute__((address_space(3))) void*)(tile + r0 * D), 16, 0, 0);
    }
  }

  // MFMA operand of lane (c, h): 8 consecutive elements 16*ks + 8h.. of row `r`.
  __device__ static __forceinline__ u32x4 read_row(const uint16_t* tile, int r, int ks, int h) {
    return *reinterpret_cast<const u32x4*>(tile + at(r, 2 * ks + h));
  }

  // MFMA operand with the tile's ROWS as the contraction index: lane (c, h)
  // gets column col0 + c at the 8 rows {slot0 + 4h + 0..3, slot0 + 8 + 4h + 0..3}
  // (accumulator order, ACC_ORDER) or slot0 + 8h + 0..7 (natural order).
  template <bool ACC_ORDER>
  __device__ static __forceinline__ u32x4 read_col(const uint16_t* tile, int slot0, int col0, int lane) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const int j = lane & 15;
    const int h = lane >> 5;
    const int d = col0 + ((lane >> 4) & 1) * 16 + 4 * (j & 3);
    const int r0 = slot0 + (ACC_ORDER ? 4 * h : 8 * h) + (j >> 2);
    const int r1 = r0 + (ACC_ORDER ? 8 : 4);
    const uint16_t* p0 = tile + at(r0, d >> 3) + (d & 4);
    const uint16_t* p1 = tile + at(r1, d >> 3) + (d & 4);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p1));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    u32x4 out = {l2[0], l2[1], h2[0], h2[1]};
    return out;
  }
};

// ---------------------------------------------------------------------------
// LDS tiles of 64 rows x D 16-bit elements whose operand addresses are AFFINE
// in the loop indices, so every ds_read uses a per-lane base register plus an
// immediate offset (no address arithmetic inside the key loop).
//
// global_load_lds fills 1024 contiguous bytes per wave instruction: a "group"
// of G = 512/D rows.  Which rows form a group, and the padding between groups,
// is chosen per access pattern so that the reads are free of bank conflicts:
//
//  RowTile  operand = 8 consecutive elements of a row, 16 lanes read 16
//           consecutive rows (A operand of X K^T-type products).  Row r lives
//           in group r % NG, so 16 consecutive rows sit in 16 different groups;
//           groups are 16 bytes apart modulo the 256-byte bank window.
//  ColTile  operand = one column at 8 rows (transpose load; rows are the
//           contraction index).  One transpose load touches 4 consecutive rows
//           x 64 bytes; those rows sit in 4 consecutive groups that are 64
//           bytes apart modulo the bank window.
// ---------------------------------------------------------------------------
template <int D>
struct RowTile {
  static constexpr int ROWS = 64;
  static constexpr int G = 512 / D;                // rows per group (4 for D=128, 8 for D=64)
  static constexpr int NG = ROWS / G;              // groups (16 / 8)
  static constexpr int GROUP_STRIDE = G * D + 8;   // elements: 1024 B + 16 B
  static constexpr int SIZE = NG * GROUP_STRIDE;   // elements
  // element offset of (row r, element e)
  __device__ static __forceinline__ int at(int r, int e) { return (r % NG) * GROUP_STRIDE + (r / NG) * D + e; }
  static constexpr int LPW = NG / 4;  // group loads per wave (4 waves fill a tile)
  // Byte offsets, from (row 0, the head's first element), of what this lane
  // fetches in each of its wave's group loads.  Loop-invariant.
  __device__ static __forceinline__ void lane_offsets(uint32_t (&off)[LPW], int64_t row_stride, int wave, int lane) {
    constexpr int CH = D / 8;
    const int sub = lane / CH, chunk = lane % CH;
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int r = sub * NG + wave * LPW + i;
      off[i] = (uint32_t)((r * row_stride + chunk * 8) * 2);
    }
  }
  // `g` (wave-uniform) points at (row 0, the head's first element) of the tile.
  __device__ static __forceinline__ void load_async(uint16_t* tile, const uint16_t* g, const uint32_t (&off)[LPW],
                                                    int wave) {
    const char* gb = reinterpret_cast<const char*>(g);
#pragma unroll
    for (int i = 0; i < LPW; ++i)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gb + off[i]),
                                       (__attribute__((address_space(3))) void*)(tile + (wave * LPW + i) * GROUP_STRIDE),
                                       16, 0, 0);
  }
};

template <int D>
struct ColTile {
  static constexpr int ROWS = 64;
  static constexpr int G = 512 / D;
  static constexpr int NG = ROWS / G;
  static constexpr int GROUP_STRIDE = G * D + 32;  // elements: 1024 B + 64 B
  static constexpr int SIZE = NG * GROUP_STRIDE;
  // rows 4m..4m+3 -> 4 consecutive groups, same position inside the group:
  // group(r) = (r & 3) + 4 * (r / (4 * G)),  sub(r) = (r / 4) % G
  __device__ static __forceinline__ int at(int r, int e) {
    return ((r & 3) + 4 * (r / (4 * G))) * GROUP_STRIDE + ((r >> 2) % G) * D + e;
  }
  static constexpr int LPW = NG / 4;
  __device__ static __forceinline__ void lane_offsets(uint32_t (&off)[LPW], int64_t row_stride, int wave, int lane) {
    constexpr int CH = D / 8;
    const int sub = lane / CH, chunk = lane % CH;
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int grp = wave * LPW + i;
      const int r = (grp >> 2) * (4 * G) + sub * 4 + (grp & 3);
      off[i] = (uint32_t)((r * row_stride + chunk * 8) * 2);
    }
  }
  __device__ static __forceinline__ void load_async(uint16_t* tile, const uint16_t* g, const uint32_t (&off)[LPW],
                                                    int wave) {
    const char* gb = reinterpret_cast<const char*>(g);
#pragma unroll
    for (int i = 0; i < LPW; ++i)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gb + off[i]),
                                       (__attribute__((address_space(3))) void*)(tile + (wave * LPW + i) * GROUP_STRIDE),
                                       16, 0, 0);
  }
  // Per-lane base of the transpose loads: lane (j = lane%16, half-wave h, 16-lane
  // group q) reads element column 16q + 4(j%4) of row (j/4) + 4h [+ slot offsets].
  __device__ static __forceinline__ int lane_base(int lane, bool acc_order) {
    const int j = lane & 15, h = lane >> 5;
    const int r = (acc_order ? 4 * h : 8 * h) + (j >> 2);
    return at(r, ((lane >> 4) & 1) * 16 + 4 * (j & 3));
  }
  // 8 contraction slots starting at row `slot0` (multiple of 16) for column
  // block `col0` (multiple of 32); `base` from lane_base().  ACC_ORDER: slots
  // are rows {4h..4h+3, 8+4h..8+4h+3} (accumulator order), else 8h..8h+7.
  template <bool ACC_ORDER>
  __device__ static __forceinline__ u32x4 read_col(const uint16_t* tile, int base, int slot0, int col0) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    // rows advance by 16 -> 4 groups (D=128) ; +8 rows (acc order) or +4 rows -> inside-group / next groups
    const int o0 = at(slot0, col0);
    const int o1 = ACC_ORDER ? at(slot0 + 8, col0) : at(slot0 + 4, col0);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + base + o0));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + base + o1));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    u32x4 out = {l2[0], l2[1], h2[0], h2[1]};
    return out;
  }
};

// The (at most two) runs of key tiles a workgroup has to visit, from the hull
// of its rows' ranges.  Tiles are BN keys wide.
struct TileRuns {
  int a0, b0, a1, b1;  // [a0, b0) then [a1, b1); empty runs have a == b
  __device__ __forceinline__ TileRuns(int lo0, int hi0, int lo1, int hi1, int bn) {
    int x0 = lo0 / bn, y0 = hi0 > 0 ? (hi0 + bn - 1) / bn : 0;
    int x1 = lo1 / bn, y1 = hi1 > 0 ? (hi1 + bn - 1) / bn : 0;
    if (y0 <= x0 || hi0 == 0) { x0 = y0 = 0; }
    if (y1 <= x1 || hi1 == 0) { x1 = y1 = 0; }
    if (y0 == x0) { x0 = x1; y0 = y1; x1 = y1 = 0; }          // only the second run
    else if (y1 > x1) {
      if (x1 < x0) { int t = x0; x0 = x1; x1 = t; t = y0; y0 = y1; y1 = t; }
      if (x1 <= y0) { y0 = max(y0, y1); x1 = y1 = 0; }         // overlapping or adjacent: merge
    }
    a0 = x0; b0 = y0; a1 = x1; b1 = y1;
  }
  __device__ __forceinline__ int count() const { return (b0 - a0) + (b1 - a1); }
  __device__ __forceinline__ int tile(int i) const { return i < b0 - a0 ? a0 + i : a1 + (i - (b0 - a0)); }
};

struct RangePair {
  int s0, len0, s1, len1;  // start and (non-negative) length of each range
  __device__ __forceinline__ bool contains(int k) const {
    return ((unsigned)(k - s0) < (unsigned)len0) | ((unsigned)(k - s1) < (unsigned)len1);
  }
};

}  // namespace dcp
