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

struct RangePair {
  int s0, len0, s1, len1;  // start and (non-negative) length of each range
  __device__ __forceinline__ bool contains(int k) const {
    return ((unsigned)(k - s0) < (unsigned)len0) | ((unsigned)(k - s1) < (unsigned)len1);
  }
};

}  // namespace dcp
