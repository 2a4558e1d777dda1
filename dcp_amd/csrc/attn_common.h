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

// The value the other half of the wave holds (lane ^ 32), by one register swap on the vector
// unit (no trip through LDS).
__device__ __forceinline__ float xor32(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // {lanes 0-31 twice, lanes 32-63 twice}
  return __uint_as_float((threadIdx.x & 32) ? r[0] : r[1]);
}
// max / sum over the two halves, the same in both
__device__ __forceinline__ float halves_max(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Minimum / maximum over the wave, as a scalar.  Four DPP steps (row_shr 1, 2, 4, 8) leave each
// 16-lane row's result in its last lane; the four row results are combined on the scalar unit.
// (Butterfly shuffles would be six dependent trips through LDS each, and a workgroup's prologue
// takes eight of these reductions.)
template <bool IS_MIN>
__device__ __forceinline__ int wave_reduce_minmax(int x) {
#define DCP_DPP_STEP(ctrl)                                                       \
  {                                                                              \
    const int y = __builtin_amdgcn_update_dpp(x, x, ctrl, 0xf, 0xf, false);      \
    x = IS_MIN ? min(x, y) : max(x, y);                                          \
  }
  DCP_DPP_STEP(0x111)  // row_shr:1 (a lane without a source keeps its own value)
  DCP_DPP_STEP(0x112)  // row_shr:2
  DCP_DPP_STEP(0x114)  // row_shr:4
  DCP_DPP_STEP(0x118)  // row_shr:8
#undef DCP_DPP_STEP
  const int r0 = __builtin_amdgcn_readlane(x, 15), r1 = __builtin_amdgcn_readlane(x, 31);
  const int r2 = __builtin_amdgcn_readlane(x, 47), r3 = __builtin_amdgcn_readlane(x, 63);
  return IS_MIN ? min(min(r0, r1), min(r2, r3)) : max(max(r0, r1), max(r2, r3));
}
__device__ __forceinline__ int wave_min(int x) { return wave_reduce_minmax<true>(x); }
__device__ __forceinline__ int wave_max(int x) { return wave_reduce_minmax<false>(x); }

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
// LDS tile of 64 rows x D 16-bit elements, filled by NW waves straight from global memory
// (global_load_lds, no register staging) and read as an MFMA operand in both
// orientations, without bank conflicts and with addresses that are a per-lane
// base plus a compile-time offset (no address arithmetic inside the loops).
//
// global_load_lds writes lane l's 16 bytes at (instruction base) + 16*l, so one
// wave instruction fills 1024 contiguous bytes: a "group" of G = 512/D rows.
// All rows of a group share their alignment in the 256-byte bank window (for
// D = 64 they alternate between its two halves), so rows that are read
// together must sit in different groups.  Groups are padded by 16 bytes, which
// puts group g at bank-window offset 16g, and row r of the tile goes to
//
//   D = 128:  group 4*(r&3) + (r>>2)&3,   position r>>4 in the group
//   D =  64:  group 4*(r&1) + (r>>2)&3,   position (r>>1)&1 + 2*(r>>4)
//
// so that, within any aligned 16 rows, row r sits at window offset
// 64*(r&3) + 16*((r>>2)&3) bytes:
//  - row operand (8 consecutive elements of a row; 16 lanes read 16
//    consecutive rows at one column): 16 different 16-byte slots;
//  - column operand (transpose load: one column at 8 rows, the rows being the
//    contraction index; 32 lanes touch 4 consecutive rows x 64 bytes): four
//    64-byte windows.
// ---------------------------------------------------------------------------
// LDS byte address of a __shared__ object
template <typename T>
__device__ __forceinline__ uint32_t lds_address(T* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)p;
}

// One 4-byte element per lane from global memory straight into LDS: lane l's value lands
// at lds_at + 4*l (lds_at wave-uniform).  Ordered by the caller like the tile loads below.
__device__ __forceinline__ void load_async_dword(uint32_t lds_at, const void* g) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_at)), "v"(g)
               : "memory");
}

// The same with a wave-uniform base address and a per-lane byte offset.
__device__ __forceinline__ void load_async_dword(uint32_t lds_at, uint32_t lane_offset, const void* base) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  const uint64_t b = ((uint64_t)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_at)), "v"(lane_offset), "s"(b)
               : "memory");
}

// A 64-bit value that every lane holds alike, moved to scalar registers.
__device__ __forceinline__ uint64_t uniform64(uint64_t a) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return ((uint64_t)hi << 32) | lo;
}

template <int D, int NW = 4>
struct KvTile {
  static constexpr int ROWS = 64;
  static constexpr int G = 512 / D;
  static constexpr int NG = ROWS / G;
  static constexpr int GROUP_STRIDE = G * D + 8;  // elements: 1024 B + 16 B
  static constexpr int SIZE = NG * GROUP_STRIDE;  // elements
  static constexpr int LPW = NG / NW;             // group loads per wave (NW waves fill a tile)
  static constexpr int ROW32 = 256;               // element offset of row r + 32 (both head dims)
  static constexpr int ROW16 = 128;               // element offset of row r + 16
  static constexpr int ROW8 = 2 * GROUP_STRIDE;   // row r + 8  (r % 16 < 8)
  static constexpr int ROW4 = GROUP_STRIDE;       // row r + 4  (r % 16 in 0..3 or 8..11)

  __device__ static __forceinline__ int at(int r, int e) {
    const int grp = D == 128 ? 4 * (r & 3) + ((r >> 2) & 3) : 4 * (r & 1) + ((r >> 2) & 3);
    const int pos = D == 128 ? (r >> 4) : ((r >> 1) & 1) + 2 * (r >> 4);
    return grp * GROUP_STRIDE + pos * D + e;
  }
  // row held at position `pos` of group `grp`
  __device__ static __forceinline__ int row_of(int grp, int pos) {
    return D == 128 ? 16 * pos + 4 * (grp & 3) + (grp >> 2)
                    : 16 * (pos >> 1) + 4 * (grp & 3) + 2 * (pos & 1) + (grp >> 2);
  }
  // Byte offsets, from (row 0, the head's first element), of what this lane
  // fetches in each of its wave's group loads.  Loop-invariant.
  __device__ static __forceinline__ void lane_offsets(uint32_t (&off)[LPW], int64_t row_stride, int wave, int lane) {
    constexpr int CH = D / 8;
#pragma unroll
    for (int i = 0; i < LPW; ++i)
      off[i] = (uint32_t)((row_of(wave * LPW + i, lane / CH) * row_stride + (lane % CH) * 8) * 2);
  }
  // `g` (wave-uniform) points at (row 0, the head's first element) of the tile.
  //
  // The load is written as assembly on purpose.  Through the builtin the compiler sees
  // an instruction that touches both global memory and LDS, and as long as one is in
  // flight it turns every LDS wait of the wave into a wait for ALL outstanding LDS
  // reads (lgkmcnt(0)), which serialises operand prefetch with the MFMAs for the whole
  // time a tile is streaming in, i.e. always.  Here the compiler tracks nothing, so the
  // kernels must (and do) order these loads themselves: s_waitcnt vmcnt(0) and a
  // workgroup barrier between a load and the first read of its stage, a barrier between
  // the last read of a stage and the load that refills it.
  // `tile_at` is the tile's LDS byte address (lds_address() of the array).
  __device__ static __forceinline__ void load_async(uint32_t tile_at, const uint16_t* g, const uint32_t (&off)[LPW],
                                                    int wave) {
    const char* gb = reinterpret_cast<const char*>(g);
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const uint32_t lds_at = __builtin_amdgcn_readfirstlane(tile_at + (wave * LPW + i) * GROUP_STRIDE * 2);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   :
                   : "s"(lds_at), "v"(gb + off[i])
                   : "memory");
    }
  }
  // The same loads one at a time, so that a kernel can spread them between its matrix
  // instructions instead of issuing a burst (a burst fills the memory pipeline's queue
  // and the wave sits at the last load until the queue drains).  The rows of group
  // load i lie 4*i rows below those of group load 0, so one per-lane byte offset
  // (lane_offset0) serves all of them and the rest of the address is wave-uniform:
  // scalar base + vector offset addressing, no per-load address arithmetic.
  __device__ static __forceinline__ uint32_t lane_offset0(int64_t row_stride, int wave, int lane) {
    constexpr int CH = D / 8;
    static_assert((LPW & (LPW - 1)) == 0 && LPW <= 4, "group loads of a wave must not carry into grp >> 2");
    return (uint32_t)((row_of(wave * LPW, lane / CH) * row_stride + (lane % CH) * 8) * 2);
  }
  // `g` (wave-uniform) points at (row 0, the head's first element) of the tile.
  __device__ static __forceinline__ void load_group(uint32_t tile_at, const uint16_t* g, uint32_t off0,
                                                    int64_t row_stride, int wave, int i) {
    const uint32_t lds_at = __builtin_amdgcn_readfirstlane(tile_at + (wave * LPW + i) * GROUP_STRIDE * 2);
    const uint64_t a = reinterpret_cast<uint64_t>(g) + (uint64_t)(i * 8) * (uint64_t)row_stride;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    const uint64_t base = ((uint64_t)hi << 32) | lo;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_at), "v"(off0), "s"(base)
                 : "memory");
  }
  // One group load whose LDS byte address and wave-uniform global base the caller has already
  // worked out (kernels that walk a tile's groups keep both as running scalars).
  __device__ static __forceinline__ void load_group_at(uint32_t lds_at, uint64_t base, uint32_t off0) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_at), "v"(off0), "s"(base)
                 : "memory");
  }
  // The same for data that is read once (non-temporal: it takes no room in the L2 that the shared
  // tiles need).
  __device__ static __forceinline__ void load_group_at_streaming(uint32_t lds_at, uint64_t base, uint32_t off0) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(lds_at), "v"(off0), "s"(base)
                 : "memory");
  }
  // LDS byte address of the wave's group load i, and the global byte step between group loads (its
  // rows lie four rows below those of load i - 1)
  __device__ static __forceinline__ uint32_t group_lds_at(uint32_t tile_at, int wave, int i) {
    return tile_at + (wave * LPW + i) * GROUP_STRIDE * 2;
  }
  __device__ static __forceinline__ uint64_t group_global_step(int64_t row_stride) { return (uint64_t)row_stride * 8; }
  // Row operand of lane (c, h): elements 16*ks + 8h.. of row 32*nt + c at
  //   tile + row_base(c, h) + nt*ROW32 + ks*16
  __device__ static __forceinline__ int row_base(int c, int h) { return at(c, 8 * h); }
  // Column operand of lane l: column 32*ct + (l & 31) at the 8 rows of k-step s2,
  //   ACC_ORDER: 16*s2 + {4h..4h+3, 8+4h..8+4h+3}   (matches accumulator rows)
  //   else:      16*s2 + 8h + 0..7
  // read as two transpose loads at tile + col_base(l) + s2*ROW16 + ct*32 (+ ROW8 or ROW4).
  __device__ static __forceinline__ int col_base(int lane, bool acc_order) {
    const int j = lane & 15, h = lane >> 5;
    return at((acc_order ? 4 * h : 8 * h) + (j >> 2), ((lane >> 4) & 1) * 16 + 4 * (j & 3));
  }
  template <bool ACC_ORDER>
  __device__ static __forceinline__ u32x4 read_col(const uint16_t* tile, int base, int s2, int ct) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const uint16_t* p0 = tile + base + s2 * ROW16 + ct * 32;
    const uint16_t* p1 = p0 + (ACC_ORDER ? ROW8 : ROW4);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p1));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    u32x4 out = {l2[0], l2[1], h2[0], h2[1]};
    return out;
  }
  __device__ static __forceinline__ u32x4 read_row(const uint16_t* tile, int base, int nt, int ks) {
    return *reinterpret_cast<const u32x4*>(tile + base + nt * ROW32 + ks * 16);
  }
};

// ---------------------------------------------------------------------------
// XCD-aware workgroup numbering.  The 256 CUs sit in 8 XCDs, each with its own
// L2, and consecutive workgroup ids are dealt round-robin to the XCDs.  Work
// items that stream the same tiles from HBM (the query tiles and grouped heads
// of one row share its K/V; the key tiles of one row share its Q/dO) should
// therefore NOT have consecutive ids: with `group` such items per shared
// stream, hardware id w is mapped to the logical item
//
//   ((w / (8*group)) * 8 + w % 8) * group + (w % (8*group)) / 8
//
// so that the `group` items of one stream all have the same w % 8 (one XCD, one
// copy in one L2) while neighbouring streams still spread over all 8 XCDs.
// The grid is rounded up to a multiple of 8*group; ids past `total` are idle.
// ---------------------------------------------------------------------------
constexpr int kNumXcd = 8;
__device__ __forceinline__ int xcd_logical_id(int w, int group, int64_t total) {
  const int per_super = kNumXcd * group;
  const int super = w / per_super, r = w - super * per_super;
  const int64_t id = ((int64_t)super * kNumXcd + (r % kNumXcd)) * group + r / kNumXcd;
  return id < total ? (int)id : -1;
}
inline int64_t xcd_grid_size(int64_t total, int group) {
  const int64_t per_super = (int64_t)kNumXcd * group;
  return (total + per_super - 1) / per_super * per_super;
}

// A persistent kernel's item body reads the kernel arguments through a pointer to the
// kernel-argument segment that is made opaque once per item, so that the compiler loads each
// field where the item uses it.  Read through the kernel's by-value parameter, every field an
// item's prologue needs is loaded once before the item loop and then occupies a scalar register
// through the whole matrix loop (the kernels end up at the scalar register limit).
// The kernel must have the parameter struct as its only argument.
template <typename Params>
using KernArgs = const __attribute__((address_space(4))) Params;
template <typename Params>
__device__ __forceinline__ KernArgs<Params>& fresh_kernel_args() {
  KernArgs<Params>* args = (KernArgs<Params>*)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(args));
  return *args;
}

// Workgroup barrier between the phases of a kernel whose LDS tiles are filled
// by global_load_lds.  It waits for this wave's LDS accesses (lgkmcnt) but, unlike
// __syncthreads(), not for its outstanding global loads, so tiles requested a phase
// or two ahead stay in flight; wait_loads() is the explicit vmcnt(0) a wave issues
// before the barrier that publishes the tiles it requested.  The "memory" clobber
// keeps the compiler from moving memory accesses across the barrier.
__device__ __forceinline__ void phase_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// s_waitcnt vmcnt(0), expcnt and lgkmcnt fields at their maximum: as a builtin, so that
// the compiler's own wait-count bookkeeping knows the tile loads have landed
__device__ __forceinline__ void wait_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

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

// A row's kv block table in LDS, and a cursor that walks the key tiles of a
// TileRuns list and yields each tile's element offset in the paged K/V buffer.
// A table lookup straight from global memory is a dependent load the wave has to
// sit out (a microsecond) before it can even request the tile; done once per tile
// it costs more than the tile's arithmetic.  The cursor touches the table only
// when it enters a new block, and then in LDS.
constexpr int kSlotTableCap = 1024;  // blocks of a row held in LDS; rows with more read the rest from global memory

__device__ __forceinline__ void load_slot_table(int* slot_lds, const int32_t* kv_table, int max_kv_blocks, int tid,
                                                int n_threads) {
  for (int i = tid; i < min(max_kv_blocks, kSlotTableCap); i += n_threads) slot_lds[i] = kv_table[i];
}

struct TileCursor {
  int index;    // position in the tile list
  int tile;     // key tile number (BN keys each)
  int pos;      // tile within its block
  int blk;      // block within the row
  int64_t off;  // element offset of the tile's first key row

  // The two sources are read through volatile pointers so that the compiler keeps them as an
  // LDS read and a global read under a (wave-uniform) branch: merged into one generic-address
  // load, the read would be followed by a wait for every outstanding global load, i.e. for the
  // tiles just requested.  The result is the same in every lane; readfirstlane moves it (and
  // all the offset arithmetic that follows) to the scalar unit.
  __device__ __forceinline__ static int slot(const int* slot_lds, const int32_t* kv_table, int blk) {
    typedef __attribute__((address_space(3))) const volatile int lds_int;
    typedef __attribute__((address_space(1))) const volatile int32_t global_int;
    int v;
    if (blk < kSlotTableCap) v = *(reinterpret_cast<lds_int*>(lds_address(slot_lds)) + blk);
    else v = *((global_int*)kv_table + blk);
    return __builtin_amdgcn_readfirstlane(v);
  }
  __device__ __forceinline__ void seek(const TileRuns& runs, int i, int tiles_per_block, const int* slot_lds,
                                       const int32_t* kv_table, int64_t slot_stride, int64_t tile_stride) {
    index = i;
    tile = runs.tile(i);
    blk = tile / tiles_per_block;
    pos = tile - blk * tiles_per_block;
    off = (int64_t)slot(slot_lds, kv_table, blk) * slot_stride + pos * tile_stride;
  }
  // to the next tile of the list (call only while index + 1 < runs.count())
  __device__ __forceinline__ void advance(const TileRuns& runs, int tiles_per_block, const int* slot_lds,
                                          const int32_t* kv_table, int64_t slot_stride, int64_t tile_stride) {
    if (__builtin_expect(index + 1 == runs.b0 - runs.a0, 0)) {  // jump to the second run
      seek(runs, index + 1, tiles_per_block, slot_lds, kv_table, slot_stride, tile_stride);
      return;
    }
    ++index;
    ++tile;
    ++pos;
    off += tile_stride;
    if (__builtin_expect(pos == tiles_per_block, 0)) {
      pos = 0;
      ++blk;
      off = (int64_t)slot(slot_lds, kv_table, blk) * slot_stride;
    }
  }
};

struct RangePair {
  int s0, len0, s1, len1;  // start and (non-negative) length of each range
  __device__ __forceinline__ bool contains(int k) const {
    return ((unsigned)(k - s0) < (unsigned)len0) | ((unsigned)(k - s1) < (unsigned)len1);
  }
  // Bit p set = key base + p (p = 0..31) lies in neither range.  A dozen vector instructions
  // for a 32-key window, after which an accumulator's initial value costs two (masked_start)
  // where a range test per element costs seven.
  __device__ __forceinline__ uint32_t closed_window(int base) const {
    auto open = [&](int s, int len) -> uint32_t {
      const int lo = min(max(s - base, 0), 32), hi = min(max(s + len - base, lo), 32);
      return (uint32_t)((1ull << hi) - (1ull << lo));  // bits lo..hi-1; the low word also when hi or lo is 32
    };
    return ~(open(s0, len0) | open(s1, len1));
  }
};
// 0.0f where bit `bit` of `closed` is clear, -inf where it is set: the bit, sign-extended to 0 / -1,
// shifted into the sign and exponent of a float.
__device__ __forceinline__ float masked_start(uint32_t closed, int bit) {
  return __builtin_bit_cast(float, (uint32_t)__builtin_amdgcn_sbfe((int32_t)closed, bit, 1) & 0xff800000u);
}

}  // namespace dcp
