// libbench_probes.so: three measurement-only kernels that bench.py runs beside the product library
// for the roofline discussion (not part of libdcp_hip.so or of its C ABI; nothing in the
// reference corresponds to them): the sustained matrix-core rate, the same with an attention kernel's instruction mix beside the
// MFMAs, and the streaming rate of HBM.
// Built by `python -m dcp_amd.build` from this one file; entry points return 0 or a DCP_ERR_*
// code and bench_probe_last_error() gives the message.
//
// Sustained matrix-core rate of the device: a kernel that does
// nothing but 32x32x16 MFMAs on operands the caller provides.  What the chip sustains depends
// on the operand values (power): constant operands run at the full shader clock, random ones
// do not.  No counterpart in the reference; used by bench.py only.
#include "attn_common.h"

namespace dcp {

// this library's own message buffer (libdcp_hip.so keeps its own)
char* last_error_buffer() {
  static thread_local char buffer[512] = {0};
  return buffer;
}

constexpr int kProbeThreads = 256;
constexpr int kProbeMfmaPerIter = 32;

// One wave per SIMD (launch one workgroup per CU).  Every lane reads 16 operand words
// (8 A, 8 B) from `operands` and issues kProbeMfmaPerIter MFMAs per iteration on four
// independent accumulators.  out[0] = shader clocks, out[1] = 100 MHz wall ticks of
// workgroup 0; out[2 + thread] = a value that depends on every accumulator.
template <int DTYPE>
__global__ __launch_bounds__(kProbeThreads, 1) void mfma_probe_kernel(const u32x4* operands, float* out, int iters) {
  u32x4 a[8], b[8];
  const size_t base = ((size_t)blockIdx.x * kProbeThreads + threadIdx.x) * 16;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = operands[base + i];
    b[i] = operands[base + 8 + i];
  }
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.0f;
  const long long w0 = wall_clock64(), c0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < kProbeMfmaPerIter; ++i) acc[i & 3] = mfma_32x32x16<DTYPE>(a[i & 7], b[(i >> 2) & 7], acc[i & 3]);
    if ((it & 63) == 63) {  // keep the sums finite
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] *= 1e-6f;
    }
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  float r = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += acc[j][i];
  out[2 + (size_t)blockIdx.x * kProbeThreads + threadIdx.x] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    out[0] = (float)(c1 - c0);
    out[1] = (float)(w1 - w0);
  }
}

// What the matrix cores sustain when every wave also issues, evenly spread between its MFMAs and
// with no dependency on anything loaded, the other instructions an attention kernel needs per
// NM MFMAs: NV plain vector instructions (FMAs), NE exponentials, NB128 16-byte and NB64 8-byte LDS
// reads per lane.  Two workgroups per CU (64 KiB of LDS each), i.e. two waves per SIMD, like the
// attention kernels.  No tile loads, no barriers, no waits on data: an upper bound for a kernel
// with that instruction mix, whatever its schedule.
template <int NM, int NV, int NE, int NB128, int NB64>
__global__ __launch_bounds__(kProbeThreads, 2) void mfma_mix_probe_kernel(const u32x4* operands, float* out, int iters,
                                                                         float s, float t) {
  __shared__ __attribute__((aligned(16))) u32x4 lds[4096];  // 64 KiB: two workgroups per CU
  for (int i = threadIdx.x; i < 4096; i += kProbeThreads) lds[i] = operands[i];
  __syncthreads();
  const size_t base = ((size_t)blockIdx.x * kProbeThreads + threadIdx.x) * 16;
  const u32x4 a = operands[base], b = operands[base + 8];
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.0f;
  float x[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) x[i] = threadIdx.x * 0.001f + i * 0.01f;
  const uint32_t at = lds_address(&lds[0]) + (threadIdx.x & 63) * 16;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      acc[m & 3] = mfma_32x32x16<DCP_DTYPE_BF16>(a, b, acc[m & 3]);
      // the m-th share of each kind: floor((m + 1) N / NM) - floor(m N / NM) instructions
#pragma unroll
      for (int k = m * NV / NM; k < (m + 1) * NV / NM; ++k) x[k & 15] = __builtin_fmaf(x[k & 15], s, t);
#pragma unroll
      for (int k = m * NE / NM; k < (m + 1) * NE / NM; ++k) x[k & 15] = fast_exp2(x[k & 15]);
#pragma unroll
      for (int k = m * NB128 / NM; k < (m + 1) * NB128 / NM; ++k) {
        u32x4 v;
        asm volatile("ds_read_b128 %0, %1 offset:1024" : "=v"(v) : "v"(at));
        asm volatile("" ::"v"(v));
      }
#pragma unroll
      for (int k = m * NB64 / NM; k < (m + 1) * NB64 / NM; ++k) {
        u32x2 v;
        asm volatile("ds_read_b64 %0, %1 offset:2048" : "=v"(v) : "v"(at));
        asm volatile("" ::"v"(v));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt lgkmcnt(0)");
    if ((it & 63) == 63) {  // keep the sums finite
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] *= 1e-6f;
    }
  }
  float r = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += acc[j][i];
#pragma unroll
  for (int i = 0; i < 16; ++i) r += x[i];
  out[2 + (size_t)blockIdx.x * kProbeThreads + threadIdx.x] = r;
}

// Plain streaming kernel for the HBM roofline discussion: NS input streams are added 16 bytes at a
// time (non-temporal loads) and written once (non-temporal store), one wave per workgroup and one
// 16-byte word per lane and stream: 1 KiB per stream and workgroup, the shape that measured fastest
// (256 lanes x 1 word: 3 % slower with one stream, 4 % with four; two words per lane: 10 % slower).
// Every stream is a sequence of blocks of `words_per_block` words; with a table, block b of stream
// s is block table[b * NS + s] of `src` (the gather / merge / sum kernels read their sources through
// such tables: where the blocks lie decides how the streams fall on the memory channels); without
// one the streams lie end to end.  What this reaches is the practical ceiling for those kernels at
// the same read : write mix.
template <int NS>
__global__ __launch_bounds__(64) void hbm_stream_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                        size_t words_per_stream, const int32_t* __restrict__ table,
                                                        unsigned chunks_per_block) {
  const size_t chunk = blockIdx.x;
  const size_t base = chunk * 64 + threadIdx.x;
  u32x4 v[NS];
  if (table) {
    const size_t b = chunk / chunks_per_block;
    const size_t within = (chunk - b * chunks_per_block) * 64 + threadIdx.x;
#pragma unroll
    for (int s = 0; s < NS; ++s)
      v[s] = __builtin_nontemporal_load(src + (size_t)table[b * NS + s] * chunks_per_block * 64 + within);
  } else {
#pragma unroll
    for (int s = 0; s < NS; ++s) v[s] = __builtin_nontemporal_load(src + s * words_per_stream + base);
  }
  u32x4 acc = v[0];
#pragma unroll
  for (int s = 1; s < NS; ++s) acc += v[s];
  __builtin_nontemporal_store(acc, dst + base);
}

}  // namespace dcp

using namespace dcp;

extern "C" const char* bench_probe_last_error(void) { return dcp::last_error_buffer(); }

// Adds `n_streams` (1, 2 or 4) equally long input streams 16 bytes at a time and writes the sum to
// `dst`: n_streams reads and one write of `bytes_per_stream` each.  `block_table` null: the streams lie
// end to end in `src`.  Otherwise a stream is made of blocks of `block_bytes` (a multiple of 1024 that
// divides bytes_per_stream) and block b of stream s is block block_table[b * n_streams + s] of `src`
// (device memory, int32).  Time it with events on `stream`.
extern "C" int bench_hbm_stream_probe(const void* src, void* dst, int n_streams, size_t bytes_per_stream,
                                      const int32_t* block_table, size_t block_bytes, void* stream) {
  DCP_REQUIRE(src && dst, "hbm_stream_probe: null argument");
  DCP_REQUIRE(bytes_per_stream > 0 && bytes_per_stream % 1024 == 0,
              "hbm_stream_probe: bytes_per_stream must be a positive multiple of 1024");
  DCP_REQUIRE(bytes_per_stream / 1024 < ((size_t)1 << 31), "hbm_stream_probe: stream too long");
  DCP_REQUIRE(!block_table || (block_bytes > 0 && block_bytes % 1024 == 0 && bytes_per_stream % block_bytes == 0),
              "hbm_stream_probe: block_bytes must be a multiple of 1024 that divides bytes_per_stream");
  const size_t words = bytes_per_stream / 16;
  const unsigned chunks_per_block = block_table ? (unsigned)(block_bytes / 1024) : 1;
  dim3 grid((unsigned)(bytes_per_stream / 1024)), block(64);
  switch (n_streams) {
    case 1:
      hipLaunchKernelGGL(hbm_stream_kernel<1>, grid, block, 0, (hipStream_t)stream, (const u32x4*)src, (u32x4*)dst, words, block_table, chunks_per_block);
      break;
    case 2:
      hipLaunchKernelGGL(hbm_stream_kernel<2>, grid, block, 0, (hipStream_t)stream, (const u32x4*)src, (u32x4*)dst, words, block_table, chunks_per_block);
      break;
    case 4:
      hipLaunchKernelGGL(hbm_stream_kernel<4>, grid, block, 0, (hipStream_t)stream, (const u32x4*)src, (u32x4*)dst, words, block_table, chunks_per_block);
      break;
    default:
      return fail(DCP_ERR_UNSUPPORTED, "hbm_stream_probe: n_streams %d unsupported (1, 2 or 4)", n_streams);
  }
  return check_launch("hbm_stream_kernel");
}

// Launches `n_workgroups` workgroups of 256 threads that do nothing but 32x32x16 MFMAs (`iters` x 32
// per wave) on operands read once from `operands`: 16 x 16 bytes per thread.  `out` receives
// 2 + n_workgroups * 256 floats: out[0] = shader clocks and out[1] = 100 MHz ticks spent in the
// loop by workgroup 0, the rest one checksum per thread.  *flop = the floating-point operations
// the launch performs; time it with events on `stream`.
extern "C" int bench_mfma_probe(const void* operands, float* out, int n_workgroups, int iters, int dtype,
                              double* flop, void* stream) {
  DCP_REQUIRE(operands && out && flop, "mfma_probe: null argument");
  DCP_REQUIRE(n_workgroups > 0 && iters > 0, "mfma_probe: sizes must be positive");
  if (dtype != DCP_DTYPE_BF16 && dtype != DCP_DTYPE_FP16)
    return fail(DCP_ERR_UNSUPPORTED, "mfma_probe: dtype %d unsupported (bf16 and fp16 only)", dtype);
  *flop = (double)n_workgroups * (kProbeThreads / 64) * (double)iters * kProbeMfmaPerIter * (2.0 * 32 * 32 * 16);
  dim3 grid(n_workgroups), block(kProbeThreads);
  if (dtype == DCP_DTYPE_BF16)
    hipLaunchKernelGGL(mfma_probe_kernel<DCP_DTYPE_BF16>, grid, block, 0, (hipStream_t)stream,
                       (const u32x4*)operands, out, iters);
  else
    hipLaunchKernelGGL(mfma_probe_kernel<DCP_DTYPE_FP16>, grid, block, 0, (hipStream_t)stream,
                       (const u32x4*)operands, out, iters);
  return check_launch("mfma_probe_kernel");
}


// The MFMA probe with an attention kernel's other instructions beside the MFMAs (see
// mfma_mix_probe_kernel): `mix` 0 = forward (per 32 MFMAs: 112 FMAs, 32 exponentials, 16 + 32 LDS
// reads), 1 = dK/dV kernel (per 32: 58, 16, 20 + 32), 2 = dQ kernel (per 48: 80, 32, 32 + 32).
// `n_workgroups` workgroups of 256 threads, two per CU; `operands` and `out` as for
// bench_mfma_probe (at least 4096 x 16 bytes of operands).  *flop = the MFMAs' operations.
extern "C" int bench_mfma_mix_probe(const void* operands, float* out, int n_workgroups, int iters, int mix, double* flop,
                                    void* stream) {
  DCP_REQUIRE(operands && out && flop, "mfma_mix_probe: null argument");
  DCP_REQUIRE(n_workgroups >= 16 && iters > 0, "mfma_mix_probe: at least 16 workgroups and one iteration");
  const int per_iter = mix == 2 ? 48 : 32;
  *flop = (double)n_workgroups * (kProbeThreads / 64) * (double)iters * per_iter * (2.0 * 32 * 32 * 16);
  dim3 grid(n_workgroups), block(kProbeThreads);
  const u32x4* ops = (const u32x4*)operands;
  switch (mix) {
    case 0:
      hipLaunchKernelGGL((mfma_mix_probe_kernel<32, 112, 32, 16, 32>), grid, block, 0, (hipStream_t)stream, ops, out, iters, 1.0001f, 0.5f);
      break;
    case 1:
      hipLaunchKernelGGL((mfma_mix_probe_kernel<32, 58, 16, 20, 32>), grid, block, 0, (hipStream_t)stream, ops, out, iters, 1.0001f, 0.5f);
      break;
    case 2:
      hipLaunchKernelGGL((mfma_mix_probe_kernel<48, 80, 32, 32, 32>), grid, block, 0, (hipStream_t)stream, ops, out, iters, 1.0001f, 0.5f);
      break;
    default:
      return fail(DCP_ERR_UNSUPPORTED, "mfma_mix_probe: mix %d unsupported (0, 1 or 2)", mix);
  }
  return check_launch("mfma_mix_probe_kernel");
}
