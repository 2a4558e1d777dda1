// Shared host/device helpers for the gfx950 kernels of libdcp_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "dcp_hip.h"

namespace dcp {

// ---- error reporting -------------------------------------------------------
char* last_error_buffer();  // thread-local, 512 bytes

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(DCP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return DCP_OK;
}

// Compute units of the current device (asked once per device; 256 if the query fails).
inline int device_cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

#define DCP_REQUIRE(cond, ...) \
  do {                         \
    if (!(cond)) return ::dcp::fail(DCP_ERR_ARG, __VA_ARGS__); \
  } while (0)

// ---- optional per-kernel timing (off by default) -----------------------------
// While enabled through dcp_profile_enable(1), every kernel launch is bracketed
// by two events recorded on the launch stream; dcp_profile_report() waits for
// them and sums the elapsed time per kernel name.  Nothing is recorded, created
// or synchronised when profiling is off.
bool profiling_enabled();
int profile_begin(const char* name, hipStream_t stream);  // the span's index, or -1 if no events could be made
void profile_end(int span, hipStream_t stream);

struct KernelTimer {
  hipStream_t stream;
  int span;
  KernelTimer(const char* name, void* s) : stream((hipStream_t)s), span(-1) {
    if (profiling_enabled()) span = profile_begin(name, stream);
  }
  ~KernelTimer() {
    if (span >= 0) profile_end(span, stream);
  }
};

// ---- 16-byte vector --------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- storage types -----------------------------------------------------------
// bf16 <-> fp32 with round-to-nearest-even (the rounding torch uses).
__device__ __forceinline__ float bf16_to_f32(uint16_t x) {
  return __uint_as_float(((uint32_t)x) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float f16_to_f32(uint16_t x) {
  _Float16 h;
  __builtin_memcpy(&h, &x, 2);
  return (float)h;
}
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  _Float16 h = (_Float16)f;
  uint16_t x;
  __builtin_memcpy(&x, &h, 2);
  return x;
}

template <int DTYPE>
struct Elem;
template <>
struct Elem<DCP_DTYPE_BF16> {
  typedef uint16_t raw;
  static __device__ __forceinline__ float load(raw x) { return bf16_to_f32(x); }
  static __device__ __forceinline__ raw store(float f) { return f32_to_bf16(f); }
};
template <>
struct Elem<DCP_DTYPE_FP16> {
  typedef uint16_t raw;
  static __device__ __forceinline__ float load(raw x) { return f16_to_f32(x); }
  static __device__ __forceinline__ raw store(float f) { return f32_to_f16(f); }
};
template <>
struct Elem<DCP_DTYPE_FP32> {
  typedef float raw;
  static __device__ __forceinline__ float load(raw x) { return x; }
  static __device__ __forceinline__ raw store(float f) { return f; }
};

inline int dtype_size(int dtype) {
  switch (dtype) {
    case DCP_DTYPE_BF16:
    case DCP_DTYPE_FP16:
      return 2;
    case DCP_DTYPE_FP32:
      return 4;
    default:
      return 0;
  }
}

}  // namespace dcp
