// A host that is neither Python nor torch: plain C++ with the HIP runtime, calling libdcp_hip.so
// through include/dcp_hip.h only.  It gathers two ragged blocks into padded slots, runs the
// range-masked attention forward over them, and sums two partial blocks; every result is checked
// against loops on the CPU.  Exit status 0 = all checks passed.  Built by the package's build
// step into tests/abi_host/abi_host_check and run by tests/test_abi_host_gpu.py.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "dcp_hip.h"

#define HIP_OK(call)                                                                  \
  do {                                                                                \
    hipError_t e_ = (call);                                                           \
    if (e_ != hipSuccess) {                                                           \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      return 2;                                                                       \
    }                                                                                 \
  } while (0)
#define DCP_OK_OR_FAIL(call)                                             \
  do {                                                                   \
    int rc_ = (call);                                                    \
    if (rc_ != 0) {                                                      \
      fprintf(stderr, "%s -> %d: %s\n", #call, rc_, dcp_last_error());   \
      return 3;                                                          \
    }                                                                    \
  } while (0)

static uint16_t to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static float rnd(uint32_t& s) {  // uniform in [-1, 1)
  s = s * 1664525u + 1013904223u;
  return (float)(s >> 8) / 8388608.0f - 1.0f;
}

template <typename T>
static T* to_device(const std::vector<T>& v) {
  T* d = nullptr;
  if (hipMalloc(&d, v.size() * sizeof(T) + 16) != hipSuccess) return nullptr;
  if (hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return d;
}

int main() {
  if (dcp_version() < 100) return 1;
  int n_dev = 0;
  HIP_OK(hipGetDeviceCount(&n_dev));
  if (n_dev < 1) {
    fprintf(stderr, "no GPU\n");
    return 2;
  }
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  // ---- problem: one sequence of 100 tokens, 2 q heads sharing 1 kv head, D = 64, causal,
  // blocks of 64 tokens: q/kv blocks of 64 and 36 tokens -------------------------------------
  const int T = 100, BS = 64, H = 2, HKV = 1, D = 64, NB = 2;
  const int lens[NB] = {64, 36};
  uint32_t seed = 12345;
  std::vector<uint16_t> q_local((size_t)T * H * D), kv_local((size_t)T * 2 * HKV * D);
  for (auto& x : q_local) x = to_bf16(rnd(seed));
  for (auto& x : kv_local) x = to_bf16(rnd(seed));
  uint16_t* d_q_local = to_device(q_local);
  uint16_t* d_kv_local = to_device(kv_local);
  uint16_t *d_q_buf, *d_kv_buf, *d_out_buf;
  float* d_lse;
  HIP_OK(hipMalloc(&d_q_buf, (size_t)NB * BS * H * D * 2));
  HIP_OK(hipMalloc(&d_kv_buf, (size_t)NB * BS * 2 * HKV * D * 2));
  HIP_OK(hipMalloc(&d_out_buf, (size_t)NB * BS * H * D * 2));
  HIP_OK(hipMalloc(&d_lse, (size_t)H * NB * BS * 4));
  HIP_OK(hipMemset(d_q_buf, 0, (size_t)NB * BS * H * D * 2));
  HIP_OK(hipMemset(d_kv_buf, 0, (size_t)NB * BS * 2 * HKV * D * 2));

  // ---- gather: local (unpadded) -> padded slots, one copy call for q and kv blocks ----------
  std::vector<int64_t> src_ptrs, dst_ptrs;
  std::vector<int32_t> src_off, src_str, dst_off, dst_str, n_el;
  int tok = 0;
  for (int b = 0; b < NB; ++b) {
    src_ptrs.push_back((int64_t)d_q_local);
    src_off.push_back(tok);
    src_str.push_back(H * D);
    dst_ptrs.push_back((int64_t)d_q_buf);
    dst_off.push_back(b * BS);
    dst_str.push_back(H * D);
    n_el.push_back(lens[b] * H * D);
    src_ptrs.push_back((int64_t)d_kv_local);
    src_off.push_back(tok);
    src_str.push_back(2 * HKV * D);
    dst_ptrs.push_back((int64_t)d_kv_buf);
    dst_off.push_back(b * BS);
    dst_str.push_back(2 * HKV * D);
    n_el.push_back(lens[b] * 2 * HKV * D);
    tok += lens[b];
  }
  int64_t *d_sp = to_device(src_ptrs), *d_dp = to_device(dst_ptrs);
  int32_t *d_so = to_device(src_off), *d_ss = to_device(src_str), *d_do = to_device(dst_off), *d_ds = to_device(dst_str),
          *d_ne = to_device(n_el);
  DCP_OK_OR_FAIL(dcp_fused_copy_varlen(d_sp, d_so, d_ss, d_dp, d_do, d_ds, d_ne, (int)src_ptrs.size(),
                                       (int64_t)BS * H * D, 2, stream));

  // ---- attention forward: row b = q block b against kv blocks 0..b, causal ranges -----------
  std::vector<int32_t> cu_q = {0, 64, 100}, cu_kv = {0, 64, 164};  // row 1 sees 64 + 36 keys
  std::vector<int32_t> range((size_t)2 * T);
  for (int t = 0; t < T; ++t) {
    range[t] = 0;          // start
    range[T + t] = t + 1;  // end (kv position within the row's concatenated blocks = global position here)
  }
  std::vector<int32_t> q_table = {0, 1}, kv_table = {0, -1, 0, 1}, out_table = {0, 1};
  int32_t *d_cuq = to_device(cu_q), *d_cukv = to_device(cu_kv), *d_rng = to_device(range), *d_qt = to_device(q_table),
          *d_kvt = to_device(kv_table), *d_ot = to_device(out_table);
  void* d_ws;
  HIP_OK(hipMalloc(&d_ws, dcp_attn_fwd_workspace_bytes()));
  const uint16_t* k_base = d_kv_buf;                 // [slot][token][2][HKV][D]: K at +0, V at +HKV*D
  const uint16_t* v_base = d_kv_buf + HKV * D;
  const float scale = 1.0f / sqrtf((float)D);
  DCP_OK_OR_FAIL(dcp_attn_fwd(d_q_buf, k_base, v_base, d_out_buf, d_lse, d_cuq, d_cukv, d_rng, 1, d_qt, d_kvt, d_ot,
                              nullptr, NB, 2, T, BS, H, HKV, D, (int64_t)BS * 2 * HKV * D, (int64_t)2 * HKV * D, NB,
                              scale, DCP_DTYPE_BF16, d_ws, dcp_attn_fwd_workspace_bytes(), stream));

  // ---- block sum: out block 0 + out block 1 (first 36 tokens) -> a third buffer -------------
  uint16_t* d_sum;
  HIP_OK(hipMalloc(&d_sum, (size_t)BS * H * D * 2));
  std::vector<int64_t> sum_src = {(int64_t)d_out_buf}, sum_dst = {(int64_t)d_sum};
  std::vector<int32_t> sum_offs = {0, 1}, sum_stride = {BS * H * D}, sum_nops = {2}, sum_dofs = {0}, sum_dstr = {1},
                       sum_n = {36 * H * D};
  int64_t *d_ssrc = to_device(sum_src), *d_sdst = to_device(sum_dst);
  int32_t *d_soffs = to_device(sum_offs), *d_sstr = to_device(sum_stride), *d_snops = to_device(sum_nops),
          *d_sdofs = to_device(sum_dofs), *d_sdstr = to_device(sum_dstr), *d_sn = to_device(sum_n);
  DCP_OK_OR_FAIL(dcp_blockwise_sum(d_ssrc, d_soffs, d_sstr, d_snops, d_sdst, d_sdofs, d_sdstr, d_sn, 1, 2,
                                   (int64_t)BS * H * D, DCP_DTYPE_BF16, stream));
  HIP_OK(hipStreamSynchronize(stream));

  // ---- checks ---------------------------------------------------------------------------------
  std::vector<uint16_t> q_buf((size_t)NB * BS * H * D), out_buf(q_buf.size()), sum_buf((size_t)BS * H * D);
  std::vector<float> lse((size_t)H * NB * BS);
  HIP_OK(hipMemcpy(q_buf.data(), d_q_buf, q_buf.size() * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(out_buf.data(), d_out_buf, out_buf.size() * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(sum_buf.data(), d_sum, sum_buf.size() * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(lse.data(), d_lse, lse.size() * 4, hipMemcpyDeviceToHost));
  int bad = 0;
  // gather is a byte copy
  tok = 0;
  for (int b = 0; b < NB; ++b) {
    if (memcmp(&q_buf[(size_t)b * BS * H * D], &q_local[(size_t)tok * H * D], (size_t)lens[b] * H * D * 2) != 0) {
      fprintf(stderr, "gathered q block %d differs\n", b);
      ++bad;
    }
    tok += lens[b];
  }
  // attention against a double-precision loop over the same (rounded) inputs
  double max_out = 0.0, max_lse = 0.0;
  for (int t = 0; t < T; ++t)
    for (int h = 0; h < H; ++h) {
      std::vector<double> s(t + 1);
      double m = -1e300;
      for (int j = 0; j <= t; ++j) {
        double acc = 0.0;
        for (int d = 0; d < D; ++d)
          acc += (double)from_bf16(q_local[((size_t)t * H + h) * D + d]) * from_bf16(kv_local[((size_t)j * 2 + 0) * HKV * D + d]);
        s[j] = acc * scale;
        if (s[j] > m) m = s[j];
      }
      double l = 0.0;
      for (int j = 0; j <= t; ++j) l += exp(s[j] - m);
      const int b = t < 64 ? 0 : 1, i = t < 64 ? t : t - 64;
      const double lse_ref = m + log(l);
      const double e_lse = fabs(lse_ref - lse[((size_t)h * NB + b) * BS + i]);
      if (e_lse > max_lse) max_lse = e_lse;
      for (int d = 0; d < D; ++d) {
        double o = 0.0;
        for (int j = 0; j <= t; ++j) o += exp(s[j] - m) / l * from_bf16(kv_local[((size_t)j * 2 + 1) * HKV * D + d]);
        const double e = fabs(o - from_bf16(out_buf[(((size_t)b * BS + i) * H + h) * D + d]));
        if (e > max_out) max_out = e;
      }
    }
  if (max_out > 2e-2 || max_lse > 1e-3) {
    fprintf(stderr, "attention: max |out| error %.4g (limit 2e-2), max |lse| error %.4g (limit 1e-3)\n", max_out, max_lse);
    ++bad;
  }
  // block sum in fp32 with one rounding
  double max_sum = 0.0;
  for (size_t i = 0; i < (size_t)36 * H * D; ++i) {
    const float want = from_bf16(to_bf16(from_bf16(out_buf[i]) + from_bf16(out_buf[(size_t)BS * H * D + i])));
    const double e = fabs((double)want - from_bf16(sum_buf[i]));
    if (e > max_sum) max_sum = e;
  }
  if (max_sum != 0.0) {
    fprintf(stderr, "block sum differs from the fp32 sum rounded once: max error %.4g\n", max_sum);
    ++bad;
  }
  // an argument error is reported through the status and the message, nothing is launched
  if (dcp_fused_copy_varlen(d_sp, d_so, d_ss, d_dp, d_do, d_ds, d_ne, 1, 16, 3, stream) == 0 ||
      strlen(dcp_last_error()) == 0) {
    fprintf(stderr, "a bad element size was not rejected\n");
    ++bad;
  }
  printf("abi_host_check: gather exact, attention max errors out %.3g lse %.3g, block sum exact: %s\n", max_out, max_lse,
         bad ? "FAILED" : "ok");
  return bad ? 1 : 0;
}
