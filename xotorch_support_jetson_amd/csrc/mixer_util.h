// Small device and host helpers shared by the mixed-layer kernel files (mixers.hip, hybrid.hip).
#pragma once
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "common.h"

namespace xot {
namespace mix {

constexpr int PAGE_TOK = 64;

__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const uint16_t* p) { return bf2f(*p); }
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(uint16_t* p, float v) { *p = f2bf(v); }

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return log1pf(expf(-fabsf(x))) + fmaxf(x, 0.0f); }
__device__ __forceinline__ float logsigmoidf_(float x) { return fminf(x, 0.0f) - log1pf(expf(-fabsf(x))); }

// sum over the workgroup; red: at least (threads / 64) floats of LDS
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = 0.0f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

// sequence of token t: the b with cu[b] <= t < cu[b + 1]
__device__ __forceinline__ int seq_of(const int* cu, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ void ld8(const float* p, float* o) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
  o[0] = a[0]; o[1] = a[1]; o[2] = a[2]; o[3] = a[3]; o[4] = b[0]; o[5] = b[1]; o[6] = b[2]; o[7] = b[3];
}
__device__ __forceinline__ void ld8(const uint16_t* p, float* o) {
  const s16x8 a = ld16(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = bf2f(a[i]);
}

// ------------------------------------------------------------------ host side
#define MCHECK(cond, ...) TORCH_CHECK(cond, "xot mixers: ", __VA_ARGS__)

inline hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }
inline bool is_act(const at::Tensor& t) { return t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat; }
inline void f32c(const at::Tensor& t, const char* name) {
  MCHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, " must be a contiguous fp32 GPU tensor");
}
inline void i32c(const at::Tensor& t, const char* name) {
  MCHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, " must be a contiguous int32 GPU tensor");
}
// fused projection output: fp32 rows of unit inner stride
inline int ld_of(const at::Tensor& P, const char* name) {
  MCHECK(P.is_cuda() && P.scalar_type() == at::kFloat && P.dim() == 2 && P.stride(1) == 1, name, " must be fp32 [T, n] rows");
  return (int)P.stride(0);
}
inline void cols_ok(const at::Tensor& P, int64_t off, int64_t n, const char* what) {
  MCHECK(off >= 0 && n >= 0 && off + n <= P.size(1), what, ": columns [", off, ", ", off + n, ") outside the projection");
}
// activation output rows (bf16 / fp32), maybe a column slice of a wider buffer
inline int act_ld(const at::Tensor& t, int64_t T, int64_t n, const char* name) {
  MCHECK(t.is_cuda() && is_act(t) && t.dim() == 2 && t.size(0) == T && t.size(1) == n && t.stride(1) == 1, name,
         " must be [T, ", n, "] bf16 / fp32 rows");
  return (int)t.stride(0);
}
// activation rows whose first n columns are written (K padding beyond stays untouched)
inline int act_ld_min(const at::Tensor& t, int64_t T, int64_t n, const char* name) {
  MCHECK(t.is_cuda() && is_act(t) && t.dim() == 2 && t.size(0) == T && t.size(1) >= n && t.stride(1) == 1, name,
         " must be [T, >= ", n, "] bf16 / fp32 rows");
  return (int)t.stride(0);
}

}  // namespace mix
}  // namespace xot
