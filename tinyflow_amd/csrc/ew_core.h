// Streaming elementwise engine: out[i] = f(a[i], b[i]).
//
// Each lane moves 16-byte vectors, four independent vectors are in flight per
// lane, and the grid is sized to the CU count with a grid-stride loop, so a
// launch is bounded by HBM bandwidth (8 or 12 bytes per element).
#pragma once

#include "internal.h"

namespace tf {
namespace ew {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;

template <class F>
__device__ inline float4 apply4(const F &f, const float4 &a, const float4 &b) {
  return make_float4(f(a.x, b.x), f(a.y, b.y), f(a.z, b.z), f(a.w, b.w));
}

// out[i] = f(a[i], b[i]) over n4 float4 vectors plus a scalar tail.
// out may alias a (in-place SGD), so no restrict qualifiers.
template <class F, bool HAS_A, bool HAS_B>
__global__ __launch_bounds__(kThreads) void ew_kernel(F f, float *out, const float *a, const float *b,
                                                     int64_t n4, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const float4 *a4 = reinterpret_cast<const float4 *>(a);
  const float4 *b4 = reinterpret_cast<const float4 *>(b);
  float4 *o4 = reinterpret_cast<float4 *>(out);
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  for (; i + (kUnroll - 1) * stride < n4; i += kUnroll * stride) {
    float4 va[kUnroll], vb[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      va[u] = HAS_A ? a4[i + u * stride] : zero;
      vb[u] = HAS_B ? b4[i + u * stride] : zero;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) o4[i + u * stride] = apply4(f, va[u], vb[u]);
  }
  for (; i < n4; i += stride) {
    const float4 va = HAS_A ? a4[i] : zero;
    const float4 vb = HAS_B ? b4[i] : zero;
    o4[i] = apply4(f, va, vb);
  }
  // scalar tail (fewer than 4 elements, or everything when a pointer is not
  // 16-byte aligned): one element per lane
  const int64_t t = n4 * 4 + (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (t < n) out[t] = f(HAS_A ? a[t] : 0.f, HAS_B ? b[t] : 0.f);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <class F, bool HAS_A, bool HAS_B>
int launch_ew(F f, float *out, const float *a, const float *b, int64_t n, hipStream_t s, const char *what) {
  if (n <= 0) return 0;
  int64_t n4 = n / 4;
  if (!aligned16(out) || (HAS_A && !aligned16(a)) || (HAS_B && !aligned16(b))) n4 = 0;
  const int64_t tail = n - n4 * 4;
  int64_t blocks = (n4 + (int64_t)kThreads * kUnroll - 1) / ((int64_t)kThreads * kUnroll);
  const int64_t cap = (int64_t)num_cus() * 8;
  if (blocks > cap) blocks = cap;
  const int64_t tail_blocks = (tail + kThreads - 1) / kThreads;
  if (blocks < tail_blocks) blocks = tail_blocks;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((ew_kernel<F, HAS_A, HAS_B>), dim3((unsigned)blocks), dim3(kThreads), 0, s, f, out, a, b,
                     n4, n);
  return finish(s, what);
}

inline int grid_for(int64_t n) {
  int64_t blocks = (n + kThreads - 1) / kThreads;
  const int64_t cap = (int64_t)num_cus() * 8;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1 : (int)blocks;
}

}  // namespace ew
}  // namespace tf
