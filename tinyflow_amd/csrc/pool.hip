// 2-D pooling forward/backward (max, and mean with padding counted).
//
// Replaces cudnnPoolingForward / cudnnPoolingBackward and the descriptor
// builder (src/gpu_op.cu:2839-3024).  NCHW; lanes run along the innermost (w / q)
// index so loads and stores coalesce.
//
// Max-pool backward runs in two passes: one lane per WINDOW records the tap that
// holds the window's maximum (among equal maxima the first one in row-major
// window order), then one lane per INPUT pixel gathers dy from the (few) windows
// that cover it and name it.  A gather needs no atomics, so the result is
// deterministic even when windows overlap (3x3 stride 2), and the forward output
// y is not needed.
//
// Element indices are 32-bit (tensors hold fewer than 2^31 elements) and are split
// into (plane, row, column) with magic-number divisions: 64-bit integer division,
// which the compiler emits for int64 indices, costs more than the memory traffic.
#include "gemm_core.h"
#include "internal.h"

#include <type_traits>

#include <algorithm>

using namespace tf;
using tf::gemm::FastDiv;

namespace {

constexpr int kThreads = 256;

struct PoolParams {
  int C, H, W, P, Q;
  int pad_h, pad_w, u, v, fh, fw;
  FastDiv div_pq, div_q, div_hw, div_w;
};

template <bool MAX>
__global__ __launch_bounds__(kThreads) void pool_forward_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                               PoolParams pp, uint32_t total) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    uint32_t nc, pix, p, q;
    pp.div_pq.divmod(i, nc, pix);
    pp.div_q.divmod(pix, p, q);
    const int h0 = (int)p * pp.u - pp.pad_h, w0 = (int)q * pp.v - pp.pad_w;
    const float *plane = x + (int64_t)nc * pp.H * pp.W;
    float acc = MAX ? -INFINITY : 0.f;
    for (int r = 0; r < pp.fh; ++r) {
      const int h = h0 + r;
      if ((unsigned)h >= (unsigned)pp.H) continue;
      for (int s = 0; s < pp.fw; ++s) {
        const int w = w0 + s;
        if ((unsigned)w >= (unsigned)pp.W) continue;
        const float val = plane[h * pp.W + w];
        if (MAX) acc = val > acc ? val : acc;
        else acc += val;
      }
    }
    y[i] = MAX ? acc : acc / (float)(pp.fh * pp.fw);
  }
}

__device__ inline int ceil_div_floor0(int a, int b) {  // ceil(a / b) clamped at 0, b > 0
  return a <= 0 ? 0 : (a + b - 1) / b;
}

// Tap (r * fw + s) that holds the first maximum of window (p, q) of `plane` in
// row-major order; 255 when the window holds no comparable value (all NaN).
__device__ inline int window_argmax(const float *__restrict__ plane, const PoolParams &pp, int p, int q) {
  const int h0 = p * pp.u - pp.pad_h, w0 = q * pp.v - pp.pad_w;
  float best = -INFINITY;
  int arg = 255;
  for (int r = 0; r < pp.fh; ++r) {
    const int h = h0 + r;
    if ((unsigned)h >= (unsigned)pp.H) continue;
    for (int s = 0; s < pp.fw; ++s) {
      const int w = w0 + s;
      if ((unsigned)w >= (unsigned)pp.W) continue;
      const float val = plane[h * pp.W + w];
      if (val > best || (arg == 255 && val == best)) {  // strict: the first maximum wins
        best = val;
        arg = r * pp.fw + s;
      }
    }
  }
  return arg;
}

// Max-pool backward, pass 1: one lane per window records the window's arg-max tap.
__global__ __launch_bounds__(kThreads) void pool_argmax_kernel(const float *__restrict__ x,
                                                              unsigned char *__restrict__ tap, PoolParams pp,
                                                              uint32_t total) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    uint32_t nc, pix, p, q;
    pp.div_pq.divmod(i, nc, pix);
    pp.div_q.divmod(pix, p, q);
    tap[i] = (unsigned char)window_argmax(x + (int64_t)nc * pp.H * pp.W, pp, (int)p, (int)q);
  }
}

// Pass 2 (max) / the whole backward (mean): one lane per INPUT pixel gathers dy
// from the windows that cover it.  With MAX and no tap array (the scratch for it
// could not be allocated) every covering window's arg-max is recomputed from x:
// slower, same bits, no memory beyond the operands.
template <bool MAX>
__global__ __launch_bounds__(kThreads) void pool_backward_kernel(const unsigned char *__restrict__ tap,
                                                                const float *__restrict__ x,
                                                                const float *__restrict__ dy,
                                                                float *__restrict__ dx, PoolParams pp,
                                                                uint32_t total) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    uint32_t nc, pix, hh, ww;
    pp.div_hw.divmod(i, nc, pix);
    pp.div_w.divmod(pix, hh, ww);
    const int h = (int)hh, w = (int)ww;
    // windows (p, q) with p*u - pad <= h <= p*u - pad + fh - 1
    const int p_lo = ceil_div_floor0(h + pp.pad_h - pp.fh + 1, pp.u);
    int p_hi = (h + pp.pad_h) / pp.u;
    if (p_hi > pp.P - 1) p_hi = pp.P - 1;
    const int q_lo = ceil_div_floor0(w + pp.pad_w - pp.fw + 1, pp.v);
    int q_hi = (w + pp.pad_w) / pp.v;
    if (q_hi > pp.Q - 1) q_hi = pp.Q - 1;
    const int64_t win_base = (int64_t)nc * pp.P * pp.Q;
    float acc = 0.f;
    for (int p = p_lo; p <= p_hi; ++p) {
      const int r = h - (p * pp.u - pp.pad_h);
      for (int q = q_lo; q <= q_hi; ++q) {
        const int64_t wi = win_base + p * pp.Q + q;
        if (MAX) {
          const int s = w - (q * pp.v - pp.pad_w);
          const int t = tap ? (int)tap[wi] : window_argmax(x + (int64_t)nc * pp.H * pp.W, pp, p, q);
          if (t == r * pp.fw + s) acc += dy[wi];
        } else {
          acc += dy[wi];
        }
      }
    }
    dx[i] = MAX ? acc : acc / (float)(pp.fh * pp.fw);
  }
}

// Max-pool backward, pass 2, for strides with u * v <= 4 (every configuration of
// the reference models): one lane owns a u x v cell of dx aligned with the stride
// grid.  The windows that can reach the cell are visited once each -- one tap byte
// and at most one dy load per window -- instead of once per dx element, which cuts
// the loads per element of dx by u * v.  The sum over windows runs in the same
// (p, q) order as in the per-element kernel, so both give the same bits.
__global__ __launch_bounds__(kThreads) void pool_backward_cell_kernel(const unsigned char *__restrict__ tap,
                                                                     const float *__restrict__ dy,
                                                                     float *__restrict__ dx, PoolParams pp,
                                                                     FastDiv div_cells, FastDiv div_cw, int cells_h,
                                                                     int cells_w, uint32_t total_cells, bool pairs) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < total_cells; i += stride) {
    uint32_t nc, cell, ci, cj;
    div_cells.divmod(i, nc, cell);
    div_cw.divmod(cell, ci, cj);
    const int h0 = (int)ci * pp.u, w0 = (int)cj * pp.v;
    const int p_lo = ceil_div_floor0(h0 + pp.pad_h - pp.fh + 1, pp.u);
    int p_hi = (h0 + pp.u - 1 + pp.pad_h) / pp.u;
    if (p_hi > pp.P - 1) p_hi = pp.P - 1;
    const int q_lo = ceil_div_floor0(w0 + pp.pad_w - pp.fw + 1, pp.v);
    int q_hi = (w0 + pp.v - 1 + pp.pad_w) / pp.v;
    if (q_hi > pp.Q - 1) q_hi = pp.Q - 1;
    const int64_t win_base = (int64_t)nc * pp.P * pp.Q;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int p = p_lo; p <= p_hi; ++p) {
      for (int q = q_lo; q <= q_hi; ++q) {
        const int64_t wi = win_base + p * pp.Q + q;
        const int t = (int)tap[wi];
        const int r = t / pp.fw, sft = t - r * pp.fw;
        const int dh = p * pp.u - pp.pad_h + r - h0, dw = q * pp.v - pp.pad_w + sft - w0;
        if (t != 255 && (unsigned)dh < (unsigned)pp.u && (unsigned)dw < (unsigned)pp.v) {
          const float g = dy[wi];
          const int slot = dh * pp.v + dw;
          // register-resident accumulators: select instead of indexing
          acc[0] += slot == 0 ? g : 0.f;
          acc[1] += slot == 1 ? g : 0.f;
          acc[2] += slot == 2 ? g : 0.f;
          acc[3] += slot == 3 ? g : 0.f;
        }
      }
    }
    float *plane = dx + (int64_t)nc * pp.H * pp.W;
    if (pairs) {  // v == 2, W even, dx 8-byte aligned: a cell row is one 8-byte store
      *reinterpret_cast<float2 *>(plane + h0 * pp.W + w0) = make_float2(acc[0], acc[1]);
      if (pp.u == 2 && h0 + 1 < pp.H)
        *reinterpret_cast<float2 *>(plane + (h0 + 1) * pp.W + w0) = make_float2(acc[2], acc[3]);
      continue;
    }
    for (int dh = 0; dh < pp.u; ++dh)
      for (int dw = 0; dw < pp.v; ++dw) {
        const int h = h0 + dh, w = w0 + dw;
        if (h < pp.H && w < pp.W) {
          const int slot = dh * pp.v + dw;
          plane[h * pp.W + w] = slot == 0 ? acc[0] : slot == 1 ? acc[1] : slot == 2 ? acc[2] : acc[3];
        }
      }
  }
}

// Max-pool backward in one pass for the window shapes of the reference models
// (3x3 and 2x2 at stride 2; template arguments, so every loop below unrolls and
// every division is by a constant) on planes too large for the whole-plane kernel
// further down (more than 128 x 128 elements).  A workgroup owns a 16 x 64 tile of dx: it
// stages the part of x that the tile's windows read in LDS, finds each window's
// arg-max tap there (same scan as window_argmax, so the same tap), keeps tap and
// dy per window in LDS, and then every lane gathers four consecutive dx elements
// from the windows that cover them, in the (p, q) order of the two-pass kernels:
// same bits, x / dy / dx cross HBM once, and no scratch memory.
constexpr int kTileH = 16, kTileW = 64;

template <int FH, int FW, int U, int V>
__global__ __launch_bounds__(kThreads) void pool_max_backward_tile_kernel(const float *__restrict__ x,
                                                                         const float *__restrict__ dy,
                                                                         float *__restrict__ dx, PoolParams pp,
                                                                         FastDiv div_tiles, FastDiv div_tw,
                                                                         bool vec4) {
  // windows that can touch the tile, and the rows / columns of x they read
  constexpr int NP = (kTileH + FH - 2) / U + 2, NQ = (kTileW + FW - 2) / V + 2;
  constexpr int RH = (NP - 1) * U + FH, RW = (NQ - 1) * V + FW;
  __shared__ float xs[RH][RW + 1];
  __shared__ float gs[NP][NQ];
  __shared__ unsigned char ts[NP][NQ];
  uint32_t nc, tile, ti, tj;
  div_tiles.divmod(blockIdx.x, nc, tile);
  div_tw.divmod(tile, ti, tj);
  const int h0 = (int)ti * kTileH, w0 = (int)tj * kTileW;
  // first window row / column that can reach the tile (may lie before window 0)
  const int p_first = (h0 + pp.pad_h - FH + 1 >= 0) ? (h0 + pp.pad_h - FH + U) / U : 0;
  const int q_first = (w0 + pp.pad_w - FW + 1 >= 0) ? (w0 + pp.pad_w - FW + V) / V : 0;
  const int xr0 = p_first * U - pp.pad_h, xc0 = q_first * V - pp.pad_w;  // may be negative
  const int tid = threadIdx.x;
  const float *plane = x + (int64_t)nc * pp.H * pp.W;
  // all loads of a lane are issued before the first one is used
  constexpr int XPT = (RH * RW + kThreads - 1) / kThreads, WPT = (NP * NQ + kThreads - 1) / kThreads;
  float xv[XPT];
#pragma unroll
  for (int e = 0; e < XPT; ++e) {
    const int i = tid + e * kThreads;
    const int r = i / RW, c = i - r * RW;
    const int h = xr0 + r, w = xc0 + c;
    xv[e] = (i < RH * RW && (unsigned)h < (unsigned)pp.H && (unsigned)w < (unsigned)pp.W) ? plane[h * pp.W + w] : 0.f;
  }
  const float *gplane = dy + (int64_t)nc * pp.P * pp.Q;
  float gv[WPT];
#pragma unroll
  for (int e = 0; e < WPT; ++e) {
    const int i = tid + e * kThreads;
    const int pi = i / NQ, qi = i - pi * NQ;
    const int p = p_first + pi, q = q_first + qi;
    gv[e] = (i < NP * NQ && p < pp.P && q < pp.Q) ? gplane[p * pp.Q + q] : 0.f;
  }
#pragma unroll
  for (int e = 0; e < XPT; ++e) {
    const int i = tid + e * kThreads;
    const int r = i / RW, c = i - r * RW;
    if (i < RH * RW) xs[r][c] = xv[e];
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < WPT; ++e) {
    const int i = tid + e * kThreads;
    if (i >= NP * NQ) break;
    const int pi = i / NQ, qi = i - pi * NQ;
    const int p = p_first + pi, q = q_first + qi;
    int arg = 255;
    const float g = gv[e];
    if (p < pp.P && q < pp.Q) {
      float best = -INFINITY;
#pragma unroll
      for (int r = 0; r < FH; ++r) {
        const int h = xr0 + pi * U + r;
#pragma unroll
        for (int sft = 0; sft < FW; ++sft) {
          const int w = xc0 + qi * V + sft;
          if ((unsigned)h < (unsigned)pp.H && (unsigned)w < (unsigned)pp.W) {
            const float val = xs[pi * U + r][qi * V + sft];
            if (val > best || (arg == 255 && val == best)) {
              best = val;
              arg = r * FW + sft;
            }
          }
        }
      }
    }
    ts[pi][qi] = (unsigned char)arg;
    gs[pi][qi] = g;
  }
  __syncthreads();
  const int h = h0 + tid / (kTileW / 4), wq = w0 + (tid % (kTileW / 4)) * 4;
  if (h >= pp.H || wq >= pp.W) return;
  float out[4];
  // windows covering row h: p*U - pad <= h <= p*U - pad + FH - 1
  const int a_h = h + pp.pad_h - FH + 1;
  const int pl = a_h <= 0 ? 0 : (a_h + U - 1) / U, ph = (h + pp.pad_h) / U;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int w = wq + k;
    const int a_w = w + pp.pad_w - FW + 1;
    const int ql = a_w <= 0 ? 0 : (a_w + V - 1) / V, qh = (w + pp.pad_w) / V;
    float acc = 0.f;
#pragma unroll
    for (int dp = 0; dp < (FH + U - 1) / U; ++dp) {
      const int p = pl + dp;
      if (p > ph) break;
      const int r = h - (p * U - pp.pad_h);
#pragma unroll
      for (int dq = 0; dq < (FW + V - 1) / V; ++dq) {
        const int q = ql + dq;
        if (q > qh) break;
        // windows past P / Q hold tap 255 and never match
        if ((int)ts[p - p_first][q - q_first] == r * FW + (w - (q * V - pp.pad_w))) acc += gs[p - p_first][q - q_first];
      }
    }
    out[k] = acc;
  }
  float *dst = dx + (int64_t)nc * pp.H * pp.W + h * pp.W + wq;
  if (vec4 && wq + 3 < pp.W) {
    *reinterpret_cast<float4 *>(dst) = make_float4(out[0], out[1], out[2], out[3]);
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (wq + k < pp.W) dst[k] = out[k];
  }
}

// One-pass max-pool backward for planes that fit in LDS whole (up to 128 x 128 with at
// most 4096 windows) and stride-2 windows of 2x2 or 3x3: one workgroup of 1024 lanes per
// (image, channel) plane
//   1. stages the plane of x with coalesced loads,
//   2. finds every window's arg-max tap there (the scan of window_argmax: same tap),
//   3. clears the plane and lets every window add its dy at its arg-max position, in
//      four rounds -- windows with (p % 2, q % 2) = (0,0), (0,1), (1,0), (1,1); the
//      windows of one round are two apart in both directions and cannot touch the
//      same element, so the adds need no atomics and every element receives its up
//      to four contributions in a fixed order,
//   4. streams the plane out as dx.
// x, dy and dx cross HBM exactly once and the work per element is a fraction of the
// gather form's (which tests up to four windows per dx element).  Overlapping windows
// are summed in round order rather than in (p, q) order, so the last bit of such a sum
// can differ from the other forms; run to run it is the same.
// VEC: H*W a multiple of 4 and 16-byte aligned planes.
constexpr int kPlaneMaxFloats = 16384, kPlaneThreads = 1024, kPlaneWindowsPerLane = 4;

template <int FH, int FW, bool VEC>
__global__ __launch_bounds__(kPlaneThreads) void pool_max_backward_plane_kernel(const float *__restrict__ x,
                                                                               const float *__restrict__ dy,
                                                                               float *__restrict__ dx,
                                                                               PoolParams pp) {
  constexpr int U = 2, V = 2;
  extern __shared__ float plane_lds[];
  typedef float f32x4p __attribute__((ext_vector_type(4)));
  const int HW = pp.H * pp.W, PQ = pp.P * pp.Q;
  const int tid = threadIdx.x;
  const float *plane = x + (int64_t)blockIdx.x * HW;
  const int n4 = VEC ? HW / 4 : 0;
  {
    const f32x4p *src = reinterpret_cast<const f32x4p *>(plane);
    f32x4p *dst = reinterpret_cast<f32x4p *>(plane_lds);
    f32x4p v[4];  // 4 x 1024 lanes x 4 floats cover the largest plane
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (tid + k * kPlaneThreads < n4) v[k] = __builtin_nontemporal_load(src + tid + k * kPlaneThreads);
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (tid + k * kPlaneThreads < n4) dst[tid + k * kPlaneThreads] = v[k];
    for (int i = n4 * 4 + tid; i < HW; i += kPlaneThreads) plane_lds[i] = plane[i];
  }
  const float *gplane = dy + (int64_t)blockIdx.x * PQ;
  float gv[kPlaneWindowsPerLane];
  int target[kPlaneWindowsPerLane];  // element of the plane that receives the window's dy, -1: none
  int round_of[kPlaneWindowsPerLane];
#pragma unroll
  for (int k = 0; k < kPlaneWindowsPerLane; ++k) {
    const int i = tid + k * kPlaneThreads;
    gv[k] = i < PQ ? gplane[i] : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kPlaneWindowsPerLane; ++k) {
    const int i = tid + k * kPlaneThreads;
    target[k] = -1;
    round_of[k] = -1;
    if (i < PQ) {
      uint32_t p, q;
      pp.div_q.divmod((uint32_t)i, p, q);
      round_of[k] = (int)((p & 1u) * 2u + (q & 1u));
      float best = -INFINITY;
#pragma unroll
      for (int r = 0; r < FH; ++r) {
        const int h = (int)p * U - pp.pad_h + r;
#pragma unroll
        for (int sft = 0; sft < FW; ++sft) {
          const int w = (int)q * V - pp.pad_w + sft;
          if ((unsigned)h < (unsigned)pp.H && (unsigned)w < (unsigned)pp.W) {
            const float val = plane_lds[h * pp.W + w];
            if (val > best || (target[k] < 0 && val == best)) {
              best = val;
              target[k] = h * pp.W + w;
            }
          }
        }
      }
    }
  }
  __syncthreads();  // every window has read its taps: the plane's LDS becomes the dx plane
  {
    f32x4p *dst = reinterpret_cast<f32x4p *>(plane_lds);
    const f32x4p zero = {0.f, 0.f, 0.f, 0.f};
    for (int i = tid; i < (HW + 3) / 4; i += kPlaneThreads) dst[i] = zero;
  }
  __syncthreads();
#pragma unroll
  for (int round = 0; round < 4; ++round) {
    if (FH > U || FW > V || round == 0) {  // disjoint windows need no rounds: all in the first
#pragma unroll
      for (int k = 0; k < kPlaneWindowsPerLane; ++k) {
        const bool mine = (FH > U || FW > V) ? round_of[k] == round : round_of[k] >= 0;
        if (mine && target[k] >= 0) plane_lds[target[k]] += gv[k];
      }
      if (FH > U || FW > V) __syncthreads();
    }
  }
  if (!(FH > U || FW > V)) __syncthreads();
  float *out_plane = dx + (int64_t)blockIdx.x * HW;
  {
    const f32x4p *src = reinterpret_cast<const f32x4p *>(plane_lds);
    f32x4p *dst = reinterpret_cast<f32x4p *>(out_plane);
    for (int i = tid; i < n4; i += kPlaneThreads) dst[i] = src[i];
    for (int i = n4 * 4 + tid; i < HW; i += kPlaneThreads) out_plane[i] = plane_lds[i];
  }
}

// Max-pool forward for the same planes and windows: the plane of x is staged in LDS
// with coalesced 16-byte loads and every window reads its taps there, so x crosses HBM
// once (the general kernel fetches each tap from memory, rows of a window a whole image
// row apart).  The scan order and the comparisons are the general kernel's: same bits.
template <int FH, int FW, bool VEC>
__global__ __launch_bounds__(kPlaneThreads) void pool_max_forward_plane_kernel(const float *__restrict__ x,
                                                                              float *__restrict__ y, PoolParams pp) {
  constexpr int U = 2, V = 2;
  extern __shared__ float plane_lds[];
  typedef float f32x4p __attribute__((ext_vector_type(4)));
  const int HW = pp.H * pp.W, PQ = pp.P * pp.Q;
  const int tid = threadIdx.x;
  const float *plane = x + (int64_t)blockIdx.x * HW;
  const int n4 = VEC ? HW / 4 : 0;
  {
    const f32x4p *src = reinterpret_cast<const f32x4p *>(plane);
    f32x4p *dst = reinterpret_cast<f32x4p *>(plane_lds);
    f32x4p v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (tid + k * kPlaneThreads < n4) v[k] = __builtin_nontemporal_load(src + tid + k * kPlaneThreads);
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (tid + k * kPlaneThreads < n4) dst[tid + k * kPlaneThreads] = v[k];
    for (int i = n4 * 4 + tid; i < HW; i += kPlaneThreads) plane_lds[i] = plane[i];
  }
  __syncthreads();
  float *out = y + (int64_t)blockIdx.x * PQ;
  for (int i = tid; i < PQ; i += kPlaneThreads) {
    uint32_t p, q;
    pp.div_q.divmod((uint32_t)i, p, q);
    float acc = -INFINITY;
#pragma unroll
    for (int r = 0; r < FH; ++r) {
      const int h = (int)p * U - pp.pad_h + r;
#pragma unroll
      for (int sft = 0; sft < FW; ++sft) {
        const int w = (int)q * V - pp.pad_w + sft;
        if ((unsigned)h < (unsigned)pp.H && (unsigned)w < (unsigned)pp.W) {
          const float val = plane_lds[h * pp.W + w];
          acc = val > acc ? val : acc;
        }
      }
    }
    out[i] = acc;
  }
}

// Global pooling (the window is the whole, unpadded plane; one output per plane), mean
// mode: a workgroup stages `planes` consecutive planes -- one contiguous run of memory --
// in LDS with coalesced loads, then one lane per plane adds its HW values in the order
// of the general kernel (same bits).  `planes` * HW <= kGlobalFloats.
constexpr int kGlobalFloats = 8192;
__global__ __launch_bounds__(kThreads) void global_mean_forward_kernel(const float *__restrict__ x,
                                                                      float *__restrict__ y, int HW, int planes,
                                                                      int total_planes) {
  __shared__ float xs[kGlobalFloats];
  const int first = blockIdx.x * planes;
  const int here = min(planes, total_planes - first);
  const float *src = x + (int64_t)first * HW;
  for (int i = threadIdx.x; i < here * HW; i += kThreads) xs[i] = src[i];
  __syncthreads();
  if ((int)threadIdx.x < here) {
    float acc = 0.f;
    for (int i = 0; i < HW; ++i) acc += xs[threadIdx.x * HW + i];
    y[first + threadIdx.x] = acc / (float)HW;
  }
}

// its backward: every element of a plane receives dy[plane] / HW
__global__ __launch_bounds__(kThreads) void global_mean_backward_kernel(const float *__restrict__ dy,
                                                                       float *__restrict__ dx, FastDiv div_hw,
                                                                       float hw, uint32_t total) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i < total) dx[i] = dy[div_hw.div(i)] / hw;
}

bool is_global_mean(const PoolDesc *d) {
  return d->mode != 0 && d->fh == d->H && d->fw == d->W && d->pad_h == 0 && d->pad_w == 0 && d->P == 1 && d->Q == 1 &&
         d->H * d->W <= kGlobalFloats;
}

int grid_for(int64_t n) {
  int64_t blocks = (n + kThreads - 1) / kThreads;
  const int64_t cap = (int64_t)num_cus() * 32;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1 : (int)blocks;
}

PoolParams params_of(const PoolDesc *d) {
  return PoolParams{d->C, d->H, d->W, d->P, d->Q, d->pad_h, d->pad_w, d->u, d->v, d->fh, d->fw,
                    FastDiv((uint32_t)(d->P * d->Q)), FastDiv((uint32_t)d->Q), FastDiv((uint32_t)(d->H * d->W)),
                    FastDiv((uint32_t)d->W)};
}

bool shape_is(const DLArray *a, int d0, int d1, int d2, int d3) {
  return a->ndim == 4 && a->shape[0] == d0 && a->shape[1] == d1 && a->shape[2] == d2 && a->shape[3] == d3;
}

// Rows of x that one workgroup of the plane kernels takes: the whole plane when it fits
// in LDS; for unpadded 2x2 / stride-2 windows, whose row pairs are independent of one
// another, otherwise the largest even divisor of H whose band fits (a band of x and its
// rows of y are contiguous in memory, so a band is a plane of fewer rows); 0: no fit.
int plane_band_rows(const PoolDesc *d) {
  const auto fits = [&](int rows, int out_rows) {
    return rows * d->W <= kPlaneMaxFloats && out_rows * d->Q <= kPlaneWindowsPerLane * kPlaneThreads;
  };
  if (fits(d->H, d->P)) return d->H;
  if (!(d->fh == 2 && d->fw == 2 && d->u == 2 && d->v == 2 && d->pad_h == 0 && d->pad_w == 0 && d->H % 2 == 0 &&
        d->P * 2 == d->H))
    return 0;
  for (int rows = d->H - 2; rows >= 2; rows -= 2)
    if (d->H % rows == 0 && fits(rows, rows / 2)) return rows;
  return 0;
}

}  // namespace

extern "C" int DLGpuPooling2DForwardGetOutShape(const int *input_shapes, int *output_shapes, int dataformat,
                                                int poolingMode, const int padding_h, const int padding_w,
                                                const int u, const int v, const int filter_h,
                                                const int filter_w, void ***list) {
  TF_REQUIRE(input_shapes && output_shapes && list, "null argument");
  TF_REQUIRE(dataformat == 0, "only NCHW (dataformat 0) is implemented");
  TF_REQUIRE(poolingMode == 0 || poolingMode == 1, "unknown pooling mode %d", poolingMode);
  TF_REQUIRE(u >= 1 && v >= 1 && filter_h >= 1 && filter_w >= 1 && padding_h >= 0 && padding_w >= 0,
             "bad window geometry");
  for (int i = 0; i < 4; ++i) TF_REQUIRE(input_shapes[i] >= 0, "negative extent");
  TF_REQUIRE(input_shapes[2] + 2 * padding_h >= filter_h && input_shapes[3] + 2 * padding_w >= filter_w,
             "window larger than padded input");
  PoolDesc *d = new PoolDesc();
  d->magic = kMagicPool;
  d->N = input_shapes[0];
  d->C = input_shapes[1];
  d->H = input_shapes[2];
  d->W = input_shapes[3];
  d->mode = poolingMode;
  d->pad_h = padding_h;
  d->pad_w = padding_w;
  d->u = u;
  d->v = v;
  d->fh = filter_h;
  d->fw = filter_w;
  d->P = 1 + (d->H + 2 * padding_h - filter_h) / u;
  d->Q = 1 + (d->W + 2 * padding_w - filter_w) / v;
  output_shapes[0] = d->N;
  output_shapes[1] = d->C;
  output_shapes[2] = d->P;
  output_shapes[3] = d->Q;
  void **slots = (void **)malloc(sizeof(void *) * 3);
  slots[0] = slots[1] = slots[2] = d;
  *list = slots;
  return 0;
}

extern "C" int DLGpuPooling2DForward(const DLArrayHandle input, DLArrayHandle output, void ***list,
                                     void **handle, void **stream) {
  announce_write(output);
  (void)handle;
  PoolDesc *d = desc_from_list<PoolDesc>(list, kMagicPool);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuPooling2DForwardGetOutShape");
  TF_REQUIRE(on_gpu(input) && on_gpu(output), "arrays must live on the GPU");
  TF_REQUIRE(shape_is(input, d->N, d->C, d->H, d->W) && shape_is(output, d->N, d->C, d->P, d->Q),
             "arrays do not match the descriptor");
  hipStream_t s = stream_of(stream);
  const int64_t total = numel(output);
  if (total == 0) return 0;
  TF_REQUIRE(numel(input) < ((int64_t)1 << 31), "tensors of 2^31 elements or more are not supported");
  const PoolParams pp = params_of(d);
  if (is_global_mean(d)) {
    const int HW = d->H * d->W, planes = std::min(kThreads, kGlobalFloats / HW);
    hipLaunchKernelGGL(global_mean_forward_kernel, dim3(cdiv(total, planes)), dim3(kThreads), 0, s,
                       (const float *)input->data, (float *)output->data, HW, planes, (int)total);
    return finish(s, "DLGpuPooling2DForward");
  }
  const bool square2 = d->u == 2 && d->v == 2 && d->fh == d->fw && (d->fh == 2 || d->fh == 3);
  const int band = (d->mode == 0 && square2) ? plane_band_rows(d) : 0;
  if (band > 0) {
    PoolParams bp = pp;  // a band of rows is a plane of fewer rows
    bp.H = band;
    bp.P = band == d->H ? d->P : band / 2;
    const int HW = band * d->W;
    const bool vec = HW % 4 == 0 && (reinterpret_cast<uintptr_t>(input->data) & 15u) == 0;
    const unsigned planes = (unsigned)(d->N * d->C * (d->H / band));
    const size_t lds = (size_t)((HW + 3) / 4 * 4) * sizeof(float);
    const float *xp = (const float *)input->data;
    float *yp = (float *)output->data;
    auto run = [&](auto f_c, auto vec_c) {
      constexpr int F = decltype(f_c)::value;
      constexpr bool VEC = decltype(vec_c)::value;
      hipLaunchKernelGGL((pool_max_forward_plane_kernel<F, F, VEC>), dim3(planes), dim3(kPlaneThreads), lds, s, xp, yp, bp);
    };
    if (d->fh == 3) { if (vec) run(std::integral_constant<int, 3>{}, std::true_type{}); else run(std::integral_constant<int, 3>{}, std::false_type{}); }
    else { if (vec) run(std::integral_constant<int, 2>{}, std::true_type{}); else run(std::integral_constant<int, 2>{}, std::false_type{}); }
    return finish(s, "DLGpuPooling2DForward");
  }
  if (d->mode == 0)
    hipLaunchKernelGGL(pool_forward_kernel<true>, dim3(grid_for(total)), dim3(kThreads), 0, s,
                       (const float *)input->data, (float *)output->data, pp, (uint32_t)total);
  else
    hipLaunchKernelGGL(pool_forward_kernel<false>, dim3(grid_for(total)), dim3(kThreads), 0, s,
                       (const float *)input->data, (float *)output->data, pp, (uint32_t)total);
  return finish(s, "DLGpuPooling2DForward");
}

extern "C" int DLGpuPooling2DBackward(const DLArrayHandle input, const DLArrayHandle output,
                                      const DLArrayHandle doutput, DLArrayHandle dinput, void ***list,
                                      void **handle, void **stream) {
  announce_write(dinput);
  (void)handle;
  PoolDesc *d = desc_from_list<PoolDesc>(list, kMagicPool);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuPooling2DForwardGetOutShape");
  TF_REQUIRE(on_gpu(input) && on_gpu(output) && on_gpu(doutput) && on_gpu(dinput),
             "arrays must live on the GPU");
  TF_REQUIRE(shape_is(input, d->N, d->C, d->H, d->W) && shape_is(dinput, d->N, d->C, d->H, d->W) &&
                 shape_is(output, d->N, d->C, d->P, d->Q) && shape_is(doutput, d->N, d->C, d->P, d->Q),
             "arrays do not match the descriptor");
  hipStream_t s = stream_of(stream);
  const int64_t total = numel(dinput);
  if (total == 0) return 0;
  TF_REQUIRE(total < ((int64_t)1 << 31), "tensors of 2^31 elements or more are not supported");
  const PoolParams pp = params_of(d);
  if (is_global_mean(d)) {
    const int HW = d->H * d->W;
    hipLaunchKernelGGL(global_mean_backward_kernel, dim3(cdiv(total, kThreads)), dim3(kThreads), 0, s,
                       (const float *)doutput->data, (float *)dinput->data, FastDiv((uint32_t)HW), (float)HW,
                       (uint32_t)total);
    return finish(s, "DLGpuPooling2DBackward");
  }
  if (d->mode == 0) {
    TF_REQUIRE(d->fh * d->fw < 255, "max-pool windows of 255 or more taps are not supported");
    const int tiles_h = cdiv(d->H, kTileH), tiles_w = cdiv(d->W, kTileW);
    const int64_t blocks = (int64_t)d->N * d->C * tiles_h * tiles_w;
    const bool square2 = d->u == 2 && d->v == 2 && d->fh == d->fw && (d->fh == 2 || d->fh == 3);
    const int band = square2 ? plane_band_rows(d) : 0;
    if (band > 0) {
      // the plane (or a band of its rows) fits in LDS: one workgroup each, nothing is read twice
      PoolParams bp = pp;
      bp.H = band;
      bp.P = band == d->H ? d->P : band / 2;
      const int HW = band * d->W;
      const bool vec = HW % 4 == 0 && ((reinterpret_cast<uintptr_t>(input->data) |
                                        reinterpret_cast<uintptr_t>(dinput->data)) & 15u) == 0;
      const unsigned planes = (unsigned)(d->N * d->C * (d->H / band));
      const size_t lds = (size_t)((HW + 3) / 4 * 4) * sizeof(float);
      const float *xp = (const float *)input->data, *gp = (const float *)doutput->data;
      float *dp = (float *)dinput->data;
      auto run = [&](auto f_c, auto vec_c) {
        constexpr int F = decltype(f_c)::value;
        constexpr bool VEC = decltype(vec_c)::value;
        hipLaunchKernelGGL((pool_max_backward_plane_kernel<F, F, VEC>), dim3(planes), dim3(kPlaneThreads), lds, s, xp, gp,
                           dp, bp);
      };
      if (d->fh == 3) { if (vec) run(std::integral_constant<int, 3>{}, std::true_type{}); else run(std::integral_constant<int, 3>{}, std::false_type{}); }
      else { if (vec) run(std::integral_constant<int, 2>{}, std::true_type{}); else run(std::integral_constant<int, 2>{}, std::false_type{}); }
      return finish(s, "DLGpuPooling2DBackward");
    }
    if (square2 && blocks < ((int64_t)1 << 31)) {
      const bool vec4 = d->W % 4 == 0 && (reinterpret_cast<uintptr_t>(dinput->data) & 15u) == 0;
      const FastDiv div_tiles((uint32_t)(tiles_h * tiles_w)), div_tw((uint32_t)tiles_w);
      const float *xp = (const float *)input->data, *gp = (const float *)doutput->data;
      float *dp = (float *)dinput->data;
      if (d->fh == 3)
        hipLaunchKernelGGL((pool_max_backward_tile_kernel<3, 3, 2, 2>), dim3((unsigned)blocks), dim3(kThreads), 0, s, xp,
                           gp, dp, pp, div_tiles, div_tw, vec4);
      else
        hipLaunchKernelGGL((pool_max_backward_tile_kernel<2, 2, 2, 2>), dim3((unsigned)blocks), dim3(kThreads), 0, s, xp,
                           gp, dp, pp, div_tiles, div_tw, vec4);
      return finish(s, "DLGpuPooling2DBackward");
    }
    const int64_t windows = numel(doutput);
    // this entry point has no way to report a failed allocation to the caller
    // (no memorytoSaving argument), so it must also work without the scratch
    unsigned char *tap = (unsigned char *)device_alloc((size_t)windows);
    if (tap)
      hipLaunchKernelGGL(pool_argmax_kernel, dim3(grid_for(windows)), dim3(kThreads), 0, s,
                         (const float *)input->data, tap, pp, (uint32_t)windows);
    if (tap && d->u * d->v <= 4) {
      const int cells_h = cdiv(d->H, d->u), cells_w = cdiv(d->W, d->v);
      const int64_t cells = (int64_t)d->N * d->C * cells_h * cells_w;
      hipLaunchKernelGGL(pool_backward_cell_kernel, dim3(grid_for(cells)), dim3(kThreads), 0, s, tap,
                         (const float *)doutput->data, (float *)dinput->data, pp,
                         FastDiv((uint32_t)(cells_h * cells_w)), FastDiv((uint32_t)cells_w), cells_h, cells_w,
                         (uint32_t)cells,
                         pp.v == 2 && pp.W % 2 == 0 && (reinterpret_cast<uintptr_t>(dinput->data) & 7u) == 0);
    } else {
      hipLaunchKernelGGL(pool_backward_kernel<true>, dim3(grid_for(total)), dim3(kThreads), 0, s, tap,
                         (const float *)input->data, (const float *)doutput->data, (float *)dinput->data, pp,
                         (uint32_t)total);
    }
    if (tap) device_free(tap);  // stream-ordered reuse
  } else {
    hipLaunchKernelGGL(pool_backward_kernel<false>, dim3(grid_for(total)), dim3(kThreads), 0, s,
                       (const unsigned char *)nullptr, (const float *)nullptr, (const float *)doutput->data,
                       (float *)dinput->data, pp, (uint32_t)total);
  }
  return finish(s, "DLGpuPooling2DBackward");
}
