// 2-D convolution forward, grad-data and grad-filter as fp32 MFMA implicit GEMMs.
//
// Replaces cudnnConvolutionForward / BackwardData / BackwardFilter as the
// reference calls them (src/gpu_op.cu:1952-2038, 1739-1824, 1653-1737) and the
// descriptor builder (src/gpu_op.cu:2040-2175).  NCHW activations, KCRS
// filters, cross-correlation, dilation 1, beta = 0.
//
// GEMM views (m x n, reduced over k); no im2col buffer is ever materialised,
// the gather happens in the tile loaders:
//   forward      y [K, (n,p,q)]    = w [K, (c,r,s)]      * x gathered
//   grad-data    dx[C, (n,h,w)]    = w^T[(k,r,s), C]     * dy gathered   (stride 1)
//                dx[C, (n,p,q)]    = w^T[k, C]           * dy            (1x1, any stride;
//                                    each result is scattered to (p*u, q*v) and the rest of
//                                    its u x v cell is zero-filled, so no flop is spent on
//                                    positions that the stride skips)
//   grad-filter  dw[K, (c,r,s)]    = dy[K, (n,p,q)]      * x gathered^T, split along
//                                    (n,p,q) into partial sums added in a fixed order
// All four lane-parallel directions ((n,p,q), (n,h,w), (c,r,s)) are contiguous
// in memory for NCHW/KCRS, so global loads and stores coalesce without any
// layout change of the activations.
#include "gemm_core.h"
#include "gemm_launch.h"
#include "internal.h"

#include <algorithm>
#include <cstring>
#include <cmath>
#include <type_traits>

using namespace tf;
using namespace tf::gemm;

namespace {
typedef float f32x2v __attribute__((ext_vector_type(2)));
typedef unsigned i32x2v __attribute__((__vector_size__(2 * sizeof(unsigned))));   // operand types of the 8- and 16-byte
typedef unsigned i32x4v __attribute__((__vector_size__(4 * sizeof(unsigned))));   // buffer builtins


// ---- gathered operand, lanes along the pixel index ------------------------------
// element(pixel, k): source tensor T[img][ch][Hs][Ws], pixel -> (img, oy, ox),
// k -> (ch, r, s) with (dy, dx) = dir * (r, s); reads T[img][ch][oy*sy+by+dy][ox*sx+bx+dx].
// MODE 0: taps are always inside the image (no padding)      -> no range test
// MODE 1: range test (zero padding)
// MODE 2: additionally the tapped coordinate must be divisible by the conv
//         stride and is divided by it (grad-data of a strided filter larger than 1x1)
template <int D, int BK, int MODE>
struct GatherAlong {
  using Map = AlongMap<D, BK>;
  static constexpr int EPT = Map::EPT;
  const float *base;
  uint32_t bytes;
  int k_extent, n_extent;
  FastDiv div_rs, div_s;     // k -> (ch, r, s): ch = k / (R*S), r = (k % (R*S)) / S
  int ch_stride;             // Hs * Ws
  FastDiv div_img, div_row;  // pixels per image, pixels per row
  int img_stride;            // elements per image of T
  int Hs, Ws;
  int sy, sx, by, bx;
  int dir;                   // +1: dy = r, dx = s (forward); -1: dy = -r, dx = -s (grad-data)
  int R, S;
  FastDiv div_u, div_v;      // MODE 2 only

  struct State {
    Map map;
    __amdgpu_buffer_rsrc_t rsrc;
    // MODE 0/1: byte offset of (img, y0, x0), OOB for a lane past the last pixel;
    // bit r of row_ok / bit s of col_ok says whether tap row r / column s lands
    // inside the image for this lane's pixel (the pixel is fixed for the whole kernel)
    uint32_t lane_off, row_ok, col_ok;
    int img_off, y0, x0;  // MODE 2
    bool ok;
  };
  __device__ inline void init(State &st, int origin, int tid) const {
    st.map.init(tid);
    st.rsrc = make_rsrc(base, bytes);
    const int pix = origin + st.map.d_local;
    st.ok = pix < n_extent;
    uint32_t img, rem, oy, ox;
    div_img.divmod((uint32_t)(st.ok ? pix : 0), img, rem);
    div_row.divmod(rem, oy, ox);
    st.img_off = (int)img * img_stride;
    st.y0 = (int)oy * sy + by;
    st.x0 = (int)ox * sx + bx;
    st.lane_off = st.ok ? (uint32_t)(st.img_off + st.y0 * Ws + st.x0) * 4u : OOB;
    st.row_ok = st.col_ok = 0;
    if (MODE == 1 && st.ok) {
      for (int r = 0; r < R; ++r)
        if ((uint32_t)(st.y0 + dir * r) < (uint32_t)Hs) st.row_ok |= 1u << r;
      for (int s = 0; s < S; ++s)
        if ((uint32_t)(st.x0 + dir * s) < (uint32_t)Ws) st.col_ok |= 1u << s;
    }
  }
  __device__ inline void load(const State &st, int k0, int k_limit, float (&reg)[EPT]) const {
    // k is wave-uniform, so its decomposition into (channel, tap row, tap column)
    // is scalar arithmetic: no memory access stands between one stage and the
    // next, and validity is folded into the offset's top bit instead of being
    // branched on -- the stage is straight-line code.
    struct Tap { int x, r, s; } t[EPT];
    uint32_t k_bad[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int k = k0 + st.map.k_of(e);
      const uint32_t kc = (uint32_t)min(k, k_extent - 1);
      uint32_t ch, rs, r, s;
      div_rs.divmod(kc, ch, rs);
      div_s.divmod(rs, r, s);
      t[e].r = (int)r;
      t[e].s = (int)s;
      t[e].x = (int)ch * ch_stride + dir * ((int)r * Ws + (int)s);
      k_bad[e] = k < k_limit ? 0u : OOB;
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      if (MODE == 0) {
        // no padding: every tap of a valid pixel is inside the image
        reg[e] = buf_load(st.rsrc, (st.lane_off + (uint32_t)t[e].x * 4u) | k_bad[e]);
      } else if (MODE == 1) {
        const uint32_t tap_bad = ~((st.row_ok >> t[e].r) & (st.col_ok >> t[e].s)) << 31;
        reg[e] = buf_load(st.rsrc, (st.lane_off + (uint32_t)t[e].x * 4u) | tap_bad | k_bad[e]);
      } else {
        // strided filter larger than 1x1 (grad-data only): the tapped coordinate
        // must be divisible by the stride and is divided by it
        const int r = t[e].r, s = t[e].s;
        const int yy = st.y0 - r, xx = st.x0 - s;
        bool ok = st.ok && yy >= 0 && xx >= 0;
        uint32_t qy, ry, qx, rx;
        div_u.divmod((uint32_t)(yy < 0 ? 0 : yy), qy, ry);
        div_v.divmod((uint32_t)(xx < 0 ? 0 : xx), qx, rx);
        ok = ok && ry == 0 && rx == 0 && qy < (uint32_t)Hs && qx < (uint32_t)Ws;
        // t.x = ch*Hs*Ws - r*Ws - s: add the taps back to get the channel offset
        const int ch_off = t[e].x + r * Ws + s;
        const uint32_t off = (uint32_t)(st.img_off + ch_off + (int)qy * Ws + (int)qx) * 4u;
        reg[e] = buf_load(st.rsrc, (ok ? off : OOB) | k_bad[e]);
      }
    }
  }
  template <int LD>
  __device__ inline void store(const State &st, float (*tile)[LD], const float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < EPT; ++e) tile[st.map.k_of(e)][st.map.d_local] = reg[e];
  }
};

// ---- gathered operand, lanes along the reduction (grad-filter's x) --------------
// element(col, k): col -> (c, r, s) fixed per lane for the whole kernel,
// k -> (img, p, q) recomputed per stage; reads x[img][c][p*u+r-pad_h][q*v+s-pad_w].
template <int D, int BK, int MODE>
struct GatherAcross {
  using Map = AcrossMap<D, BK>;
  static constexpr int EPT = Map::EPT;
  const float *base;
  uint32_t bytes;
  int k_extent, n_extent;    // N*P*Q, C*R*S
  FastDiv div_pq, div_q, div_rs, div_s;
  int img_stride, chan_stride;  // C*H*W, H*W
  int H, W, u, v, pad_h, pad_w;

  struct State {
    Map map;
    __amdgpu_buffer_rsrc_t rsrc;
    int col_off[EPT];  // c * H * W, or -1 past the last column
    int taps[EPT];     // packed (r, s)
  };
  __device__ inline void init(State &st, int origin, int tid) const {
    st.map.init(tid);
    st.rsrc = make_rsrc(base, bytes);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int col = origin + st.map.d_of(e);
      const bool ok = col < n_extent;
      uint32_t c, rs, r, s;
      div_rs.divmod((uint32_t)(ok ? col : 0), c, rs);
      div_s.divmod(rs, r, s);
      st.col_off[e] = ok ? (int)c * chan_stride : -1;
      st.taps[e] = (int)((r << 16) | s);
    }
  }
  __device__ inline void load(const State &st, int k0, int k_limit, float (&reg)[EPT]) const {
    const int kidx = k0 + st.map.k_local;
    const bool k_ok = kidx < k_limit;
    uint32_t img, rem, p, q;
    div_pq.divmod((uint32_t)(k_ok ? kidx : 0), img, rem);
    div_q.divmod(rem, p, q);
    const int y0 = (int)p * u - pad_h, x0 = (int)q * v - pad_w;
    const int img_off = (int)img * img_stride;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int yy = y0 + (st.taps[e] >> 16), xx = x0 + (st.taps[e] & 0xffff);
      bool ok = k_ok && st.col_off[e] >= 0;
      if (MODE != 0) ok = ok && (uint32_t)yy < (uint32_t)H && (uint32_t)xx < (uint32_t)W;
      const uint32_t off = (uint32_t)(img_off + st.col_off[e] + yy * W + xx) * 4u;
      reg[e] = buf_load(st.rsrc, ok ? off : OOB);
    }
  }
  template <int LD>
  __device__ inline void store(const State &st, float (*tile)[LD], const float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < EPT; ++e) tile[st.map.k_local][st.map.d_of(e)] = reg[e];
  }
};

// ---- grad-filter's dy operand: element(m = out channel, k = (img, pq)) -----------
template <int D, int BK>
struct DyAcross {
  using Map = AcrossMap<D, BK>;
  static constexpr int EPT = Map::EPT;
  const float *base;
  uint32_t bytes;
  int k_extent, m_extent;  // N*P*Q, K
  FastDiv div_pq;
  int img_stride, PQ;      // K*P*Q

  struct State {
    Map map;
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t row_off[EPT];
  };
  __device__ inline void init(State &st, int origin, int tid) const {
    st.map.init(tid);
    st.rsrc = make_rsrc(base, bytes);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int m = origin + st.map.d_of(e);
      st.row_off[e] = m < m_extent ? (uint32_t)m * (uint32_t)PQ * 4u : OOB;
    }
  }
  __device__ inline void load(const State &st, int k0, int k_limit, float (&reg)[EPT]) const {
    const int kidx = k0 + st.map.k_local;
    const bool k_ok = kidx < k_limit;
    uint32_t img, pq;
    div_pq.divmod((uint32_t)(k_ok ? kidx : 0), img, pq);
    const uint32_t k_off = k_ok ? (uint32_t)((int)img * img_stride + (int)pq) * 4u : OOB;
#pragma unroll
    for (int e = 0; e < EPT; ++e)
      reg[e] = buf_load(st.rsrc, (st.row_off[e] + k_off) | ((st.row_off[e] | k_off) & OOB));
  }
  template <int LD>
  __device__ inline void store(const State &st, float (*tile)[LD], const float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < EPT; ++e) tile[st.map.k_local][st.map.d_of(e)] = reg[e];
  }
};

// ---- epilogues ----------------------------------------------------------------------
// D[m = channel][n = (img, pixel)] -> out[img][m][pixel], through a buffer
// descriptor (see StoreRowMajor): invalid rows / columns get an out-of-range offset.
struct StoreNCHW {
  float *out;
  int m_extent, n_extent;
  FastDiv div_hw;        // pixels per image in the column index (HW, or HW rounded up to 4: ragged segments)
  int HW;
  int64_t split_stride;  // elements between the partial outputs of consecutive k-splits
  struct State {
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t col_off[4];  // byte offset of (img, channel 0, pixel), or OOB
  };
  template <int TN>
  __device__ inline void init(State &st, int n_wave, int lane, int split) const {
    st.rsrc = make_rsrc(out + (int64_t)split * split_stride, (uint32_t)split_stride * 4u);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n_wave + 32 * j + (lane & 31);
      uint32_t img, pix;
      div_hw.divmod((uint32_t)(n < n_extent ? n : 0), img, pix);
      st.col_off[j] = (n < n_extent && pix < (uint32_t)HW) ? (img * (uint32_t)m_extent * (uint32_t)HW + pix) * 4u : OOB;
    }
  }
  __device__ inline void store(const State &st, int m, int /*n*/, int j, float v) const {
    const uint32_t off = st.col_off[j] + (uint32_t)m * (uint32_t)HW * 4u;
    buf_store(st.rsrc, (m < m_extent ? off : OOB) | (st.col_off[j] & OOB), v);
  }
};

// D[m = c][n = (img, p, q)] -> dx[img][c][p*u][q*v]; the other positions of the
// u x v cell anchored there receive 0 (1x1 filter: they have no contribution).
struct StoreScatter {
  float *out;
  int m_extent, n_extent;  // C, N*P*Q
  FastDiv div_pq, div_q;
  int H, W, u, v;
  bool pairs;  // u = v = 2 with even H and W: every cell is a full, 8-byte aligned 2 x 2 block
  int pq_valid;  // real P*Q (div_pq may divide by P*Q rounded up to 4: ragged segments)
  struct State {
    int col_base[4];
    int rows[4], cols[4];
  };
  template <int TN>
  __device__ inline void init(State &st, int n_wave, int lane, int /*split*/) const {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n_wave + 32 * j + (lane & 31);
      uint32_t img, rem, p, q;
      div_pq.divmod((uint32_t)(n < n_extent ? n : 0), img, rem);
      div_q.divmod(rem, p, q);
      const int h0 = (int)p * u, w0 = (int)q * v;
      st.col_base[j] = (n < n_extent && rem < (uint32_t)pq_valid) ? ((int)img * m_extent * H + h0) * W + w0 : -1;
      st.rows[j] = min(u, H - h0);
      st.cols[j] = min(v, W - w0);
    }
  }
  __device__ inline void store(const State &st, int m, int /*n*/, int j, float val) const {
    if (m < m_extent && st.col_base[j] >= 0) {
      float *cell = out + st.col_base[j] + m * H * W;
      if (pairs) {  // two 8-byte stores instead of four 4-byte ones
        *reinterpret_cast<float2 *>(cell) = make_float2(val, 0.f);
        *reinterpret_cast<float2 *>(cell + W) = make_float2(0.f, 0.f);
        return;
      }
      for (int dy = 0; dy < st.rows[j]; ++dy)
        for (int dx = 0; dx < st.cols[j]; ++dx) cell[dy * W + dx] = (dy | dx) == 0 ? val : 0.f;
    }
  }
};

// wt[(k*RS + rs) * C + c] = w[(k*C + c) * RS + rs]
__global__ __launch_bounds__(256) void filter_to_krsc_kernel(const float *__restrict__ w, float *__restrict__ wt,
                                                            int K, int C, int RS) {
  const int total = K * C * RS;
  const int stride = gridDim.x * 256;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const int c = i % C;
    const int t = i / C;
    const int rs = t % RS;
    const int k = t / RS;
    wt[i] = w[(k * C + c) * RS + rs];
  }
}

// ---- Winograd F(2x2, 3x3) and F(4x4, 3x3) --------------------------------------------
// A 3x3 / stride-1 correlation evaluated on m x m output tiles (m = 2 or 4):
//   Y = A^T [ (G g G^T) .* (B^T d B) ] A      d: (m+2) x (m+2) input patch, g: 3x3 filter
// The (m+2)^2 positions of the transformed domain are independent matrix products
//   M[pos][mo][t] = sum_cr U[pos][mo][cr] * V[pos][cr][t]     t = (image, tile row, tile column)
// with 2.25x (m = 2) or 4x (m = 4) fewer multiplications than the direct form; they run as one launch of
// the tile engine with the position on blockIdx.y.  Forward uses it with
// (mo, cr) = (K, C) on x; grad-data with (mo, cr) = (C, K) on dy and the filter
// rotated by 180 degrees.  U, V and M live in scratch memory.
template <class L>
struct Batched : L {
  int64_t batch_stride;  // elements between the operands of consecutive problems
  __device__ inline void init(typename L::State &st, int origin, int tid) const {
    L one = *this;
    one.base += (int64_t)blockIdx.y * batch_stride;
    one.init(st, origin, tid);
  }
};
struct StoreBatched : StoreRowMajor {
  int64_t batch_stride;
  template <int TN>
  __device__ inline void init(State &st, int n0, int lane, int split) const {
    StoreRowMajor one = *this;
    one.out += (int64_t)blockIdx.y * batch_stride;
    one.template init<TN>(st, n0, lane, split);
  }
};

// The 1-D transforms of F(m x m, 3 x 3) for output tiles of m = 2 and m = 4 (patches of
// 4 and 6); every 2-D transform below applies one of them to the columns and then to
// the rows.  F(4x4) needs 4x instead of 2.25x fewer multiplications and moves 2.25x
// instead of 4x the input through the transformed domain; its rounding error is a
// few times that of F(2x2) (see the choice of points below), so the planner uses it
// up to 512 channels only.
template <int TILE>
struct Wino;
template <>
struct Wino<2> {
  static constexpr int A = 4;
  // B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]
  __device__ static inline void bt(const float (&d)[4], float (&t)[4]) {
#pragma clang fp contract(off)
    t[0] = d[0] - d[2];
    t[1] = d[1] + d[2];
    t[2] = d[2] - d[1];
    t[3] = d[1] - d[3];
  }
  // G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1]
  __device__ static inline void g(const float (&f)[3], float (&u)[4]) {
#pragma clang fp contract(off)  // the same bits wherever this is inlined (a kept block must equal a fresh one)
    u[0] = f[0];
    u[1] = 0.5f * (f[0] + f[1] + f[2]);
    u[2] = 0.5f * (f[0] - f[1] + f[2]);
    u[3] = f[2];
  }
  // A^T = [1 1 1 0; 0 1 -1 -1]
  __device__ static inline void at(const float (&m)[4], float (&y)[2]) {
    y[0] = m[0] + m[1] + m[2];
    y[1] = m[1] - m[2] - m[3];
  }
  // the transposes, for grad-filter: A y and G^T u
  __device__ static inline void a(const float (&y)[2], float (&m)[4]) {
#pragma clang fp contract(off)
    m[0] = y[0];
    m[1] = y[0] + y[1];
    m[2] = y[0] - y[1];
    m[3] = -y[1];
  }
  __device__ static inline void gt(const float (&u)[4], float (&f)[3]) {
    f[0] = u[0] + 0.5f * (u[1] + u[2]);
    f[1] = 0.5f * (u[1] - u[2]);
    f[2] = 0.5f * (u[1] + u[2]) + u[3];
  }
};
template <>
struct Wino<4> {
  static constexpr int A = 6;
  // Interpolation points 0, +-3/4, +-3/2 and infinity rather than the customary 0, +-1, +-2:
  // the transform coefficients stay between 1/4 and 4 (instead of 1/24 ... 8), which
  // cuts the fp32 rounding error by about four (measured against float64: 2e-6 of
  // the output scale at 256 channels, against 8e-6), and B^T, A^T are still exact
  // in binary.
  // B^T = [81/64 0 -45/16 0 1 0; 0 -27/16 -9/4 3/4 1 0; 0 27/16 -9/4 -3/4 1 0;
  //        0 -27/32 -9/16 3/2 1 0; 0 27/32 -9/16 -3/2 1 0; 0 81/64 0 -45/16 0 1]
  __device__ static inline void bt(const float (&d)[6], float (&t)[6]) {
#pragma clang fp contract(off)  // the same bits in every kernel this is inlined into
    const float e1 = d[4] - 2.25f * d[2], o1 = 0.75f * d[3] - 1.6875f * d[1];
    const float e2 = d[4] - 0.5625f * d[2], o2 = 1.5f * d[3] - 0.84375f * d[1];
    t[0] = 1.265625f * d[0] - 2.8125f * d[2] + d[4];
    t[1] = e1 + o1;
    t[2] = e1 - o1;
    t[3] = e2 + o2;
    t[4] = e2 - o2;
    t[5] = 1.265625f * d[1] - 2.8125f * d[3] + d[5];
  }
  // G = [64/81 0 0; -128/243 -32/81 -8/27; -128/243 32/81 -8/27; 32/243 16/81 8/27;
  //      32/243 -16/81 8/27; 0 0 1]
  __device__ static inline void g(const float (&f)[3], float (&u)[6]) {
#pragma clang fp contract(off)  // the same bits wherever this is inlined (a kept block must equal a fresh one)
    const float e1 = (-128.f / 243.f) * f[0] - (8.f / 27.f) * f[2], o1 = (32.f / 81.f) * f[1];
    const float e2 = (32.f / 243.f) * f[0] + (8.f / 27.f) * f[2], o2 = (16.f / 81.f) * f[1];
    u[0] = (64.f / 81.f) * f[0];
    u[1] = e1 - o1;
    u[2] = e1 + o1;
    u[3] = e2 + o2;
    u[4] = e2 - o2;
    u[5] = f[2];
  }
  // A^T = [1 1 1 1 1 0; 0 3/4 -3/4 3/2 -3/2 0; 0 9/16 9/16 9/4 9/4 0; 0 27/64 -27/64 27/8 -27/8 1]
  __device__ static inline void at(const float (&m)[6], float (&y)[4]) {
    const float a = m[1] + m[2], b = m[1] - m[2], c = m[3] + m[4], e = m[3] - m[4];
    y[0] = m[0] + a + c;
    y[1] = 0.75f * b + 1.5f * e;
    y[2] = 0.5625f * a + 2.25f * c;
    y[3] = 0.421875f * b + 3.375f * e + m[5];
  }
  // the transposes, for grad-filter: A y and G^T u
  __device__ static inline void a(const float (&y)[4], float (&m)[6]) {
#pragma clang fp contract(off)  // the same bits in every kernel this is inlined into
    const float e1 = y[0] + 0.5625f * y[2], o1 = 0.75f * y[1] + 0.421875f * y[3];
    const float e2 = y[0] + 2.25f * y[2], o2 = 1.5f * y[1] + 3.375f * y[3];
    m[0] = y[0];
    m[1] = e1 + o1;
    m[2] = e1 - o1;
    m[3] = e2 + o2;
    m[4] = e2 - o2;
    m[5] = y[3];
  }
  __device__ static inline void gt(const float (&u)[6], float (&f)[3]) {
    const float s12 = u[1] + u[2], s34 = u[3] + u[4];
    f[0] = (64.f / 81.f) * u[0] - (128.f / 243.f) * s12 + (32.f / 243.f) * s34;
    f[1] = (32.f / 81.f) * (u[2] - u[1]) + (16.f / 81.f) * (u[3] - u[4]);
    f[2] = (8.f / 27.f) * (s34 - s12) + u[5];
  }
};

// U[pos][k][c] = (G g G^T)[pos], one lane per filter g = w[k][c] (grad-data: rotated by
// 180 degrees).  Forward reads U as [mo = k][cr = c], grad-data as its transpose
// [cr = k][mo = c].
// With `U_rot` the same launch also writes the transform of the rotated filter there
// (what a later grad-data call of the same step needs), from the nine taps it has loaded.
template <int TILE>
__global__ __launch_bounds__(256) void wino_filter_kernel(const float *__restrict__ w, float *__restrict__ U,
                                                         int K, int C, bool for_dgrad,
                                                         float *__restrict__ U_rot = nullptr) {
  constexpr int A = Wino<TILE>::A;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= K * C) return;
  float taps[9];
#pragma unroll
  for (int q = 0; q < 9; ++q) taps[q] = w[(int64_t)idx * 9 + q];
  const int64_t plane = (int64_t)K * C;
  auto transform = [&](bool rotated, float *dst) {
    float t[A][3];  // G g, column by column
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      float col[3], u[A];
#pragma unroll
      for (int r = 0; r < 3; ++r) col[r] = rotated ? taps[(2 - r) * 3 + (2 - q)] : taps[r * 3 + q];
      Wino<TILE>::g(col, u);
#pragma unroll
      for (int i = 0; i < A; ++i) t[i][q] = u[i];
    }
#pragma unroll
    for (int i = 0; i < A; ++i) {
      float u[A];
      Wino<TILE>::g(t[i], u);
#pragma unroll
      for (int j = 0; j < A; ++j) dst[(i * A + j) * plane + idx] = u[j];
    }
  };
  transform(for_dgrad, U);
  if (U_rot) transform(true, U_rot);
}

// V[pos][cr][t] = (B^T d B)[pos]; d is the patch of in[image][cr] whose corner is
// (TILE*tile_row - pad_h, TILE*tile_col - pad_w), zero outside the image.  One lane per
// (cr = blockIdx.y, t); columns T..Tp-1 of the padded row are written as zeros.
// ROW16 (TILE 4 only; pad_w = 1): the four middle columns of a patch row start at a
// multiple of 4 and are fetched as one 16-byte load (W a multiple of 4, `in` 16-byte
// aligned) or, with `halves`, as two 8-byte loads (W even, `in` 8-byte aligned).
// WITH_DM (padding 1 on both sides, so that the patch's inner TILE x TILE block is the
// output tile of the same index): the input is a dy, and the launch also writes what
// grad-filter wants of it, dM[pos][cr][t] = (A y A^T)[pos] with y that inner block --
// grad-data and grad-filter of one layer then read dy once between them.
//
// Addressing: `in`, V and dM are read and written through buffer descriptors, a 32-bit
// per-lane byte offset plus, for the position planes of V and dM, a uniform plane offset
// -- one store instruction per value instead of a 64-bit vector address computed for
// each (every array of a Winograd launch is under 4 GiB: wino_shape bounds the scratch).
template <int TILE, bool ROW16 = false, bool HALVES = false, bool WITH_DM = false>
__global__ __launch_bounds__(256) void wino_input_kernel(const float *__restrict__ in, float *__restrict__ V, int Cr,
                                                        int H, int W, FastDiv div_tiles, FastDiv div_tw, int pad_h,
                                                        int pad_w, int T, int Tp, uint32_t in_bytes,
                                                        float *__restrict__ dM = nullptr) {
  static_assert(!ROW16 || TILE == 4, "ROW16 is the 6-wide patch whose columns 1..4 start at a multiple of 4");
  constexpr int A = Wino<TILE>::A;
  const uint32_t t = blockIdx.x * 256 + threadIdx.x;
  const int cr = blockIdx.y;
  if (t >= (uint32_t)Tp) return;
  const __amdgpu_buffer_rsrc_t rin = gemm::make_rsrc(in, in_bytes);
  float d[A][A];
#pragma unroll
  for (int i = 0; i < A; ++i)
#pragma unroll
    for (int j = 0; j < A; ++j) d[i][j] = 0.f;
  if (t < (uint32_t)T) {
    uint32_t img, rem, th, tw;
    div_tiles.divmod(t, img, rem);
    div_tw.divmod(rem, th, tw);
    const uint32_t plane = (img * (uint32_t)Cr + (uint32_t)cr) * (uint32_t)(H * W);  // first element of the plane
    const int h0 = TILE * (int)th - pad_h, w0 = TILE * (int)tw - pad_w;
    if constexpr (ROW16) {
      const int wq = w0 + 1;  // = 4 * tw < W
#pragma unroll
      for (int i = 0; i < A; ++i) {
        const int h = h0 + i;
        if (h < 0 || h >= H) continue;
        const uint32_t row = (plane + (uint32_t)(h * W + wq)) * 4u;  // byte offset of column wq
        if (wq > 0) d[i][0] = gemm::buf_load(rin, row - 4u);
        if constexpr (HALVES) {  // the last tile of a row may hold only two columns
          const f32x2v lo = __builtin_bit_cast(f32x2v, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)row, 0, 0));
          d[i][1] = lo.x;
          d[i][2] = lo.y;
          if (wq + 2 < W) {
            const f32x2v hi = __builtin_bit_cast(f32x2v, __builtin_amdgcn_raw_buffer_load_b64(rin, (int)row + 8, 0, 0));
            d[i][3] = hi.x;
            d[i][4] = hi.y;
          }
        } else {
          const gemm::f32x4v mid = gemm::buf_load4(rin, row);
          d[i][1] = mid.x;
          d[i][2] = mid.y;
          d[i][3] = mid.z;
          d[i][4] = mid.w;
        }
        if (wq + 4 < W) d[i][5] = gemm::buf_load(rin, row + 16u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < A; ++i)
#pragma unroll
        for (int j = 0; j < A; ++j) {
          const int h = h0 + i, x = w0 + j;
          if (h >= 0 && h < H && x >= 0 && x < W) d[i][j] = gemm::buf_load(rin, (plane + (uint32_t)(h * W + x)) * 4u);
        }
    }
  }
  float r[A][A];  // B^T d, column by column
#pragma unroll
  for (int j = 0; j < A; ++j) {
    float col[A], o[A];
#pragma unroll
    for (int i = 0; i < A; ++i) col[i] = d[i][j];
    Wino<TILE>::bt(col, o);
#pragma unroll
    for (int i = 0; i < A; ++i) r[i][j] = o[i];
  }
  const uint32_t plane_bytes = (uint32_t)Cr * (uint32_t)Tp * 4u;   // one position of V (and of dM)
  const uint32_t lane_off = ((uint32_t)cr * (uint32_t)Tp + t) * 4u;
  const __amdgpu_buffer_rsrc_t rv = gemm::make_rsrc(V, (uint32_t)(A * A) * plane_bytes);
#pragma unroll
  for (int i = 0; i < A; ++i) {
    float o[A];
    Wino<TILE>::bt(r[i], o);
#pragma unroll
    for (int j = 0; j < A; ++j)
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, o[j]), rv, (int)lane_off,
                                            (int)((uint32_t)(i * A + j) * plane_bytes), 0);
  }
  if constexpr (WITH_DM) {
    float q[A][TILE];  // A y, column by column
#pragma unroll
    for (int b = 0; b < TILE; ++b) {
      float col[TILE], o[A];
#pragma unroll
      for (int a = 0; a < TILE; ++a) col[a] = d[a + 1][b + 1];
      Wino<TILE>::a(col, o);
#pragma unroll
      for (int i = 0; i < A; ++i) q[i][b] = o[i];
    }
    const __amdgpu_buffer_rsrc_t rm = gemm::make_rsrc(dM, (uint32_t)(A * A) * plane_bytes);
#pragma unroll
    for (int i = 0; i < A; ++i) {
      float o[A];
      Wino<TILE>::a(q[i], o);
#pragma unroll
      for (int j = 0; j < A; ++j)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, o[j]), rm, (int)lane_off,
                                              (int)((uint32_t)(i * A + j) * plane_bytes), 0);
    }
  }
}

// out[image][mo][TILE*tile_row + a][TILE*tile_col + b] = (A^T m A)[a][b], m[pos] = M[pos][mo][t].
// One lane per (mo = blockIdx.y, t); `rows_vec`: Q is a multiple of TILE and out is
// aligned to a tile row, which is then one 8- or 16-byte store.
template <int TILE>
__global__ __launch_bounds__(256) void wino_output_kernel(const float *__restrict__ M, float *__restrict__ out, int Mo,
                                                         int P, int Q, FastDiv div_tiles, FastDiv div_tw, int T,
                                                         int Tp, bool rows_vec, uint32_t out_bytes) {
  constexpr int A = Wino<TILE>::A;
  const uint32_t t = blockIdx.x * 256 + threadIdx.x;
  const int mo = blockIdx.y;
  if (t >= (uint32_t)T) return;
  // buffer addressing as in wino_input_kernel: uniform plane offsets for M, uniform row offsets for out
  const uint32_t plane_bytes = (uint32_t)Mo * (uint32_t)Tp * 4u;
  const uint32_t lane_off = ((uint32_t)mo * (uint32_t)Tp + t) * 4u;
  const __amdgpu_buffer_rsrc_t rm = gemm::make_rsrc(M, (uint32_t)(A * A) * plane_bytes);
  float m[A][A];
#pragma unroll
  for (int i = 0; i < A; ++i)
#pragma unroll
    for (int j = 0; j < A; ++j)
      m[i][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                              rm, (int)lane_off, (int)((uint32_t)(i * A + j) * plane_bytes), 2));
  float s[TILE][A];  // A^T m, column by column
#pragma unroll
  for (int j = 0; j < A; ++j) {
    float col[A], o[TILE];
#pragma unroll
    for (int i = 0; i < A; ++i) col[i] = m[i][j];
    Wino<TILE>::at(col, o);
#pragma unroll
    for (int a = 0; a < TILE; ++a) s[a][j] = o[a];
  }
  uint32_t img, rem, th, tw;
  div_tiles.divmod(t, img, rem);
  div_tw.divmod(rem, th, tw);
  const int p0 = TILE * (int)th, q0 = TILE * (int)tw;
  const __amdgpu_buffer_rsrc_t ro = gemm::make_rsrc(out, out_bytes);
  const uint32_t dst = (((img * (uint32_t)Mo + (uint32_t)mo) * (uint32_t)P + (uint32_t)p0) * (uint32_t)Q + (uint32_t)q0) * 4u;
#pragma unroll
  for (int a = 0; a < TILE; ++a) {
    if (p0 + a >= P) break;
    float y[TILE];
    Wino<TILE>::at(s[a], y);
    const int row_off = a * Q * 4;
    if (rows_vec) {
      // (the row offset goes into the per-lane offset, not into the scalar operand: 16-byte stores
      // with a scalar offset register now and then stored a wrong first word at full-size layers,
      // when the next row's arithmetic reused the data registers)
      if constexpr (TILE == 2) {
        const f32x2v v = {y[0], y[1]};
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(i32x2v, v), ro, (int)dst + row_off, 0, 0);
      } else {
        const gemm::f32x4v v = {y[0], y[1], y[2], y[3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4v, v), ro, (int)dst + row_off, 0, 0);
      }
    } else {
#pragma unroll
      for (int b2 = 0; b2 < TILE; ++b2)
        if (q0 + b2 < Q) gemm::buf_store(ro, dst + (uint32_t)(row_off + b2 * 4), y[b2]);
    }
  }
}

// Grad-filter in the same domain: dU[pos][k][c] = sum_t dM[pos][k][t] * V[pos][c][t] with
// dM = A dY A^T (dY the m x m tile of dy, zero beyond the edge) and V the transformed
// input as in forward; then dw = G^T dU G.  `rows_vec`: Q is a multiple of TILE and dy
// aligned to a tile row, which is then one 8- or 16-byte load.
template <int TILE>
__global__ __launch_bounds__(256) void wino_dy_kernel(const float *__restrict__ dy, float *__restrict__ dM, int K,
                                                     int P, int Q, FastDiv div_tiles, FastDiv div_tw, int T, int Tp,
                                                     bool rows_vec) {
  constexpr int A = Wino<TILE>::A;
  const uint32_t t = blockIdx.x * 256 + threadIdx.x;
  const int k = blockIdx.y;
  if (t >= (uint32_t)Tp) return;
  float y[TILE][TILE];
#pragma unroll
  for (int a = 0; a < TILE; ++a)
#pragma unroll
    for (int b = 0; b < TILE; ++b) y[a][b] = 0.f;
  if (t < (uint32_t)T) {
    uint32_t img, rem, th, tw;
    div_tiles.divmod(t, img, rem);
    div_tw.divmod(rem, th, tw);
    const int p0 = TILE * (int)th, q0 = TILE * (int)tw;
    const float *src = dy + (((int64_t)img * K + k) * P + p0) * Q + q0;
#pragma unroll
    for (int a = 0; a < TILE; ++a) {
      if (p0 + a >= P) break;
      if (rows_vec) {
        if constexpr (TILE == 2) {
          const float2 v = *reinterpret_cast<const float2 *>(src + a * Q);
          y[a][0] = v.x;
          y[a][1] = v.y;
        } else {
          const float4 v = *reinterpret_cast<const float4 *>(src + a * Q);
          y[a][0] = v.x;
          y[a][1] = v.y;
          y[a][2] = v.z;
          y[a][3] = v.w;
        }
      } else {
#pragma unroll
        for (int b = 0; b < TILE; ++b)
          if (q0 + b < Q) y[a][b] = src[a * Q + b];
      }
    }
  }
  float r[A][TILE];  // A dY, column by column
#pragma unroll
  for (int b = 0; b < TILE; ++b) {
    float col[TILE], o[A];
#pragma unroll
    for (int a = 0; a < TILE; ++a) col[a] = y[a][b];
    Wino<TILE>::a(col, o);
#pragma unroll
    for (int i = 0; i < A; ++i) r[i][b] = o[i];
  }
  const uint32_t plane_bytes = (uint32_t)K * (uint32_t)Tp * 4u;
  const uint32_t lane_off = ((uint32_t)k * (uint32_t)Tp + t) * 4u;
  const __amdgpu_buffer_rsrc_t rm = gemm::make_rsrc(dM, (uint32_t)(A * A) * plane_bytes);
#pragma unroll
  for (int i = 0; i < A; ++i) {
    float o[A];
    Wino<TILE>::a(r[i], o);
#pragma unroll
    for (int j = 0; j < A; ++j)
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, o[j]), rm, (int)lane_off,
                                            (int)((uint32_t)(i * A + j) * plane_bytes), 0);
  }
}

// dw[k][c] = G^T (sum over k-splits of dU[split][pos][k][c]) G.  A workgroup owns 64
// filters; lane group g adds the splits of a quarter of the positions in split order
// (fixed, so the result does not depend on timing), then 64 lanes transform.  KC = K*C.
template <int TILE>
__global__ __launch_bounds__(256) void wino_dfilter_kernel(const float *__restrict__ dU, float *__restrict__ dw,
                                                          int KC, int splits) {
  constexpr int A = Wino<TILE>::A, POS = A * A, PPG = POS / 4;  // 16 or 36 positions, 4 or 9 per lane group
  __shared__ float u[POS][64];
  const int lane = threadIdx.x & 63, group = threadIdx.x >> 6;
  const int idx = blockIdx.x * 64 + lane;
  if (idx < KC) {
    float acc[PPG];
#pragma unroll
    for (int j = 0; j < PPG; ++j) acc[j] = dU[(int64_t)(group * PPG + j) * KC + idx];
    for (int sp = 1; sp < splits; ++sp)
#pragma unroll
      for (int j = 0; j < PPG; ++j) acc[j] += dU[((int64_t)sp * POS + group * PPG + j) * KC + idx];
#pragma unroll
    for (int j = 0; j < PPG; ++j) u[group * PPG + j][lane] = acc[j];
  }
  __syncthreads();
  if (group != 0 || idx >= KC) return;
  float r[3][A];  // G^T dU, column by column
#pragma unroll
  for (int j = 0; j < A; ++j) {
    float col[A], o[3];
#pragma unroll
    for (int i = 0; i < A; ++i) col[i] = u[i * A + j][lane];
    Wino<TILE>::gt(col, o);
#pragma unroll
    for (int i = 0; i < 3; ++i) r[i][j] = o[i];
  }
  float *dst = dw + (int64_t)idx * 9;
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    float o[3];
    Wino<TILE>::gt(r[i], o);
#pragma unroll
    for (int j = 0; j < 3; ++j) dst[i * 3 + j] = o[j];
  }
}

// ---- host side --------------------------------------------------------------------------

template <int V>
using IC = std::integral_constant<int, V>;

// Tile shapes and the stage depth that goes with each (measured): 16-deep stages
// for the wide tiles, 32-deep for the 64 x 64 tile, whose per-stage overhead is
// otherwise as large as its eight MFMAs per wave.
inline int stage_depth(int bm, int bn) { return (bm == 64 && bn == 64) ? 32 : 16; }

// Forward, the 1x1 grad-data and the Winograd products run the 64 x 64 tile with 16-deep
// stages when the reduction (per k-split) is short (at most 512): half the LDS per workgroup lets eight instead of four share a CU,
// which covers the prologue and epilogue that dominate such a workgroup's life (measured
// -4 % on those launches; +6 % on reductions of 1024, which keep 32).  Plans, k-split
// ranges and fold decisions are made for 32-deep stages either way (their ranges are
// multiples of 32, hence of 16), so only the kernel's stage loop differs.
inline int run_depth(int bm, int bn, int K) {
  static const bool on = [] {
    const char *e = getenv("TINYFLOW_SHORT_STAGES");
    return !(e && *e && atoi(e) == 0);
  }();
  return (on && bm == 64 && bn == 64 && K <= 512) ? 16 : stage_depth(bm, bn);
}

template <class F>
void with_tile(int bm, int bn, F &&f, int depth = 0) {
  if (bm == 128 && bn == 128) f(IC<128>{}, IC<128>{}, IC<16>{});
  else if (bm == 64 && bn == 128) f(IC<64>{}, IC<128>{}, IC<16>{});
  else if (depth == 16) f(IC<64>{}, IC<64>{}, IC<16>{});
  else f(IC<64>{}, IC<64>{}, IC<32>{});
}

// Events a measuring caller wants recorded around the next contraction kernel only
// (not around the layout or split-sum passes that may accompany it).
thread_local hipEvent_t next_kernel_start = nullptr, next_kernel_stop = nullptr;

template <int BM, int BN, int BK, class AL, class BL, class EP>
void launch(const AL &al, const BL &bl, const EP &ep, int K, const Geometry &g, hipStream_t s, int batch = 1) {
  if (next_kernel_start) (void)hipEventRecord(next_kernel_start, s);
  hipLaunchKernelGGL((gemm_kernel<BM, BN, BK, AL, BL, EP>), dim3(g.blocks(), batch), dim3(THREADS), 0, s, al, bl, ep,
                     K, g.k_per_split, g.tiles_m, g.tiles_n, g.fold());
  if (next_kernel_stop) (void)hipEventRecord(next_kernel_stop, s);
  next_kernel_start = next_kernel_stop = nullptr;
}

bool shape_is(const DLArray *a, int d0, int d1, int d2, int d3) {
  return a->ndim == 4 && a->shape[0] == d0 && a->shape[1] == d1 && a->shape[2] == d2 && a->shape[3] == d3;
}

constexpr int64_t kMaxBytes = (int64_t)1 << 31;  // buffer offsets are 31-bit

// Launch plan of each of the three convolutions of a descriptor: which loader
// mode / epilogue, which tile and how many k-splits.  The entry points and the
// introspection call below both use it, so they cannot disagree.
struct ConvPlan {
  const char *variant;   // short name of the loader / epilogue combination
  const char *a_loader, *b_loader, *epilogue;  // as they appear in the kernel symbol
  int b_mode;            // MODE template argument of the gathered operand, -1 if none
  bool a_vec, b_vec;     // operand fetched with the 16-byte loaders (shape permitting)
  int bm, bn, splits;
  int M, N, K;
  int seg = 0;            // pixels per image as the 16-byte loaders index them: P*Q, or P*Q rounded up
                          // to a multiple of 4 (ragged segments); 0 when they are not used
  bool winograd = false;  // 3x3 / stride-1 layers: transformed-domain products (bm x bn is their tile)
  int wino_tile = 2;      // F(2x2, 3x3) or F(4x4, 3x3)
};

// Pixels per image as the 16-byte loaders index a [image][channel][pixel] block: the
// real count when it is a multiple of 4; otherwise rounded up (ragged segments, see
// gemm_core.h) as long as the padding columns cost at most an eighth more work.
int vector_segment(int pixels) {
  if (pixels % 4 == 0) return pixels;
  const int padded = (pixels + 3) / 4 * 4;
  return padded * 8 <= pixels * 9 ? padded : 0;
}

// Tile and k-split selection.  Every ResNet/VGG layer offers several workable
// (tile, splits) pairs and the best one is worth 10-30 % on the small-image stages,
// so the choice is made by a cost model rather than by a rule of thumb.  The model
// (microseconds) was fitted to sweeps of all pairs over the ResNet-50 layers at batch
// 16 / 64 / 128 and the VGG-16 layers at batch 32 on MI355X, first to the measured
// times (rms error 14 %), then nudged so that its picks cost least (within 1 % of the
// sweeps' optimum on ResNet-50 batch 64, 2 % at batch 128):
//   workgroup time   = a(tile) * (k per split + 24), a = 0.065 / 0.0332 / 0.0178 us
//                      per reduction step for 128x128 / 64x128 / 64x64
//   rounds           = workgroups / CUs, rounded up once a CU holds more than one
//   latency hiding   = a CU that only ever holds 1 / 2 / 3 workgroups runs them at
//                      0.68 / 0.87 / 0.95 of the rate it reaches with four or more
//   split-sum pass   = (2 * splits + 1) * output bytes at 6.5 TB/s
// It depends on the problem shape and the CU count only, so a given layer always
// gets the same plan and results stay bit-reproducible from run to run.  The batched
// products of the Winograd forms (batch > 1) keep the constants they were tuned with.
double predict_us(int M, int N, int K, int bm, int bn, int splits, bool wgrad, bool padded, bool scatter,
                  double out_bytes, int batch = 1) {
  const Geometry g = make_geometry(M, N, K, bm, bn, splits, stage_depth(bm, bn));
  const bool one = batch == 1;
  double a = (bm == 128 && bn == 128) ? (one ? 0.065 : 0.0705) : (bm == 64 && bn == 128) ? (one ? 0.0332 : 0.0406)
                                                                                           : (one ? 0.0178 : 0.0229);
  if (padded) a *= one ? 1.17 : 1.04;
  if (wgrad) a *= bm == 128 ? (one ? 0.906 : 0.98) : (one ? 1.24 : 1.05);
  const double block_us = a * (g.k_per_split + (one ? 23.8 : 9.0));
  const double per_cu = (double)g.blocks() * batch / num_cus();
  const double whole = std::ceil(per_cu);
  const double rounds = per_cu <= 1.0 ? 1.0 : std::min(whole, per_cu + (one ? 0.85 : 0.94));
  const double hiding = one ? (whole <= 1 ? 0.675 : whole <= 2 ? 0.865 : whole <= 3 ? 0.953 : 1.0)
                            : (whole <= 1 ? 0.656 : whole <= 2 ? 0.84 : whole <= 3 ? 0.92 : 1.0);
  double t = rounds * block_us / hiding;
  if (g.splits > 1) t += (2.0 * g.splits + 1.0) * out_bytes / (one ? 6485.0 : 6000.0) * 1e-3;
  if (scatter && bm * bn > 4096) t *= 1.0 + (one ? 0.045 : 0.164) * (bm * bn / 4096.0 - 1.0);
  return t;
}

// Fills p.bm / p.bn / p.splits with the cheapest candidate.  `may_split` is false
// where the epilogue cannot write partial sums (scatter); grad-filter only has
// the square tiles.
double choose_tile_and_splits(ConvPlan &p, bool wgrad, bool padded, bool scatter, bool may_split,
                              double out_bytes) {
  static const int tiles[3][2] = {{128, 128}, {64, 128}, {64, 64}};
  const size_t max_scratch = (size_t)512 << 20;
  double best = 1e30;
  p.bm = p.bn = 64;
  p.splits = 1;
  for (auto &t : tiles) {
    const int bm = t[0], bn = t[1];
    if (wgrad && bm != bn) continue;
    if (bm == 128 && (p.M <= 64 || (wgrad && p.N <= 64))) continue;
    const int n_tiles = cdiv(p.M, bm) * cdiv(p.N, bn);
    int cand[16], n_cand = 0;
    cand[n_cand++] = 1;
    if (may_split) {
      if (wgrad) {
        // aim at 1, 1.5, 2, 3, 4 and 6 workgroups per CU
        static const int per_cu_x2[] = {2, 3, 4, 6, 8, 12};
        for (int x : per_cu_x2) cand[n_cand++] = std::max(1, (num_cus() * x / 2 + n_tiles / 2) / n_tiles);
      } else {
        static const int few[] = {2, 3, 4, 5, 6, 8, 10, 12};
        for (int x : few) cand[n_cand++] = x;
      }
    }
    for (int i = 0; i < n_cand; ++i) {
      const int splits = cand[i];
      if (splits > 1 && (p.K / splits < 64 || (double)splits * out_bytes > (double)max_scratch)) continue;
      const double us = predict_us(p.M, p.N, p.K, bm, bn, splits, wgrad, padded, scatter, out_bytes);
      if (us < best) {
        best = us;
        p.bm = bm;
        p.bn = bn;
        p.splits = make_geometry(p.M, p.N, p.K, bm, bn, splits, stage_depth(bm, bn)).splits;
      }
    }
  }
  return best;
}

// Geometry of the Winograd form of a 3x3 / stride-1 convolution (forward) or of its
// grad-data (the same correlation on dy with padding 2 - pad and the rotated filter).
struct WinoShape {
  int Mo, Cr;              // output / reduction channels of the correlation
  int in_h, in_w, out_h, out_w, pad_h, pad_w;
  int tile, positions;     // output tile edge m (2 or 4) and (m + 2)^2
  int TH, TW, T, Tp;       // output tiles per image column / row, in total, padded to 4
  size_t u_elems, v_elems, m_elems;  // scratch, each rounded up to 64 floats
};
constexpr int kMaxChannelsF4 = 512;  // F(4x4) only up to this many reduction channels (grad-filter: channels
                                     // on either side), which bounds its rounding error
constexpr size_t kMaxWinogradScratch = (size_t)2 << 30;

bool wino_shape(const ConvDesc *d, bool dgrad, WinoShape &w, bool wgrad = false, int tile = 2) {
  if (tile != 2 && tile != 4) return false;
  w.tile = tile;
  w.positions = (tile + 2) * (tile + 2);
  if (d->R != 3 || d->S != 3 || d->u != 1 || d->v != 1 || d->pad_h > 2 || d->pad_w > 2) return false;
  w.Mo = dgrad ? d->C : d->K;
  w.Cr = dgrad ? d->K : d->C;
  w.in_h = dgrad ? d->P : d->H;
  w.in_w = dgrad ? d->Q : d->W;
  w.out_h = dgrad ? d->H : d->P;
  w.out_w = dgrad ? d->W : d->Q;
  w.pad_h = dgrad ? 2 - d->pad_h : d->pad_h;
  w.pad_w = dgrad ? 2 - d->pad_w : d->pad_w;
  // 16-byte loads of U: rows of Cr floats (forward), of Mo floats (grad-data, transposed)
  // (grad-filter reduces over the tiles instead and has no such condition)
  if (w.Cr < 1 || w.Cr > 65535 || w.Mo < 1 || w.Mo > 65535) return false;
  if (!wgrad && (w.Cr % 4 != 0 || (dgrad && w.Mo % 4 != 0))) return false;
  if (tile == 4 && (w.Cr > kMaxChannelsF4 || (wgrad && w.Mo > kMaxChannelsF4))) return false;
  w.TH = cdiv(w.out_h, tile);
  w.TW = cdiv(w.out_w, tile);
  const int64_t T = (int64_t)d->N * w.TH * w.TW;
  if (T < 1 || T > (1 << 28)) return false;
  w.T = (int)T;
  w.Tp = (w.T + 3) / 4 * 4;
  auto round64 = [](int64_t n) { return (size_t)((n + 63) / 64 * 64); };
  w.u_elems = wgrad ? 0 : round64((int64_t)w.positions * w.Mo * w.Cr);
  w.v_elems = round64((int64_t)w.positions * w.Cr * w.Tp);
  w.m_elems = round64((int64_t)w.positions * w.Mo * w.Tp);
  if ((w.u_elems + w.v_elems + w.m_elems) * 4 > kMaxWinogradScratch) return false;
  return true;
}

// Decides between the direct and the Winograd forms and fills the plan of the latter.
// Model: the transformed-domain products as one batched launch of the tile engine,
// plus the transform passes at their measured memory rate.  TINYFLOW_WINOGRAD in the
// environment forces the choice (tests and measurements): 0 direct, 1 Winograd with
// the model's tile, 2 / 4 that tile where the shape allows it; TINYFLOW_WINOGRAD_MAX_TILE=2
// keeps the planner to F(2x2) for callers who want its rounding error (that of the
// direct form) rather than F(4x4)'s (about twice that: measured on the full-size
// ResNet-50 / VGG-16 layers against float64, the largest error is at most 1.5 times
// that of a one-accumulator fp32 loop for the direct form and at most 2.7 times for F(4x4)).
void consider_winograd(ConvPlan &p, const ConvDesc *d, bool dgrad, double direct_us, const char *variant2,
                       const char *variant4) {
  const char *force = getenv("TINYFLOW_WINOGRAD");
  const int forced = force && *force ? atoi(force) : -1;
  if (forced == 0) return;
  static const int tiles[3][2] = {{128, 128}, {64, 128}, {64, 64}};
  double best_us = 1e30;
  int best_tile = 0, best_bm = 64, best_bn = 64;
  WinoShape best_w;
  const char *cap = getenv("TINYFLOW_WINOGRAD_MAX_TILE");
  const int max_tile = cap && *cap ? atoi(cap) : 4;
  for (int tile : {2, 4}) {
    if ((forced == 2 || forced == 4) ? tile != forced : tile > max_tile) continue;
    WinoShape w;
    if (!wino_shape(d, dgrad, w, false, tile)) continue;
    double best = 1e30;
    int bm = 64, bn = 64;
    for (auto &t : tiles) {
      if (t[0] == 128 && w.Mo <= 64) continue;
      const double us = predict_us(w.Mo, w.Tp, w.Cr, t[0], t[1], 1, false, false, false, 0.0, w.positions);
      if (us < best) {
        best = us;
        bm = t[0];
        bn = t[1];
      }
    }
    const double in_bytes = 4.0 * d->N * w.Cr * w.in_h * w.in_w, out_bytes = 4.0 * d->N * w.Mo * w.out_h * w.out_w;
    const double moved = in_bytes + out_bytes + 4.0 * (w.v_elems + w.m_elems) + 8.0 * w.u_elems;
    // short reductions: the products themselves stream V and M once more
    const double stream_us = 4.0 * (w.v_elems + w.m_elems) / 5.0e6;
    const double wino_us = std::max(best, stream_us) + moved / 4.0e6 + 6.0;
    if (wino_us < best_us) {
      best_us = wino_us;
      best_tile = tile;
      best_bm = bm;
      best_bn = bn;
      best_w = w;
    }
  }
  if (best_tile == 0 || (forced < 0 && best_us >= direct_us)) return;
  p.winograd = true;
  p.wino_tile = best_tile;
  p.variant = best_tile == 2 ? variant2 : variant4;
  p.bm = best_bm;
  p.bn = best_bn;
  p.splits = 1;
  p.M = best_w.Mo;
  p.N = best_w.Tp;
  p.K = best_w.Cr;
}

// Grad-filter in the Winograd domain: batched [K x Tp] * [Tp x C] products, split
// along the tile index where 16 x tiles leave CUs idle.
void consider_winograd_wgrad(ConvPlan &p, const ConvDesc *d, double direct_us) {
  const char *force = getenv("TINYFLOW_WINOGRAD");
  const int forced = force && *force ? atoi(force) : -1;
  if (forced == 0) return;
  const char *cap = getenv("TINYFLOW_WINOGRAD_MAX_TILE");
  const int max_tile = cap && *cap ? atoi(cap) : 4;
  static const int tiles[3][2] = {{128, 128}, {64, 128}, {64, 64}};
  static const int cand[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64};
  double best_us = 1e30;
  int best_tile = 0, best_bm = 64, best_bn = 64, best_splits = 1, best_tp = 0;
  for (int tile : {2, 4}) {
    // a forced 4 falls back to 2 where the shape does not allow it, so that "forced"
    // always means some Winograd form for grad-filter
    WinoShape w;
    if (!wino_shape(d, false, w, true, tile)) continue;
    if (forced == 2 && tile != 2) continue;
    if (forced < 0 && tile > max_tile) continue;
    const double out_bytes = 4.0 * w.positions * d->K * d->C;
    double best = 1e30;
    int bm = 64, bn = 64, splits_of_best = 1;
    for (auto &t : tiles) {
      if (t[0] == 128 && d->K <= 64) continue;
      if (t[1] == 128 && d->C <= 64) continue;
      for (int splits : cand) {
        if (splits > 1 && (w.Tp / splits < 64 || splits * out_bytes > 256e6)) continue;
        double us = predict_us(d->K, d->C, w.Tp, t[0], t[1], splits, false, false, false, out_bytes, w.positions);
        // the kernel that folds the splits and applies G^T . G runs one workgroup per 64
        // filters; with few filters (64 x 64: 64 workgroups) it cannot pull the partial
        // sums at the memory rate (about 25 GB/s per workgroup, measured), which is what
        // the split term of predict_us assumes
        const double fold_rate = std::min(6.0e6, std::ceil(d->K * (double)d->C / 64.0) * 25.0e3);  // bytes per us
        if (splits > 1) us += splits * out_bytes * (1.0 / fold_rate - 1.0 / 6.0e6);
        if (us < best) {
          best = us;
          bm = t[0];
          bn = t[1];
          splits_of_best = make_geometry(d->K, d->C, w.Tp, bm, bn, splits, stage_depth(bm, bn)).splits;
        }
      }
    }
    const double moved = 4.0 * d->N * ((double)d->C * d->H * d->W + (double)d->K * d->P * d->Q) +
                         4.0 * (w.v_elems + w.m_elems);
    const double stream_us = 4.0 * (w.v_elems + w.m_elems) / 5.0e6;
    double wino_us = std::max(best, stream_us) + moved / 4.0e6 + 6.0;
    if (forced == 4 && tile == 4) wino_us = 0.0;
    if (wino_us < best_us) {
      best_us = wino_us;
      best_tile = tile;
      best_bm = bm;
      best_bn = bn;
      best_splits = splits_of_best;
      best_tp = w.Tp;
    }
  }
  if (best_tile == 0 || (forced < 0 && best_us >= direct_us)) return;
  p.winograd = true;
  p.wino_tile = best_tile;
  p.variant = best_tile == 2 ? "wgrad_winograd" : "wgrad_winograd4x4";
  p.bm = best_bm;
  p.bn = best_bn;
  p.splits = best_splits;
  p.M = d->K;
  p.N = d->C;
  p.K = best_tp;
}

ConvPlan plan_forward(const ConvDesc *d) {
  ConvPlan p;
  p.M = d->K;
  p.N = d->N * d->P * d->Q;
  p.K = d->C * d->R * d->S;
  const bool padded = d->pad_h || d->pad_w;
  // filter rows of C*R*S floats; a 1x1 / stride-1 / unpadded input is a plain
  // [image][channel][pixel] block
  p.a_vec = p.K % 4 == 0;
  p.seg = vector_segment(d->P * d->Q);
  p.b_vec = p.a_vec && !padded && d->R * d->S == 1 && d->u == 1 && d->v == 1 && p.seg != 0 &&
            (int64_t)d->N * p.seg < (1ll << 31);
  if (p.b_vec) p.N = d->N * p.seg;  // columns in the loaders' (possibly padded) index space
  else p.seg = 0;
  const double direct_us = choose_tile_and_splits(p, false, padded, false, true, 4.0 * p.M * d->N * d->P * d->Q);
  p.variant = padded ? "fwd_pad" : "fwd_nopad";
  p.epilogue = "StoreNCHW";
  p.a_loader = p.a_vec ? "Across4" : "PlainAcross";
  p.b_loader = p.b_vec ? "Along4" : "GatherAlong";
  p.b_mode = p.b_vec ? -1 : padded ? 1 : 0;
  consider_winograd(p, d, false, direct_us, "fwd_winograd", "fwd_winograd4x4");
  return p;
}

ConvPlan plan_dgrad(const ConvDesc *d) {
  ConvPlan p;
  const int RS = d->R * d->S;
  p.M = d->C;
  p.K = d->K * RS;
  p.splits = 1;
  p.epilogue = "StoreNCHW";
  p.b_mode = 0;
  p.a_vec = d->C % 4 == 0;  // the [(k, r, s)][c] filter has rows of C floats
  p.b_vec = false;
  double direct_us = -1.0;
  if (RS == 1) {
    p.N = d->N * d->P * d->Q;
    const bool dense = d->u == 1 && d->v == 1;
    // dy is read compactly, [image][out channel][pixel]
    p.seg = vector_segment(d->P * d->Q);
    p.b_vec = p.a_vec && p.seg != 0 && (int64_t)d->N * p.seg < (1ll << 31);
    p.a_vec = p.b_vec;
    if (p.b_vec) p.N = d->N * p.seg;
    else p.seg = 0;
    choose_tile_and_splits(p, false, false, !dense, dense, 4.0 * p.M * d->N * d->H * d->W);
    p.variant = dense ? "dgrad_1x1" : "dgrad_1x1_scatter";
    if (!dense) p.epilogue = "StoreScatter";
  } else {
    p.N = d->N * d->H * d->W;
    if (d->u == 1 && d->v == 1) {
      direct_us = choose_tile_and_splits(p, false, true, false, true, 4.0 * p.M * p.N);
      p.variant = "dgrad_pad";
      p.b_mode = 1;
    } else {
      p.bm = p.bn = 64;
      p.variant = "dgrad_strided";
      p.b_mode = 2;
      p.a_vec = false;
    }
  }
  p.a_loader = p.a_vec ? "Along4" : "PlainAlong";
  p.b_loader = p.b_vec ? "Along4" : "GatherAlong";
  if (p.b_vec) p.b_mode = -1;
  if (direct_us >= 0.0) consider_winograd(p, d, true, direct_us, "dgrad_winograd", "dgrad_winograd4x4");
  return p;
}

ConvPlan plan_wgrad(const ConvDesc *d) {
  ConvPlan p;
  p.M = d->K;
  p.N = d->C * d->R * d->S;
  p.K = d->N * d->P * d->Q;
  const bool padded = d->pad_h || d->pad_w;
  // dy is [image][out channel][pixel]; x is the same kind of block for a 1x1 /
  // stride-1 / unpadded filter.  Both operands then share the reduction index, which
  // may be the padded one of ragged segments; a gathered x keeps the real index, so dy
  // is vectorised next to it only when its segments are whole.
  const int PQ = d->P * d->Q;
  p.seg = vector_segment(PQ);
  p.b_vec = p.seg != 0 && !padded && d->R * d->S == 1 && d->u == 1 && d->v == 1 && (int64_t)d->N * p.seg < (1ll << 31);
  p.a_vec = p.b_vec || PQ % 4 == 0;
  if (!p.b_vec) p.seg = p.a_vec ? PQ : 0;
  p.K = d->N * (p.seg ? p.seg : PQ);
  const double direct_us = choose_tile_and_splits(p, true, padded, false, true, 4.0 * p.M * p.N);
  p.variant = padded ? "wgrad_pad" : "wgrad_nopad";
  p.epilogue = "StoreRowMajor";
  p.a_loader = p.a_vec ? "Across4" : "DyAcross";
  p.b_loader = p.b_vec ? "Across4" : "GatherAcross";
  p.b_mode = p.b_vec ? -1 : padded ? 1 : 0;
  consider_winograd_wgrad(p, d, direct_us);
  return p;
}

// Runs the planned Winograd form: filter and input transforms, the batched products,
// the output transform.  Scratch follows the usual convention (shortfall reported
// through memorytoSaving, nothing written).
// The grad-filter call of a training step needs the transformed input V = B^T x B of the
// forward call of that step again.  Once a descriptor has seen a grad-filter call in a
// Winograd form, its forward calls with the same tile put V in a block of its own and
// keep it (keep_set: valid until anything writes to x), and grad-filter takes it over
// instead of transforming x a second time.  The values are the ones it would compute.
// Nothing is kept under a device-memory budget or with TINYFLOW_KEEP_TRANSFORMED_INPUT=0.
// Launches the input transform x -> V (and, with dM, the grad-filter form of the same
// array, see WITH_DM) in the variant the row length and alignment allow.
void launch_wino_input(int tile, const float *in, float *V, float *dM, int images, int Cr, int H, int W, int pad_h,
                       int pad_w, const FastDiv &div_tiles, const FastDiv &div_tw, int T, int Tp, hipStream_t s) {
  const dim3 grid(cdiv(Tp, 256), Cr), block(256);
  const uint32_t in_bytes = (uint32_t)((size_t)images * Cr * H * W * sizeof(float));  // under 4 GiB: smaller than V
  if (tile == 2) {
    hipLaunchKernelGGL(wino_input_kernel<2>, grid, block, 0, s, in, V, Cr, H, W, div_tiles, div_tw, pad_h, pad_w, T, Tp,
                       in_bytes, nullptr);
    return;
  }
  const bool row16 = pad_w == 1 && W % 4 == 0 && (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
  const bool halves = !row16 && pad_w == 1 && W % 2 == 0 && (reinterpret_cast<uintptr_t>(in) & 7u) == 0;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, s, in, V, Cr, H, W, div_tiles, div_tw, pad_h, pad_w, T, Tp, in_bytes, dM);
  };
  if (dM) {
    if (row16) go(wino_input_kernel<4, true, false, true>);
    else if (halves) go(wino_input_kernel<4, true, true, true>);
    else go(wino_input_kernel<4, false, false, true>);
  } else {
    if (row16) go(wino_input_kernel<4, true, false, false>);
    else if (halves) go(wino_input_kernel<4, true, true, false>);
    else go(wino_input_kernel<4, false, false, false>);
  }
}

// dy of a 3x3 / stride-1 layer padded by 1: grad-data's patches and grad-filter's tiles
// have the same index, so one pass over dy can serve both (F(4x4) forms of both)
bool dy_transforms_shareable(const ConvDesc *d) {
  return d->pad_h == 1 && d->pad_w == 1 && d->H == d->P && d->W == d->Q;
}

bool keeping_transformed_input() {
  static const bool on = [] {
    const char *e = getenv("TINYFLOW_KEEP_TRANSFORMED_INPUT");
    return !(e && *e && atoi(e) == 0);
  }();
  return on && !device_budget_active();
}

int run_winograd(ConvDesc *d, bool dgrad, const ConvPlan &plan, const float *in, const float *filter,
                 float *out, int *memorytoSaving, hipStream_t s) {
  WinoShape w;
  if (!wino_shape(d, dgrad, w, false, plan.wino_tile)) return -1;
  const size_t bytes = (w.u_elems + w.v_elems + w.m_elems) * sizeof(float);
  float *kept_V = nullptr;
  if (!dgrad && d->grad_filter_tile == w.tile && keeping_transformed_input() && keep_has_room(w.v_elems * sizeof(float)))
    kept_V = (float *)device_alloc(w.v_elems * sizeof(float));  // no room: this call keeps nothing
  // The transformed filter: a forward call also writes the one grad-data will want (a block
  // of its own, valid until anything writes to the filter); grad-data takes that over.
  float *U_for_dgrad = nullptr, *U_kept = nullptr;
  if (dgrad) d->grad_data_tile = w.tile;
  if (dgrad && keeping_transformed_input()) U_kept = (float *)keep_take(&d->kept_u, filter, s, w.tile);
  if (!dgrad && d->grad_data_tile == w.tile && keeping_transformed_input() && keep_has_room(w.u_elems * sizeof(float)))
    U_for_dgrad = (float *)device_alloc(w.u_elems * sizeof(float));
  // dy: grad-filter may have left grad-data's transform of it, or will want its own
  float *V_kept = nullptr, *dM_for_wgrad = nullptr;
  if (dgrad && w.tile == 4 && dy_transforms_shareable(d) && keeping_transformed_input()) {
    V_kept = (float *)keep_take(&d->kept_dy, in, s, kKeptDyForDgrad | 4);
    if (!V_kept && d->grad_filter_tile == 4 && keep_has_room(w.v_elems * sizeof(float)))
      dM_for_wgrad = (float *)device_alloc(w.v_elems * sizeof(float));
  }
  const size_t own = bytes - ((kept_V || V_kept) ? w.v_elems * sizeof(float) : 0) - (U_kept ? w.u_elems * sizeof(float) : 0);
  float *scratch = (float *)device_alloc(own);
  if (!scratch) {
    if (kept_V) device_free(kept_V);
    if (U_for_dgrad) device_free(U_for_dgrad);
    if (U_kept) device_free(U_kept);
    if (V_kept) device_free(V_kept);
    if (dM_for_wgrad) device_free(dM_for_wgrad);
    if (memorytoSaving) *memorytoSaving = shortfall(bytes);
    return 0;
  }
  float *next = scratch;
  float *U = U_kept ? U_kept : next;
  if (!U_kept) next += w.u_elems;
  float *V = kept_V ? kept_V : V_kept ? V_kept : next;
  if (!kept_V && !V_kept) next += w.v_elems;
  float *Mt = next;
  const FastDiv div_tiles((uint32_t)(w.TH * w.TW)), div_tw((uint32_t)w.TW);
  const dim3 fgrid(cdiv(d->K * d->C, 256)), ogrid(cdiv(w.T, 256), w.Mo), block(256);
  if (!U_kept) {
    if (w.tile == 2)
      hipLaunchKernelGGL(wino_filter_kernel<2>, fgrid, block, 0, s, filter, U, d->K, d->C, dgrad, U_for_dgrad);
    else
      hipLaunchKernelGGL(wino_filter_kernel<4>, fgrid, block, 0, s, filter, U, d->K, d->C, dgrad, U_for_dgrad);
  }
  if (!V_kept)
    launch_wino_input(w.tile, in, V, dM_for_wgrad, d->N, w.Cr, w.in_h, w.in_w, w.pad_h, w.pad_w, div_tiles, div_tw, w.T, w.Tp,
                      s);
  with_tile(plan.bm, plan.bn, [&](auto bm_c, auto bn_c, auto bk_c) {
    constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value, BK = decltype(bk_c)::value;
    const Geometry g = make_geometry(w.Mo, w.Tp, w.Cr, BM, BN, 1, BK);
    const uint32_t u_bytes = (uint32_t)((size_t)w.Mo * w.Cr * 4);
    const Batched<Along4<BN, BK>> bl{{V, (uint32_t)((size_t)w.Cr * w.Tp * 4), w.Tp, w.Tp, w.Cr, FastDiv(ONE_SEGMENT), 0},
                                     (int64_t)w.Cr * w.Tp};
    const StoreBatched ep{{Mt, w.Tp, w.Mo, w.Tp, 0}, (int64_t)w.Mo * w.Tp};
    if (dgrad) {
      const Batched<Along4<BM, BK>> al{{U, u_bytes, w.Mo, w.Mo, w.Cr, FastDiv(ONE_SEGMENT), 0}, (int64_t)w.Mo * w.Cr};
      launch<BM, BN, BK>(al, bl, ep, w.Cr, g, s, w.positions);
    } else {
      const Batched<Across4<BM, BK>> al{{U, u_bytes, w.Cr, w.Mo, w.Cr, FastDiv(ONE_SEGMENT), 0}, (int64_t)w.Mo * w.Cr};
      launch<BM, BN, BK>(al, bl, ep, w.Cr, g, s, w.positions);
    }
  }, run_depth(plan.bm, plan.bn, w.Cr));
  const bool rows_vec = w.out_w % w.tile == 0 && (reinterpret_cast<uintptr_t>(out) & (uintptr_t)(4 * w.tile - 1)) == 0;
  const uint32_t out_bytes = (uint32_t)((size_t)d->N * w.Mo * w.out_h * w.out_w * sizeof(float));  // smaller than M
  if (w.tile == 2)
    hipLaunchKernelGGL(wino_output_kernel<2>, ogrid, block, 0, s, (const float *)Mt, out, w.Mo, w.out_h, w.out_w,
                       div_tiles, div_tw, w.T, w.Tp, rows_vec, out_bytes);
  else
    hipLaunchKernelGGL(wino_output_kernel<4>, ogrid, block, 0, s, (const float *)Mt, out, w.Mo, w.out_h, w.out_w,
                       div_tiles, div_tw, w.T, w.Tp, rows_vec, out_bytes);
  device_free(scratch);
  if (U_kept) device_free(U_kept);
  if (V_kept) device_free(V_kept);
  if (dM_for_wgrad)
    keep_set(&d->kept_dy, dM_for_wgrad, w.v_elems * sizeof(float), in, (size_t)d->N * d->K * d->P * d->Q * sizeof(float),
             s, kKeptDyForWgrad | 4);
  if (kept_V)
    keep_set(&d->kept_v, kept_V, w.v_elems * sizeof(float), in, (size_t)d->N * d->C * d->H * d->W * sizeof(float), s,
             w.tile);
  if (U_for_dgrad)
    keep_set(&d->kept_u, U_for_dgrad, w.u_elems * sizeof(float), filter, (size_t)d->K * d->C * 9 * sizeof(float), s,
             w.tile);
  return 0;
}

int run_winograd_wgrad(ConvDesc *d, const ConvPlan &plan, const float *x, const float *dy, float *dw,
                       int *memorytoSaving, hipStream_t s) {
  WinoShape w;
  if (!wino_shape(d, false, w, true, plan.wino_tile)) return -1;
  d->grad_filter_tile = w.tile;
  // V of this step's forward call, if it is still there, belongs to this x, this tile and this stream
  float *kept_V = nullptr;
  if (keeping_transformed_input()) kept_V = (float *)keep_take(&d->kept_v, x, s, w.tile);
  // dy: grad-data may have left grad-filter's transform of it, or will want its own
  float *dM_kept = nullptr, *V_for_dgrad = nullptr;
  if (w.tile == 4 && dy_transforms_shareable(d) && keeping_transformed_input()) {
    dM_kept = (float *)keep_take(&d->kept_dy, dy, s, kKeptDyForWgrad | 4);
    if (!dM_kept && d->grad_data_tile == 4 && keep_has_room(w.m_elems * sizeof(float)))
      V_for_dgrad = (float *)device_alloc(w.m_elems * sizeof(float));
  }
  const int KC = d->K * d->C;
  const int bk = stage_depth(plan.bm, plan.bn);
  const Geometry g = make_geometry(d->K, d->C, w.Tp, plan.bm, plan.bn, plan.splits, bk);
  const size_t du_elems = (size_t)g.splits * w.positions * KC;
  const size_t bytes = ((kept_V ? 0 : w.v_elems) + (dM_kept ? 0 : w.m_elems) + du_elems) * sizeof(float);
  float *scratch = (float *)device_alloc(bytes);
  if (!scratch) {
    if (kept_V) device_free(kept_V);
    if (dM_kept) device_free(dM_kept);
    if (V_for_dgrad) device_free(V_for_dgrad);
    if (memorytoSaving) *memorytoSaving = shortfall(bytes);
    return 0;
  }
  float *next = scratch;
  float *V = kept_V ? kept_V : next;
  if (!kept_V) next += w.v_elems;
  float *dM = dM_kept ? dM_kept : next;
  if (!dM_kept) next += w.m_elems;
  float *dU = next;
  const FastDiv div_tiles((uint32_t)(w.TH * w.TW)), div_tw((uint32_t)w.TW);
  const bool rows_vec = d->Q % w.tile == 0 && (reinterpret_cast<uintptr_t>(dy) & (uintptr_t)(4 * w.tile - 1)) == 0;
  const dim3 block(256);
  if (!kept_V)
    launch_wino_input(w.tile, x, V, nullptr, d->N, d->C, d->H, d->W, d->pad_h, d->pad_w, div_tiles, div_tw, w.T, w.Tp, s);
  if (dM_kept)
    ;  // dM is grad-data's by-product
  else if (V_for_dgrad)  // one pass over dy writes grad-data's V (kept) and dM
    launch_wino_input(4, dy, V_for_dgrad, dM, d->N, d->K, d->P, d->Q, 2 - d->pad_h, 2 - d->pad_w, div_tiles, div_tw, w.T, w.Tp,
                      s);
  else if (w.tile == 2)
    hipLaunchKernelGGL(wino_dy_kernel<2>, dim3(cdiv(w.Tp, 256), d->K), block, 0, s, dy, dM, d->K, d->P, d->Q, div_tiles,
                       div_tw, w.T, w.Tp, rows_vec);
  else
    hipLaunchKernelGGL(wino_dy_kernel<4>, dim3(cdiv(w.Tp, 256), d->K), block, 0, s, dy, dM, d->K, d->P, d->Q, div_tiles,
                       div_tw, w.T, w.Tp, rows_vec);
  with_tile(plan.bm, plan.bn, [&](auto bm_c, auto bn_c, auto bk_c) {
    constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value, BK = decltype(bk_c)::value;
    const Batched<Across4<BM, BK>> al{{dM, (uint32_t)((size_t)d->K * w.Tp * 4), w.Tp, d->K, w.Tp, FastDiv(ONE_SEGMENT), 0},
                                      (int64_t)d->K * w.Tp};
    const Batched<Across4<BN, BK>> bl{{V, (uint32_t)((size_t)d->C * w.Tp * 4), w.Tp, d->C, w.Tp, FastDiv(ONE_SEGMENT), 0},
                                      (int64_t)d->C * w.Tp};
    const StoreBatched ep{{dU, d->C, d->K, d->C, (int64_t)w.positions * KC}, (int64_t)KC};
    launch<BM, BN, BK>(al, bl, ep, w.Tp, g, s, w.positions);
  }, run_depth(plan.bm, plan.bn, g.k_per_split));
  if (w.tile == 2)
    hipLaunchKernelGGL(wino_dfilter_kernel<2>, dim3(cdiv(KC, 64)), block, 0, s, (const float *)dU, dw, KC, g.splits);
  else
    hipLaunchKernelGGL(wino_dfilter_kernel<4>, dim3(cdiv(KC, 64)), block, 0, s, (const float *)dU, dw, KC, g.splits);
  device_free(scratch);
  if (kept_V) device_free(kept_V);
  if (dM_kept) device_free(dM_kept);
  if (V_for_dgrad)
    keep_set(&d->kept_dy, V_for_dgrad, w.m_elems * sizeof(float), dy, (size_t)d->N * d->K * d->P * d->Q * sizeof(float), s,
             kKeptDyForDgrad | 4);
  return 0;
}

}  // namespace

// Introspection for benchmarks (no counterpart in the reference): describes the
// kernel that `which` (0 forward, 1 grad-data, 2 grad-filter) launches for this
// descriptor as "<variant> <bm>x<bn> s<splits> | <kernel symbol>", where the symbol
// is spelled the way a profiler prints it (anonymous-namespace qualifiers
// dropped), and returns the algorithmic flop count 2*N*K*C*R*S*P*Q through *flops.
extern "C" int DLGpuConvolutionDescribeKernel(void ***list, int which, char *name, int name_len,
                                              double *flops) {
  ConvDesc *d = desc_from_list<ConvDesc>(list, kMagicConv);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuConvolution2DForwardGetOutShape");
  TF_REQUIRE(which >= 0 && which <= 2 && name && name_len > 0, "bad arguments");
  const ConvPlan p = which == 0 ? plan_forward(d) : which == 1 ? plan_dgrad(d) : plan_wgrad(d);
  // forward and the 1x1 grad-data run short reductions with 16-deep stages (run_depth)
  const bool short_stages = !p.winograd && (which == 0 || (which == 1 && d->R * d->S == 1));
  const int bk = short_stages ? run_depth(p.bm, p.bn, p.K) : stage_depth(p.bm, p.bn);
  if (p.winograd) {
    // the batched product is the contraction kernel; its flop count is what it
    // executes (16 or 36 products), 2.25x or 4x below the direct form's
    const int reduction = which == 2 ? make_geometry(p.M, p.N, p.K, p.bm, p.bn, p.splits, stage_depth(p.bm, p.bn)).k_per_split
                                     : p.K;
    const int bk = run_depth(p.bm, p.bn, reduction);
    snprintf(name, (size_t)name_len,
             "%s %dx%d s%d | gemm_kernel<%d, %d, %d, Batched<%s<%d, %d%s>>, Batched<%s<%d, %d%s>>, StoreBatched>",
             p.variant, p.bm, p.bn, p.splits, p.bm, p.bn, bk, which == 1 ? "Along4" : "Across4", p.bm, bk,
             which == 1 ? "" : ", false", which == 2 ? "Across4" : "Along4", p.bn, bk, which == 2 ? ", false" : "");
    if (flops) {
      WinoShape w;
      wino_shape(d, which == 1, w, which == 2, p.wino_tile);
      *flops = 2.0 * w.positions * d->K * (double)d->C * w.T;
    }
    return 0;
  }
  // Across4 carries its RAGGED flag in the symbol (a profiler prints defaulted arguments too)
  char b_args[32];
  const bool ragged_wgrad = which == 2 && p.b_vec && p.seg != d->P * d->Q;
  const char *a_flag = strcmp(p.a_loader, "Across4") == 0 ? (ragged_wgrad ? ", true" : ", false") : "";
  const char *b_flag = strcmp(p.b_loader, "Across4") == 0 ? (ragged_wgrad ? ", true" : ", false") : "";
  if (p.b_mode >= 0) snprintf(b_args, sizeof b_args, "%d, %d, %d", p.bn, bk, p.b_mode);
  else snprintf(b_args, sizeof b_args, "%d, %d%s", p.bn, bk, b_flag);
  snprintf(name, (size_t)name_len, "%s %dx%d s%d | gemm_kernel<%d, %d, %d, %s<%d, %d%s>, %s<%s>, %s>", p.variant,
           p.bm, p.bn, p.splits, p.bm, p.bn, bk, p.a_loader, p.bm, bk, a_flag, p.b_loader, b_args, p.epilogue);
  if (flops)
    *flops = 2.0 * d->N * d->K * d->C * d->R * d->S * (double)d->P * d->Q;
  return 0;
}

extern "C" int DLGpuConvolutionTimeNextKernel(void *start_event, void *stop_event) {
  next_kernel_start = (hipEvent_t)start_event;
  next_kernel_stop = (hipEvent_t)stop_event;
  return 0;
}

extern "C" int DLGpuConvolution2DForwardGetOutShape(const int *input_shapes, const int *filter_shapes,
                                                    int *output_shapes, int dataformat, int padding,
                                                    const int u, const int v, void ***list) {
  TF_REQUIRE(input_shapes && filter_shapes && output_shapes && list, "null argument");
  TF_REQUIRE(dataformat == 0, "only NCHW (dataformat 0) is implemented");
  TF_REQUIRE(u >= 1 && v >= 1, "strides must be positive");
  for (int i = 0; i < 4; ++i)
    TF_REQUIRE(input_shapes[i] >= 0 && filter_shapes[i] >= 0, "negative extent");
  TF_REQUIRE(filter_shapes[1] == input_shapes[1], "filter expects %d input channels, input has %d",
             filter_shapes[1], input_shapes[1]);
  TF_REQUIRE(filter_shapes[2] >= 1 && filter_shapes[3] >= 1 && filter_shapes[2] <= 32 && filter_shapes[3] <= 32,
             "filter extents must lie in 1..32");
  ConvDesc desc;
  ConvDesc *d = &desc;
  d->magic = kMagicConv;
  d->N = input_shapes[0];
  d->C = input_shapes[1];
  d->H = input_shapes[2];
  d->W = input_shapes[3];
  d->K = filter_shapes[0];
  d->R = filter_shapes[2];
  d->S = filter_shapes[3];
  d->pad_h = padding == 1 ? d->R / 2 : 0;  // "SAME" is a symmetric k/2, "VALID" is 0
  d->pad_w = padding == 1 ? d->S / 2 : 0;
  d->u = u;
  d->v = v;
  TF_REQUIRE(d->H + 2 * d->pad_h >= d->R && d->W + 2 * d->pad_w >= d->S, "filter larger than padded input");
  d->P = 1 + (d->H + 2 * d->pad_h - d->R) / u;
  d->Q = 1 + (d->W + 2 * d->pad_w - d->S) / v;
  d = new ConvDesc(desc);
  output_shapes[0] = d->N;
  output_shapes[1] = d->K;
  output_shapes[2] = d->P;
  output_shapes[3] = d->Q;
  // four slots like the reference's {x, w, conv, y} descriptor list
  void **slots = (void **)malloc(sizeof(void *) * 4);
  for (int i = 0; i < 4; ++i) slots[i] = d;
  *list = slots;
  return 0;
}

static int check_conv_arrays(const ConvDesc *d, const DLArray *x, const DLArray *w, const DLArray *y) {
  TF_REQUIRE(on_gpu(x) && on_gpu(w) && on_gpu(y), "arrays must live on the GPU");
  TF_REQUIRE(shape_is(x, d->N, d->C, d->H, d->W), "input does not match the descriptor (N,C,H,W)");
  TF_REQUIRE(shape_is(w, d->K, d->C, d->R, d->S), "filter does not match the descriptor (K,C,R,S)");
  TF_REQUIRE(shape_is(y, d->N, d->K, d->P, d->Q), "output does not match the descriptor (N,K,P,Q)");
  TF_REQUIRE(numel(x) * 4 < kMaxBytes && numel(y) * 4 < kMaxBytes && numel(w) * 4 < kMaxBytes,
             "tensors of 2 GiB or more are not supported");
  return 0;
}

extern "C" int DLGpuConvolution2DForward(const DLArrayHandle input, const DLArrayHandle filter,
                                         DLArrayHandle output, void ***list, void **handle,
                                         int *memorytoSaving, void **stream) {
  announce_write(output);
  (void)handle;
  ConvDesc *d = desc_from_list<ConvDesc>(list, kMagicConv);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuConvolution2DForwardGetOutShape");
  if (check_conv_arrays(d, input, filter, output) != 0) return -1;
  hipStream_t s = stream_of(stream);
  const ConvPlan plan = plan_forward(d);
  const int M = plan.M, N = plan.N, K = plan.K;
  if (M == 0 || N == 0) return 0;
  if (K == 0) return DLGpuArraySet(output, 0.f, stream);
  if (plan.winograd) {
    if (run_winograd(d, false, plan, (const float *)input->data, (const float *)filter->data, (float *)output->data,
                     memorytoSaving, s) != 0)
      return -1;
    return finish(s, "DLGpuConvolution2DForward");
  }
  const int bm = plan.bm, bn = plan.bn;
  Geometry g = make_geometry(M, N, K, bm, bn, plan.splits, stage_depth(bm, bn));
  if (fold_tickets(s)) plan_fold(g, K, stage_depth(bm, bn), 1);  // no ticket words: the unfolded plan
  FoldBuffers fb;
  if (const int rc = acquire_fold(g, bm, bn, 1, s, fb)) {
    if (rc == 1 && memorytoSaving) *memorytoSaving = shortfall(fb.bytes);
    return rc == 1 ? 0 : -1;
  }
  float *partial = nullptr;
  if (g.splits > 1) {
    const size_t bytes = (size_t)g.splits * numel(output) * sizeof(float);
    partial = (float *)device_alloc(bytes);
    if (!partial) {
      if (memorytoSaving) *memorytoSaving = shortfall(bytes);
      return 0;
    }
  }
  const bool padded = d->pad_h != 0 || d->pad_w != 0;
  const int PQ = d->P * d->Q;
  // (a plan with ragged segments counts its columns in the padded index space, so it
  // keeps the 16-byte loaders whatever the alignment: they only need 4 bytes)
  const bool aligned = (vec4_ok(filter->data, 0) && vec4_ok(input->data, 0)) || (plan.seg != 0 && plan.seg != PQ);
  const bool a_vec = plan.a_vec && aligned, b_vec = plan.b_vec && aligned;
  const uint32_t w_bytes = (uint32_t)(numel(filter) * 4), x_bytes = (uint32_t)(numel(input) * 4);
  with_tile(bm, bn, [&](auto bm_c, auto bn_c, auto bk_c) {
    constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value, BK = decltype(bk_c)::value;
    // with the 16-byte loader the columns are (image, pixel) in its segment index space
    const int seg = b_vec ? plan.seg : PQ;
    StoreNCHW ep{partial ? partial : (float *)output->data, M, N, FastDiv((uint32_t)seg), PQ, numel(output)};
    auto with_b = [&](const auto &al, auto a_is_vec) {
      if constexpr (decltype(a_is_vec)::value) {  // a vectorised input only comes with a vectorised filter
        if (b_vec) {
          Along4<BN, BK> bl{(const float *)input->data, x_bytes, PQ, N, K, FastDiv((uint32_t)seg), d->C * PQ};
          launch<BM, BN, BK>(al, bl, ep, K, g, s);
          return;
        }
      }
      auto run = [&](auto mode_c) {
        constexpr int MODE = decltype(mode_c)::value;
        GatherAlong<BN, BK, MODE> bl{(const float *)input->data, x_bytes, K, N,
                                 FastDiv((uint32_t)(d->R * d->S)), FastDiv((uint32_t)d->S), d->H * d->W,
                                 FastDiv((uint32_t)PQ), FastDiv((uint32_t)d->Q),
                                 d->C * d->H * d->W, d->H, d->W, d->u, d->v, -d->pad_h, -d->pad_w,
                                 1, d->R, d->S, FastDiv(1), FastDiv(1)};
        launch<BM, BN, BK>(al, bl, ep, K, g, s);
      };
      if (padded) run(IC<1>{}); else run(IC<0>{});
    };
    if (a_vec)
      with_b(Across4<BM, BK>{(const float *)filter->data, w_bytes, K, M, K, FastDiv(ONE_SEGMENT), 0},
             std::true_type{});
    else
      with_b(PlainAcross<BM, BK>{(const float *)filter->data, w_bytes, K, M, K}, std::false_type{});
  }, run_depth(bm, bn, K));
  if (partial) {
    launch_split_sum(partial, (float *)output->data, numel(output), g.splits, s);
    device_free(partial);
  }
  release_fold(fb);
  return finish(s, "DLGpuConvolution2DForward");
}

extern "C" int DLGpuConvolutionBackwardData(const DLArrayHandle input, const DLArrayHandle doutput,
                                            const DLArrayHandle filter, DLArrayHandle dinput, void ***list,
                                            void **handle, int *memorytoSaving, void **stream) {
  announce_write(dinput);
  (void)handle;
  ConvDesc *d = desc_from_list<ConvDesc>(list, kMagicConv);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuConvolution2DForwardGetOutShape");
  if (check_conv_arrays(d, input, filter, doutput) != 0) return -1;
  TF_REQUIRE(on_gpu(dinput) && same_shape(dinput, input), "dinput must have the input's shape");
  hipStream_t s = stream_of(stream);
  const int RS = d->R * d->S;
  const ConvPlan plan = plan_dgrad(d);
  const int M = plan.M, K = plan.K;
  if (numel(dinput) == 0) return 0;
  if (numel(doutput) == 0) return DLGpuArraySet(dinput, 0.f, stream);
  if (plan.winograd) {
    if (run_winograd(d, true, plan, (const float *)doutput->data, (const float *)filter->data, (float *)dinput->data,
                     memorytoSaving, s) != 0)
      return -1;
    return finish(s, "DLGpuConvolutionBackwardData");
  }

  const uint32_t w_bytes = (uint32_t)(numel(filter) * 4), dy_bytes = (uint32_t)(numel(doutput) * 4);
  const int PQ = d->P * d->Q;
  // a strided filter larger than 1x1 always runs on the small tile, unsplit
  const bool strided_taps = RS > 1 && !(d->u == 1 && d->v == 1);
  const int g_bm = strided_taps ? 64 : plan.bm, g_bn = strided_taps ? 64 : plan.bn;
  Geometry g = make_geometry(M, plan.N, K, g_bm, g_bn, strided_taps ? 1 : plan.splits, stage_depth(g_bm, g_bn));
  if (fold_tickets(s)) plan_fold(g, K, stage_depth(g_bm, g_bn), 1);  // no ticket words: the unfolded plan
  // Scratch: the re-laid filter, the fold pieces or the k-split partials.  Whichever of them
  // cannot be had, the call reports all of them, so that a caller who makes that much room
  // can repeat it.
  const size_t wt_bytes = RS > 1 ? (size_t)numel(filter) * sizeof(float) : 0;
  const size_t partial_bytes = g.splits > 1 ? (size_t)g.splits * numel(dinput) * sizeof(float) : 0;
  const size_t fold_bytes = g.fold_pieces > 1 ? g.fold_scratch_bytes(g_bm, g_bn, 1) : 0;
  const size_t all_bytes = (wt_bytes ? block_bytes(wt_bytes) : 0) + (partial_bytes ? block_bytes(partial_bytes) : 0) +
                           (fold_bytes ? block_bytes(fold_bytes) : 0);
  // filter as [(k, r, s)][c]; a 1x1 filter already has that layout
  const float *wt = (const float *)filter->data;
  float *wt_scratch = nullptr;
  if (wt_bytes) {
    wt_scratch = (float *)device_alloc(wt_bytes);
    if (!wt_scratch) {
      if (memorytoSaving) *memorytoSaving = shortfall(all_bytes);
      return 0;
    }
    const int total = (int)numel(filter);
    hipLaunchKernelGGL(filter_to_krsc_kernel, dim3(min(cdiv(total, 256), num_cus() * 8)), dim3(256), 0, s,
                       (const float *)filter->data, wt_scratch, d->K, d->C, RS);
    wt = wt_scratch;
  }
  FoldBuffers fb;
  if (const int rc = acquire_fold(g, g_bm, g_bn, 1, s, fb)) {
    if (wt_scratch) device_free(wt_scratch);
    if (rc == 1 && memorytoSaving) *memorytoSaving = shortfall(all_bytes);
    return rc == 1 ? 0 : -1;
  }
  float *partial = nullptr;
  if (partial_bytes) {
    partial = (float *)device_alloc(partial_bytes);
    if (!partial) {
      if (wt_scratch) device_free(wt_scratch);
      release_fold(fb);
      if (memorytoSaving) *memorytoSaving = shortfall(all_bytes);
      return 0;
    }
  }
  float *dst = partial ? partial : (float *)dinput->data;
  const int64_t dx_count = numel(dinput);

  // (a plan with ragged segments keeps the 16-byte loaders whatever the alignment)
  const bool aligned = (vec4_ok(wt, 0) && vec4_ok(doutput->data, 0)) || (plan.seg != 0 && plan.seg != PQ);
  const bool a_vec = plan.a_vec && aligned, b_vec = plan.b_vec && aligned;
  const FastDiv whole(ONE_SEGMENT);
  if (RS == 1) {
    // 1x1 filter (pad 0): compact GEMM over the output pixels + scatter
    const int N = plan.N;
    const int bm = plan.bm, bn = plan.bn;
    const int seg = (a_vec && b_vec) ? plan.seg : PQ;  // pixels per image in the column index
    with_tile(bm, bn, [&](auto bm_c, auto bn_c, auto bk_c) {
      constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value, BK = decltype(bk_c)::value;
      auto with_epilogue = [&](const auto &al, const auto &bl) {
        if (d->u == 1 && d->v == 1) {
          StoreNCHW ep{dst, M, N, FastDiv((uint32_t)seg), PQ, dx_count};
          launch<BM, BN, BK>(al, bl, ep, K, g, s);
        } else {
          StoreScatter ep{(float *)dinput->data, M, N, FastDiv((uint32_t)seg), FastDiv((uint32_t)d->Q),
                          d->H, d->W, d->u, d->v,
                          d->u == 2 && d->v == 2 && d->H % 2 == 0 && d->W % 2 == 0 &&
                              (reinterpret_cast<uintptr_t>(dinput->data) & 7u) == 0,
                          PQ};
          launch<BM, BN, BK>(al, bl, ep, K, g, s);
        }
      };
      if (a_vec && b_vec) {
        with_epilogue(Along4<BM, BK>{wt, w_bytes, d->C, M, K, whole, 0},
                      Along4<BN, BK>{(const float *)doutput->data, dy_bytes, PQ, N, K, FastDiv((uint32_t)seg),
                                     d->K * PQ});
      } else {
        with_epilogue(PlainAlong<BM, BK>{wt, w_bytes, d->C, M, K},
                      GatherAlong<BN, BK, 0>{(const float *)doutput->data, dy_bytes, K, N, FastDiv(1), FastDiv(1),
                                             PQ, FastDiv((uint32_t)PQ), FastDiv((uint32_t)d->Q), d->K * PQ, d->P,
                                             d->Q, 1, 1, 0, 0, -1, 1, 1, FastDiv(1), FastDiv(1)});
      }
    }, run_depth(bm, bn, K));
  } else {
    const int N = plan.N;
    const int HW = d->H * d->W;
    const int bm = plan.bm, bn = plan.bn;
    StoreNCHW ep{dst, M, N, FastDiv((uint32_t)HW), HW, dx_count};
    if (d->u == 1 && d->v == 1) {
      with_tile(bm, bn, [&](auto bm_c, auto bn_c, auto bk_c) {
        constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value, BK = decltype(bk_c)::value;
        GatherAlong<BN, BK, 1> bl{(const float *)doutput->data, dy_bytes, K, N, FastDiv((uint32_t)RS),
                              FastDiv((uint32_t)d->S), PQ,
                              FastDiv((uint32_t)HW), FastDiv((uint32_t)d->W), d->K * PQ, d->P, d->Q,
                              1, 1, d->pad_h, d->pad_w, -1, d->R, d->S, FastDiv(1), FastDiv(1)};
        if (a_vec) launch<BM, BN, BK>(Along4<BM, BK>{wt, w_bytes, d->C, M, K, whole, 0}, bl, ep, K, g, s);
        else launch<BM, BN, BK>(PlainAlong<BM, BK>{wt, w_bytes, d->C, M, K}, bl, ep, K, g, s);
      });
    } else {
      // strided filter larger than 1x1: every input pixel, taps filtered by divisibility
      PlainAlong<64, 32> al{wt, w_bytes, d->C, M, K};
      GatherAlong<64, 32, 2> bl{(const float *)doutput->data, dy_bytes, K, N, FastDiv((uint32_t)RS),
                            FastDiv((uint32_t)d->S), PQ,
                            FastDiv((uint32_t)HW), FastDiv((uint32_t)d->W), d->K * PQ, d->P, d->Q,
                            1, 1, d->pad_h, d->pad_w, -1, d->R, d->S,
                            FastDiv((uint32_t)d->u), FastDiv((uint32_t)d->v)};
      launch<64, 64, 32>(al, bl, ep, K, g, s);
    }
  }
  if (partial) {
    launch_split_sum(partial, (float *)dinput->data, dx_count, g.splits, s);
    device_free(partial);
  }
  release_fold(fb);
  if (wt_scratch) device_free(wt_scratch);
  return finish(s, "DLGpuConvolutionBackwardData");
}

extern "C" int DLGpuConvolutionBackwardFilter(const DLArrayHandle input, const DLArrayHandle doutput,
                                              const DLArrayHandle filter, DLArrayHandle dfilter, void ***list,
                                              void **handle, int *memorytoSaving, void **stream) {
  announce_write(dfilter);
  (void)handle;
  ConvDesc *d = desc_from_list<ConvDesc>(list, kMagicConv);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuConvolution2DForwardGetOutShape");
  if (check_conv_arrays(d, input, filter, doutput) != 0) return -1;
  TF_REQUIRE(on_gpu(dfilter) && same_shape(dfilter, filter), "dfilter must have the filter's shape");
  hipStream_t s = stream_of(stream);
  const int PQ = d->P * d->Q, RS = d->R * d->S;
  const ConvPlan plan = plan_wgrad(d);
  const int M = plan.M, N = plan.N, K = plan.K;
  if (M == 0 || N == 0) return 0;
  if (K == 0) return DLGpuArraySet(dfilter, 0.f, stream);
  if (plan.winograd) {
    if (run_winograd_wgrad(d, plan, (const float *)input->data, (const float *)doutput->data, (float *)dfilter->data,
                           memorytoSaving, s) != 0)
      return -1;
    return finish(s, "DLGpuConvolutionBackwardFilter");
  }

  const int bm = plan.bm, bn = plan.bn;
  Geometry g = make_geometry(M, N, K, bm, bn, plan.splits, stage_depth(bm, bn));
  if (fold_tickets(s)) plan_fold(g, K, stage_depth(bm, bn), 1);  // no ticket words: the unfolded plan
  FoldBuffers fb;
  if (const int rc = acquire_fold(g, bm, bn, 1, s, fb)) {
    if (rc == 1 && memorytoSaving) *memorytoSaving = shortfall(fb.bytes);
    return rc == 1 ? 0 : -1;
  }
  float *dst = (float *)dfilter->data;
  float *partial = nullptr;
  if (g.splits > 1) {
    const size_t bytes = (size_t)g.splits * M * N * sizeof(float);
    partial = (float *)device_alloc(bytes);
    if (!partial) {
      release_fold(fb);
      if (memorytoSaving) *memorytoSaving = shortfall(bytes);
      return 0;
    }
    dst = partial;
  }
  const bool padded = d->pad_h != 0 || d->pad_w != 0;
  const bool ragged = plan.seg != 0 && plan.seg != PQ;  // both operands in the padded reduction index
  const bool aligned = (vec4_ok(doutput->data, 0) && vec4_ok(input->data, 0)) || ragged;
  const bool a_vec = plan.a_vec && aligned, b_vec = plan.b_vec && aligned;
  const uint32_t dy_bytes = (uint32_t)(numel(doutput) * 4), x_bytes = (uint32_t)(numel(input) * 4);
  with_tile(bm, bn, [&](auto bm_c, auto bn_c, auto bk_c) {
    constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value, BK = decltype(bk_c)::value;
    if constexpr (BM == BN) {  // only the square tiles are used for grad-filter
      StoreRowMajor ep{dst, N, M, N, (int64_t)M * N};
      if (ragged) {  // 1x1, stride 1, pixels per image not a multiple of 4: masked 16-byte loads on both sides
        const FastDiv div_seg((uint32_t)plan.seg);
        Across4<BM, BK, true> al{(const float *)doutput->data, dy_bytes, PQ, M, K, div_seg, d->K * PQ, PQ};
        Across4<BN, BK, true> bl{(const float *)input->data, x_bytes, PQ, N, K, div_seg, d->C * PQ, PQ};
        launch<BM, BN, BK>(al, bl, ep, K, g, s);
        return;
      }
      auto with_b = [&](const auto &al, auto a_is_vec) {
        if constexpr (decltype(a_is_vec)::value) {
          if (b_vec) {
            Across4<BN, BK> bl{(const float *)input->data, x_bytes, PQ, N, K, FastDiv((uint32_t)PQ), d->C * PQ};
            launch<BM, BN, BK>(al, bl, ep, K, g, s);
            return;
          }
        }
        auto run = [&](auto mode_c) {
          constexpr int MODE = decltype(mode_c)::value;
          GatherAcross<BN, BK, MODE> bl{(const float *)input->data, x_bytes, K, N,
                                    FastDiv((uint32_t)PQ), FastDiv((uint32_t)d->Q), FastDiv((uint32_t)RS),
                                    FastDiv((uint32_t)d->S), d->C * d->H * d->W, d->H * d->W,
                                    d->H, d->W, d->u, d->v, d->pad_h, d->pad_w};
          launch<BM, BN, BK>(al, bl, ep, K, g, s);
        };
        if (padded) run(IC<1>{}); else run(IC<0>{});
      };
      if (a_vec)
        with_b(Across4<BM, BK>{(const float *)doutput->data, dy_bytes, PQ, M, K, FastDiv((uint32_t)PQ), d->K * PQ},
               std::true_type{});
      else
        with_b(DyAcross<BM, BK>{(const float *)doutput->data, dy_bytes, K, M, FastDiv((uint32_t)PQ), d->K * PQ, PQ},
               std::false_type{});
    }
  });
  if (partial) {
    launch_split_sum(partial, (float *)dfilter->data, (int64_t)M * N, g.splits, s);
    device_free(partial);
  }
  release_fold(fb);
  return finish(s, "DLGpuConvolutionBackwardFilter");
}
