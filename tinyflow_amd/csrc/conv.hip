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
#include "internal.h"

#include <mutex>
#include <type_traits>
#include <vector>

using namespace tf;
using namespace tf::gemm;

namespace {

inline int pack_taps(int dy, int dx) { return (int)(((uint32_t)(dy & 0xffff) << 16) | (uint32_t)(dx & 0xffff)); }
__device__ inline int tap_y(int packed) { return packed >> 16; }                 // sign-extending
__device__ inline int tap_x(int packed) { return (int)(short)(packed & 0xffff); }

// ---- gathered operand, lanes along the pixel index ------------------------------
// element(pixel, k): source tensor T[img][ch][Hs][Ws], pixel -> (img, oy, ox),
// k -> (ch, dy, dx) through a table; reads T[img][ch][oy*sy+by+dy][ox*sx+bx+dx].
// MODE 0: taps are always inside the image (no padding)      -> no range test
// MODE 1: range test (zero padding)
// MODE 2: additionally the tapped coordinate must be divisible by the conv
//         stride and is divided by it (grad-data of a strided filter larger than 1x1)
template <int D, int MODE>
struct GatherAlong {
  using Map = AlongMap<D>;
  static constexpr int EPT = Map::EPT;
  const float *base;
  uint32_t bytes;
  const int2 *tab;  // [k_extent]: .x = ch * Hs * Ws, .y = packed (dy, dx)
  int k_extent, n_extent;
  FastDiv div_img, div_row;  // pixels per image, pixels per row
  int img_stride;            // elements per image of T
  int Hs, Ws;
  int sy, sx, by, bx;
  FastDiv div_u, div_v;      // MODE 2 only

  struct State {
    Map map;
    __amdgpu_buffer_rsrc_t rsrc;
    int img_off, y0, x0;
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
  }
  __device__ inline void load(const State &st, int k0, float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int k = k0 + st.map.k_of(e);       // wave-uniform
      const bool k_ok = k < k_extent;
      const int2 t = tab[k_ok ? k : 0];
      int yy = st.y0 + tap_y(t.y), xx = st.x0 + tap_x(t.y);
      bool ok = st.ok && k_ok;
      if (MODE == 2) {
        ok = ok && yy >= 0 && xx >= 0;
        uint32_t qy, ry, qx, rx;
        div_u.divmod((uint32_t)(yy < 0 ? 0 : yy), qy, ry);
        div_v.divmod((uint32_t)(xx < 0 ? 0 : xx), qx, rx);
        ok = ok && ry == 0 && rx == 0;
        yy = (int)qy;
        xx = (int)qx;
      }
      if (MODE != 0) ok = ok && (uint32_t)yy < (uint32_t)Hs && (uint32_t)xx < (uint32_t)Ws;
      const uint32_t off = (uint32_t)(st.img_off + t.x + yy * Ws + xx) * 4u;
      reg[e] = buf_load(st.rsrc, ok ? off : OOB);
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
template <int D, int MODE>
struct GatherAcross {
  using Map = AcrossMap<D>;
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
  __device__ inline void load(const State &st, int k0, float (&reg)[EPT]) const {
    const int kidx = k0 + st.map.k_local;
    const bool k_ok = kidx < k_extent;
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
template <int D>
struct DyAcross {
  using Map = AcrossMap<D>;
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
  __device__ inline void load(const State &st, int k0, float (&reg)[EPT]) const {
    const int kidx = k0 + st.map.k_local;
    const bool k_ok = kidx < k_extent;
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
// D[m = channel][n = (img, pixel)] -> out[img][m][pixel]
struct StoreNCHW {
  float *out;
  int m_extent, n_extent;
  FastDiv div_hw;
  int HW;
  struct State {
    int col_base[4];  // img * CH * HW + pixel, or -1
  };
  template <int TN>
  __device__ inline void init(State &st, int n_wave, int lane, int /*split*/) const {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n_wave + 32 * j + (lane & 31);
      uint32_t img, pix;
      div_hw.divmod((uint32_t)(n < n_extent ? n : 0), img, pix);
      st.col_base[j] = n < n_extent ? (int)img * m_extent * HW + (int)pix : -1;
    }
  }
  __device__ inline void store(const State &st, int m, int /*n*/, int j, float v) const {
    if (m < m_extent && st.col_base[j] >= 0) out[st.col_base[j] + m * HW] = v;
  }
};

// D[m = c][n = (img, p, q)] -> dx[img][c][p*u][q*v]; the other positions of the
// u x v cell anchored there receive 0 (1x1 filter: they have no contribution).
struct StoreScatter {
  float *out;
  int m_extent, n_extent;  // C, N*P*Q
  FastDiv div_pq, div_q;
  int H, W, u, v;
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
      st.col_base[j] = n < n_extent ? ((int)img * m_extent * H + h0) * W + w0 : -1;
      st.rows[j] = min(u, H - h0);
      st.cols[j] = min(v, W - w0);
    }
  }
  __device__ inline void store(const State &st, int m, int /*n*/, int j, float val) const {
    if (m < m_extent && st.col_base[j] >= 0) {
      float *cell = out + st.col_base[j] + m * H * W;
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

// ---- host side --------------------------------------------------------------------------

template <int V>
using IC = std::integral_constant<int, V>;

template <class F>
void with_tile(int bm, int bn, F &&f) {
  if (bm == 128 && bn == 128) f(IC<128>{}, IC<128>{});
  else if (bm == 64 && bn == 128) f(IC<64>{}, IC<128>{});
  else f(IC<64>{}, IC<64>{});
}

// Largest tile that still yields about 1.5 workgroups per CU; the smallest otherwise.
void pick_tile(int M, int N, int &bm, int &bn) {
  static const int cand[3][2] = {{128, 128}, {64, 128}, {64, 64}};
  const int want = num_cus() * 3 / 2;
  for (auto &c : cand) {
    if (c[0] == 128 && M <= 64) continue;
    bm = c[0];
    bn = c[1];
    if (cdiv(M, bm) * cdiv(N, bn) >= want) return;
  }
}

template <int BM, int BN, class AL, class BL, class EP>
void launch(const AL &al, const BL &bl, const EP &ep, int K, const Geometry &g, hipStream_t s) {
  hipLaunchKernelGGL((gemm_kernel<BM, BN, AL, BL, EP>), dim3(g.blocks()), dim3(THREADS), 0, s, al, bl, ep, K,
                     g.k_per_split, g.tiles_m, g.tiles_n);
}

std::mutex g_tab_mu;

int upload_table(const std::vector<int> &host, int **dev) {
  TF_HIP(hipMalloc((void **)dev, host.size() * sizeof(int)));
  TF_HIP(hipMemcpy(*dev, host.data(), host.size() * sizeof(int), hipMemcpyHostToDevice));
  return 0;
}

// Reduction-index tables of a descriptor, built on first use and kept for its lifetime.
int ensure_tables(ConvDesc *d) {
  std::lock_guard<std::mutex> g(g_tab_mu);
  if (!d->fwd_tab) {
    std::vector<int> t((size_t)d->C * d->R * d->S * 2);
    size_t i = 0;
    for (int c = 0; c < d->C; ++c)
      for (int r = 0; r < d->R; ++r)
        for (int s = 0; s < d->S; ++s) {
          t[i++] = c * d->H * d->W;
          t[i++] = pack_taps(r, s);
        }
    if (upload_table(t, &d->fwd_tab) != 0) return -1;
  }
  if (!d->dgrad_tab) {
    std::vector<int> t((size_t)d->K * d->R * d->S * 2);
    size_t i = 0;
    for (int k = 0; k < d->K; ++k)
      for (int r = 0; r < d->R; ++r)
        for (int s = 0; s < d->S; ++s) {
          t[i++] = k * d->P * d->Q;
          t[i++] = pack_taps(-r, -s);
        }
    if (upload_table(t, &d->dgrad_tab) != 0) return -1;
  }
  return 0;
}

bool shape_is(const DLArray *a, int d0, int d1, int d2, int d3) {
  return a->ndim == 4 && a->shape[0] == d0 && a->shape[1] == d1 && a->shape[2] == d2 && a->shape[3] == d3;
}

constexpr int64_t kMaxBytes = (int64_t)1 << 31;  // buffer offsets are 31-bit

// Launch plan of each of the three convolutions of a descriptor: which loader
// mode / epilogue, which tile and how many k-splits.  The entry points and the
// introspection call below both use it, so they cannot disagree.
struct ConvPlan {
  const char *variant;
  int bm, bn, splits;
  int M, N, K;
};

ConvPlan plan_forward(const ConvDesc *d) {
  ConvPlan p;
  p.M = d->K;
  p.N = d->N * d->P * d->Q;
  p.K = d->C * d->R * d->S;
  pick_tile(p.M, p.N, p.bm, p.bn);
  p.splits = 1;
  p.variant = (d->pad_h || d->pad_w) ? "fwd_pad" : "fwd_nopad";
  return p;
}

ConvPlan plan_dgrad(const ConvDesc *d) {
  ConvPlan p;
  const int RS = d->R * d->S;
  p.M = d->C;
  p.K = d->K * RS;
  p.splits = 1;
  if (RS == 1) {
    p.N = d->N * d->P * d->Q;
    pick_tile(p.M, p.N, p.bm, p.bn);
    p.variant = (d->u == 1 && d->v == 1) ? "dgrad_1x1" : "dgrad_1x1_scatter";
  } else {
    p.N = d->N * d->H * d->W;
    if (d->u == 1 && d->v == 1) {
      pick_tile(p.M, p.N, p.bm, p.bn);
      p.variant = "dgrad_pad";
    } else {
      p.bm = p.bn = 64;
      p.variant = "dgrad_strided";
    }
  }
  return p;
}

ConvPlan plan_wgrad(const ConvDesc *d) {
  ConvPlan p;
  p.M = d->K;
  p.N = d->C * d->R * d->S;
  p.K = d->N * d->P * d->Q;
  const bool big = p.M > 64 && p.N > 64;
  p.bm = p.bn = big ? 128 : 64;
  const int tiles = cdiv(p.M, p.bm) * cdiv(p.N, p.bn);
  p.splits = make_geometry(p.M, p.N, p.K, p.bm, p.bn, choose_splits(tiles, p.K, 8 * BK)).splits;
  p.variant = (d->pad_h || d->pad_w) ? "wgrad_pad" : "wgrad_nopad";
  return p;
}

}  // namespace

// Introspection for benchmarks (no counterpart in the reference): writes a short
// name of the kernel variant that `which` (0 forward, 1 grad-data, 2 grad-filter)
// launches for this descriptor, e.g. "wgrad_pad_128x128_s37", and returns the
// algorithmic flop count 2*N*K*C*R*S*P*Q through *flops.
extern "C" int DLGpuConvolutionDescribeKernel(void ***list, int which, char *name, int name_len,
                                              double *flops) {
  ConvDesc *d = desc_from_list<ConvDesc>(list, kMagicConv);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuConvolution2DForwardGetOutShape");
  TF_REQUIRE(which >= 0 && which <= 2 && name && name_len > 0, "bad arguments");
  const ConvPlan p = which == 0 ? plan_forward(d) : which == 1 ? plan_dgrad(d) : plan_wgrad(d);
  snprintf(name, (size_t)name_len, "%s_%dx%d_s%d", p.variant, p.bm, p.bn, p.splits);
  if (flops)
    *flops = 2.0 * d->N * d->K * d->C * d->R * d->S * (double)d->P * d->Q;
  return 0;
}

extern "C" int DLGpuConvolution2DForwardGetOutShape(const int *input_shapes, const int *filter_shapes,
                                                    int *output_shapes, int dataformat, int padding,
                                                    const int u, const int v, void ***list) {
  TF_REQUIRE(input_shapes && filter_shapes && output_shapes && list, "null argument");
  TF_REQUIRE(dataformat == 0, "only NCHW (dataformat 0) is implemented");
  TF_REQUIRE(u >= 1 && v >= 1, "strides must be positive");
  ConvDesc *d = new ConvDesc();
  d->magic = kMagicConv;
  d->N = input_shapes[0];
  d->C = input_shapes[1];
  d->H = input_shapes[2];
  d->W = input_shapes[3];
  d->K = filter_shapes[0];
  d->R = filter_shapes[2];
  d->S = filter_shapes[3];
  TF_REQUIRE(filter_shapes[1] == d->C, "filter expects %d input channels, input has %d", filter_shapes[1], d->C);
  d->pad_h = padding == 1 ? d->R / 2 : 0;  // "SAME" is a symmetric k/2, "VALID" is 0
  d->pad_w = padding == 1 ? d->S / 2 : 0;
  d->u = u;
  d->v = v;
  TF_REQUIRE(d->H + 2 * d->pad_h >= d->R && d->W + 2 * d->pad_w >= d->S, "filter larger than padded input");
  d->P = 1 + (d->H + 2 * d->pad_h - d->R) / u;
  d->Q = 1 + (d->W + 2 * d->pad_w - d->S) / v;
  TF_REQUIRE(d->R < 32768 && d->S < 32768, "filter extent too large");
  d->fwd_tab = nullptr;
  d->dgrad_tab = nullptr;
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
  (void)handle;
  (void)memorytoSaving;
  ConvDesc *d = desc_from_list<ConvDesc>(list, kMagicConv);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuConvolution2DForwardGetOutShape");
  if (check_conv_arrays(d, input, filter, output) != 0) return -1;
  if (ensure_tables(d) != 0) return -1;
  hipStream_t s = stream_of(stream);
  const ConvPlan plan = plan_forward(d);
  const int M = plan.M, N = plan.N, K = plan.K;
  if (M == 0 || N == 0) return 0;
  const int bm = plan.bm, bn = plan.bn;
  const Geometry g = make_geometry(M, N, K, bm, bn, 1);
  const bool padded = d->pad_h != 0 || d->pad_w != 0;
  with_tile(bm, bn, [&](auto bm_c, auto bn_c) {
    constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value;
    PlainAcross<BM> al{(const float *)filter->data, (uint32_t)(numel(filter) * 4), K, M, K};
    StoreNCHW ep{(float *)output->data, M, N, FastDiv((uint32_t)(d->P * d->Q)), d->P * d->Q};
    auto run = [&](auto mode_c) {
      constexpr int MODE = decltype(mode_c)::value;
      GatherAlong<BN, MODE> bl{(const float *)input->data, (uint32_t)(numel(input) * 4),
                               (const int2 *)d->fwd_tab, K, N,
                               FastDiv((uint32_t)(d->P * d->Q)), FastDiv((uint32_t)d->Q),
                               d->C * d->H * d->W, d->H, d->W, d->u, d->v, -d->pad_h, -d->pad_w,
                               FastDiv(1), FastDiv(1)};
      launch<BM, BN>(al, bl, ep, K, g, s);
    };
    if (padded) run(IC<1>{}); else run(IC<0>{});
  });
  return finish(s, "DLGpuConvolution2DForward");
}

extern "C" int DLGpuConvolutionBackwardData(const DLArrayHandle input, const DLArrayHandle doutput,
                                            const DLArrayHandle filter, DLArrayHandle dinput, void ***list,
                                            void **handle, int *memorytoSaving, void **stream) {
  (void)handle;
  ConvDesc *d = desc_from_list<ConvDesc>(list, kMagicConv);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuConvolution2DForwardGetOutShape");
  if (check_conv_arrays(d, input, filter, doutput) != 0) return -1;
  TF_REQUIRE(on_gpu(dinput) && same_shape(dinput, input), "dinput must have the input's shape");
  if (ensure_tables(d) != 0) return -1;
  hipStream_t s = stream_of(stream);
  const int RS = d->R * d->S;
  const ConvPlan plan = plan_dgrad(d);
  const int M = plan.M, K = plan.K;
  if (numel(dinput) == 0) return 0;
  if (numel(doutput) == 0) return DLGpuArraySet(dinput, 0.f, stream);

  // filter as [(k, r, s)][c]; a 1x1 filter already has that layout
  const float *wt = (const float *)filter->data;
  float *wt_scratch = nullptr;
  if (RS > 1) {
    const size_t bytes = (size_t)numel(filter) * sizeof(float);
    wt_scratch = (float *)device_alloc(bytes);
    if (!wt_scratch) {
      if (memorytoSaving) *memorytoSaving = (int)bytes;
      return 0;
    }
    const int total = (int)numel(filter);
    hipLaunchKernelGGL(filter_to_krsc_kernel, dim3(min(cdiv(total, 256), num_cus() * 8)), dim3(256), 0, s,
                       (const float *)filter->data, wt_scratch, d->K, d->C, RS);
    wt = wt_scratch;
  }
  const uint32_t w_bytes = (uint32_t)(numel(filter) * 4), dy_bytes = (uint32_t)(numel(doutput) * 4);
  const int PQ = d->P * d->Q;

  if (RS == 1) {
    // 1x1 filter (pad 0): compact GEMM over the output pixels + scatter
    const int N = plan.N;
    const int bm = plan.bm, bn = plan.bn;
    const Geometry g = make_geometry(M, N, K, bm, bn, 1);
    with_tile(bm, bn, [&](auto bm_c, auto bn_c) {
      constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value;
      PlainAlong<BM> al{wt, w_bytes, d->C, M, K};
      GatherAlong<BN, 0> bl{(const float *)doutput->data, dy_bytes, (const int2 *)d->dgrad_tab, K, N,
                            FastDiv((uint32_t)PQ), FastDiv((uint32_t)d->Q), d->K * PQ, d->P, d->Q,
                            1, 1, 0, 0, FastDiv(1), FastDiv(1)};
      if (d->u == 1 && d->v == 1) {
        StoreNCHW ep{(float *)dinput->data, M, N, FastDiv((uint32_t)PQ), PQ};
        launch<BM, BN>(al, bl, ep, K, g, s);
      } else {
        StoreScatter ep{(float *)dinput->data, M, N, FastDiv((uint32_t)PQ), FastDiv((uint32_t)d->Q),
                        d->H, d->W, d->u, d->v};
        launch<BM, BN>(al, bl, ep, K, g, s);
      }
    });
  } else {
    const int N = plan.N;
    const int HW = d->H * d->W;
    const int bm = plan.bm, bn = plan.bn;
    StoreNCHW ep{(float *)dinput->data, M, N, FastDiv((uint32_t)HW), HW};
    if (d->u == 1 && d->v == 1) {
      const Geometry g = make_geometry(M, N, K, bm, bn, 1);
      with_tile(bm, bn, [&](auto bm_c, auto bn_c) {
        constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value;
        PlainAlong<BM> al{wt, w_bytes, d->C, M, K};
        GatherAlong<BN, 1> bl{(const float *)doutput->data, dy_bytes, (const int2 *)d->dgrad_tab, K, N,
                              FastDiv((uint32_t)HW), FastDiv((uint32_t)d->W), d->K * PQ, d->P, d->Q,
                              1, 1, d->pad_h, d->pad_w, FastDiv(1), FastDiv(1)};
        launch<BM, BN>(al, bl, ep, K, g, s);
      });
    } else {
      // strided filter larger than 1x1: every input pixel, taps filtered by divisibility
      const Geometry g = make_geometry(M, N, K, 64, 64, 1);
      PlainAlong<64> al{wt, w_bytes, d->C, M, K};
      GatherAlong<64, 2> bl{(const float *)doutput->data, dy_bytes, (const int2 *)d->dgrad_tab, K, N,
                            FastDiv((uint32_t)HW), FastDiv((uint32_t)d->W), d->K * PQ, d->P, d->Q,
                            1, 1, d->pad_h, d->pad_w, FastDiv((uint32_t)d->u), FastDiv((uint32_t)d->v)};
      launch<64, 64>(al, bl, ep, K, g, s);
    }
  }
  if (wt_scratch) device_free(wt_scratch);
  return finish(s, "DLGpuConvolutionBackwardData");
}

extern "C" int DLGpuConvolutionBackwardFilter(const DLArrayHandle input, const DLArrayHandle doutput,
                                              const DLArrayHandle filter, DLArrayHandle dfilter, void ***list,
                                              void **handle, int *memorytoSaving, void **stream) {
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

  const int bm = plan.bm, bn = plan.bn;
  Geometry g = make_geometry(M, N, K, bm, bn, plan.splits);
  float *dst = (float *)dfilter->data;
  float *partial = nullptr;
  if (g.splits > 1) {
    const size_t bytes = (size_t)g.splits * M * N * sizeof(float);
    partial = (float *)device_alloc(bytes);
    if (!partial) {
      if (memorytoSaving) *memorytoSaving = (int)bytes;
      return 0;
    }
    dst = partial;
  }
  const bool padded = d->pad_h != 0 || d->pad_w != 0;
  with_tile(bm, bn, [&](auto bm_c, auto bn_c) {
    constexpr int BM = decltype(bm_c)::value, BN = decltype(bn_c)::value;
    if constexpr (BM == BN) {  // only the square tiles are used for grad-filter
      DyAcross<BM> al{(const float *)doutput->data, (uint32_t)(numel(doutput) * 4), K, M,
                      FastDiv((uint32_t)PQ), d->K * PQ, PQ};
      StoreRowMajor ep{dst, N, M, N, (int64_t)M * N};
      auto run = [&](auto mode_c) {
        constexpr int MODE = decltype(mode_c)::value;
        GatherAcross<BN, MODE> bl{(const float *)input->data, (uint32_t)(numel(input) * 4), K, N,
                                  FastDiv((uint32_t)PQ), FastDiv((uint32_t)d->Q), FastDiv((uint32_t)RS),
                                  FastDiv((uint32_t)d->S), d->C * d->H * d->W, d->H * d->W,
                                  d->H, d->W, d->u, d->v, d->pad_h, d->pad_w};
        launch<BM, BN>(al, bl, ep, K, g, s);
      };
      if (padded) run(IC<1>{}); else run(IC<0>{});
    }
  });
  if (partial) {
    launch_split_sum(partial, (float *)dfilter->data, (int64_t)M * N, g.splits, s);
    device_free(partial);
  }
  return finish(s, "DLGpuConvolutionBackwardFilter");
}
