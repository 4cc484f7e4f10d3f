/*
 * CPU oracle, brute force -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Direct seven-loop evaluation of the three convolution definitions exactly as
 * written in the reference's call sites (cross-correlation, NCHW activations,
 * KCRS filters, symmetric zero padding, dilation 1):
 *   forward      src/gpu_op.cu:1952-2038  (cudnnConvolutionForward)
 *   grad-data    src/gpu_op.cu:1739-1824  (cudnnConvolutionBackwardData, beta 0)
 *   grad-filter  src/gpu_op.cu:1653-1737  (cudnnConvolutionBackwardFilter, beta 0)
 * No im2col, no GEMM, double accumulation: it shares no structure with the numpy
 * oracle (oracle/ops.py) or with the HIP kernels, and pins both on small inputs.
 *
 * Built by oracle/build_oracle.py into oracle/_build/libconv_direct.so.
 */
#include <stddef.h>

#define X_AT(n, c, h, w) x[(((size_t)(n) * C + (c)) * H + (h)) * W + (w)]
#define W_AT(k, c, r, s) wt[(((size_t)(k) * C + (c)) * R + (r)) * S + (s)]
#define Y_AT(n, k, p, q) y[(((size_t)(n) * K + (k)) * P + (p)) * Q + (q)]

void conv_direct_forward(const double *x, const double *wt, double *y, int N, int C, int H, int W, int K,
                         int R, int S, int P, int Q, int pad_h, int pad_w, int u, int v) {
  for (int n = 0; n < N; ++n)
    for (int k = 0; k < K; ++k)
      for (int p = 0; p < P; ++p)
        for (int q = 0; q < Q; ++q) {
          double acc = 0.0;
          for (int c = 0; c < C; ++c)
            for (int r = 0; r < R; ++r)
              for (int s = 0; s < S; ++s) {
                const int h = p * u + r - pad_h, w = q * v + s - pad_w;
                if (h >= 0 && h < H && w >= 0 && w < W) acc += X_AT(n, c, h, w) * W_AT(k, c, r, s);
              }
          Y_AT(n, k, p, q) = acc;
        }
}

/* dx[n,c,h,w] = sum over (k,p,q,r,s) with h = p*u + r - pad_h, w = q*v + s - pad_w */
void conv_direct_backward_data(const double *y /* dy */, const double *wt, double *x /* dx */, int N, int C,
                               int H, int W, int K, int R, int S, int P, int Q, int pad_h, int pad_w, int u,
                               int v) {
  for (size_t i = 0; i < (size_t)N * C * H * W; ++i) x[i] = 0.0;
  for (int n = 0; n < N; ++n)
    for (int k = 0; k < K; ++k)
      for (int p = 0; p < P; ++p)
        for (int q = 0; q < Q; ++q)
          for (int c = 0; c < C; ++c)
            for (int r = 0; r < R; ++r)
              for (int s = 0; s < S; ++s) {
                const int h = p * u + r - pad_h, w = q * v + s - pad_w;
                if (h >= 0 && h < H && w >= 0 && w < W) X_AT(n, c, h, w) += Y_AT(n, k, p, q) * W_AT(k, c, r, s);
              }
}

void conv_direct_backward_filter(const double *x, const double *y /* dy */, double *wt /* dw */, int N, int C,
                                 int H, int W, int K, int R, int S, int P, int Q, int pad_h, int pad_w, int u,
                                 int v) {
  for (int k = 0; k < K; ++k)
    for (int c = 0; c < C; ++c)
      for (int r = 0; r < R; ++r)
        for (int s = 0; s < S; ++s) {
          double acc = 0.0;
          for (int n = 0; n < N; ++n)
            for (int p = 0; p < P; ++p)
              for (int q = 0; q < Q; ++q) {
                const int h = p * u + r - pad_h, w = q * v + s - pad_w;
                if (h >= 0 && h < H && w >= 0 && w < W) acc += Y_AT(n, k, p, q) * X_AT(n, c, h, w);
              }
          W_AT(k, c, r, s) = acc;
        }
}
