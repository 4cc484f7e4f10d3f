// Batch normalisation forward (training) and backward with gamma = 1, beta = 0,
// eps = 1e-5 and biased variance -- the only configuration the reference uses
// (src/gpu_op.cu:4224-4458: scale/bias are rebuilt as ones/zeros on every call,
// the scale/bias gradients cuDNN returns are discarded, there are no running
// statistics).
//
// per-activation mode (what every reference model graph passes): one statistic
//   per (c,h,w) position over the batch.  x is an [N, L] matrix, L = C*H*W; a lane
//   owns one column, keeps its N values in registers, and the whole op is a
//   single pass: forward reads x and writes y (8 B/element), backward reads x, dy
//   and writes dx (12 B/element).  Lanes of a wave read 64 consecutive columns,
//   so every access is a full 256-byte line.
// spatial mode: one statistic per channel over (N,H,W).  Three kernels: per-(channel,
//   image-chunk) partial sums (fp32 per lane, fp64 across lanes and chunks), a tiny
//   one that folds the chunks of every channel in a fixed order, and a streaming
//   normalise pass over the flat tensor (12 B/element forward, 20 backward).
//
// Saved statistics protocol (as the reference): forward allocates mean and
// inverse-std buffers and publishes them through *mean_p / *Variance_p; backward
// consumes and releases them.
#include "gemm_core.h"
#include "internal.h"

#include <type_traits>

using namespace tf;
using tf::gemm::FastDiv;

namespace {

constexpr int kThreads = 256;
constexpr float kEps = 1e-5f;
constexpr int kNonTemporal = 2;  // cache-policy operand of a buffer access: a stream that is read once
typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- per-activation

// NREG >= N values of one column live in registers.  The three tensors are addressed
// through buffer descriptors: one per-lane column offset (a VGPR computed once) plus a
// uniform row offset (a scalar) per access, instead of a 64-bit vector address per
// access -- the address arithmetic was more than half of the kernel's instructions and
// cost as many registers as a quarter of the data.  A descriptor covers exactly the N
// rows, so rows N..NREG-1 read as zero and their stores are dropped by the bounds
// check: no per-row branch.  Needs NREG * L * 4 < 2^32 (the row offsets are 32-bit).
// RELU: y = max(bn(x), 0) in the same pass (the fused entry points below).
// FULL: N == NREG, no row needs masking in the variance.
template <int NREG, bool RELU, bool FULL>
__global__ __launch_bounds__(kThreads) void bn_pa_forward_kernel(const float *__restrict__ x,
                                                                float *__restrict__ y,
                                                                float *__restrict__ save_mean,
                                                                float *__restrict__ save_istd, int N, uint32_t L) {
  const uint32_t l = blockIdx.x * kThreads + threadIdx.x;
  if (l >= L) return;
  const uint32_t col = l * 4u, row = L * 4u;
  const __amdgpu_buffer_rsrc_t rx = gemm::make_rsrc(x, (uint32_t)N * row), ry = gemm::make_rsrc(y, (uint32_t)N * row);
  float v[NREG];
#pragma unroll
  for (int n = 0; n < NREG; ++n)
    v[n] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, (int)col, (int)(n * row), kNonTemporal));
  float s = 0.f;
#pragma unroll
  for (int n = 0; n < NREG; ++n) s += v[n];
  const float mean = s / (float)N;
  float q = 0.f;
#pragma unroll
  for (int n = 0; n < NREG; ++n) {
    const float dlt = (FULL || n < N) ? v[n] - mean : 0.f;
    q += dlt * dlt;
  }
  const float istd = 1.0f / sqrtf(q / (float)N + kEps);
  save_mean[l] = mean;
  save_istd[l] = istd;
#pragma unroll
  for (int n = 0; n < NREG; ++n) {
    const float out = (v[n] - mean) * istd;
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, (RELU && out < 0.f) ? 0.f : out), ry, (int)col,
                                          (int)(n * row), 0);
  }
}

// any N: three sweeps over the column (the second and third hit the cache)
template <bool RELU>
__global__ __launch_bounds__(kThreads) void bn_pa_forward_stream_kernel(const float *__restrict__ x,
                                                                       float *__restrict__ y,
                                                                       float *__restrict__ save_mean,
                                                                       float *__restrict__ save_istd, int N,
                                                                       int64_t L) {
  const int64_t l = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (l >= L) return;
  float s = 0.f;
  for (int n = 0; n < N; ++n) s += x[(int64_t)n * L + l];
  const float mean = s / (float)N;
  float q = 0.f;
  for (int n = 0; n < N; ++n) {
    const float dlt = x[(int64_t)n * L + l] - mean;
    q += dlt * dlt;
  }
  const float istd = 1.0f / sqrtf(q / (float)N + kEps);
  save_mean[l] = mean;
  save_istd[l] = istd;
  for (int n = 0; n < N; ++n) {
    const float out = (x[(int64_t)n * L + l] - mean) * istd;
    y[(int64_t)n * L + l] = (RELU && out < 0.f) ? 0.f : out;
  }
}

// dx = istd/N * (N*dy - sum(dy) - xhat * sum(dy*xhat))
// RELU: dy is first masked with bn(x) > 0, i.e. the gradient of max(bn(x), 0).
// Addressing as in the forward kernel; a row beyond N reads dy = 0 and adds nothing.
template <int NREG, bool RELU>
__global__ __launch_bounds__(kThreads) void bn_pa_backward_kernel(const float *__restrict__ x,
                                                                 const float *__restrict__ dy,
                                                                 float *__restrict__ dx,
                                                                 const float *__restrict__ save_mean,
                                                                 const float *__restrict__ save_istd, int N,
                                                                 uint32_t L) {
  const uint32_t l = blockIdx.x * kThreads + threadIdx.x;
  if (l >= L) return;
  const uint32_t col = l * 4u, row = L * 4u, all = (uint32_t)N * row;
  const __amdgpu_buffer_rsrc_t rx = gemm::make_rsrc(x, all), rg = gemm::make_rsrc(dy, all),
                               ro = gemm::make_rsrc(dx, all);
  const float mean = save_mean[l], istd = save_istd[l];
  float xh[NREG], g[NREG];
#pragma unroll
  for (int n = 0; n < NREG; ++n) {
    xh[n] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, (int)col, (int)(n * row), kNonTemporal));
    g[n] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rg, (int)col, (int)(n * row), kNonTemporal));
  }
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int n = 0; n < NREG; ++n) {
    xh[n] = (xh[n] - mean) * istd;
    if (RELU) g[n] = xh[n] > 0.f ? g[n] : 0.f;
    s1 += g[n];
    s2 += g[n] * xh[n];
  }
  const float m = (float)N;
  const float scale = istd / m;
#pragma unroll
  for (int n = 0; n < NREG; ++n)
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, scale * (m * g[n] - s1 - xh[n] * s2)), ro, (int)col,
                                          (int)(n * row), 0);
}

template <bool RELU>
__global__ __launch_bounds__(kThreads) void bn_pa_backward_stream_kernel(const float *__restrict__ x,
                                                                        const float *__restrict__ dy,
                                                                        float *__restrict__ dx,
                                                                        const float *__restrict__ save_mean,
                                                                        const float *__restrict__ save_istd,
                                                                        int N, int64_t L) {
  const int64_t l = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (l >= L) return;
  const float mean = save_mean[l], istd = save_istd[l];
  float s1 = 0.f, s2 = 0.f;
  for (int n = 0; n < N; ++n) {
    const float xh = (x[(int64_t)n * L + l] - mean) * istd;
    float g = dy[(int64_t)n * L + l];
    if (RELU) g = xh > 0.f ? g : 0.f;
    s1 += g;
    s2 += g * xh;
  }
  const float m = (float)N;
  const float scale = istd / m;
  for (int n = 0; n < N; ++n) {
    const float xh = (x[(int64_t)n * L + l] - mean) * istd;
    float g = dy[(int64_t)n * L + l];
    if (RELU) g = xh > 0.f ? g : 0.f;
    dx[(int64_t)n * L + l] = scale * (m * g - s1 - xh * s2);
  }
}

// ------------------------------------------------------------------------ spatial

__device__ inline double wave_sum_d(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// Sum of a pair over the 256 lanes of a block, valid in thread 0.
__device__ inline void block_sum2(double &a, double &b, double (*smem)[2]) {
  a = wave_sum_d(a);
  b = wave_sum_d(b);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    smem[wave][0] = a;
    smem[wave][1] = b;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    a = (smem[0][0] + smem[1][0]) + (smem[2][0] + smem[3][0]);
    b = (smem[0][1] + smem[1][1]) + (smem[2][1] + smem[3][1]);
  }
}

// One unit of the spatial kernels: a 16-byte vector (feature maps whose size is a
// multiple of 4) or a single float.
template <bool VEC>
struct Unit;
template <>
struct Unit<true> {
  static constexpr int W = 4;
  static __device__ inline void load(const float *p, float (&v)[4]) {
    const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  static __device__ inline void store(float *p, const float (&v)[4]) {
    const f32x4 t = {v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4 *>(p) = t;
  }
};
template <>
struct Unit<false> {
  static constexpr int W = 1;
  static __device__ inline void load(const float *p, float (&v)[1]) { v[0] = *p; }
  static __device__ inline void store(float *p, const float (&v)[1]) { *p = v[0]; }
};

// x viewed as [N, C, HW]; block (c, chunk) sums images [chunk*ipc, ...) of channel c.
// FWD: partial = (sum (x - p), sum (x - p)^2) with the pivot p = the channel's first
// element (image 0, pixel 0): sums of shifted values lose nothing to cancellation
// when |mean| is much larger than the standard deviation, where sum x^2 - m*mean^2
// in fp32 would.  BWD: partial = (sum dy, sum dy*xhat).
// The (image, pixel) pairs of a chunk are walked as one flat index so that small
// feature maps (7x7) keep all lanes busy; VEC: 16-byte loads when HW is a multiple
// of 4.  Lanes accumulate in fp32 (a few hundred terms each), the block and the
// chunks are combined in fp64.
template <bool BWD, bool VEC>
__global__ __launch_bounds__(kThreads) void bn_sp_partial_kernel(const float *__restrict__ x,
                                                                const float *__restrict__ dy,
                                                                const float *__restrict__ save_mean,
                                                                const float *__restrict__ save_istd,
                                                                double *__restrict__ partial, int N, int C,
                                                                int HW, int images_per_chunk, FastDiv div_row) {
  __shared__ double smem[4][2];
  const int c = blockIdx.x;
  const int n0 = blockIdx.y * images_per_chunk;
  int n1 = n0 + images_per_chunk;
  if (n1 > N) n1 = N;
  const float mean = BWD ? save_mean[c] : 0.f, istd = BWD ? save_istd[c] : 0.f;
  const float pivot = BWD ? 0.f : x[(int64_t)c * HW];
  constexpr int W = Unit<VEC>::W;
  const uint32_t row_units = (uint32_t)HW / W;                 // div_row divides by this
  const uint32_t total = (uint32_t)(n1 - n0) * row_units;
  float a0 = 0.f, b0 = 0.f;
  for (uint32_t idx = threadIdx.x; idx < total; idx += kThreads) {
    uint32_t img, unit;
    div_row.divmod(idx, img, unit);
    const int64_t at = ((int64_t)(n0 + (int)img) * C + c) * HW + (int64_t)unit * W;
    float xv[W], gv[W] = {};
    Unit<VEC>::load(x + at, xv);
    if (BWD) Unit<VEC>::load(dy + at, gv);
#pragma unroll
    for (int k = 0; k < W; ++k) {
      if (BWD) {
        a0 += gv[k];
        b0 += gv[k] * ((xv[k] - mean) * istd);
      } else {
        const float t = xv[k] - pivot;
        a0 += t;
        b0 += t * t;
      }
    }
  }
  double a = (double)a0, b = (double)b0;
  block_sum2(a, b, smem);
  if (threadIdx.x == 0) {
    partial[((int64_t)blockIdx.y * C + c) * 2 + 0] = a;
    partial[((int64_t)blockIdx.y * C + c) * 2 + 1] = b;
  }
}

// Folds the chunk partials of every channel, in chunk order, into the two floats
// the apply pass needs: forward (mean, 1/sqrt(var + eps)), which are also the saved
// statistics; backward (sum dy, sum dy*xhat).
template <bool BWD>
__global__ __launch_bounds__(kThreads) void bn_sp_finish_kernel(const double *__restrict__ partial,
                                                               const float *__restrict__ x,
                                                               float *__restrict__ out0, float *__restrict__ out1,
                                                               int N, int C, int HW, int chunks) {
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= C) return;
  double s = 0.0, q = 0.0;
  for (int k = 0; k < chunks; ++k) {
    s += partial[((int64_t)k * C + c) * 2 + 0];
    q += partial[((int64_t)k * C + c) * 2 + 1];
  }
  if (BWD) {
    out0[c] = (float)s;
    out1[c] = (float)q;
  } else {
    const double m = (double)N * (double)HW;
    const double shifted_mean = s / m;  // mean of x - pivot; the variance does not depend on the pivot
    double var = q / m - shifted_mean * shifted_mean;
    if (var < 0.0) var = 0.0;
    out0[c] = (float)((double)x[(int64_t)c * HW] + shifted_mean);
    out1[c] = (float)(1.0 / sqrt(var + (double)kEps));
  }
}

// Apply pass over the flat tensor, one contiguous run of 1024 units (16 KiB when
// VEC) per workgroup as in the elementwise engine; a unit (float4 or float) lies
// inside one (image, channel) row, whose channel is (unit / units per row) % C.
// FWD: y = (x - mean) * istd.  BWD: dx = istd/m * (m*dy - s1 - xhat*s2).
template <bool BWD, bool VEC>
__global__ __launch_bounds__(kThreads) void bn_sp_apply_kernel(const float *__restrict__ x,
                                                              const float *__restrict__ dy,
                                                              float *__restrict__ out,
                                                              const float *__restrict__ p_mean,
                                                              const float *__restrict__ p_istd,
                                                              const float *__restrict__ p_s1,
                                                              const float *__restrict__ p_s2, float m,
                                                              FastDiv div_row, FastDiv div_c, uint32_t units) {
  constexpr int W = Unit<VEC>::W;
  constexpr int kUnroll = 4;
  const uint32_t base = blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
  float xv[kUnroll][W], gv[kUnroll][W] = {};
  uint32_t ch[kUnroll] = {};
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const uint32_t unit = base + u * kThreads;
    if (unit >= units) continue;
    uint32_t img;
    div_c.divmod(div_row.div(unit), img, ch[u]);
    Unit<VEC>::load(x + (int64_t)unit * W, xv[u]);
    if (BWD) Unit<VEC>::load(dy + (int64_t)unit * W, gv[u]);
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const uint32_t unit = base + u * kThreads;
    if (unit >= units) continue;
    const float mean = p_mean[ch[u]], istd = p_istd[ch[u]];
    float r[W];
    if (BWD) {
      const float s1 = p_s1[ch[u]], s2 = p_s2[ch[u]];
      const float scale = istd / m;
#pragma unroll
      for (int k = 0; k < W; ++k) {
        const float xh = (xv[u][k] - mean) * istd;
        r[k] = scale * (m * gv[u][k] - s1 - xh * s2);
      }
    } else {
#pragma unroll
      for (int k = 0; k < W; ++k) r[k] = (xv[u][k] - mean) * istd;
    }
    Unit<VEC>::store(out + (int64_t)unit * W, r);
  }
}

template <int NREG, bool RELU>
void pa_forward(dim3 grid, dim3 block, hipStream_t s, const float *x, float *y, float *mean, float *istd, int N,
                uint32_t L) {
  if (N == NREG)
    hipLaunchKernelGGL((bn_pa_forward_kernel<NREG, RELU, true>), grid, block, 0, s, x, y, mean, istd, N, L);
  else
    hipLaunchKernelGGL((bn_pa_forward_kernel<NREG, RELU, false>), grid, block, 0, s, x, y, mean, istd, N, L);
}

// The register kernels address row n at the 32-bit byte offset n * L * 4.
bool pa_rows_addressable(int nreg, int64_t L) { return (int64_t)nreg * L * 4 < ((int64_t)1 << 32); }

int sp_chunks(int N, int C) {
  // about four workgroups per CU in the partial pass
  int chunks = cdiv((int64_t)num_cus() * 4, C);
  if (chunks > N) chunks = N;
  return chunks < 1 ? 1 : chunks;
}

int check_bn_arrays(const BNDesc *d, const DLArray *a, const DLArray *b) {
  TF_REQUIRE(on_gpu(a) && on_gpu(b), "arrays must live on the GPU");
  const int64_t n = (int64_t)d->N * d->C * d->HW;
  TF_REQUIRE(numel(a) == n && numel(b) == n, "arrays do not match the descriptor");
  // the spatial kernels index units with 32-bit fast division
  TF_REQUIRE(d->mode == 0 || n < (int64_t(1) << 31), "spatial mode supports fewer than 2^31 elements");
  return 0;
}

}  // namespace

extern "C" int DLGpuBatchNormalizationGetCudnnlist(const int *input_shapes, int sizeofshape, int dataformat,
                                                   int batchNormMode, void **mean_p, void **Variance_p,
                                                   void ***list) {
  (void)mean_p;
  (void)Variance_p;
  TF_REQUIRE(input_shapes && list, "null argument");
  TF_REQUIRE(sizeofshape >= 2 && sizeofshape <= 5, "rank %d not supported", sizeofshape);
  TF_REQUIRE(dataformat == 0, "only NCHW (dataformat 0) is implemented");
  TF_REQUIRE(batchNormMode == 0 || batchNormMode == 1, "unknown batch-norm mode %d", batchNormMode);
  int64_t hw = 1;
  for (int i = 0; i < sizeofshape; ++i) {
    TF_REQUIRE(input_shapes[i] >= 0, "negative extent");
    if (i >= 2) hw *= input_shapes[i];
    TF_REQUIRE(hw <= INT32_MAX, "spatial extent too large");
  }
  BNDesc *d = new BNDesc();
  d->magic = kMagicBN;
  d->mode = batchNormMode;
  d->N = input_shapes[0];
  d->C = input_shapes[1];
  d->HW = (int)hw;
  d->stat_count = batchNormMode == 0 ? (int64_t)d->C * d->HW : d->C;
  d->saved_mean = d->saved_istd = nullptr;
  void **slots = (void **)malloc(sizeof(void *) * 3);
  slots[0] = slots[1] = slots[2] = d;
  *list = slots;
  return 0;
}

static int bn_forward_impl(const DLArrayHandle input, DLArrayHandle output, int batchNormMode, int n,
                           void **mean_p, void **Variance_p, void ***list, void **handle, int *memorytoSaving,
                           void **stream, bool relu, const char *what) {
  (void)handle;
  (void)n;  // would weight running statistics, which the reference never keeps
  BNDesc *d = desc_from_list<BNDesc>(list, kMagicBN);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuBatchNormalizationGetCudnnlist");
  TF_REQUIRE(d->mode == batchNormMode, "mode differs from the descriptor");
  TF_REQUIRE(mean_p && Variance_p, "null statistics cell");
  TF_REQUIRE(!relu || d->mode == 0, "the fused batch-norm + ReLU entry points implement per-activation mode only");
  if (check_bn_arrays(d, input, output) != 0) return -1;
  hipStream_t s = stream_of(stream);
  const size_t stat_bytes = (size_t)d->stat_count * sizeof(float);
  if (d->saved_mean) {  // a forward whose backward never ran: recycle its statistics
    device_free(d->saved_mean);
    device_free(d->saved_istd);
    d->saved_mean = d->saved_istd = nullptr;
  }
  // Everything this call allocates, which is what it reports when any of it cannot be had:
  // a caller that makes that much room must be able to repeat the call.
  const int sp_real_chunks = (d->mode == 0 || numel(input) == 0) ? 0 : cdiv(d->N, cdiv(d->N, sp_chunks(d->N, d->C)));
  const size_t sp_partial_bytes = (size_t)sp_real_chunks * d->C * 2 * sizeof(double);
  const size_t all_bytes = 2 * block_bytes(stat_bytes) + (sp_partial_bytes ? block_bytes(sp_partial_bytes) : 0);
  float *mean = (float *)device_alloc(stat_bytes);
  float *istd = mean ? (float *)device_alloc(stat_bytes) : nullptr;
  if (!mean || !istd) {
    if (mean) device_free(mean);
    if (memorytoSaving) *memorytoSaving = shortfall(all_bytes);
    return 0;
  }
  *mean_p = d->saved_mean = mean;
  *Variance_p = d->saved_istd = istd;
  const float *x = (const float *)input->data;
  float *y = (float *)output->data;
  if (numel(input) == 0) return 0;
  if (d->mode == 0) {
    const int64_t L = d->stat_count;
    const dim3 grid(cdiv(L, kThreads)), block(kThreads);
    auto run = [&](auto relu_c) {
      constexpr bool RELU = decltype(relu_c)::value;
      const uint32_t l32 = (uint32_t)L;
      if (d->N <= 32 && pa_rows_addressable(32, L))
        pa_forward<32, RELU>(grid, block, s, x, y, mean, istd, d->N, l32);
      else if (d->N <= 64 && pa_rows_addressable(64, L))
        pa_forward<64, RELU>(grid, block, s, x, y, mean, istd, d->N, l32);
      else if (d->N <= 128 && pa_rows_addressable(128, L))
        pa_forward<128, RELU>(grid, block, s, x, y, mean, istd, d->N, l32);
      else
        hipLaunchKernelGGL(bn_pa_forward_stream_kernel<RELU>, grid, block, 0, s, x, y, mean, istd, d->N, L);
    };
    if (relu) run(std::true_type{}); else run(std::false_type{});
  } else {
    const int chunks = sp_chunks(d->N, d->C);
    const int ipc = cdiv(d->N, chunks);
    const int real_chunks = sp_real_chunks;
    double *partial = (double *)device_alloc(sp_partial_bytes);
    if (!partial) {
      device_free(mean);
      device_free(istd);
      *mean_p = d->saved_mean = nullptr;
      *Variance_p = d->saved_istd = nullptr;
      if (memorytoSaving) *memorytoSaving = shortfall(all_bytes);
      return 0;
    }
    const bool vec = d->HW % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
    const int W = vec ? 4 : 1;
    const FastDiv div_row((uint32_t)(d->HW / W)), div_c((uint32_t)d->C);
    const uint32_t units = (uint32_t)((int64_t)d->N * d->C * d->HW / W);
    const dim3 pgrid(d->C, real_chunks), agrid((units + kThreads * 4 - 1) / (kThreads * 4));
    auto run = [&](auto vec_c) {
      constexpr bool VEC = decltype(vec_c)::value;
      hipLaunchKernelGGL((bn_sp_partial_kernel<false, VEC>), pgrid, dim3(kThreads), 0, s, x, (const float *)nullptr,
                         (const float *)nullptr, (const float *)nullptr, partial, d->N, d->C, d->HW, ipc, div_row);
      hipLaunchKernelGGL(bn_sp_finish_kernel<false>, dim3(cdiv(d->C, kThreads)), dim3(kThreads), 0, s, partial, x,
                         mean, istd, d->N, d->C, d->HW, real_chunks);
      hipLaunchKernelGGL((bn_sp_apply_kernel<false, VEC>), agrid, dim3(kThreads), 0, s, x, (const float *)nullptr, y,
                         (const float *)mean, (const float *)istd, (const float *)nullptr, (const float *)nullptr,
                         0.f, div_row, div_c, units);
    };
    if (vec) run(std::true_type{}); else run(std::false_type{});
    device_free(partial);
  }
  return finish(s, what);
}

extern "C" int DLGpuBatchNormalizationForward(const DLArrayHandle input, DLArrayHandle output,
                                              int batchNormMode, int n, void **mean_p, void **Variance_p,
                                              void ***list, void **handle, int *memorytoSaving,
                                              void **stream) {
  announce_write(output);
  return bn_forward_impl(input, output, batchNormMode, n, mean_p, Variance_p, list, handle, memorytoSaving, stream,
                         false, "DLGpuBatchNormalizationForward");
}

// No counterpart in the reference: y = max(bn(x), 0) in one pass over x (8 bytes per
// element instead of 16 for the two ops), per-activation mode.  Same statistics
// protocol as the plain forward; pairs with DLGpuBatchNormalizationReluBackward.
extern "C" int DLGpuBatchNormalizationReluForward(const DLArrayHandle input, DLArrayHandle output,
                                                  int batchNormMode, int n, void **mean_p, void **Variance_p,
                                                  void ***list, void **handle, int *memorytoSaving,
                                                  void **stream) {
  announce_write(output);
  return bn_forward_impl(input, output, batchNormMode, n, mean_p, Variance_p, list, handle, memorytoSaving, stream,
                         true, "DLGpuBatchNormalizationReluForward");
}

static int bn_backward_impl(const DLArrayHandle input, const DLArrayHandle doutput, DLArrayHandle dinput,
                            int batchNormMode, void **mean_p, void **Variance_p, void ***list, void **handle,
                            int *memorytoSaving, void **stream, bool relu, const char *what) {
  (void)handle;
  BNDesc *d = desc_from_list<BNDesc>(list, kMagicBN);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuBatchNormalizationGetCudnnlist");
  TF_REQUIRE(d->mode == batchNormMode, "mode differs from the descriptor");
  // the cells start out pointing at host integers, so "non-null" proves nothing:
  // they must hold exactly what the last forward published
  TF_REQUIRE(mean_p && Variance_p && d->saved_mean && *mean_p == d->saved_mean &&
                 *Variance_p == d->saved_istd,
             "no saved statistics: backward needs the forward pass of the same step");
  TF_REQUIRE(!relu || d->mode == 0, "the fused batch-norm + ReLU entry points implement per-activation mode only");
  if (check_bn_arrays(d, input, doutput) != 0) return -1;
  TF_REQUIRE(on_gpu(dinput) && numel(dinput) == numel(input), "dinput must have the input's shape");
  hipStream_t s = stream_of(stream);
  const float *x = (const float *)input->data, *dy = (const float *)doutput->data;
  float *dx = (float *)dinput->data;
  const float *mean = (const float *)*mean_p, *istd = (const float *)*Variance_p;
  if (numel(input) != 0) {
    if (d->mode == 0) {
      const int64_t L = d->stat_count;
      const dim3 grid(cdiv(L, kThreads)), block(kThreads);
      auto run = [&](auto relu_c) {
        constexpr bool RELU = decltype(relu_c)::value;
        const uint32_t l32 = (uint32_t)L;
        if (d->N <= 32 && pa_rows_addressable(32, L))
          hipLaunchKernelGGL((bn_pa_backward_kernel<32, RELU>), grid, block, 0, s, x, dy, dx, mean, istd, d->N, l32);
        else if (d->N <= 64 && pa_rows_addressable(64, L))
          hipLaunchKernelGGL((bn_pa_backward_kernel<64, RELU>), grid, block, 0, s, x, dy, dx, mean, istd, d->N, l32);
        else if (d->N <= 128 && pa_rows_addressable(128, L))
          hipLaunchKernelGGL((bn_pa_backward_kernel<128, RELU>), grid, block, 0, s, x, dy, dx, mean, istd, d->N, l32);
        else
          hipLaunchKernelGGL(bn_pa_backward_stream_kernel<RELU>, grid, block, 0, s, x, dy, dx, mean, istd, d->N, L);
      };
      if (relu) run(std::true_type{}); else run(std::false_type{});
    } else {
      const int chunks = sp_chunks(d->N, d->C);
      const int ipc = cdiv(d->N, chunks);
      const int real_chunks = cdiv(d->N, ipc);
      const size_t pbytes = (size_t)real_chunks * d->C * 2 * sizeof(double) + (size_t)d->C * 2 * sizeof(float);
      double *partial = (double *)device_alloc(pbytes);
      if (!partial) {
        if (memorytoSaving) *memorytoSaving = shortfall(pbytes);
        return 0;  // statistics stay published so the call can be repeated
      }
      // the two per-channel sums of the apply pass live behind the chunk partials
      float *sums = reinterpret_cast<float *>(partial + (size_t)real_chunks * d->C * 2);
      const bool vec = d->HW % 4 == 0 &&
                       ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy) |
                         reinterpret_cast<uintptr_t>(dx)) & 15u) == 0;
      const int W = vec ? 4 : 1;
      const FastDiv div_row((uint32_t)(d->HW / W)), div_c((uint32_t)d->C);
      const uint32_t units = (uint32_t)((int64_t)d->N * d->C * d->HW / W);
      const dim3 pgrid(d->C, real_chunks), agrid((units + kThreads * 4 - 1) / (kThreads * 4));
      const float m = (float)((double)d->N * (double)d->HW);
      auto run = [&](auto vec_c) {
        constexpr bool VEC = decltype(vec_c)::value;
        hipLaunchKernelGGL((bn_sp_partial_kernel<true, VEC>), pgrid, dim3(kThreads), 0, s, x, dy, mean, istd, partial,
                           d->N, d->C, d->HW, ipc, div_row);
        hipLaunchKernelGGL(bn_sp_finish_kernel<true>, dim3(cdiv(d->C, kThreads)), dim3(kThreads), 0, s, partial, x,
                           sums, sums + d->C, d->N, d->C, d->HW, real_chunks);
        hipLaunchKernelGGL((bn_sp_apply_kernel<true, VEC>), agrid, dim3(kThreads), 0, s, x, dy, dx, mean, istd,
                           (const float *)sums, (const float *)(sums + d->C), m, div_row, div_c, units);
      };
      if (vec) run(std::true_type{}); else run(std::false_type{});
      device_free(partial);
    }
  }
  // the saved statistics are consumed (stream-ordered release)
  device_free(d->saved_mean);
  device_free(d->saved_istd);
  *mean_p = d->saved_mean = nullptr;
  *Variance_p = d->saved_istd = nullptr;
  return finish(s, what);
}

extern "C" int DLGpuBatchNormalizationBackward(const DLArrayHandle input, const DLArrayHandle doutput,
                                               DLArrayHandle dinput, int batchNormMode, void **mean_p,
                                               void **Variance_p, void ***list, void **handle,
                                               int *memorytoSaving, void **stream) {
  announce_write(dinput);
  return bn_backward_impl(input, doutput, dinput, batchNormMode, mean_p, Variance_p, list, handle, memorytoSaving,
                          stream, false, "DLGpuBatchNormalizationBackward");
}

// No counterpart in the reference: gradient of max(bn(x), 0) with respect to x.
// doutput is the gradient of the ReLU output; the ReLU mask bn(x) > 0 is rebuilt
// from x and the saved statistics, so neither bn(x) nor the ReLU output is read
// (12 bytes per element instead of 24 for the two ops).
extern "C" int DLGpuBatchNormalizationReluBackward(const DLArrayHandle input, const DLArrayHandle doutput,
                                                   DLArrayHandle dinput, int batchNormMode, void **mean_p,
                                                   void **Variance_p, void ***list, void **handle,
                                                   int *memorytoSaving, void **stream) {
  announce_write(dinput);
  return bn_backward_impl(input, doutput, dinput, batchNormMode, mean_p, Variance_p, list, handle, memorytoSaving,
                          stream, true, "DLGpuBatchNormalizationReluBackward");
}
