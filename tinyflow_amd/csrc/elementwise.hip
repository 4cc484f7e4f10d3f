// Bandwidth-bound elementwise kernels: array set, add / multiply (tensor and
// constant), ReLU and its gradient, broadcasts, cross-entropy terms, SGD and Adam.
//
// All of them stream their operands once: each lane moves 16-byte vectors,
// four independent vectors are in flight per lane and the grid is sized to the
// CU count with a grid-stride loop, so a launch is bounded by HBM bandwidth
// (8 or 12 bytes per element) rather than by the number of workgroups.
//
// Reference kernels replaced: src/gpu_op.cu:39-52 (set, broadcast),
// :108-123 (channel broadcast), :193-235 (add/mul/relu), :4461-4533 (Adam),
// :4538-4597 (cross), :4600-4625 (SGD); one thread per element, 1024-thread
// blocks capped at 4096 blocks there.
#include "ew_core.h"
#include "gemm_core.h"
#include "internal.h"

#include <algorithm>
#include <mutex>
#include <unordered_map>
#include <vector>

using namespace tf;
using tf::gemm::FastDiv;

using namespace tf::ew;

namespace {

struct OpSet { float v; __device__ float operator()(float, float) const { return v; } };
struct OpAdd { __device__ float operator()(float a, float b) const { return a + b; } };
// max(a + b, 0): the sum keeps a negative zero, like the separate ReLU kernel does
struct OpAddRelu { __device__ float operator()(float a, float b) const { const float t = a + b; return t < 0.f ? 0.f : t; } };
struct OpMul { __device__ float operator()(float a, float b) const { return a * b; } };
struct OpAddC { float v; __device__ float operator()(float a, float) const { return a + v; } };
struct OpMulC { float v; __device__ float operator()(float a, float) const { return a * v; } };
struct OpRelu { __device__ float operator()(float a, float) const { return a < 0.f ? 0.f : a; } };
// gradient mask is x > 0 (reference kernel gpu_op.cu:230-235 and its test
// tests/test_gpu_op.py:145-155); a = x, b = upstream gradient
struct OpReluGrad { __device__ float operator()(float a, float b) const { return a > 0.f ? b : 0.f; } };
// a = parameter, b = gradient
struct OpSgd { float lr; __device__ float operator()(float a, float b) const { return a - lr * b; } };
// a = x (probabilities), b = y (labels)
struct OpCross { float s; __device__ float operator()(float a, float b) const { return logf(a) * b * (-1.f) * s; } };

// out[i] = in[i % in_count].  Indices are 32-bit and divided by magic numbers: a
// 64-bit integer division per element would cost more than the memory traffic.
__global__ __launch_bounds__(kThreads) void broadcast_tail_kernel(const float *__restrict__ in, FastDiv in_count,
                                                                 float *__restrict__ out, uint32_t n) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    uint32_t q, r;
    in_count.divmod(i, q, r);
    out[i] = in[r];
  }
}

// out[n, c, inner] = in[c]; one float4 per lane when inner % 4 == 0
template <bool VEC>
__global__ __launch_bounds__(kThreads) void broadcast_channel_kernel(const float *__restrict__ in, FastDiv channels,
                                                                    FastDiv units_per_row,
                                                                    float *__restrict__ out, uint32_t n_units) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < n_units; i += stride) {
    uint32_t row, img, c;
    row = units_per_row.div(i);
    channels.divmod(row, img, c);
    const float v = in[c];
    if (VEC) reinterpret_cast<float4 *>(out)[i] = make_float4(v, v, v, v);
    else out[i] = v;
  }
}

// out[i] = -s * y[i] / x[i] * dout[i]
__global__ __launch_bounds__(kThreads) void cross_backward_kernel(const float *__restrict__ x,
                                                                 const float *__restrict__ y,
                                                                 const float *__restrict__ dout,
                                                                 float *__restrict__ out, float s, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    out[i] = y[i] * (-1.f) * s * (1.0f / x[i]) * dout[i];
}

// m = b1*m + (1-b1)*g ; v = b2*v + (1-b2)*g*g
__global__ __launch_bounds__(kThreads) void adam_mv_kernel(float *m, float *v, const float *__restrict__ g,
                                                          float b1, float b2, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    const float gi = g[i];
    m[i] = m[i] * b1 + gi * (1.f - b1);
    v[i] = v[i] * b2 + gi * gi * (1.f - b2);
  }
}

// w -= lr * (m / (1-b1t)) / (sqrt(v / (1-b2t)) + e)
__global__ __launch_bounds__(kThreads) void adam_kernel(float *w, const float *__restrict__ m,
                                                       const float *__restrict__ v, float b1t, float b2t,
                                                       float e, float lr, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    w[i] = w[i] - lr * m[i] / (1.f - b1t) / (sqrtf(v[i] / (1.f - b2t)) + e);
}

// Fused multi-tensor SGD over a flat index space:
// w[number[i]][offset[i]] -= lr * g[number[i]][offset[i]]
__global__ __launch_bounds__(kThreads) void sgd_multi_kernel(float **w, float **g,
                                                            const int *__restrict__ number,
                                                            const int *__restrict__ offset, float lr,
                                                            int count) {
  const int stride = gridDim.x * kThreads;
  for (int i = blockIdx.x * kThreads + threadIdx.x; i < count; i += stride) {
    const int t = number[i], o = offset[i];
    w[t][o] = w[t][o] - lr * g[t][o];
  }
}

// Fused multi-tensor Adam over the same flat index space, one lane per parameter
// and one pass over w, m, v, g (28 bytes per parameter):
//   m = b1*m + (1-b1)*g;  v = b2*v + (1-b2)*g*g
//   w -= (lr * m / (1-b1t)) / (sqrt(v / (1-b2t)) + e)
__global__ __launch_bounds__(kThreads) void adam_multi_kernel(float **w, float **m, float **v, float **g,
                                                             const int *__restrict__ number,
                                                             const int *__restrict__ offset, float b1, float b2,
                                                             float b1t, float b2t, float e, float lr, int count) {
  const int stride = gridDim.x * kThreads;
  for (int i = blockIdx.x * kThreads + threadIdx.x; i < count; i += stride) {
    const int t = number[i], o = offset[i];
    const float gi = g[t][o];
    const float mm = m[t][o] * b1 + gi * (1.f - b1);
    const float vv = v[t][o] * b2 + gi * gi * (1.f - b2);
    m[t][o] = mm;
    v[t][o] = vv;
    w[t][o] = w[t][o] - (lr * mm / (1.f - b1t)) / (sqrtf(vv / (1.f - b2t)) + e);
  }
}

// ---- fused multi-tensor updates, run form -----------------------------------------
// The per-parameter (tensor number, offset) tables of the fused optimizers describe,
// in every real use, whole tensors laid end to end: runs of consecutive offsets
// inside one tensor.  DLGpuGetIndextoVaribaleNumberCudaPointer detects that on the
// host arrays and records the runs cut into pieces of kRunPiece elements; a launch
// whose tables were built that way gives one workgroup one piece and streams it like
// the single-tensor engine (16-byte vectors, 12 bytes per parameter for SGD) instead
// of reading two 4-byte indices per parameter.  Same arithmetic per element, so the
// result has the bits of the indexed form.
constexpr int kRunPiece = kVecPerBlock * 4;  // 4096 elements = 16 KiB per operand
struct RunPiece {
  int tensor;   // index into the pointer tables
  int offset;   // first element of the piece inside the tensor
  int length;   // elements, <= kRunPiece
};
struct RunTable {
  RunPiece *pieces = nullptr;  // device
  int n_pieces = 0;
  int count = 0;               // parameters covered (must equal the launch's count)
  bool tables_are_dummies = false;  // the per-element tables behind this key were never uploaded
};
std::mutex run_mu;
std::unordered_map<const void *, RunTable> run_tables;  // keyed by the device `number` table

template <int NPTR, class F>
__global__ __launch_bounds__(kThreads) void multi_tensor_kernel(F f, float *const *p0, float *const *p1,
                                                               float *const *p2, float *const *p3,
                                                               const RunPiece *__restrict__ pieces) {
  const RunPiece piece = pieces[blockIdx.x];
  float *t0 = p0[piece.tensor] + piece.offset;
  float *t1 = p1[piece.tensor] + piece.offset;
  float *t2 = NPTR > 2 ? p2[piece.tensor] + piece.offset : nullptr;
  float *t3 = NPTR > 2 ? p3[piece.tensor] + piece.offset : nullptr;
  bool vec = ((reinterpret_cast<uintptr_t>(t0) | reinterpret_cast<uintptr_t>(t1)) & 15u) == 0;
  if (NPTR > 2) vec = vec && ((reinterpret_cast<uintptr_t>(t2) | reinterpret_cast<uintptr_t>(t3)) & 15u) == 0;
  const int n4 = vec ? piece.length / 4 : 0;
  for (int i = threadIdx.x; i < n4; i += kThreads) f.template apply<f32x4>(t0, t1, t2, t3, i);
  for (int i = n4 * 4 + threadIdx.x; i < piece.length; i += kThreads) f.template apply<float>(t0, t1, t2, t3, i);
}

struct MultiSgd {
  float lr;
  template <class V>
  __device__ inline void apply(float *w, float *g, float *, float *, int i) const {
    V *w4 = reinterpret_cast<V *>(w);
    const V gv = __builtin_nontemporal_load(reinterpret_cast<const V *>(g) + i);
    w4[i] = w4[i] - lr * gv;
  }
};
struct MultiAdam {
  float b1, b2, b1t, b2t, e, lr;
  template <class V>
  __device__ inline void apply(float *w, float *m, float *v, float *g, int i) const {
    V *w4 = reinterpret_cast<V *>(w), *m4 = reinterpret_cast<V *>(m), *v4 = reinterpret_cast<V *>(v);
    const V gi = __builtin_nontemporal_load(reinterpret_cast<const V *>(g) + i);
    const V mm = m4[i] * b1 + gi * (1.f - b1);
    const V vv = v4[i] * b2 + gi * gi * (1.f - b2);
    m4[i] = mm;
    v4[i] = vv;
    V root = vv / (1.f - b2t);
    if constexpr (sizeof(V) == sizeof(float)) {
      root = sqrtf(root);
    } else {
      root.x = sqrtf(root.x); root.y = sqrtf(root.y); root.z = sqrtf(root.z); root.w = sqrtf(root.w);
    }
    w4[i] = w4[i] - (lr * mm / (1.f - b1t)) / (root + e);
  }
};

// Run table of the launch whose tables start at `number_table`, if its host arrays were
// runs: 1 found, 0 none (use the indexed kernel), -1 the tables exist only as runs and
// the launch's count is not the one they were built for.
int find_run_table(const void *number_table, int count, RunTable &out) {
  std::lock_guard<std::mutex> g(run_mu);
  auto it = run_tables.find(number_table);
  if (it == run_tables.end()) return 0;
  if (it->second.count != count || it->second.n_pieces == 0) return it->second.tables_are_dummies ? -1 : 0;
  out = it->second;
  return 1;
}

}  // namespace

extern "C" int DLGpuArraySet(DLArrayHandle arr, float value, void **stream) {
  announce_write(arr);
  TF_REQUIRE(on_gpu(arr), "array must live on the GPU");
  hipStream_t s = stream_of(stream);
  return launch_ew<OpSet, false, false>(OpSet{value}, (float *)arr->data, nullptr, nullptr, numel(arr), s,
                                        "DLGpuArraySet");
}

extern "C" int DLGpuMatrixElementwiseAdd(const DLArrayHandle a, const DLArrayHandle b, DLArrayHandle out,
                                         void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(a) && on_gpu(b) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(same_shape(a, out) && same_shape(b, out), "shape mismatch");
  return launch_ew<OpAdd, true, true>(OpAdd{}, (float *)out->data, (const float *)a->data,
                                      (const float *)b->data, numel(out), stream_of(stream),
                                      "DLGpuMatrixElementwiseAdd");
}

// No counterpart in the reference: max(a + b, 0), the join of a residual block and
// the ReLU that follows it, in one pass (12 bytes per element instead of 20).
extern "C" int DLGpuMatrixElementwiseAddRelu(const DLArrayHandle a, const DLArrayHandle b, DLArrayHandle out,
                                             void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(a) && on_gpu(b) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(same_shape(a, out) && same_shape(b, out), "shape mismatch");
  return launch_ew<OpAddRelu, true, true>(OpAddRelu{}, (float *)out->data, (const float *)a->data,
                                          (const float *)b->data, numel(out), stream_of(stream),
                                          "DLGpuMatrixElementwiseAddRelu");
}

extern "C" int DLGpuMatrixElementwiseAddByConst(const DLArrayHandle in, float val, DLArrayHandle out,
                                                void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(same_shape(in, out), "shape mismatch");
  return launch_ew<OpAddC, true, false>(OpAddC{val}, (float *)out->data, (const float *)in->data, nullptr,
                                        numel(out), stream_of(stream), "DLGpuMatrixElementwiseAddByConst");
}

extern "C" int DLGpuMatrixElementwiseMultiply(const DLArrayHandle a, const DLArrayHandle b, DLArrayHandle out,
                                              void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(a) && on_gpu(b) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(same_shape(a, out) && same_shape(b, out), "shape mismatch");
  return launch_ew<OpMul, true, true>(OpMul{}, (float *)out->data, (const float *)a->data,
                                      (const float *)b->data, numel(out), stream_of(stream),
                                      "DLGpuMatrixElementwiseMultiply");
}

extern "C" int DLGpuMatrixMultiplyByConst(const DLArrayHandle in, float val, DLArrayHandle out,
                                          void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(same_shape(in, out), "shape mismatch");
  return launch_ew<OpMulC, true, false>(OpMulC{val}, (float *)out->data, (const float *)in->data, nullptr,
                                        numel(out), stream_of(stream), "DLGpuMatrixMultiplyByConst");
}

// The two stream-less entry points run on the legacy default stream, which is
// ordered after all work already enqueued on the blocking streams created by
// DLGpuCreatecudaStream and before any work enqueued on them later.
extern "C" int DLGpuRelu(const DLArrayHandle in, DLArrayHandle out) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(same_shape(in, out), "shape mismatch");
  return launch_ew<OpRelu, true, false>(OpRelu{}, (float *)out->data, (const float *)in->data, nullptr,
                                        numel(out), streamless_launch_stream(), "DLGpuRelu");
}

extern "C" int DLGpuReluGradient(const DLArrayHandle in, const DLArrayHandle grad, DLArrayHandle out) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(grad) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(same_shape(in, out) && same_shape(grad, out), "shape mismatch");
  return launch_ew<OpReluGrad, true, true>(OpReluGrad{}, (float *)out->data, (const float *)in->data,
                                           (const float *)grad->data, numel(out), streamless_launch_stream(),
                                           "DLGpuReluGradient");
}

extern "C" int DLGpuSgdUpdate(DLArrayHandle w, const DLArrayHandle g, float lr, void **stream) {
  announce_write(w);
  TF_REQUIRE(on_gpu(w) && on_gpu(g), "arrays must live on the GPU");
  TF_REQUIRE(numel(w) == numel(g), "parameter and gradient differ in size");
  return launch_ew<OpSgd, true, true>(OpSgd{lr}, (float *)w->data, (const float *)w->data,
                                      (const float *)g->data, numel(w), stream_of(stream), "DLGpuSgdUpdate");
}

extern "C" int DLGpuCross(const DLArrayHandle x, const DLArrayHandle y, DLArrayHandle out, float b,
                          void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(x) && on_gpu(y) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(numel(x) == numel(out) && numel(y) == numel(out), "shape mismatch");
  return launch_ew<OpCross, true, true>(OpCross{b}, (float *)out->data, (const float *)x->data,
                                        (const float *)y->data, numel(out), stream_of(stream), "DLGpuCross");
}

extern "C" int DLGpuCrossBackward(const DLArrayHandle x, const DLArrayHandle y, const DLArrayHandle dout,
                                  DLArrayHandle out, float b, void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(x) && on_gpu(y) && on_gpu(dout) && on_gpu(out), "arrays must live on the GPU");
  const int64_t n = numel(out);
  TF_REQUIRE(numel(x) == n && numel(y) == n && numel(dout) == n, "shape mismatch");
  hipStream_t s = stream_of(stream);
  if (n == 0) return 0;
  hipLaunchKernelGGL(cross_backward_kernel, dim3(grid_for(n)), dim3(kThreads), 0, s, (const float *)x->data,
                     (const float *)y->data, (const float *)dout->data, (float *)out->data, b, n);
  return finish(s, "DLGpuCrossBackward");
}

extern "C" int DLGpuBroadcastTo0(const DLArrayHandle in, DLArrayHandle out, void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  const int64_t in_count = numel(in), n = numel(out);
  TF_REQUIRE(in_count > 0 && in_count <= INT32_MAX, "bad input size");
  if (!(in->ndim == 1 && in->shape[0] == 1)) {
    TF_REQUIRE(in->ndim <= out->ndim, "input has more dims than output");
    for (int i = 0; i < in->ndim; ++i)
      TF_REQUIRE(in->shape[in->ndim - 1 - i] == out->shape[out->ndim - 1 - i],
                 "input must match the trailing dims of the output");
  }
  hipStream_t s = stream_of(stream);
  if (n == 0) return 0;
  TF_REQUIRE(n < ((int64_t)1 << 31), "tensors of 2^31 elements or more are not supported");
  hipLaunchKernelGGL(broadcast_tail_kernel, dim3(grid_for(n)), dim3(kThreads), 0, s, (const float *)in->data,
                     FastDiv((uint32_t)in_count), (float *)out->data, (uint32_t)n);
  return finish(s, "DLGpuBroadcastTo0");
}

extern "C" int DLGpuBroadcastTo1(const DLArrayHandle in, DLArrayHandle out, void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(in->ndim == 1 && out->ndim >= 2 && in->shape[0] == out->shape[1],
             "input must be (C,) and output (N, C, ...)");
  int64_t inner = 1;
  for (int i = 2; i < out->ndim; ++i) inner *= out->shape[i];
  const int64_t n = numel(out);
  TF_REQUIRE(inner <= INT32_MAX, "inner extent too large");
  hipStream_t s = stream_of(stream);
  if (n == 0) return 0;
  TF_REQUIRE(n < ((int64_t)1 << 31), "tensors of 2^31 elements or more are not supported");
  const FastDiv channels((uint32_t)out->shape[1]);
  if (inner % 4 == 0 && aligned16(out->data)) {
    const int64_t units = n / 4;
    hipLaunchKernelGGL(broadcast_channel_kernel<true>, dim3(grid_for(units)), dim3(kThreads), 0, s,
                       (const float *)in->data, channels, FastDiv((uint32_t)(inner / 4)), (float *)out->data,
                       (uint32_t)units);
  } else {
    hipLaunchKernelGGL(broadcast_channel_kernel<false>, dim3(grid_for(n)), dim3(kThreads), 0, s,
                       (const float *)in->data, channels, FastDiv((uint32_t)inner), (float *)out->data,
                       (uint32_t)n);
  }
  return finish(s, "DLGpuBroadcastTo1");
}

extern "C" int DLGpuAdam_mv(DLArrayHandle m, DLArrayHandle v, const DLArrayHandle g, float b1, float b2,
                            void **stream) {
  announce_write(m);
  announce_write(v);
  TF_REQUIRE(on_gpu(m) && on_gpu(v) && on_gpu(g), "arrays must live on the GPU");
  const int64_t n = numel(g);
  TF_REQUIRE(numel(m) == n && numel(v) == n, "shape mismatch");
  hipStream_t s = stream_of(stream);
  if (n == 0) return 0;
  hipLaunchKernelGGL(adam_mv_kernel, dim3(grid_for(n)), dim3(kThreads), 0, s, (float *)m->data,
                     (float *)v->data, (const float *)g->data, b1, b2, n);
  return finish(s, "DLGpuAdam_mv");
}

extern "C" int DLGpuAdam(DLArrayHandle w, const DLArrayHandle m, const DLArrayHandle v, float b1t, float b2t,
                         float e, float lr, void **stream) {
  announce_write(w);
  TF_REQUIRE(on_gpu(w) && on_gpu(m) && on_gpu(v), "arrays must live on the GPU");
  const int64_t n = numel(w);
  TF_REQUIRE(numel(m) == n && numel(v) == n, "shape mismatch");
  hipStream_t s = stream_of(stream);
  if (n == 0) return 0;
  hipLaunchKernelGGL(adam_kernel, dim3(grid_for(n)), dim3(kThreads), 0, s, (float *)w->data,
                     (const float *)m->data, (const float *)v->data, b1t, b2t, e, lr, n);
  return finish(s, "DLGpuAdam");
}

// ---- fused multi-tensor SGD --------------------------------------------------
// Tables of the fused optimizers.  The reference allocates them with cudaMalloc and
// never gives them back (src/gpu_op.cu:4628-4700); here they come from the pool (so
// the allocator's statistics and budget see them) and DLGpuFreeIndexCudaPointer /
// DLGpuFreeNCudaPointer release them.

namespace {

// Records `pieces` under the key `d_number`; false when the device has no room.
bool publish_runs(const std::vector<RunPiece> &pieces, int count, const void *d_number, bool tables_are_dummies) {
  RunTable t;
  t.n_pieces = (int)pieces.size();
  t.count = count;
  t.tables_are_dummies = tables_are_dummies;
  t.pieces = (RunPiece *)device_alloc(pieces.size() * sizeof(RunPiece));
  if (!t.pieces) return false;
  if (hipMemcpy(t.pieces, pieces.data(), pieces.size() * sizeof(RunPiece), hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipGetLastError();
    device_free(t.pieces);
    return false;
  }
  std::lock_guard<std::mutex> g(run_mu);
  run_tables[d_number] = t;
  return true;
}

void append_run(std::vector<RunPiece> &pieces, int tensor, int first_offset, int64_t length) {
  for (int64_t start = 0; start < length; start += kRunPiece)
    pieces.push_back(RunPiece{tensor, first_offset + (int)start, (int)std::min<int64_t>(kRunPiece, length - start)});
}

// The two-pointer result cell of the index tables around device blocks a and b.
int index_cell(void ***result, void *a, void *b) {
  *result = (void **)malloc(sizeof(void *) * 2);
  TF_REQUIRE(*result, "host allocation failed");
  (*result)[0] = a;
  (*result)[1] = b;
  return 0;
}

}  // namespace

extern "C" int DLGpuGetIndextoVaribaleNumberCudaPointer(int *index_to_number, int *prefix, int count,
                                                        void ***result) {
  TF_REQUIRE(index_to_number && prefix && result && count >= 0, "bad arguments");
  // the tables as runs of consecutive offsets inside one tensor, cut into pieces
  std::vector<RunPiece> pieces;
  for (int i = 0; i < count;) {
    int j = i + 1;
    while (j < count && index_to_number[j] == index_to_number[i] && prefix[j] == prefix[i] + (j - i)) ++j;
    append_run(pieces, index_to_number[i], prefix[i], j - i);
    i = j;
  }
  // worth it only when the pieces are long on average (scattered indices stay with the indexed kernel)
  const bool as_runs = !pieces.empty() && (int64_t)pieces.size() * 256 <= (int64_t)count + 256 * 1024;
  // A launch that finds its run table never reads the per-element tables, so they are
  // uploaded only for the indexed kernel; the run form keeps two one-word blocks whose
  // addresses identify the tables.
  const size_t bytes = as_runs ? sizeof(int) : sizeof(int) * (size_t)(count > 0 ? count : 1);
  int *d_number = (int *)device_alloc(bytes), *d_prefix = (int *)device_alloc(bytes);
  if (!d_number || !d_prefix) {
    if (d_number) device_free(d_number);
    if (d_prefix) device_free(d_prefix);
    TF_REQUIRE(false, "no device memory for %zu bytes of index tables", 2 * bytes);
  }
  bool published = as_runs && publish_runs(pieces, count, d_number, true);
  if (as_runs && !published) {
    device_free(d_number);
    device_free(d_prefix);
    TF_REQUIRE(false, "no device memory for the run table");
  }
  if (!as_runs && count > 0) {
    TF_HIP(hipMemcpy(d_number, index_to_number, sizeof(int) * (size_t)count, hipMemcpyHostToDevice));
    TF_HIP(hipMemcpy(d_prefix, prefix, sizeof(int) * (size_t)count, hipMemcpyHostToDevice));
  }
  return index_cell(result, d_number, d_prefix);
}

// No counterpart in the reference: the same index tables for whole tensors laid end to
// end, built from the tensors' element counts, so that neither the caller nor the
// library materialises a per-parameter array.  The result is used and released like
// DLGpuGetIndextoVaribaleNumberCudaPointer's; `*count` receives the parameter total
// to pass to DLGpuSgd_o / DLGpuAdam_o.
extern "C" int DLGpuGetTensorRunsCudaPointer(const int64_t *sizes, int n_tensors, int *count, void ***result) {
  TF_REQUIRE(sizes && result && count && n_tensors >= 0, "bad arguments");
  int64_t total = 0;
  std::vector<RunPiece> pieces;
  for (int t = 0; t < n_tensors; ++t) {
    TF_REQUIRE(sizes[t] >= 0 && sizes[t] <= INT32_MAX, "tensor %d has a bad size", t);
    append_run(pieces, t, 0, sizes[t]);
    total += sizes[t];
  }
  TF_REQUIRE(total <= INT32_MAX, "2^31 parameters or more in one fused update");
  int *d_number = (int *)device_alloc(sizeof(int)), *d_prefix = (int *)device_alloc(sizeof(int));
  if (!d_number || !d_prefix || (!pieces.empty() && !publish_runs(pieces, (int)total, d_number, true))) {
    if (d_number) device_free(d_number);
    if (d_prefix) device_free(d_prefix);
    TF_REQUIRE(false, "no device memory for the run table");
  }
  *count = (int)total;
  return index_cell(result, d_number, d_prefix);
}

// No counterpart in the reference (which never releases these tables): gives back the
// device blocks and the host cell of DLGpuGetIndextoVaribaleNumberCudaPointer /
// DLGpuGetTensorRunsCudaPointer.  The caller must not use `indexlist` afterwards.
extern "C" int DLGpuFreeIndexCudaPointer(void ***indexlist) {
  TF_REQUIRE(indexlist, "bad arguments");
  if (!*indexlist) return 0;
  TF_HIP(hipStreamSynchronize(streamless_launch_stream()));  // the last fused update may still read them
  RunPiece *pieces = nullptr;
  {
    std::lock_guard<std::mutex> g(run_mu);
    auto it = run_tables.find((*indexlist)[0]);
    if (it != run_tables.end()) {
      pieces = it->second.pieces;
      run_tables.erase(it);
    }
  }
  if (pieces) device_free(pieces);
  for (int i = 0; i < 2; ++i)
    if ((*indexlist)[i]) device_free((*indexlist)[i]);
  free(*indexlist);
  *indexlist = nullptr;
  return 0;
}

namespace {
int pointer_tables(void **const *host, int n_tables, int number, void ****result) {
  float **dev[4] = {nullptr, nullptr, nullptr, nullptr};
  const size_t bytes = sizeof(float *) * (size_t)(number > 0 ? number : 1);
  bool ok = true;
  for (int i = 0; i < n_tables && ok; ++i) {
    dev[i] = (float **)device_alloc(bytes);
    ok = dev[i] && (number == 0 || hipMemcpy(dev[i], host[i], sizeof(float *) * (size_t)number,
                                             hipMemcpyHostToDevice) == hipSuccess);
  }
  void ***cell = ok ? (void ***)malloc(sizeof(void **) * n_tables) : nullptr;
  if (!cell) {
    (void)hipGetLastError();
    for (int i = 0; i < n_tables; ++i)
      if (dev[i]) device_free(dev[i]);
    TF_REQUIRE(false, "no memory for %d pointer tables of %d entries", n_tables, number);
  }
  for (int i = 0; i < n_tables; ++i) cell[i] = (void **)dev[i];
  *result = cell;
  return 0;
}
}  // namespace

extern "C" int DLGpuGetN2CudaPointer(void **output, void **g, int number, void ****result) {
  TF_REQUIRE(output && g && result && number >= 0, "bad arguments");
  void **host[2] = {output, g};
  return pointer_tables(host, 2, number, result);
}

extern "C" int DLGpuGetN4CudaPointer(void **output, void **m, void **v, void **g, int number, void ****result) {
  TF_REQUIRE(output && m && v && g && result && number >= 0, "bad arguments");
  void **host[4] = {output, m, v, g};
  return pointer_tables(host, 4, number, result);
}

// No counterpart in the reference: releases the `n_tables` (2 or 4) device pointer
// tables and the host cell of DLGpuGetN2CudaPointer / DLGpuGetN4CudaPointer.
extern "C" int DLGpuFreeNCudaPointer(void ****list, int n_tables) {
  TF_REQUIRE(list && (n_tables == 2 || n_tables == 4), "bad arguments");
  if (!*list) return 0;
  TF_HIP(hipStreamSynchronize(streamless_launch_stream()));  // the last fused update may still read them
  for (int i = 0; i < n_tables; ++i)
    if ((*list)[i]) device_free((*list)[i]);
  free(*list);
  *list = nullptr;
  return 0;
}

extern "C" int DLGpuAdam_o(void ****n4list, const void ***indexlist, const int count, const float b1,
                           const float b2, const float b1t, const float b2t, const float e,
                           const float learning_rate) {
  note_write_everything();  // the pointer tables name the written tensors, not their sizes
  TF_REQUIRE(n4list && *n4list && indexlist && *indexlist && count >= 0, "bad arguments");
  if (count == 0) return 0;
  // no stream argument: ordered against all streams that run kernels
  hipStream_t s = streamless_launch_stream();
  RunTable runs;
  const int found = find_run_table((*indexlist)[0], count, runs);
  TF_REQUIRE(found >= 0, "count %d is not the count the index tables were built for", count);
  if (found) {
    hipLaunchKernelGGL((multi_tensor_kernel<4, MultiAdam>), dim3(runs.n_pieces), dim3(kThreads), 0, s,
                       MultiAdam{b1, b2, b1t, b2t, e, learning_rate}, (float *const *)((*n4list)[0]),
                       (float *const *)((*n4list)[1]), (float *const *)((*n4list)[2]),
                       (float *const *)((*n4list)[3]), (const RunPiece *)runs.pieces);
    return finish(s, "DLGpuAdam_o");
  }
  hipLaunchKernelGGL(adam_multi_kernel, dim3(grid_for(count)), dim3(kThreads), 0, s,
                     (float **)((*n4list)[0]), (float **)((*n4list)[1]), (float **)((*n4list)[2]),
                     (float **)((*n4list)[3]), (const int *)((*indexlist)[0]), (const int *)((*indexlist)[1]), b1,
                     b2, b1t, b2t, e, learning_rate, count);
  return finish(s, "DLGpuAdam_o");
}

extern "C" int DLGpuSgd_o(void ****n2list, const void ***indexlist, const int count,
                          const float learning_rate) {
  note_write_everything();  // the pointer tables name the written tensors, not their sizes
  TF_REQUIRE(n2list && *n2list && indexlist && *indexlist && count >= 0, "bad arguments");
  if (count == 0) return 0;
  // no stream argument: ordered against all streams that run kernels
  hipStream_t s = streamless_launch_stream();
  RunTable runs;
  const int found = find_run_table((*indexlist)[0], count, runs);
  TF_REQUIRE(found >= 0, "count %d is not the count the index tables were built for", count);
  if (found) {
    hipLaunchKernelGGL((multi_tensor_kernel<2, MultiSgd>), dim3(runs.n_pieces), dim3(kThreads), 0, s,
                       MultiSgd{learning_rate}, (float *const *)((*n2list)[0]), (float *const *)((*n2list)[1]),
                       (float *const *)nullptr, (float *const *)nullptr, (const RunPiece *)runs.pieces);
    return finish(s, "DLGpuSgd_o");
  }
  hipLaunchKernelGGL(sgd_multi_kernel, dim3(grid_for(count)), dim3(kThreads), 0, s,
                     (float **)((*n2list)[0]), (float **)((*n2list)[1]), (const int *)((*indexlist)[0]),
                     (const int *)((*indexlist)[1]), learning_rate, count);
  return finish(s, "DLGpuSgd_o");
}
