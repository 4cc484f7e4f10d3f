// Activation forward/backward: ReLU (the mode every conv net of the reference
// uses), sigmoid, tanh, and softmax over c*h*w per instance.
//
// Replaces cudnnActivationForward/Backward and cudnnSoftmaxForward/Backward as
// called at src/gpu_op.cu:3211-3274 and 3475-3544, and the descriptor builder at
// :3364-3471.  The ReLU gradient reads x and dy and writes dx (12 bytes per
// element); the forward output y, which cuDNN also takes, is not needed.
//
// Once a descriptor has seen a backward call, its ReLU forward calls also write one
// bit per element (x > 0) into a kept block, and the backward call of the same step
// reads dy and those bits instead of dy and x: 8.125 bytes per element instead of 12,
// with the same result bit for bit.  The block follows the rule of every kept
// by-product: it is dropped as soon as any entry point writes or frees x.
#include <atomic>
#include <cstdlib>

#include "ew_core.h"
#include "internal.h"

using namespace tf;
using namespace tf::ew;

namespace {

struct FwdRelu { __device__ float operator()(float a, float) const { return a < 0.f ? 0.f : a; } };
struct FwdSigmoid { __device__ float operator()(float a, float) const { return 1.f / (1.f + expf(-a)); } };
struct FwdTanh { __device__ float operator()(float a, float) const { return tanhf(a); } };
// a = x, b = dy: the mask is x > 0, identical to cuDNN's y > 0 for ReLU
struct BwdRelu { __device__ float operator()(float a, float b) const { return a > 0.f ? b : 0.f; } };
// a = y, b = dy
struct BwdSigmoid { __device__ float operator()(float a, float b) const { return b * a * (1.f - a); } };
struct BwdTanh { __device__ float operator()(float a, float b) const { return b * (1.f - a * a); } };

// ---- ReLU with kept sign bits ---------------------------------------------------
// Work split as in ew_kernel: workgroup b owns the 1024 float4 from b*1024, lane t the
// four at b*1024 + u*256 + t.  The lane's 16 bits (bit 4u+c for component c of vector
// u) are one uint16 at index b*256 + t, so a wave writes and reads 128 contiguous bytes.
typedef unsigned short mask_t;

inline int64_t mask_blocks(int64_t n4) { return (n4 + kVecPerBlock - 1) / kVecPerBlock; }
inline size_t mask_bytes(int64_t n4) { return (size_t)mask_blocks(n4) * kThreads * sizeof(mask_t); }

__device__ inline unsigned sign_bits(const f32x4 &v) {
  return (v.x > 0.f ? 1u : 0u) | (v.y > 0.f ? 2u : 0u) | (v.z > 0.f ? 4u : 0u) | (v.w > 0.f ? 8u : 0u);
}

__device__ inline f32x4 pass_where_set(const f32x4 &dy, unsigned bits) {
  f32x4 r;
  r.x = (bits & 1u) ? dy.x : 0.f;
  r.y = (bits & 2u) ? dy.y : 0.f;
  r.z = (bits & 4u) ? dy.z : 0.f;
  r.w = (bits & 8u) ? dy.w : 0.f;
  return r;
}

__global__ __launch_bounds__(kThreads) void relu_forward_mask_kernel(const float *x, float *y, mask_t *mask,
                                                                    int64_t n4) {
  const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x);
  f32x4 *y4 = reinterpret_cast<f32x4 *>(y);
  const FwdRelu f;
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  const int64_t base = (int64_t)blockIdx.x * kVecPerBlock + threadIdx.x;
  unsigned bits = 0;
  if (base + (kUnroll - 1) * kThreads < n4) {
    f32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) v[u] = load_stream(x4 + base + u * kThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      bits |= sign_bits(v[u]) << (4 * u);
      store_stream(apply4(f, v[u], zero), y4 + base + u * kThreads);
    }
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + u * kThreads;
      if (i < n4) {
        const f32x4 v = load_stream(x4 + i);
        bits |= sign_bits(v) << (4 * u);
        store_stream(apply4(f, v, zero), y4 + i);
      }
    }
  }
  mask[(int64_t)blockIdx.x * kThreads + threadIdx.x] = (mask_t)bits;
}

__global__ __launch_bounds__(kThreads) void relu_backward_mask_kernel(const mask_t *mask, const float *dy,
                                                                     float *dx, int64_t n4) {
  const f32x4 *dy4 = reinterpret_cast<const f32x4 *>(dy);
  f32x4 *dx4 = reinterpret_cast<f32x4 *>(dx);
  const int64_t base = (int64_t)blockIdx.x * kVecPerBlock + threadIdx.x;
  const unsigned bits = __builtin_nontemporal_load(mask + (int64_t)blockIdx.x * kThreads + threadIdx.x);
  if (base + (kUnroll - 1) * kThreads < n4) {
    f32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) v[u] = load_stream(dy4 + base + u * kThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      store_stream(pass_where_set(v[u], bits >> (4 * u)), dx4 + base + u * kThreads);
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + u * kThreads;
      if (i < n4) store_stream(pass_where_set(load_stream(dy4 + i), bits >> (4 * u)), dx4 + i);
    }
  }
}

// arrays below this size gain nothing from a second, smaller read
constexpr int64_t kMaskMinElems = 1 << 16;
constexpr int kMaskTag = 1;

std::atomic<long long> g_masks_kept{0}, g_masks_used{0};

bool keeping_relu_mask() {
  static const bool on = [] {
    const char *e = getenv("TINYFLOW_KEEP_RELU_MASK");
    return !(e && *e && atoi(e) == 0);
  }();
  return on && !device_budget_active();
}

bool mask_shape_ok(int64_t n, const void *a, const void *b) {
  return n >= kMaskMinElems && n % 4 == 0 && aligned16(a) && aligned16(b);
}

}  // namespace

// How many ReLU forward calls kept their sign bits, and how many backward calls used
// them, since the library was loaded.  Either pointer may be null.
extern "C" int DLGpuReluMaskCounts(long long *kept, long long *used) {
  if (kept) *kept = g_masks_kept.load();
  if (used) *used = g_masks_used.load();
  return 0;
}

extern "C" int DLGpuActivationGetCudnnlist(const int *input_shapes, const int sizeofshape, int dataformat,
                                           int activationMode, void ***list) {
  TF_REQUIRE(input_shapes && list, "null argument");
  TF_REQUIRE(sizeofshape >= 1 && sizeofshape <= 5, "rank %d not supported", sizeofshape);
  TF_REQUIRE(activationMode >= 0 && activationMode <= 3, "unknown activation mode %d", activationMode);
  (void)dataformat;  // softmax runs over all non-batch dims, elementwise modes ignore layout
  ActDesc *d = new ActDesc();
  d->magic = kMagicAct;
  d->mode = activationMode;
  d->n = input_shapes[0];
  d->inner = 1;
  for (int i = 1; i < sizeofshape; ++i) d->inner *= input_shapes[i];
  void **slots = (void **)malloc(sizeof(void *) * 2);
  slots[0] = slots[1] = d;
  *list = slots;
  return 0;
}

extern "C" int DLGpuActivationForward(const DLArrayHandle input, DLArrayHandle output, int activationMode,
                                      void ***list, void **handle, void **stream) {
  announce_write(output);
  (void)handle;
  ActDesc *d = desc_from_list<ActDesc>(list, kMagicAct);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuActivationGetCudnnlist");
  TF_REQUIRE(on_gpu(input) && on_gpu(output), "arrays must live on the GPU");
  const int64_t n = numel(input);
  TF_REQUIRE(n == numel(output) && n == d->n * d->inner, "arrays do not match the descriptor");
  hipStream_t s = stream_of(stream);
  const float *x = (const float *)input->data;
  float *y = (float *)output->data;
  switch (activationMode) {
    case 0: return launch_ew<FwdSigmoid, true, false>(FwdSigmoid{}, y, x, nullptr, n, s, "DLGpuActivationForward");
    case 1: {
      const size_t bytes = mask_bytes(n / 4);
      if (d->backward_seen && x != y && mask_shape_ok(n, x, y) && keeping_relu_mask() && keep_has_room(bytes)) {
        if (mask_t *mask = (mask_t *)device_alloc(bytes)) {
          hipLaunchKernelGGL(relu_forward_mask_kernel, dim3((unsigned)mask_blocks(n / 4)), dim3(kThreads), 0, s, x,
                             y, mask, n / 4);
          keep_set(&d->kept_mask, mask, bytes, x, (size_t)n * sizeof(float), s, kMaskTag);
          g_masks_kept.fetch_add(1);
          return finish(s, "DLGpuActivationForward");
        }
      }
      return launch_ew<FwdRelu, true, false>(FwdRelu{}, y, x, nullptr, n, s, "DLGpuActivationForward");
    }
    case 2: return launch_ew<FwdTanh, true, false>(FwdTanh{}, y, x, nullptr, n, s, "DLGpuActivationForward");
    case 3:
      TF_REQUIRE(d->inner <= INT32_MAX, "instance too large");
      launch_softmax_rows(x, y, d->n, (int)d->inner, s);
      return finish(s, "DLGpuActivationForward");
  }
  TF_REQUIRE(false, "unknown activation mode %d", activationMode);
}

extern "C" int DLGpuActivationBackward(const DLArrayHandle input, DLArrayHandle dinput,
                                       const DLArrayHandle output, const DLArrayHandle doutput,
                                       int activationMode, void ***list, void **handle, void **stream) {
  announce_write(dinput);
  (void)handle;
  ActDesc *d = desc_from_list<ActDesc>(list, kMagicAct);
  TF_REQUIRE(d, "descriptor list was not created by DLGpuActivationGetCudnnlist");
  TF_REQUIRE(on_gpu(input) && on_gpu(dinput) && on_gpu(output) && on_gpu(doutput),
             "arrays must live on the GPU");
  const int64_t n = numel(input);
  TF_REQUIRE(n == numel(dinput) && n == numel(output) && n == numel(doutput) && n == d->n * d->inner,
             "arrays do not match the descriptor");
  hipStream_t s = stream_of(stream);
  const float *x = (const float *)input->data, *y = (const float *)output->data;
  const float *dy = (const float *)doutput->data;
  float *dx = (float *)dinput->data;
  switch (activationMode) {
    case 0: return launch_ew<BwdSigmoid, true, true>(BwdSigmoid{}, dx, y, dy, n, s, "DLGpuActivationBackward");
    case 1: {
      d->backward_seen = true;
      // the bits describe x as the forward call read it; the registry has dropped them if
      // anything wrote x since (this call's own dx included, announced above)
      if (mask_t *mask = (mask_t *)keep_take(&d->kept_mask, x, s, kMaskTag)) {
        const bool usable = n % 4 == 0 && aligned16(dy) && aligned16(dx);
        if (usable) {
          hipLaunchKernelGGL(relu_backward_mask_kernel, dim3((unsigned)mask_blocks(n / 4)), dim3(kThreads), 0, s,
                             mask, dy, dx, n / 4);
          g_masks_used.fetch_add(1);
        }
        device_free(mask);
        if (usable) return finish(s, "DLGpuActivationBackward");
      }
      return launch_ew<BwdRelu, true, true>(BwdRelu{}, dx, x, dy, n, s, "DLGpuActivationBackward");
    }
    case 2: return launch_ew<BwdTanh, true, true>(BwdTanh{}, dx, y, dy, n, s, "DLGpuActivationBackward");
    case 3:
      TF_REQUIRE(d->inner <= INT32_MAX, "instance too large");
      launch_softmax_rows_backward(y, dy, dx, d->n, (int)d->inner, s);
      return finish(s, "DLGpuActivationBackward");
  }
  TF_REQUIRE(false, "unknown activation mode %d", activationMode);
}
