// Activation forward/backward: ReLU (the mode every conv net of the reference
// uses), sigmoid, tanh, and softmax over c*h*w per instance.
//
// Replaces cudnnActivationForward/Backward and cudnnSoftmaxForward/Backward as
// called at src/gpu_op.cu:3211-3274 and 3475-3544, and the descriptor builder at
// :3364-3471.  The ReLU gradient reads x and dy and writes dx (12 bytes per
// element); the forward output y, which cuDNN also takes, is not needed.
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

}  // namespace

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
    case 1: return launch_ew<FwdRelu, true, false>(FwdRelu{}, y, x, nullptr, n, s, "DLGpuActivationForward");
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
    case 1: return launch_ew<BwdRelu, true, true>(BwdRelu{}, dx, x, dy, n, s, "DLGpuActivationBackward");
    case 2: return launch_ew<BwdTanh, true, true>(BwdTanh{}, dx, y, dy, n, s, "DLGpuActivationBackward");
    case 3:
      TF_REQUIRE(d->inner <= INT32_MAX, "instance too large");
      launch_softmax_rows_backward(y, dy, dx, d->n, (int)d->inner, s);
      return finish(s, "DLGpuActivationBackward");
  }
  TF_REQUIRE(false, "unknown activation mode %d", activationMode);
}
