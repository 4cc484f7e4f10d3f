// Dropout forward / backward and channel concatenation.
//
// Dropout replaces cudnnDropoutForward / cudnnDropoutBackward as the reference
// calls them (src/gpu_op.cu:3547-3693; input descriptor :3276-3362): each
// element is dropped with probability `dropout`, survivors are scaled by
// 1 / (1 - dropout), and backward applies the same mask and scale to the
// gradient.  The mask lives in the reserve space as one bit per element
// (forward allocates it and publishes it through *reserveSpace_p, backward
// consumes and releases it, as in the reference).
//
// Random bits come from Philox4x32-10 (Salmon et al., SC'11), a counter-based
// generator: element i uses word i % 4 of the block with counter (i / 4, 0, 0, 0)
// and key (seed, 0), and is kept when that word is >= dropout * 2^32.  The
// mask is a pure function of (seed, element index, dropout), so any grid shape
// reproduces it; cuDNN's own generator is not reproducible outside cuDNN.
//
// Concatenation along axis 1 replaces src/gpu_op.cu:967-1084.
#include "gemm_core.h"
#include "internal.h"

using namespace tf;
using tf::gemm::FastDiv;

namespace {

constexpr int kThreads = 256;
constexpr int kMagicInput = 0x7466496e;    // 'tfIn'
constexpr int kMagicDropout = 0x74664472;  // 'tfDr'

struct DropoutDesc;
struct InputDesc {
  int magic;
  int64_t count;
  // mask + list published by the last forward through this descriptor and not yet
  // consumed by a backward (the binding makes new cells for every forward, so the
  // descriptor, which lives as long as its node, is where an unconsumed pair is found)
  DropoutDesc *pending;
  void **pending_slots;
};

struct DropoutDesc {
  int magic;
  int64_t count;
  float scale;
  void *reserve;
};

struct u32x4 {
  uint32_t x, y, z, w;
};

__device__ inline u32x4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0;
    c1 = lo1;
    c2 = n2;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return {c0, c1, c2, c3};
}

// One lane owns 8 consecutive elements = one mask byte (two Philox blocks).
template <bool FORWARD>
__global__ __launch_bounds__(kThreads) void dropout_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                          unsigned char *__restrict__ mask, int64_t count,
                                                          uint32_t seed, uint32_t threshold, float scale) {
  const int64_t group = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int64_t base = group * 8;
  if (base >= count) return;
  unsigned bits;
  if (FORWARD) {
    const u32x4 r0 = philox4x32_10((uint32_t)(2 * group), (uint32_t)((2 * group) >> 32), 0u, 0u, seed, 0u);
    const u32x4 r1 = philox4x32_10((uint32_t)(2 * group + 1), (uint32_t)((2 * group + 1) >> 32), 0u, 0u, seed, 0u);
    const uint32_t r[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
    bits = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) bits |= (r[j] >= threshold ? 1u : 0u) << j;
    mask[group] = (unsigned char)bits;
  } else {
    bits = mask[group];
  }
  if (base + 8 <= count && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0) {
    const float4 a = reinterpret_cast<const float4 *>(in + base)[0], b = reinterpret_cast<const float4 *>(in + base)[1];
    float4 oa, ob;
    oa.x = (bits & 1u) ? a.x * scale : 0.f;
    oa.y = (bits & 2u) ? a.y * scale : 0.f;
    oa.z = (bits & 4u) ? a.z * scale : 0.f;
    oa.w = (bits & 8u) ? a.w * scale : 0.f;
    ob.x = (bits & 16u) ? b.x * scale : 0.f;
    ob.y = (bits & 32u) ? b.y * scale : 0.f;
    ob.z = (bits & 64u) ? b.z * scale : 0.f;
    ob.w = (bits & 128u) ? b.w * scale : 0.f;
    reinterpret_cast<float4 *>(out + base)[0] = oa;
    reinterpret_cast<float4 *>(out + base)[1] = ob;
  } else {
    for (int j = 0; j < 8 && base + j < count; ++j) out[base + j] = ((bits >> j) & 1u) ? in[base + j] * scale : 0.f;
  }
}

// out[o, :] = [a[o, :ca], b[o, :cb]] with ca / cb elements per outer index
__global__ __launch_bounds__(kThreads) void concat_kernel(const float *__restrict__ a, uint32_t ca,
                                                         const float *__restrict__ b, uint32_t cb, FastDiv row,
                                                         float *__restrict__ out, uint32_t total) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    uint32_t o, j;
    row.divmod(i, o, j);
    out[i] = j < ca ? a[(int64_t)o * ca + j] : b[(int64_t)o * cb + (j - ca)];
  }
}

// din[o, :] = dout[o, offset : offset + width]
__global__ __launch_bounds__(kThreads) void slice_kernel(const float *__restrict__ dout, int64_t row, int64_t offset,
                                                        FastDiv width, float *__restrict__ din, uint32_t total) {
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    uint32_t o, j;
    width.divmod(i, o, j);
    din[i] = dout[(int64_t)o * row + offset + j];
  }
}

int grid_for(int64_t n) {
  int64_t blocks = (n + kThreads - 1) / kThreads;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1 : (int)blocks;
}

// Per-outer-index widths of the two inputs of a concatenation along axis 1.
int concat_geometry(const DLArray *a, const DLArray *b, int64_t &outer, int64_t &ca, int64_t &cb) {
  TF_REQUIRE(on_gpu(a) && on_gpu(b), "arrays must live on the GPU");
  TF_REQUIRE(a->ndim == b->ndim && a->ndim >= 2, "inputs must have the same rank (>= 2)");
  for (int i = 0; i < a->ndim; ++i)
    if (i != 1) TF_REQUIRE(a->shape[i] == b->shape[i], "inputs differ outside axis 1");
  outer = a->shape[0];
  ca = outer ? numel(a) / outer : 0;
  cb = outer ? numel(b) / outer : 0;
  return 0;
}

}  // namespace

extern "C" int DLGpuGetInputDescriptor(const int *input_shapes, int sizeofshape, int dataformat, void ***inputd) {
  (void)dataformat;  // the element count is all dropout needs; the layout does not matter
  TF_REQUIRE(input_shapes && inputd, "null argument");
  TF_REQUIRE(sizeofshape >= 1 && sizeofshape <= 8, "rank %d not supported", sizeofshape);
  InputDesc *d = new InputDesc();
  d->magic = kMagicInput;
  d->count = 1;
  for (int i = 0; i < sizeofshape; ++i) {
    TF_REQUIRE(input_shapes[i] >= 0, "negative extent");
    d->count *= input_shapes[i];
  }
  void **slots = (void **)malloc(sizeof(void *));
  slots[0] = d;
  *inputd = slots;
  return 0;
}

extern "C" int DLGpuDropoutForward(const DLArrayHandle input, DLArrayHandle output, int dataformat, float dropout,
                                   int seed, void **reserveSpace_p, void ***inputd, void ***cudnnlist,
                                   void **handle, int *memorytoSaving, void **stream) {
  announce_write(output);
  (void)dataformat;
  (void)handle;
  InputDesc *in = desc_from_list<InputDesc>(inputd, kMagicInput);
  TF_REQUIRE(in, "descriptor was not created by DLGpuGetInputDescriptor");
  TF_REQUIRE(reserveSpace_p && cudnnlist, "null argument");
  TF_REQUIRE(on_gpu(input) && on_gpu(output), "arrays must live on the GPU");
  TF_REQUIRE(numel(input) == in->count && numel(output) == in->count, "arrays do not match the descriptor");
  TF_REQUIRE(dropout >= 0.f && dropout < 1.f, "dropout probability %g outside [0, 1)", (double)dropout);
  hipStream_t s = stream_of(stream);
  // a forward whose backward never ran (an evaluation-only pass): release its mask and
  // list before publishing new ones (a backward on the old cells is then refused)
  // The mask goes back to the pool; the two small host records are only invalidated,
  // not freed, because the caller's old cells still point at them.
  if (in->pending) {
    device_free(in->pending->reserve);
    in->pending->reserve = nullptr;
    in->pending->magic = 0;
    in->pending = nullptr;
    in->pending_slots = nullptr;
  }
  const int64_t groups = (in->count + 7) / 8;
  unsigned char *mask = (unsigned char *)device_alloc((size_t)(groups > 0 ? groups : 1));
  if (!mask) {
    if (memorytoSaving) *memorytoSaving = shortfall(groups);
    return 0;
  }
  DropoutDesc *d = new DropoutDesc();
  d->magic = kMagicDropout;
  d->count = in->count;
  d->scale = 1.0f / (1.0f - dropout);
  d->reserve = mask;
  *reserveSpace_p = mask;
  void **slots = (void **)malloc(sizeof(void *) * 2);
  slots[0] = d;
  slots[1] = in;
  *cudnnlist = slots;
  in->pending = d;
  in->pending_slots = slots;
  if (groups > 0) {
    // drop when the 32-bit draw is below dropout * 2^32
    const double t = (double)dropout * 4294967296.0;
    const uint32_t threshold = t >= 4294967295.0 ? 0xffffffffu : (uint32_t)t;
    hipLaunchKernelGGL(dropout_kernel<true>, dim3((unsigned)((groups + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       s, (const float *)input->data, (float *)output->data, mask, in->count, (uint32_t)seed,
                       threshold, d->scale);
  }
  return finish(s, "DLGpuDropoutForward");
}

extern "C" int DLGpuDropoutBackward(const DLArrayHandle doutput, DLArrayHandle dinput, void **reserveSpace_p,
                                    void ***cudnnlist, void **handle, void **stream) {
  announce_write(dinput);
  (void)handle;
  DropoutDesc *d = desc_from_list<DropoutDesc>(cudnnlist, kMagicDropout);
  TF_REQUIRE(d, "list was not created by DLGpuDropoutForward (or was consumed already)");
  TF_REQUIRE(reserveSpace_p && *reserveSpace_p == d->reserve, "reserve space does not belong to this list");
  TF_REQUIRE(on_gpu(doutput) && on_gpu(dinput), "arrays must live on the GPU");
  TF_REQUIRE(numel(doutput) == d->count && numel(dinput) == d->count, "arrays do not match the forward pass");
  hipStream_t s = stream_of(stream);
  const int64_t groups = (d->count + 7) / 8;
  if (groups > 0)
    hipLaunchKernelGGL(dropout_kernel<false>, dim3((unsigned)((groups + kThreads - 1) / kThreads)), dim3(kThreads),
                       0, s, (const float *)doutput->data, (float *)dinput->data, (unsigned char *)d->reserve,
                       d->count, 0u, 0u, d->scale);
  // the mask and the list are consumed (stream-ordered release), as in the reference
  if (InputDesc *in = reinterpret_cast<InputDesc *>((*cudnnlist)[1]); in && in->magic == kMagicInput && in->pending == d) {
    in->pending = nullptr;
    in->pending_slots = nullptr;
  }
  device_free(d->reserve);
  *reserveSpace_p = nullptr;
  d->magic = 0;
  delete d;
  free(*cudnnlist);
  *cudnnlist = nullptr;
  return finish(s, "DLGpuDropoutBackward");
}

extern "C" int DLGpuConcatForward(const DLArrayHandle input1, const DLArrayHandle input2, DLArrayHandle output,
                                  void **stream) {
  announce_write(output);
  int64_t outer, ca, cb;
  if (concat_geometry(input1, input2, outer, ca, cb) != 0) return -1;
  TF_REQUIRE(on_gpu(output) && numel(output) == numel(input1) + numel(input2), "output has the wrong size");
  hipStream_t s = stream_of(stream);
  const int64_t total = numel(output);
  TF_REQUIRE(total < ((int64_t)1 << 31), "tensors of 2^31 elements or more are not supported");
  if (total > 0)
    hipLaunchKernelGGL(concat_kernel, dim3(grid_for(total)), dim3(kThreads), 0, s, (const float *)input1->data,
                       (uint32_t)ca, (const float *)input2->data, (uint32_t)cb, FastDiv((uint32_t)(ca + cb)),
                       (float *)output->data, (uint32_t)total);
  return finish(s, "DLGpuConcatForward");
}

static int concat_backward(const DLArray *input1, const DLArray *input2, const DLArray *doutput, DLArray *dinput,
                           bool second, void **stream, const char *what) {
  int64_t outer, ca, cb;
  if (concat_geometry(input1, input2, outer, ca, cb) != 0) return -1;
  TF_REQUIRE(on_gpu(doutput) && numel(doutput) == numel(input1) + numel(input2), "doutput has the wrong size");
  const int64_t width = second ? cb : ca;
  TF_REQUIRE(on_gpu(dinput) && numel(dinput) == outer * width, "dinput has the wrong size");
  hipStream_t s = stream_of(stream);
  const int64_t total = outer * width;
  TF_REQUIRE(numel(doutput) < ((int64_t)1 << 31), "tensors of 2^31 elements or more are not supported");
  if (total > 0)
    hipLaunchKernelGGL(slice_kernel, dim3(grid_for(total)), dim3(kThreads), 0, s, (const float *)doutput->data,
                       ca + cb, second ? ca : 0, FastDiv((uint32_t)width), (float *)dinput->data, (uint32_t)total);
  return finish(s, what);
}

extern "C" int DLGpuConcataBackward(const DLArrayHandle input1, const DLArrayHandle input2,
                                    const DLArrayHandle doutput, DLArrayHandle dinput1, void **stream) {
  announce_write(dinput1);
  return concat_backward(input1, input2, doutput, dinput1, false, stream, "DLGpuConcataBackward");
}

extern "C" int DLGpuConcatbBackward(const DLArrayHandle input1, const DLArrayHandle input2,
                                    const DLArrayHandle doutput, DLArrayHandle dinput2, void **stream) {
  announce_write(dinput2);
  return concat_backward(input1, input2, doutput, dinput2, true, stream, "DLGpuConcatbBackward");
}
