// Sum reductions (bias gradients) and the softmax / softmax-cross-entropy rows.
//
// Every reduction is a fixed-order, two-stage tree (per-lane serial sums, wave
// shuffles, then a second pass over per-chunk partials): no atomics, so results
// are run-to-run deterministic.  The input is read exactly once, which makes the
// bias gradient HBM-bound at 4*(|dy| + C) bytes.
//
// Reference code replaced: src/gpu_op.cu:179-189, 950-963 (axis-0 sum),
// :369-524 (broadcast backward), :628-881 (cudnnReduceTensor ADD),
// :237-302, 1235-1287 (softmax, softmax cross entropy).
#include "internal.h"

#include <mutex>

using namespace tf;

namespace {

constexpr int kThreads = 256;

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_down(v, off, 64));
  return v;
}

// Sum of all lanes of a 256-thread block, valid in thread 0.
__device__ inline float block_sum(float v, float *smem /*[4]*/) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float r = 0.f;
  if (threadIdx.x == 0) r = (smem[0] + smem[1]) + (smem[2] + smem[3]);
  __syncthreads();
  return r;
}

// in viewed as [A, B] (C == 1): partial[chunk*B + j] = sum over rows of the chunk
__global__ __launch_bounds__(kThreads) void colsum_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                         int A, int B, int rows_per_chunk) {
  const int j = blockIdx.x * kThreads + threadIdx.x;
  if (j >= B) return;
  const int a0 = blockIdx.y * rows_per_chunk;
  int a1 = a0 + rows_per_chunk;
  if (a1 > A) a1 = A;
  const float *p = in + (int64_t)a0 * B + j;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  int a = a0;
  for (; a + 3 < a1; a += 4) {
    s0 += p[0];
    s1 += p[(int64_t)B];
    s2 += p[(int64_t)2 * B];
    s3 += p[(int64_t)3 * B];
    p += (int64_t)4 * B;
  }
  for (; a < a1; ++a) {
    s0 += p[0];
    p += B;
  }
  out[(int64_t)blockIdx.y * B + j] = (s0 + s1) + (s2 + s3);
}

// in viewed as [A, B, C]: partial[chunk*B + b] = sum_{a in chunk, c} in[a, b, c]
// one block per (b, chunk)
template <bool VEC>
__global__ __launch_bounds__(kThreads) void midsum_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                         int A, int B, int C, int rows_per_chunk) {
  __shared__ float smem[4];
  const int b = blockIdx.x;
  const int a0 = blockIdx.y * rows_per_chunk;
  int a1 = a0 + rows_per_chunk;
  if (a1 > A) a1 = A;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int a = a0; a < a1; ++a) {
    const float *row = in + ((int64_t)a * B + b) * C;
    if (VEC) {
      const float4 *row4 = reinterpret_cast<const float4 *>(row);
      const int c4 = C >> 2;
      for (int c = threadIdx.x; c < c4; c += kThreads) {
        const float4 v = row4[c];
        s0 += v.x;
        s1 += v.y;
        s2 += v.z;
        s3 += v.w;
      }
    } else {
      for (int c = threadIdx.x; c < C; c += kThreads) s0 += row[c];
    }
  }
  const float total = block_sum((s0 + s1) + (s2 + s3), smem);
  if (threadIdx.x == 0) out[(int64_t)blockIdx.y * B + b] = total;
}

// out[j] = sum_chunk partial[chunk*B + j], chunks added in index order
__global__ __launch_bounds__(kThreads) void finalsum_kernel(const float *__restrict__ partial,
                                                           float *__restrict__ out, int B, int chunks) {
  const int j = blockIdx.x * kThreads + threadIdx.x;
  if (j >= B) return;
  float s = 0.f;
  for (int c = 0; c < chunks; ++c) s += partial[(int64_t)c * B + j];
  out[j] = s;
}

// Row softmax: one wave per row, max-subtracted.
__global__ __launch_bounds__(kThreads) void softmax_rows_kernel(const float *__restrict__ in,
                                                               float *__restrict__ out, int64_t rows, int cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float *x = in + row * cols;
  float *y = out + row * cols;
  float m = -INFINITY;
  for (int c = lane; c < cols; c += 64) m = fmaxf(m, x[c]);
  m = __shfl(wave_max(m), 0, 64);
  float s = 0.f;
  for (int c = lane; c < cols; c += 64) s += expf(x[c] - m);
  s = __shfl(wave_sum(s), 0, 64);
  for (int c = lane; c < cols; c += 64) y[c] = expf(x[c] - m) / s;
}

// Softmax backward per row: dx = y * (dy - sum_j dy_j * y_j)
__global__ __launch_bounds__(kThreads) void softmax_rows_backward_kernel(const float *__restrict__ y,
                                                                        const float *__restrict__ dy,
                                                                        float *__restrict__ dx, int64_t rows,
                                                                        int cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float *yr = y + row * cols;
  const float *dyr = dy + row * cols;
  float *dxr = dx + row * cols;
  float s = 0.f;
  for (int c = lane; c < cols; c += 64) s += dyr[c] * yr[c];
  s = __shfl(wave_sum(s), 0, 64);
  for (int c = lane; c < cols; c += 64) dxr[c] = yr[c] * (dyr[c] - s);
}

// out[0] = mean_rows( -sum_c label * log_softmax(logit) ), single block of 1024
// threads; each wave walks rows wave, wave+16, ... and the 16 wave totals are
// added in wave order.
__global__ __launch_bounds__(1024) void softmax_xent_kernel(const float *__restrict__ logits,
                                                           const float *__restrict__ labels,
                                                           float *__restrict__ out, int rows, int cols) {
  __shared__ float wave_total[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float total = 0.f;
  for (int r = wave; r < rows; r += 16) {
    const float *x = logits + (int64_t)r * cols;
    const float *t = labels + (int64_t)r * cols;
    float m = -INFINITY;
    for (int c = lane; c < cols; c += 64) m = fmaxf(m, x[c]);
    m = __shfl(wave_max(m), 0, 64);
    float s = 0.f;
    for (int c = lane; c < cols; c += 64) s += expf(x[c] - m);
    s = __shfl(wave_sum(s), 0, 64);
    const float log_s = logf(s);
    float l = 0.f;
    for (int c = lane; c < cols; c += 64) l -= t[c] * ((x[c] - m) - log_s);
    total += wave_sum(l);
  }
  if (lane == 0) wave_total[wave] = total;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int w = 0; w < 16; ++w) s += wave_total[w];
    out[0] = s / (float)rows;
  }
}

// The same loss in two launches for more than 16 rows: one wave per row writes the
// row's term (same arithmetic as above), then one workgroup adds the terms the way
// the single-workgroup kernel does (wave w takes rows w, w+16, ... in order, the 16
// wave totals are added in wave order), so both forms give the same bits.
__global__ __launch_bounds__(kThreads) void softmax_xent_rows_kernel(const float *__restrict__ logits,
                                                                    const float *__restrict__ labels,
                                                                    float *__restrict__ row_loss, int rows,
                                                                    int cols) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  if (r >= rows) return;
  const float *x = logits + (int64_t)r * cols;
  const float *t = labels + (int64_t)r * cols;
  float m = -INFINITY;
  for (int c = lane; c < cols; c += 64) m = fmaxf(m, x[c]);
  m = __shfl(wave_max(m), 0, 64);
  float s = 0.f;
  for (int c = lane; c < cols; c += 64) s += expf(x[c] - m);
  s = __shfl(wave_sum(s), 0, 64);
  const float log_s = logf(s);
  float l = 0.f;
  for (int c = lane; c < cols; c += 64) l -= t[c] * ((x[c] - m) - log_s);
  l = wave_sum(l);
  if (lane == 0) row_loss[r] = l;
}

__global__ __launch_bounds__(1024) void xent_mean_kernel(const float *__restrict__ row_loss, float *__restrict__ out,
                                                        int rows) {
  __shared__ float wave_total[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    float total = 0.f;
    for (int r = wave; r < rows; r += 16) total += row_loss[r];
    wave_total[wave] = total;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int w = 0; w < 16; ++w) s += wave_total[w];
    out[0] = s / (float)rows;
  }
}

__global__ __launch_bounds__(kThreads) void zero_kernel(float *out, int n) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) out[i] = 0.f;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// How a sum over A rows (and C inner elements) per output is cut into chunks of rows
// that separate workgroups sum, so that a short output still fills a part of `cus`
// compute units (4 workgroups per unit are aimed at); the chunks' partial sums
// (chunks x B floats) are then added in chunk order.  Pure host arithmetic.
void chunk_rule(int64_t A, int64_t B, int64_t C, int cus, int &chunks, int &rows_per_chunk) {
  const int target_blocks = cus * 4;
  chunks = 1;
  const int64_t blocks_per_chunk = (C == 1) ? (B + kThreads - 1) / kThreads : B;
  if (blocks_per_chunk < target_blocks) {
    chunks = (int)((target_blocks + blocks_per_chunk - 1) / blocks_per_chunk);
    // keep at least 8 rows per chunk (column sums) / 1 row (mid sums)
    const int64_t max_chunks = (C == 1) ? (A + 7) / 8 : A;
    if (chunks > max_chunks) chunks = (int)max_chunks;
    if (chunks < 1) chunks = 1;
  }
  rows_per_chunk = (int)((A + chunks - 1) / chunks);
  chunks = (int)((A + rows_per_chunk - 1) / rows_per_chunk);
}

// out[b] = sum_{a, c} in[a, b, c]; 0 on success, 1 when scratch is exhausted
// (then *scratch_bytes holds the size wanted), -1 on launch failure.  A caller
// that cannot report exhausted scratch passes scratch_bytes == nullptr: the sum
// then runs as a single chunk, which needs no scratch (slower on short outputs,
// and the additions associate differently than in the chunked run).
//
// `fixed` / `fixed_bytes` name a caller-owned scratch area to use instead of the
// pool (the entry point that must not allocate): the chunking is the same, so the
// result has the same bits; when the partial sums do not fit, -2 is returned and
// nothing is launched.
int reduce_abc(const float *in, float *out, int64_t A, int64_t B, int64_t C, hipStream_t s,
               size_t *scratch_bytes, const char *what, float *fixed = nullptr, size_t fixed_bytes = 0) {
  if (B == 0) return 0;
  if (A > INT32_MAX || B > INT32_MAX || C > INT32_MAX) {
    fprintf(stderr, "[tinyflow_amd] %s: extents of 2^31 or more are not supported\n", what);
    return -1;
  }
  if (A == 0 || C == 0) {  // empty sum: a fill kernel, which (unlike a memset node) is safe under graph capture
    hipLaunchKernelGGL(zero_kernel, dim3(cdiv(B, kThreads)), dim3(kThreads), 0, s, out, (int)B);
    return finish(s, what);
  }
  const int64_t blocks_per_chunk = (C == 1) ? (B + kThreads - 1) / kThreads : B;
  int chunks, rows_per_chunk;
  chunk_rule(A, B, C, num_cus(), chunks, rows_per_chunk);
  float *partial = out;
  if (chunks > 1) {
    const size_t bytes = (size_t)chunks * (size_t)B * sizeof(float);
    if (fixed) {
      if (bytes > fixed_bytes) {
        if (scratch_bytes) *scratch_bytes = bytes;
        return -2;
      }
      partial = fixed;
    } else {
      partial = (float *)device_alloc(bytes);
    }
    if (!partial) {
      if (scratch_bytes) {
        *scratch_bytes = bytes;
        return 1;
      }
      partial = out;
      chunks = 1;
      rows_per_chunk = (int)A;
    }
  }
  if (C == 1) {
    hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)blocks_per_chunk, chunks), dim3(kThreads), 0, s, in,
                       partial, (int)A, (int)B, rows_per_chunk);
  } else if (C % 4 == 0 && aligned16(in)) {
    hipLaunchKernelGGL(midsum_kernel<true>, dim3((unsigned)B, chunks), dim3(kThreads), 0, s, in, partial,
                       (int)A, (int)B, (int)C, rows_per_chunk);
  } else {
    hipLaunchKernelGGL(midsum_kernel<false>, dim3((unsigned)B, chunks), dim3(kThreads), 0, s, in, partial,
                       (int)A, (int)B, (int)C, rows_per_chunk);
  }
  if (chunks > 1) {
    hipLaunchKernelGGL(finalsum_kernel, dim3(cdiv(B, kThreads)), dim3(kThreads), 0, s, partial, out, (int)B,
                       chunks);
    if (!fixed) device_free(partial);  // stream-ordered reuse: later users are enqueued behind finalsum
  }
  return finish(s, what);
}

}  // namespace

extern "C" int DLGpuReduceSumAxisZero(const DLArrayHandle in, DLArrayHandle out) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(in->ndim >= 1, "input needs at least one dim");
  const int64_t A = in->shape[0];
  const int64_t B = numel(in) / (A > 0 ? A : 1);
  TF_REQUIRE(numel(out) == (in->ndim == 1 ? 1 : B), "output must be input.shape[1:]");
  // 1-D input (n,) -> (1,): one column of n rows
  return reduce_abc((const float *)in->data, (float *)out->data, A, in->ndim == 1 ? 1 : B, 1, nullptr, nullptr,
                    "DLGpuReduceSumAxisZero");
}

// ---- the entry point that allocates nothing -----------------------------------
// The column sums' per-chunk partials live in a file-scope device array instead of
// pool memory.  Each device holds its own copy of the array at its own address, so
// the address is looked up once per device (hipGetSymbolAddress with that device
// current) and that pointer, never the symbol, is what the kernels receive.
// 1.5 MiB: on a 256-unit part chunks x columns stays under 256 Ki + columns floats, so
// every column sum of up to 131 072 columns fits, and so does any sum that runs as one
// chunk; a wider chunked sum is refused (DLGpuReduceSumAxisZeroNoAllocBytes tells).
constexpr size_t kFixedScratchBytes = 3u << 19;
static __device__ __align__(256) unsigned char scratch[kFixedScratchBytes];

namespace {
constexpr int kMaxDevices = 16;
std::mutex fixed_mu;
float *fixed_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device; nullptr (with a message) on failure.
float *fixed_scratch_of_current_device(const char *what) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fprintf(stderr, "[tinyflow_amd] %s: no current device (or device index above %d)\n", what, kMaxDevices - 1);
    return nullptr;
  }
  std::lock_guard<std::mutex> g(fixed_mu);
  if (!fixed_ptr[dev]) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      fprintf(stderr, "[tinyflow_amd] %s: hipGetSymbolAddress failed: %s\n", what, hipGetErrorString(e));
      return nullptr;
    }
    fixed_ptr[dev] = (float *)p;
  }
  return fixed_ptr[dev];
}
}  // namespace

// Pure host arithmetic, no GPU call when cus > 0: the bytes of partial sums the column
// sum of a (rows, cols) array keeps in the built-in area on a part of `cus` compute
// units (0: the current device's count), and the size of that area.  The entry point
// below refuses a shape with *wanted > *limit.
extern "C" int DLGpuReduceSumAxisZeroNoAllocBytes(int64_t rows, int64_t cols, int cus, int64_t *wanted,
                                                  int64_t *limit) {
  TF_REQUIRE(wanted && limit && rows >= 0 && cols >= 0 && cus >= 0, "bad arguments");
  TF_REQUIRE(rows <= INT32_MAX && cols <= INT32_MAX, "extents of 2^31 or more are not supported");
  *limit = (int64_t)kFixedScratchBytes;
  *wanted = 0;
  if (rows == 0 || cols == 0) return 0;
  int chunks, rows_per_chunk;
  chunk_rule(rows, cols, 1, cus > 0 ? cus : num_cus(), chunks, rows_per_chunk);
  if (chunks > 1) *wanted = (int64_t)chunks * cols * (int64_t)sizeof(float);
  return 0;
}

extern "C" int DLGpuReduceSumAxisZeroNoAlloc(const DLArrayHandle in, DLArrayHandle out, void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(in->ndim >= 1, "input needs at least one dim");
  const int64_t A = in->shape[0];
  const int64_t B = numel(in) / (A > 0 ? A : 1);
  TF_REQUIRE(numel(out) == (in->ndim == 1 ? 1 : B), "output must be input.shape[1:]");
  float *fixed = fixed_scratch_of_current_device("DLGpuReduceSumAxisZeroNoAlloc");
  if (!fixed) return -1;
  size_t want = 0;
  const int rc = reduce_abc((const float *)in->data, (float *)out->data, A, in->ndim == 1 ? 1 : B, 1,
                            stream_of(stream), &want, "DLGpuReduceSumAxisZeroNoAlloc", fixed, kFixedScratchBytes);
  TF_REQUIRE(rc != -2, "partial sums need %zu bytes, the built-in scratch area holds %zu", want,
             kFixedScratchBytes);
  return rc;
}

extern "C" int DLGpuBroadcastToBackward0(const DLArrayHandle in, DLArrayHandle out) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  const int64_t B = numel(out);
  TF_REQUIRE(B > 0 && numel(in) % B == 0, "output size must divide input size");
  if (!(out->ndim == 1 && out->shape[0] == 1)) {
    TF_REQUIRE(out->ndim <= in->ndim, "output has more dims than input");
    for (int i = 0; i < out->ndim; ++i)
      TF_REQUIRE(in->shape[in->ndim - 1 - i] == out->shape[out->ndim - 1 - i],
                 "output must match the trailing dims of the input");
  }
  return reduce_abc((const float *)in->data, (float *)out->data, numel(in) / B, B, 1, nullptr, nullptr,
                    "DLGpuBroadcastToBackward0");
}

extern "C" int DLGpuBroadcastToBackward1(const DLArrayHandle in, DLArrayHandle out) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(out->ndim == 1 && in->ndim >= 2 && out->shape[0] == in->shape[1],
             "input must be (N, C, ...) and output (C,)");
  int64_t inner = 1;
  for (int i = 2; i < in->ndim; ++i) inner *= in->shape[i];
  return reduce_abc((const float *)in->data, (float *)out->data, in->shape[0], in->shape[1], inner, nullptr,
                    nullptr, "DLGpuBroadcastToBackward1");
}

extern "C" int DLGReduceSumGetCudnnlist(const int *input_shapes, const int *output_shapes, const int ndim,
                                        int dataformat, void ***list, void **handle) {
  (void)dataformat;
  (void)handle;
  TF_REQUIRE(input_shapes && output_shapes && list, "null argument");
  TF_REQUIRE(ndim >= 1 && ndim <= 5, "rank %d not supported", ndim);
  for (int i = 0; i < ndim; ++i)
    TF_REQUIRE(input_shapes[i] >= 0 && (output_shapes[i] == input_shapes[i] || output_shapes[i] == 1),
               "output dim %d must be 1 or equal to the input dim", i);
  ReduceDesc *d = new ReduceDesc();
  d->magic = kMagicReduce;
  d->ndim = ndim;
  for (int i = 0; i < ndim; ++i) {
    d->in[i] = input_shapes[i];
    d->out[i] = output_shapes[i];
  }
  // same five-slot list as the reference; every slot points at the descriptor
  void **slots = (void **)malloc(sizeof(void *) * 5);
  for (int i = 0; i < 5; ++i) slots[i] = d;
  *list = slots;
  return 0;
}

extern "C" int DLGpuReduceSum(const DLArrayHandle in, DLArrayHandle out, void ***list, void **handle,
                              int *memorytoSaving, void **stream) {
  announce_write(out);
  (void)handle;
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  ReduceDesc *d = desc_from_list<ReduceDesc>(list, kMagicReduce);
  TF_REQUIRE(d, "descriptor list was not created by DLGReduceSumGetCudnnlist");
  int64_t in_count = 1, out_count = 1;
  for (int i = 0; i < d->ndim; ++i) {
    in_count *= d->in[i];
    out_count *= d->out[i];
  }
  TF_REQUIRE(numel(in) == in_count && numel(out) == out_count, "arrays do not match the descriptor");
  // Collapse to [A, B, C]: a reduced prefix, one run of kept dims, a reduced
  // suffix.  Dims of extent 1 carry no data and fit anywhere.
  int64_t A = 1, B = 1, C = 1;
  int phase = 0;  // 0 prefix (reduced), 1 kept run, 2 suffix (reduced)
  for (int i = 0; i < d->ndim; ++i) {
    if (d->in[i] == 1) continue;
    const bool kept = d->out[i] == d->in[i];
    if (kept) {
      TF_REQUIRE(phase <= 1, "kept dims must be contiguous (reduce pattern not supported)");
      phase = 1;
      B *= d->in[i];
    } else if (phase == 0) {
      A *= d->in[i];
    } else {
      phase = 2;
      C *= d->in[i];
    }
  }
  size_t want = 0;
  const int rc = reduce_abc((const float *)in->data, (float *)out->data, A, B, C, stream_of(stream), &want,
                            "DLGpuReduceSum");
  if (rc == 1) {
    if (memorytoSaving) *memorytoSaving = shortfall(want);
    return 0;
  }
  return rc;
}

extern "C" int DLGpuSoftmax(const DLArrayHandle in, DLArrayHandle out, void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(in) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(in->ndim == 2 && same_shape(in, out), "softmax needs matching 2-D arrays");
  const int64_t rows = in->shape[0];
  const int cols = (int)in->shape[1];
  hipStream_t s = stream_of(stream);
  if (rows == 0 || cols == 0) return 0;
  hipLaunchKernelGGL(softmax_rows_kernel, dim3(cdiv(rows, kThreads / 64)), dim3(kThreads), 0, s,
                     (const float *)in->data, (float *)out->data, rows, cols);
  return finish(s, "DLGpuSoftmax");
}

extern "C" int DLGpuSoftmaxCrossEntropy(const DLArrayHandle logits, const DLArrayHandle labels,
                                        DLArrayHandle out, void **stream) {
  announce_write(out);
  TF_REQUIRE(on_gpu(logits) && on_gpu(labels) && on_gpu(out), "arrays must live on the GPU");
  TF_REQUIRE(logits->ndim == 2 && same_shape(logits, labels), "logits and labels must be matching 2-D arrays");
  TF_REQUIRE(numel(out) == 1, "output must hold one element");
  hipStream_t s = stream_of(stream);
  const int rows = (int)logits->shape[0], cols = (int)logits->shape[1];
  // this entry point cannot report exhausted scratch: without it the one-launch form runs
  float *row_loss = rows > 16 ? (float *)device_alloc((size_t)rows * sizeof(float)) : nullptr;
  if (row_loss) {
    hipLaunchKernelGGL(softmax_xent_rows_kernel, dim3(cdiv(rows, kThreads / 64)), dim3(kThreads), 0, s,
                       (const float *)logits->data, (const float *)labels->data, row_loss, rows, cols);
    hipLaunchKernelGGL(xent_mean_kernel, dim3(1), dim3(1024), 0, s, (const float *)row_loss, (float *)out->data, rows);
    device_free(row_loss);
  } else {
    hipLaunchKernelGGL(softmax_xent_kernel, dim3(1), dim3(1024), 0, s, (const float *)logits->data,
                       (const float *)labels->data, (float *)out->data, rows, cols);
  }
  return finish(s, "DLGpuSoftmaxCrossEntropy");
}

// Used by activation.hip for the softmax activation mode.
namespace tf {
int launch_softmax_rows(const float *in, float *out, int64_t rows, int cols, hipStream_t s) {
  if (rows == 0 || cols == 0) return 0;
  hipLaunchKernelGGL(softmax_rows_kernel, dim3(cdiv(rows, kThreads / 64)), dim3(kThreads), 0, s, in, out, rows,
                     cols);
  return 0;
}
int launch_softmax_rows_backward(const float *y, const float *dy, float *dx, int64_t rows, int cols,
                                 hipStream_t s) {
  if (rows == 0 || cols == 0) return 0;
  hipLaunchKernelGGL(softmax_rows_backward_kernel, dim3(cdiv(rows, kThreads / 64)), dim3(kThreads), 0, s, y, dy,
                     dx, rows, cols);
  return 0;
}
}  // namespace tf
