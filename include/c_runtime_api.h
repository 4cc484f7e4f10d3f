/*
 * C-ABI of libc_runtime_api.so, the MI355X (gfx950) drop-in for tinyflow's
 * native runtime on the training hot path (backward pass + gradient kernels).
 *
 * Every entry point below replaces the reference function of the same name;
 * the citation after each declaration is the reference declaration
 * (src/c_runtime_api.h) and its CUDA/cuDNN implementation (src/gpu_op.cu,
 * src/c_runtime_api.cc).  The binding sets no argtypes, so arguments arrive
 * under ctypes defaults: Python int -> C int, bool -> int, c_float -> float,
 * DLContext by value, everything else a pointer.  All functions return int:
 * 0 on success, -1 on a rejected call (shape mismatch, unsupported layout,
 * HIP failure) -- the reference asserts or exits in those places.
 *
 * Conventions shared by all op entry points
 *  - tensors are dense row-major fp32, activations NCHW, filters KCRS;
 *  - `void **stream` points at a cell whose content is the hipStream_t
 *    (written by DLGpuCreatecudaStream); ops enqueue on it and return without
 *    waiting.  Results become host-visible through DLArrayCopyFromTo, which
 *    orders itself after all enqueued work, so the observable behaviour of the
 *    reference (which synchronises after every op) is preserved.  Setting the
 *    environment variable TINYFLOW_SYNC_EVERY_OP=1 restores a literal
 *    synchronise-after-every-op mode;
 *  - `void ***list` is an opaque descriptor list created by the matching
 *    *GetOutShape / *GetCudnnlist call (cuDNN descriptors in the reference,
 *    plain structs here); it is never freed, as in the reference;
 *  - `int *memorytoSaving` is left at 0 unless device scratch could not be
 *    allocated, in which case it receives the byte count wanted and the op
 *    returns 0 without writing its output (reference: gpu_op.cu:1704-1712);
 *  - the `handle` arguments (cudnn/cublas handles in the reference) are opaque
 *    cells created by DLGpuCreatecudnnHandle / DLGpuCreatecublasHandle; only
 *    their bound stream is used.
 *
 * Enum values sent by the binding (reference: pycode/tinyflow/gpu_op.py):
 *   dataformat  NCHW=0, NHWC=1 (only NCHW is implemented for 4-D ops)
 *   padding     "SAME"=1 (symmetric k/2), "VALID"=0   (gpu_op.py:443-448)
 *   poolingMode max=0, mean=1 (count includes padding) (gpu_op.py:610-613)
 *   activation  sigmoid=0, relu=1, tanh=2, softmax=3   (gpu_op.py:501-510)
 *   batchNorm   pre_activation(per-activation)=0, spatial=1 (gpu_op.py:778-783)
 */
#ifndef TINYFLOW_AMD_C_RUNTIME_API_H_
#define TINYFLOW_AMD_C_RUNTIME_API_H_

#include "dlarray.h"

#ifdef __cplusplus
#include <cstdbool>
extern "C" {
#else
#include <stdbool.h>
#endif

typedef int64_t index_t;

/* ------------------------------------------------------------------ arrays */

/* Allocate an fp32 array (device memory for kGPU, pinned host memory for
 * kCPU).  On out-of-memory: *memorytoSaving = bytes wanted, *out untouched,
 * returns 0.  ref: c_runtime_api.h:53-54, c_runtime_api.cc:93-121,
 * cuda_device_api.cc:31-45, cpu_device_api.cc:12-22 */
int DLArrayAlloc(const index_t *shape, index_t ndim, DLContext ctx,
                 DLArrayHandle *out, int *memorytoSaving);

/* ref: c_runtime_api.h:61, c_runtime_api.cc:123-128 */
int DLArrayFree(DLArrayHandle handle);

/* Copy between host/device arrays of equal byte size.  stream == NULL: fully
 * synchronous.  Otherwise `stream` points at a stream cell; the copy runs on
 * that stream, ordered after everything enqueued on the kernel streams, and the
 * call returns after it completed -- except a device-to-device copy on a stream
 * that op entry points launch on, which stays asynchronous (later ops on that
 * stream are ordered behind it).
 * ref: c_runtime_api.h:70-71, c_runtime_api.cc:130-164 */
int DLArrayCopyFromTo(DLArrayHandle from, DLArrayHandle to, DLStreamHandle stream);

/* No counterpart in the reference: the rule above as a pure function, so that it
 * can be checked without a GPU.  kind: 0 host->device, 1 device->host,
 * 2 device->device; returns 1 when DLArrayCopyFromTo waits for the copy. */
int DLArrayCopyWaitsForCompletion(int kind, int stream_runs_kernels, int sync_every_op);

/* No counterpart in the reference.  Host -> device copy into an array that came from
 * DLArrayAlloc and has not been used since (the prefetch of the swap path): only
 * the previous life of the destination's storage has to be over, not everything
 * that is enqueued, so the copy overlaps with the compute stream.  `stream` is a
 * stream cell as for DLArrayCopyFromTo (not NULL); returns after the copy. */
int DLArrayCopyIntoFresh(DLArrayHandle from, DLArrayHandle to, DLStreamHandle stream);

/* No counterpart in the reference.  Call right after DLArrayAlloc on an array that
 * DLArrayCopyIntoFresh will fill later: records, now, the fence that covers the
 * last release of the array's storage, so that the copy waits for nothing enqueued
 * after this call.  Without it DLArrayCopyIntoFresh waits like DLArrayCopyFromTo. */
int DLArrayPrepareFresh(DLArrayHandle arr);

/* ref: c_runtime_api.h:564, gpu_op.cu:4896-4898 */
int getInt(int *intp);

/* No counterpart in the reference (which is bounded by the physical card): a
 * device-memory budget for the allocator behind DLArrayAlloc and the ops'
 * scratch, so that a 16 GB device can be imitated on a larger one; bytes <= 0
 * removes it.  The environment variable TINYFLOW_GPU_MEM_LIMIT_MB sets the same
 * budget at start-up. */
int DLGpuSetDeviceMemoryLimit(int64_t bytes);

/* No counterpart in the reference: allocator statistics in bytes -- held from
 * HIP (in use + cached), in use, and the high-water mark of bytes in use since
 * the last call that passed reset_peak != 0. */
int DLGpuGetDeviceMemoryStats(int64_t *reserved, int64_t *in_use, int64_t *peak_in_use,
                              int reset_peak);

/* Pageable-vs-pinned host<->device bandwidth probe (prints GB/s).
 * ref: c_runtime_api.h:565, gpu_op.cu:4915-5005 */
int testPcie();

/* ----------------------------------------------------- streams and handles */

/* ref: c_runtime_api.h:230-235, gpu_op.cu:1352-1429 */
int DLGpuCreatecudaStream(void **stream);
int DLGpuDestroycudaStream(void **stream);
int DLGpuCreatecudnnHandle(void **handle, void **stream);
int DLGpuDestroycudnnHandle(void **handle);
int DLGpuCreatecublasHandle(void **handle, void **stream);
int DLGpuDestroycublasHandle(void **handle);

/* ------------------------------------------------------------- elementwise */

/* arr[i] = value.  ref: c_runtime_api.h:79, gpu_op.cu:39-45, 331-341 */
int DLGpuArraySet(DLArrayHandle arr, float value, void **stream);

/* out[i] = in[i % count(in)] (trailing-dims broadcast, FC bias).
 * ref: c_runtime_api.h:87, gpu_op.cu:47-52, 343-367 */
int DLGpuBroadcastTo0(const DLArrayHandle input, DLArrayHandle output, void **stream);

/* out[n,c,...] = in[c] (per-channel broadcast, conv bias).
 * ref: c_runtime_api.h:91, gpu_op.cu:108-123, 450-471 */
int DLGpuBroadcastTo1(const DLArrayHandle input, DLArrayHandle output, void **stream);

/* Sum over the leading dims down to the output's trailing shape.
 * ref: c_runtime_api.h:89, gpu_op.cu:369-447 */
int DLGpuBroadcastToBackward0(const DLArrayHandle input, DLArrayHandle output);

/* out[c] = sum over n and trailing dims of in[n,c,...].
 * ref: c_runtime_api.h:93, gpu_op.cu:473-524 */
int DLGpuBroadcastToBackward1(const DLArrayHandle input, DLArrayHandle output);

/* out[j] = sum_i in[i, j].  ref: c_runtime_api.h:101, gpu_op.cu:179-189, 950-963 */
int DLGpuReduceSumAxisZero(const DLArrayHandle input, DLArrayHandle output);

/* The same column sums with the same bits, for callers that cannot allocate
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  The per-chunk partial sums live
 * in a 1.5 MiB device array built into the library (one copy per GPU, held until
 * the process ends) instead of pool memory; no hipMalloc / hipFree / memset is
 * issued.  A shape whose partial sums do not fit returns -1 with a message and
 * launches nothing (on a 256-unit part: chunked sums over more than 131 072
 * columns; sums that run as one chunk need no scratch and always fit).  Calls on
 * one GPU share the array: calls that overlap on different streams race. */
int DLGpuReduceSumAxisZeroNoAlloc(const DLArrayHandle input, DLArrayHandle output, void **stream);
/* The rule behind that limit as pure host arithmetic (no GPU call when cus > 0):
 * bytes of partial sums a (rows, cols) column sum keeps on a part of `cus` compute
 * units (0: the current device), and the size of the built-in area.  No
 * counterpart in the reference. */
int DLGpuReduceSumAxisZeroNoAllocBytes(int64_t rows, int64_t cols, int cus, int64_t *wanted, int64_t *limit);

/* ref: c_runtime_api.h:110-141, gpu_op.cu:193-219, 1090-1164 */
int DLGpuMatrixElementwiseAdd(const DLArrayHandle matA, const DLArrayHandle matB,
                              DLArrayHandle output, void **stream);
int DLGpuMatrixElementwiseAddByConst(const DLArrayHandle input, float val,
                                     DLArrayHandle output, void **stream);
/* No counterpart in the reference: output = max(matA + matB, 0), a residual join and
 * the ReLU behind it as one pass; equals the two separate ops bit for bit. */
int DLGpuMatrixElementwiseAddRelu(const DLArrayHandle matA, const DLArrayHandle matB,
                                  DLArrayHandle output, void **stream);
int DLGpuMatrixElementwiseMultiply(const DLArrayHandle matA, const DLArrayHandle matB,
                                   DLArrayHandle output, void **stream);
int DLGpuMatrixMultiplyByConst(const DLArrayHandle input, float val,
                               DLArrayHandle output, void **stream);

/* out = max(in, 0) / out = in > 0 ? grad : 0.  Neither takes a stream; both run
 * on the default stream, ordered after all work already enqueued on the streams
 * created by DLGpuCreatecudaStream and before any work enqueued there later.  ref: c_runtime_api.h:162-172, gpu_op.cu:221-235, 1201-1233 */
int DLGpuRelu(const DLArrayHandle input, DLArrayHandle output);
int DLGpuReluGradient(const DLArrayHandle input, const DLArrayHandle in_grad,
                      DLArrayHandle output);

/* ------------------------------------------------ softmax / cross entropy */

/* Row softmax of a 2-D array (max-subtracted).
 * ref: c_runtime_api.h:180, gpu_op.cu:237-255, 1235-1254 */
int DLGpuSoftmax(const DLArrayHandle input, DLArrayHandle output, void **stream);

/* out[0] = mean_n( -sum_c y_[n,c] * log softmax(y)[n,c] ); output shape (1,).
 * ref: c_runtime_api.h:190-192, gpu_op.cu:261-302, 1256-1287 */
int DLGpuSoftmaxCrossEntropy(const DLArrayHandle input_a, const DLArrayHandle input_b,
                             DLArrayHandle output, void **stream);

/* out = -b * y * log(x) / out = -b * y / x * dout.
 * ref: c_runtime_api.h:544-552, gpu_op.cu:4538-4597 */
int DLGpuCross(const DLArrayHandle x, const DLArrayHandle y, DLArrayHandle output,
               float b, void **stream);
int DLGpuCrossBackward(const DLArrayHandle x, const DLArrayHandle y,
                       const DLArrayHandle doutput, DLArrayHandle output,
                       float b, void **stream);

/* ------------------------------------------------------------------ matmul */

/* C = op(A) * op(B), row-major 2-D, alpha = 1, beta = 0.
 * ref: c_runtime_api.h:152-154, gpu_op.cu:1166-1199 (cublasSgemm) */
int DLGpuMatrixMultiply(const DLArrayHandle matA, bool transposeA,
                        const DLArrayHandle matB, bool transposeB,
                        DLArrayHandle matC, void **handle, void **stream);

/* ---------------------------------------------------------- reduce (bias) */

/* Describe a sum-reduction from input_shapes to output_shapes (same rank;
 * output dims of size 1 are reduced).
 * ref: c_runtime_api.h:218-223, gpu_op.cu:628-807 */
int DLGReduceSumGetCudnnlist(const int *input_shapes, const int *output_shapes,
                             const int sizeofshape, int dataformat,
                             void ***list, void **handle);
/* ref: c_runtime_api.h:224, gpu_op.cu:812-881 (cudnnReduceTensor ADD) */
int DLGpuReduceSum(const DLArrayHandle input, DLArrayHandle output, void ***list,
                   void **handle, int *memorytoSaving, void **stream);

/* ------------------------------------------------------------- convolution */

/* Output shape of a 2-D cross-correlation and its descriptor list.
 * out = 1 + (in + 2*pad - k) / stride, pad = k/2 when padding == 1 else 0.
 * ref: c_runtime_api.h:385-392, gpu_op.cu:2040-2175 */
int DLGpuConvolution2DForwardGetOutShape(const int *input_shapes, const int *filter_shapes,
                                         int *output_shapes, int dataformat, int padding,
                                         const int u, const int v, void ***list);

/* y[n,k,p,q] = sum_{c,r,s} x[n,c,p*u+r-pad,q*v+s-pad] * w[k,c,r,s].
 * ref: c_runtime_api.h:260-264, gpu_op.cu:1952-2038 (cudnnConvolutionForward) */
int DLGpuConvolution2DForward(const DLArrayHandle input, const DLArrayHandle filter,
                              DLArrayHandle output, void ***list, void **handle,
                              int *memorytoSaving, void **stream);

/* dw[k,c,r,s] = sum_{n,p,q} dy[n,k,p,q] * x[n,c,p*u+r-pad,q*v+s-pad] (overwrite).
 * ref: c_runtime_api.h:244-249, gpu_op.cu:1653-1737 (cudnnConvolutionBackwardFilter) */
int DLGpuConvolutionBackwardFilter(const DLArrayHandle input, const DLArrayHandle doutput,
                                   const DLArrayHandle filter, DLArrayHandle dfilter,
                                   void ***list, void **handle, int *memorytoSaving,
                                   void **stream);

/* dx[n,c,h,w] = sum_{k,r,s} dy[n,k,p,q] * w[k,c,r,s], h = p*u+r-pad (overwrite).
 * ref: c_runtime_api.h:251-256, gpu_op.cu:1739-1824 (cudnnConvolutionBackwardData) */
int DLGpuConvolutionBackwardData(const DLArrayHandle input, const DLArrayHandle doutput,
                                 const DLArrayHandle filter, DLArrayHandle dinput,
                                 void ***list, void **handle, int *memorytoSaving,
                                 void **stream);

/* No counterpart in the reference: introspection for benchmarks.  Writes the name
 * of the kernel variant, tile and k-split count that conv `which` (0 forward,
 * 1 grad-data, 2 grad-filter) launches for this descriptor, and its algorithmic
 * flop count 2*N*K*C*R*S*P*Q. */
int DLGpuConvolutionDescribeKernel(void ***list, int which, char *name, int name_len,
                                   double *flops);

/* No counterpart in the reference: measurement aid.  The next convolution entry
 * point called on this host thread records the two HIP events (hipEvent_t, either
 * may be NULL) on its stream immediately before and after its contraction kernel,
 * leaving out the layout and split-sum passes that may accompany it, so a caller
 * can time exactly the kernel a profiler lists under the described symbol. */
int DLGpuConvolutionTimeNextKernel(void *start_event, void *stop_event);

/* No counterpart in the reference: introspection for tests.  A Winograd forward call
 * may keep its transformed input for the grad-filter call of the same step on the same,
 * unmodified input array (any entry point that writes or frees the array drops it).
 * Reports how many such blocks were kept and how many were taken over since the
 * library was loaded, and how many are held right now; any pointer may be NULL. */
int DLGpuKeptByproductCounts(long long *kept_blocks, long long *taken_blocks, int *held_now);

/* ----------------------------------------------------------------- pooling */

/* out = 1 + (in + 2*pad - window) / stride.
 * ref: c_runtime_api.h:407-417, gpu_op.cu:2880-2982 */
int DLGpuPooling2DForwardGetOutShape(const int *input_shapes, int *output_shapes,
                                     int dataformat, int poolingMode,
                                     const int padding_h, const int padding_w,
                                     const int u, const int v,
                                     const int filter_h, const int filter_w, void ***list);

/* ref: c_runtime_api.h:306-309, gpu_op.cu:2839-2878 (cudnnPoolingForward) */
int DLGpuPooling2DForward(const DLArrayHandle input, DLArrayHandle output,
                          void ***list, void **handle, void **stream);

/* max: dy routed to the first maximum (row-major window scan) of each window;
 * mean: dy / (fh*fw) spread over the window.
 * ref: c_runtime_api.h:326-331, gpu_op.cu:2984-3024 (cudnnPoolingBackward) */
int DLGpuPooling2DBackward(const DLArrayHandle input, const DLArrayHandle output,
                           const DLArrayHandle doutput, DLArrayHandle dinput,
                           void ***list, void **handle, void **stream);

/* -------------------------------------------------------------- activation */

/* ref: c_runtime_api.h:370-374, gpu_op.cu:3364-3471 */
int DLGpuActivationGetCudnnlist(const int *input_shapes, const int sizeofshape,
                                int dataformat, int activationMode, void ***list);

/* ref: c_runtime_api.h:350-354, gpu_op.cu:3211-3274 */
int DLGpuActivationForward(const DLArrayHandle input, DLArrayHandle output,
                           int activationMode, void ***list, void **handle, void **stream);

/* relu: dx = x > 0 ? dy : 0; sigmoid: dy*y*(1-y); tanh: dy*(1-y*y);
 * softmax: dx = y * (dy - sum_j dy_j*y_j) per instance.
 * ref: c_runtime_api.h:356-362, gpu_op.cu:3475-3544 */
int DLGpuActivationBackward(const DLArrayHandle input, DLArrayHandle dinput,
                            const DLArrayHandle output, const DLArrayHandle doutput,
                            int activationMode, void ***list, void **handle, void **stream);

/* No counterpart in the reference: introspection for tests and for the benchmark's
 * byte accounting.  Once a ReLU descriptor has seen a backward call, its forward calls
 * also write one bit per element (x > 0) into a block of the library's own, and the
 * backward call of the same step on the same, unmodified x reads dy and the bits
 * instead of dy and x, with the same result bit for bit (any entry point that writes
 * or frees x drops the bits, and the call reads x as before).  Nothing is kept under a
 * device-memory budget or with TINYFLOW_KEEP_RELU_MASK=0 in the environment.
 * Reports how many forward calls kept their bits and how many backward calls used
 * them since the library was loaded; either pointer may be NULL. */
int DLGpuReluMaskCounts(long long *kept, long long *used);

/* ------------------------------------------------------ batch normalisation */

/* gamma = 1, beta = 0, eps = 1e-5, biased variance; no running statistics.
 * Forward allocates the saved mean / inverse-std buffers and stores them in
 * *mean_p / *Variance_p; backward consumes and releases them, so every forward
 * is followed by exactly one backward (or the buffers stay allocated).
 * ref: c_runtime_api.h:485-510, gpu_op.cu:4111-4458 */
int DLGpuBatchNormalizationGetCudnnlist(const int *input_shapes, int sizeofshape,
                                        int dataformat, int batchNormMode,
                                        void **mean_p, void **Variance_p, void ***list);
int DLGpuBatchNormalizationForward(const DLArrayHandle input, DLArrayHandle output,
                                   int batchNormMode, int n, void **mean_p,
                                   void **Variance_p, void ***list, void **handle,
                                   int *memorytoSaving, void **stream);
int DLGpuBatchNormalizationBackward(const DLArrayHandle input, const DLArrayHandle doutput,
                                    DLArrayHandle dinput, int batchNormMode, void **mean_p,
                                    void **Variance_p, void ***list, void **handle,
                                    int *memorytoSaving, void **stream);

/* No counterpart in the reference: batch norm and the ReLU that follows it as one
 * pass (per-activation mode only).  Forward writes max(bn(x), 0); backward takes
 * the gradient of that output and rebuilds the ReLU mask from x and the saved
 * statistics.  Same arguments and statistics protocol as the plain pair above; the
 * results equal those of the two separate ops bit for bit. */
int DLGpuBatchNormalizationReluForward(const DLArrayHandle input, DLArrayHandle output,
                                       int batchNormMode, int n, void **mean_p, void **Variance_p,
                                       void ***list, void **handle, int *memorytoSaving,
                                       void **stream);
int DLGpuBatchNormalizationReluBackward(const DLArrayHandle input, const DLArrayHandle doutput,
                                        DLArrayHandle dinput, int batchNormMode, void **mean_p,
                                        void **Variance_p, void ***list, void **handle,
                                        int *memorytoSaving, void **stream);

/* ----------------------------------------------------- dropout, concatenation */

/* Element-count descriptor that dropout takes in place of the reference's cuDNN
 * tensor descriptor.  ref: c_runtime_api.h:365-368, gpu_op.cu:3276-3362 */
int DLGpuGetInputDescriptor(const int *input_shapes, int sizeofshape, int dataformat,
                            void ***inputd);

/* out = x * keep / (1 - dropout); keep ~ Bernoulli(1 - dropout) drawn from
 * Philox4x32-10 keyed by `seed` (counter = element index / 4).  The bit mask is
 * allocated here, published through *reserveSpace_p and listed in *cudnnlist.
 * ref: c_runtime_api.h:435-443, gpu_op.cu:3547-3640 */
int DLGpuDropoutForward(const DLArrayHandle input, DLArrayHandle output, int dataformat,
                        float dropout, int seed, void **reserveSpace_p, void ***inputd,
                        void ***cudnnlist, void **handle, int *memorytoSaving, void **stream);

/* dinput = doutput * keep / (1 - dropout); consumes the mask and the list.
 * ref: c_runtime_api.h:445-449, gpu_op.cu:3647-3693 */
int DLGpuDropoutBackward(const DLArrayHandle doutput, DLArrayHandle dinput, void **reserveSpace_p,
                         void ***cudnnlist, void **handle, void **stream);

/* Concatenation of two tensors along axis 1 and the two slices that are its
 * gradients.  ref: c_runtime_api.h:226-228, gpu_op.cu:967-1084 */
int DLGpuConcatForward(const DLArrayHandle input1, const DLArrayHandle input2, DLArrayHandle output,
                       void **stream);
int DLGpuConcataBackward(const DLArrayHandle input1, const DLArrayHandle input2,
                         const DLArrayHandle doutput, DLArrayHandle dinput1, void **stream);
int DLGpuConcatbBackward(const DLArrayHandle input1, const DLArrayHandle input2,
                         const DLArrayHandle doutput, DLArrayHandle dinput2, void **stream);

/* --------------------------------------------------------------- optimizers */

/* w[i] -= lr * g[i] in place.  ref: c_runtime_api.h:539-543, gpu_op.cu:4600-4625 */
int DLGpuSgdUpdate(DLArrayHandle output, const DLArrayHandle m, float b, void **stream);

/* Fused multi-tensor SGD: one launch over the flattened parameter index space.
 * Tables are built once by the two *CudaPointer calls.
 * ref: c_runtime_api.h:534-537, 555-562, gpu_op.cu:4628-4672, 4824-4863 */
int DLGpuGetIndextoVaribaleNumberCudaPointer(int *index_to_number, int *prefix,
                                             int count, void ***result);
int DLGpuGetN2CudaPointer(void **output, void **g, int number, void ****result);
int DLGpuSgd_o(void ****n2list, const void ***indexlist, const int count,
               const float learning_rate);

/* Adam, two-kernel form: m,v update then parameter update.
 * ref: c_runtime_api.h:512-522, gpu_op.cu:4461-4533 */
int DLGpuAdam_mv(DLArrayHandle m, DLArrayHandle v, const DLArrayHandle g,
                 float b1, float b2, void **stream);
int DLGpuAdam(DLArrayHandle output, const DLArrayHandle m, const DLArrayHandle v,
              float b1t, float b2t, float e, float learning_rate, void **stream);

/* Fused multi-tensor Adam: one launch and one pass over (w, m, v, g) of every
 * parameter tensor, addressed through the same index tables as DLGpuSgd_o.
 * ref: c_runtime_api.h:524-532, 560, gpu_op.cu:4674-4700, 4745-4781, 4865-4893 */
int DLGpuGetN4CudaPointer(void **output, void **m, void **v, void **g, int number, void ****result);
int DLGpuAdam_o(void ****n4list, const void ***indexlist, const int count,
                const float b1, const float b2, const float b1t, const float b2t,
                const float e, const float learning_rate);

/* No counterpart in the reference, which allocates the tables above with cudaMalloc
 * and never gives them back (gpu_op.cu:4628-4700): release calls for the index tables
 * and for the 2 or 4 pointer tables (device blocks and host cell; the cell is set to
 * NULL), and index tables for whole tensors laid end to end built from the tensors'
 * element counts instead of from per-parameter arrays (*count receives the total to
 * pass to DLGpuSgd_o / DLGpuAdam_o).  The tables come from the library's device pool,
 * so DLGpuGetDeviceMemoryStats and a memory limit see them. */
int DLGpuGetTensorRunsCudaPointer(const int64_t *sizes, int n_tensors, int *count, void ***result);
int DLGpuFreeIndexCudaPointer(void ***indexlist);
int DLGpuFreeNCudaPointer(void ****list, int n_tables);

#ifdef __cplusplus
}
#endif
#endif /* TINYFLOW_AMD_C_RUNTIME_API_H_ */
