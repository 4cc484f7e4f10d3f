"""One thin wrapper per C entry point of libc_runtime_api.so.

Same function names, argument order and string -> enum maps as the reference
binding ``pycode/tinyflow/gpu_op.py`` for the entry points of the training hot
path, so graph code written against the reference calls through unchanged.
Ops that can run out of device scratch return the byte count wanted (0 = ok),
as the reference wrappers do.
"""
import ctypes

import numpy as np

from ._base import _LIB, c_array, check_call
from . import ndarray as _nd

_DATAFORMAT = {"NCHW": 0, "NHWC": 1}            # reference gpu_op.py:437-442
_PADDING = {"SAME": 1, "VALID": 0}              # reference gpu_op.py:443-448
_POOLING = {"max": 0, "mean": 1}                # reference gpu_op.py:610-615
_ACTIVATION = {"sigmoid": 0, "relu": 1, "tanh": 2, "softmax": 3}  # gpu_op.py:501-510
_BATCHNORM = {"pre_activation": 0, "spatial": 1}                  # gpu_op.py:778-783


def _enum(table, key):
    assert key in table, "unknown option %r (expected one of %s)" % (key, sorted(table))
    return table[key]


def _cell(depth):
    """A chain of ``depth`` pointers ending at an int: the out-parameter cells the
    C side writes handles, streams and descriptor lists into."""
    cell = ctypes.c_int(0)
    for _ in range(depth):
        cell = ctypes.pointer(cell)
    return cell


def _nd_args(*arrays):
    for a in arrays:
        assert isinstance(a, _nd.NDArray)


# ------------------------------------------------------------ streams / handles

def create_cudaStream():
    stream = _cell(2)
    check_call(_LIB.DLGpuCreatecudaStream(stream))
    return stream


def destroy_cudaStream(cudaStream):
    check_call(_LIB.DLGpuDestroycudaStream(cudaStream))


def create_cudnnHandle(cudaStream):
    handle = _cell(2)
    check_call(_LIB.DLGpuCreatecudnnHandle(handle, cudaStream))
    return handle


def destroy_cudnnHandle(cudnnHandle):
    check_call(_LIB.DLGpuDestroycudnnHandle(cudnnHandle))


def create_cublasHandle(cudaStream):
    handle = _cell(2)
    check_call(_LIB.DLGpuCreatecublasHandle(handle, cudaStream))
    return handle


def destroy_cublasHandle(cublasHandle):
    check_call(_LIB.DLGpuDestroycublasHandle(cublasHandle))


# ------------------------------------------------------------------ elementwise

def array_set(arr, value, cudaStream):
    _nd_args(arr)
    check_call(_LIB.DLGpuArraySet(arr.handle, ctypes.c_float(value), cudaStream))


def broadcast_to(in_arr, out_arr, type, cudaStream):
    _nd_args(in_arr, out_arr)
    if type == "NHWC":
        check_call(_LIB.DLGpuBroadcastTo0(in_arr.handle, out_arr.handle, cudaStream))
    elif type == "NCHW":
        check_call(_LIB.DLGpuBroadcastTo1(in_arr.handle, out_arr.handle, cudaStream))
    else:
        assert 0, type


def broadcast_to_backward(in_arr, out_arr, type):
    _nd_args(in_arr, out_arr)
    if type == "NHWC":
        check_call(_LIB.DLGpuBroadcastToBackward0(in_arr.handle, out_arr.handle))
    elif type == "NCHW":
        check_call(_LIB.DLGpuBroadcastToBackward1(in_arr.handle, out_arr.handle))
    else:
        assert 0, type


def reduce_sum_axis_zero(in_arr, out_arr):
    _nd_args(in_arr, out_arr)
    check_call(_LIB.DLGpuReduceSumAxisZero(in_arr.handle, out_arr.handle))


def reduce_sum_axis_zero_no_alloc(in_arr, out_arr, cudaStream):
    """reduce_sum_axis_zero for callers that cannot allocate: partial sums go to a
    device array built into the library (extension: no counterpart in the reference)"""
    _nd_args(in_arr, out_arr)
    check_call(_LIB.DLGpuReduceSumAxisZeroNoAlloc(in_arr.handle, out_arr.handle, cudaStream))


def matrix_elementwise_add(matA, matB, matC, cudaStream):
    _nd_args(matA, matB, matC)
    check_call(_LIB.DLGpuMatrixElementwiseAdd(matA.handle, matB.handle, matC.handle, cudaStream))


def matrix_elementwise_add_relu(matA, matB, matC, cudaStream):
    """max(matA + matB, 0) in one pass (extension: no counterpart in the reference)"""
    _nd_args(matA, matB, matC)
    check_call(_LIB.DLGpuMatrixElementwiseAddRelu(matA.handle, matB.handle, matC.handle, cudaStream))


def matrix_elementwise_add_by_const(in_mat, val, out_mat, cudaStream):
    _nd_args(in_mat, out_mat)
    check_call(_LIB.DLGpuMatrixElementwiseAddByConst(in_mat.handle, ctypes.c_float(val),
                                                     out_mat.handle, cudaStream))


def matrix_elementwise_multiply(matA, matB, matC, cudaStream):
    _nd_args(matA, matB, matC)
    check_call(_LIB.DLGpuMatrixElementwiseMultiply(matA.handle, matB.handle, matC.handle, cudaStream))


def matrix_elementwise_multiply_by_const(in_mat, val, out_mat, cudaStream):
    _nd_args(in_mat, out_mat)
    check_call(_LIB.DLGpuMatrixMultiplyByConst(in_mat.handle, ctypes.c_float(val), out_mat.handle,
                                               cudaStream))


def matrix_multiply(matA, transA, matB, transB, matC, cublasHandle, cudaStream):
    _nd_args(matA, matB, matC)
    check_call(_LIB.DLGpuMatrixMultiply(matA.handle, bool(transA), matB.handle, bool(transB),
                                        matC.handle, cublasHandle, cudaStream))


def relu(in_arr, out_arr):
    _nd_args(in_arr, out_arr)
    check_call(_LIB.DLGpuRelu(in_arr.handle, out_arr.handle))


def relu_gradient(in_arr, in_grad_arr, out_arr):
    _nd_args(in_arr, in_grad_arr, out_arr)
    check_call(_LIB.DLGpuReluGradient(in_arr.handle, in_grad_arr.handle, out_arr.handle))


def softmax(in_arr, out_arr, cudaStream):
    _nd_args(in_arr, out_arr)
    check_call(_LIB.DLGpuSoftmax(in_arr.handle, out_arr.handle, cudaStream))


def softmax_cross_entropy(in_arr_a, in_arr_b, out_arr, cudaStream):
    _nd_args(in_arr_a, in_arr_b, out_arr)
    check_call(_LIB.DLGpuSoftmaxCrossEntropy(in_arr_a.handle, in_arr_b.handle, out_arr.handle,
                                             cudaStream))


def cross(x, y, output, mean, cudaStream):
    _nd_args(x, y, output)
    check_call(_LIB.DLGpuCross(x.handle, y.handle, output.handle, ctypes.c_float(mean), cudaStream))


def cross_backward(x, y, doutput, output, mean, cudaStream):
    _nd_args(x, y, doutput, output)
    check_call(_LIB.DLGpuCrossBackward(x.handle, y.handle, doutput.handle, output.handle,
                                       ctypes.c_float(mean), cudaStream))


# ---------------------------------------------------------------- reduce (bias)

def reduce_sum_get_real_shape(input_shapes, output_shapes, dataformat):
    """Rank-matched (input, output) shapes for a bias-gradient reduction
    (reference gpu_op.py:83-119): NCHW keeps the channel axis 1, NHWC the last axis."""
    assert len(output_shapes) == 1
    n = len(input_shapes)
    if dataformat == "NCHW":
        assert input_shapes[1] == output_shapes[0] and 3 <= n <= 5
        return tuple(input_shapes), (1, output_shapes[0]) + (1,) * (n - 2)
    if dataformat == "NHWC":
        if n == 1:
            assert output_shapes[0] == 1
            return (1, 1, input_shapes[0]), (1, 1, 1)
        if n == 2:
            if output_shapes[0] != 1:
                assert input_shapes[1] == output_shapes[0]
            return (1, input_shapes[0], input_shapes[1]), (1, 1, output_shapes[0])
        assert 3 <= n <= 5 and input_shapes[-1] == output_shapes[0]
        return tuple(input_shapes), (1,) * (n - 1) + (output_shapes[0],)
    assert 0, dataformat


def reduce_sum_get_cudnnlist(input_shapes, output_shapes, dataformat, cudnnHandle):
    fmt = _enum(_DATAFORMAT, dataformat)
    cudnnlist = _cell(3)
    check_call(_LIB.DLGReduceSumGetCudnnlist(c_array(ctypes.c_int, input_shapes),
                                             c_array(ctypes.c_int, output_shapes),
                                             len(input_shapes), fmt, cudnnlist, cudnnHandle))
    return cudnnlist


def reduce_sum_new(in_arr, out_arr, cudnnlist, cudnnHandle, cudaStream):
    _nd_args(in_arr, out_arr)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuReduceSum(in_arr.handle, out_arr.handle, cudnnlist, cudnnHandle,
                                   ctypes.byref(wanted), cudaStream))
    return wanted.value


# ------------------------------------------------------------------ convolution

def convolution_2d_forward_get_out_shape(input_shapes, filter_shapes, dataformat, padding, u, v):
    fmt = _enum(_DATAFORMAT, dataformat)
    pad = _enum(_PADDING, padding)
    assert len(input_shapes) == 4 and len(filter_shapes) == 4
    c_out = c_array(ctypes.c_int, (0, 0, 0, 0))
    cudnnlist = _cell(3)
    check_call(_LIB.DLGpuConvolution2DForwardGetOutShape(
        c_array(ctypes.c_int, input_shapes), c_array(ctypes.c_int, filter_shapes), c_out, fmt, pad,
        u, v, cudnnlist))
    return tuple(c_out), cudnnlist


def convolution_2d_forward(in_arr, in_filter, out_arr, cudnnlist, cudnnHandle, cudaStream):
    _nd_args(in_arr, in_filter, out_arr)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuConvolution2DForward(in_arr.handle, in_filter.handle, out_arr.handle,
                                              cudnnlist, cudnnHandle, ctypes.byref(wanted), cudaStream))
    return wanted.value


def convolution_backward_filter(in_arr, dout_arr, in_filter, in_dfilter, cudnnlist, cudnnHandle,
                                cudaStream):
    _nd_args(in_arr, dout_arr, in_filter, in_dfilter)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuConvolutionBackwardFilter(in_arr.handle, dout_arr.handle, in_filter.handle,
                                                   in_dfilter.handle, cudnnlist, cudnnHandle,
                                                   ctypes.byref(wanted), cudaStream))
    return wanted.value


def convolution_backward_data(in_arr, dout_arr, in_filter, dinput_arr, cudnnlist, cudnnHandle,
                              cudaStream):
    _nd_args(in_arr, dout_arr, in_filter, dinput_arr)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuConvolutionBackwardData(in_arr.handle, dout_arr.handle, in_filter.handle,
                                                 dinput_arr.handle, cudnnlist, cudnnHandle,
                                                 ctypes.byref(wanted), cudaStream))
    return wanted.value


# ---------------------------------------------------------------------- pooling

def pooling_2d_forward_get_out_shape(input_shapes, dataformat, poolingMode, padding_h, padding_w,
                                     u, v, filter_h, filter_w):
    fmt = _enum(_DATAFORMAT, dataformat)
    mode = _enum(_POOLING, poolingMode)
    assert len(input_shapes) == 4
    c_out = c_array(ctypes.c_int, (0, 0, 0, 0))
    cudnnlist = _cell(3)
    check_call(_LIB.DLGpuPooling2DForwardGetOutShape(
        c_array(ctypes.c_int, input_shapes), c_out, fmt, mode, padding_h, padding_w, u, v,
        filter_h, filter_w, cudnnlist))
    return tuple(c_out), cudnnlist


def pooling_2d_forward(in_arr, out_arr, cudnnlist, cudnnHandle, cudaStream):
    _nd_args(in_arr, out_arr)
    check_call(_LIB.DLGpuPooling2DForward(in_arr.handle, out_arr.handle, cudnnlist, cudnnHandle,
                                          cudaStream))


def pooling_2d_backward(in_arr, out_arr, dout_arr, din_arr, cudnnlist, cudnnHandle, cudaStream):
    _nd_args(in_arr, out_arr, dout_arr, din_arr)
    check_call(_LIB.DLGpuPooling2DBackward(in_arr.handle, out_arr.handle, dout_arr.handle,
                                           din_arr.handle, cudnnlist, cudnnHandle, cudaStream))


# ------------------------------------------------------------------- activation

def activation_get_cudnnlist(input_shapes, dataformat, activationMode):
    fmt = _enum(_DATAFORMAT, dataformat)
    mode = _enum(_ACTIVATION, activationMode)
    cudnnlist = _cell(3)
    check_call(_LIB.DLGpuActivationGetCudnnlist(c_array(ctypes.c_int, input_shapes),
                                                len(input_shapes), fmt, mode, cudnnlist))
    return cudnnlist


def activation_forward(input, output, activationMode, cudnnlist, cudnnHandle, cudaStream):
    _nd_args(input, output)
    mode = _enum(_ACTIVATION, activationMode)
    check_call(_LIB.DLGpuActivationForward(input.handle, output.handle, mode, cudnnlist, cudnnHandle,
                                           cudaStream))


def activation_backward(input, dinput, output, doutput, activationMode, cudnnlist, cudnnHandle,
                        cudaStream):
    _nd_args(input, dinput, output, doutput)
    mode = _enum(_ACTIVATION, activationMode)
    check_call(_LIB.DLGpuActivationBackward(input.handle, dinput.handle, output.handle,
                                            doutput.handle, mode, cudnnlist, cudnnHandle, cudaStream))


# ---------------------------------------------------------- batch normalisation

def bn_get_cudnnlist(input_shapes, dataformat, batchNormMode):
    fmt = _enum(_DATAFORMAT, dataformat)
    mode = _enum(_BATCHNORM, batchNormMode)
    mean_p = _cell(2)
    var_p = _cell(2)
    cudnnlist = _cell(3)
    check_call(_LIB.DLGpuBatchNormalizationGetCudnnlist(c_array(ctypes.c_int, input_shapes),
                                                        len(input_shapes), fmt, mode, mean_p, var_p,
                                                        cudnnlist))
    return mean_p, var_p, cudnnlist


def bn_forward(input, output, batchNormMode, n, mean_p, var_p, cudnnlist, cudnnHandle, cudaStream):
    _nd_args(input, output)
    mode = _enum(_BATCHNORM, batchNormMode)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuBatchNormalizationForward(input.handle, output.handle, mode, n, mean_p, var_p,
                                                   cudnnlist, cudnnHandle, ctypes.byref(wanted),
                                                   cudaStream))
    return wanted.value


def bn_backward(input, doutput, dinput, batchNormMode, mean_p, var_p, cudnnlist, cudnnHandle,
                cudaStream):
    _nd_args(input, doutput, dinput)
    mode = _enum(_BATCHNORM, batchNormMode)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuBatchNormalizationBackward(input.handle, doutput.handle, dinput.handle, mode,
                                                    mean_p, var_p, cudnnlist, cudnnHandle,
                                                    ctypes.byref(wanted), cudaStream))
    return wanted.value


def bn_relu_forward(input, output, batchNormMode, n, mean_p, var_p, cudnnlist, cudnnHandle, cudaStream):
    """max(bn(x), 0) in one pass (extension: no counterpart in the reference); same
    arguments as ``bn_forward``."""
    _nd_args(input, output)
    mode = _enum(_BATCHNORM, batchNormMode)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuBatchNormalizationReluForward(input.handle, output.handle, mode, n, mean_p, var_p,
                                                       cudnnlist, cudnnHandle, ctypes.byref(wanted), cudaStream))
    return wanted.value


def bn_relu_backward(input, doutput, dinput, batchNormMode, mean_p, var_p, cudnnlist, cudnnHandle, cudaStream):
    """Gradient of ``bn_relu_forward`` with respect to its input (extension); ``doutput``
    is the gradient of the ReLU output."""
    _nd_args(input, doutput, dinput)
    mode = _enum(_BATCHNORM, batchNormMode)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuBatchNormalizationReluBackward(input.handle, doutput.handle, dinput.handle, mode,
                                                        mean_p, var_p, cudnnlist, cudnnHandle,
                                                        ctypes.byref(wanted), cudaStream))
    return wanted.value


# ------------------------------------------------------------------- optimizers

def sgd_update(output, g, learning_rate, cudaStream):
    _nd_args(output, g)
    check_call(_LIB.DLGpuSgdUpdate(output.handle, g.handle, ctypes.c_float(learning_rate), cudaStream))


def adam_mv(m, v, g, b1, b2, cudaStream):
    _nd_args(m, v, g)
    check_call(_LIB.DLGpuAdam_mv(m.handle, v.handle, g.handle, ctypes.c_float(b1), ctypes.c_float(b2),
                                 cudaStream))


def adam_compute(output, m, v, b1t, b2t, e, learning_rate, cudaStream):
    _nd_args(output, m, v)
    check_call(_LIB.DLGpuAdam(output.handle, m.handle, v.handle, ctypes.c_float(b1t),
                              ctypes.c_float(b2t), ctypes.c_float(e), ctypes.c_float(learning_rate),
                              cudaStream))


def _int_table(values):
    """C int array for a list, or the buffer of a numpy array (int32 copy if needed)."""
    if isinstance(values, np.ndarray):
        arr = np.ascontiguousarray(values, dtype=np.int32)
        return arr, arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int))
    arr = c_array(ctypes.c_int, values)
    return arr, arr


def get_index_to_VaribaleNumber_cuda_pointer(index_to_Variable, prefix_list, index_count):
    """Device tables index -> (tensor number, offset inside the tensor) for the fused
    optimizers; the two tables may be lists (as the reference passes them) or numpy arrays."""
    result = _cell(3)
    keep_a, number = _int_table(index_to_Variable)
    keep_b, offset = _int_table(prefix_list)
    check_call(_LIB.DLGpuGetIndextoVaribaleNumberCudaPointer(number, offset, ctypes.c_int(index_count), result))
    del keep_a, keep_b
    return result


def get_tensor_runs_cuda_pointer(sizes):
    """Index tables of the fused optimizers for whole tensors of ``sizes`` elements
    laid end to end (no counterpart in the reference, which builds per-parameter
    lists: gpu_op.py:887-945).  Returns (tables, parameter count)."""
    result = _cell(3)
    count = ctypes.c_int(0)
    arr = (ctypes.c_int64 * len(sizes))(*[int(n) for n in sizes])
    check_call(_LIB.DLGpuGetTensorRunsCudaPointer(arr, ctypes.c_int(len(sizes)), ctypes.byref(count), result))
    return result, count.value


def free_index_cuda_pointer(tables):
    """Releases the tables of ``get_index_to_VaribaleNumber_cuda_pointer`` /
    ``get_tensor_runs_cuda_pointer`` (no counterpart in the reference)."""
    check_call(_LIB.DLGpuFreeIndexCudaPointer(tables))


def free_n_cuda_pointer(pointers, n_tables):
    """Releases the pointer tables of ``get_n2_cuda_pointer`` (n_tables = 2) or
    ``get_n4_cuda_pointer`` (4) (no counterpart in the reference)."""
    check_call(_LIB.DLGpuFreeNCudaPointer(pointers, ctypes.c_int(n_tables)))


def get_n2_cuda_pointer(output, g, number):
    result = _cell(4)
    check_call(_LIB.DLGpuGetN2CudaPointer(c_array(ctypes.c_void_p, output), c_array(ctypes.c_void_p, g),
                                          ctypes.c_int(number), result))
    return result


def get_n4_cuda_pointer(output, m, v, g, number):
    result = _cell(4)
    check_call(_LIB.DLGpuGetN4CudaPointer(c_array(ctypes.c_void_p, output), c_array(ctypes.c_void_p, m),
                                          c_array(ctypes.c_void_p, v), c_array(ctypes.c_void_p, g),
                                          ctypes.c_int(number), result))
    return result


def sgd_compute_o(n2list, indexinfolist, count, learning_rate):
    check_call(_LIB.DLGpuSgd_o(n2list, indexinfolist, ctypes.c_int(count), ctypes.c_float(learning_rate)))


def adam_compute_o(n4list, indexinfolist, count, b1, b2, b1t, b2t, e, learning_rate):
    check_call(_LIB.DLGpuAdam_o(n4list, indexinfolist, ctypes.c_int(count), ctypes.c_float(b1),
                                ctypes.c_float(b2), ctypes.c_float(b1t), ctypes.c_float(b2t),
                                ctypes.c_float(e), ctypes.c_float(learning_rate)))


def getInt(intp):
    return _LIB.getInt(intp)


def testPcie():
    check_call(_LIB.testPcie())


# ------------------------------------------------------- dropout, concatenation

def get_input_descriptor(input_shapes, dataformat):
    """reference gpu_op.py:557-570"""
    fmt = _enum(_DATAFORMAT, dataformat)
    inputd = _cell(3)
    check_call(_LIB.DLGpuGetInputDescriptor(c_array(ctypes.c_int, input_shapes), len(input_shapes), fmt, inputd))
    return inputd


def dropout_forward(input, output, dataformat, dropout, seed, inputd, cudnnHandle, cudaStream):
    """Returns (reserveSpace_p, cudnnlist, bytes wanted); reference gpu_op.py:657-685."""
    _nd_args(input, output)
    fmt = _enum(_DATAFORMAT, dataformat)
    assert seed >= 0
    reserveSpace_p = _cell(2)
    cudnnlist = _cell(3)
    wanted = ctypes.c_int(0)
    check_call(_LIB.DLGpuDropoutForward(input.handle, output.handle, fmt, ctypes.c_float(dropout),
                                        ctypes.c_int(seed), reserveSpace_p, inputd, cudnnlist, cudnnHandle,
                                        ctypes.byref(wanted), cudaStream))
    return reserveSpace_p, cudnnlist, wanted.value


def dropout_backward(doutput, dinput, reserveSpace_p, cudnnlist, cudnnHandle, cudaStream):
    """reference gpu_op.py:688-692"""
    _nd_args(doutput, dinput)
    check_call(_LIB.DLGpuDropoutBackward(doutput.handle, dinput.handle, reserveSpace_p, cudnnlist,
                                         cudnnHandle, cudaStream))


def concat_forward(in_arr_a, in_arr_b, out_arr, cudaStream):
    """reference gpu_op.py:746-751"""
    _nd_args(in_arr_a, in_arr_b, out_arr)
    check_call(_LIB.DLGpuConcatForward(in_arr_a.handle, in_arr_b.handle, out_arr.handle, cudaStream))


def concat_a_backward(in_arr_a, in_arr_b, out_arr, din_arr_a, cudaStream):
    """reference gpu_op.py:752-758; ``out_arr`` is the gradient of the concatenation"""
    _nd_args(in_arr_a, in_arr_b, out_arr, din_arr_a)
    check_call(_LIB.DLGpuConcataBackward(in_arr_a.handle, in_arr_b.handle, out_arr.handle, din_arr_a.handle,
                                         cudaStream))


def concat_b_backward(in_arr_a, in_arr_b, out_arr, din_arr_b, cudaStream):
    """reference gpu_op.py:760-768"""
    _nd_args(in_arr_a, in_arr_b, out_arr, din_arr_b)
    check_call(_LIB.DLGpuConcatbBackward(in_arr_a.handle, in_arr_b.handle, out_arr.handle, din_arr_b.handle,
                                         cudaStream))


# --------------------------------------------------- allocator budget (extension)

def set_device_memory_limit(nbytes):
    """Budget of the device allocator in bytes (0 or None: unlimited).  No
    counterpart in the reference; lets a 16 GB card be imitated on a larger one."""
    check_call(_LIB.DLGpuSetDeviceMemoryLimit(ctypes.c_int64(int(nbytes or 0))))


def relu_mask_counts():
    """(kept, used): ReLU forward calls that kept their sign bits for the backward call, and
    backward calls that read those bits instead of x, since the library was loaded."""
    kept, used = ctypes.c_longlong(0), ctypes.c_longlong(0)
    check_call(_LIB.DLGpuReluMaskCounts(ctypes.byref(kept), ctypes.byref(used)))
    return kept.value, used.value


def device_memory_stats(reset_peak=False):
    """(reserved, in_use, peak_in_use) bytes of the device allocator."""
    vals = [ctypes.c_int64(0) for _ in range(3)]
    check_call(_LIB.DLGpuGetDeviceMemoryStats(ctypes.byref(vals[0]), ctypes.byref(vals[1]),
                                              ctypes.byref(vals[2]), int(bool(reset_peak))))
    return tuple(v.value for v in vals)
