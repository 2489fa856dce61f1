"""One thin Python function per operator symbol of the C ABI.

Mirror of the reference's python/athena/gpu_links/*.py: same function names, argument
order and defaults (cited per function), so a graph op written against the reference's
`gpu_links` runs unchanged on this library.  Return values of the C calls are checked
here (the reference's wrappers ignore them).
"""
import ctypes

from . import ndarray as _nd
from ._base import _LIB, check_call

__all__ = [
    "array_set", "matrix_elementwise_add", "matrix_elementwise_add_by_const",
    "matrix_elementwise_multiply", "matrix_elementwise_multiply_by_const", "array_reshape",
    "relu", "relu_gradient", "matrix_multiply", "softmax", "softmax_cross_entropy",
    "softmax_cross_entropy_gradient", "CuDNN_conv2d", "CuDNN_conv2d_gradient_of_data",
    "CuDNN_conv2d_gradient_of_filter", "conv2d", "conv2d_gradient_of_data",
    "conv2d_gradient_of_filter", "CuDNN_Batch_Normalization", "CuDNN_Batch_Normalization_gradient",
    "max_pooling2d", "max_pooling2d_gradient", "CuDNN_max_pooling2d", "CuDNN_max_pooling2d_gradient",
    "concat", "concat_gradient", "matrix_slice", "matrix_slice_gradient",
    "sgd_update", "momentum_update", "adagrad_update", "adam_update",
    "average_pooling2d", "average_pooling2d_gradient", "CuDNN_average_pooling2d",
    "CuDNN_average_pooling2d_gradient", "broadcast_to", "reduce_sum_axis_zero", "_reduce_sum_axis_zero",
    "conv2d_broadcast_to", "conv2d_reduce_sum", "broadcast_shape", "reduce_sum", "pad", "pad_gradient",
    "matrix_transpose", "batch_matrix_multiply", "one_hot", "where", "embedding_lookup",
    "embedding_lookup_gradient", "matrix_elementwise_divide", "matrix_elementwise_divide_const",
    "matrix_opposite", "matrix_sqrt", "matrix_rsqrt", "tanh", "sigmoid",
    "batch_norm_relu", "batch_norm_relu_gradient", "conv2d_batch_norm_stats", "batch_norm_from_stats",
    "optimizer_update_multi",
    "CuDNN_Dropout", "CuDNN_Dropout_gradient", "CuSparse_Csrmv", "CuSparse_Csrmm",
]


def _h(arr):
    assert isinstance(arr, _nd.NDArray)
    return arr.handle


def _s(stream):
    return stream.handle if stream else None


def _p(profiler):
    return ctypes.byref(profiler) if profiler else None


# ---- graph-closure ops (gpu_links/ArraySetLink.py:8, AddElewiseLink.py, AddConstLink.py,
#      MultiplyElewiseLink.py, MultiplyConstLink.py, ReshapeLink.py:8) ----
def array_set(arr, value, stream=None, profiler=None):
    check_call(_LIB.DLGpuArraySet(_h(arr), ctypes.c_float(value), _s(stream), _p(profiler)))


def matrix_elementwise_add(matA, matB, matC, stream=None, profiler=None):
    check_call(_LIB.DLGpuMatrixElementwiseAdd(_h(matA), _h(matB), _h(matC), _s(stream), _p(profiler)))


def matrix_elementwise_add_by_const(in_mat, val, out_mat, stream=None, profiler=None):
    check_call(_LIB.DLGpuMatrixElementwiseAddByConst(_h(in_mat), ctypes.c_float(val), _h(out_mat),
                                                     _s(stream), _p(profiler)))


def matrix_elementwise_multiply(matA, matB, matC, stream=None, profiler=None):
    check_call(_LIB.DLGpuMatrixElementwiseMultiply(_h(matA), _h(matB), _h(matC), _s(stream), _p(profiler)))


def matrix_elementwise_multiply_by_const(in_mat, val, out_mat, stream=None, profiler=None):
    check_call(_LIB.DLGpuMatrixMultiplyByConst(_h(in_mat), ctypes.c_float(val), _h(out_mat),
                                               _s(stream), _p(profiler)))


def array_reshape(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuReshape(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


# ---- Relu (gpu_links/ReluLink.py:8,14) ----
def relu(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuRelu(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def relu_gradient(in_arr, in_grad_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuReluGradient(_h(in_arr), _h(in_grad_arr), _h(out_arr), _s(stream), _p(profiler)))


# ---- MatMul (gpu_links/MatrixMultLink.py:8) ----
def matrix_multiply(matA, transA, matB, transB, matC, stream=None, profiler=None):
    check_call(_LIB.DLGpuMatrixMultiply(_h(matA), ctypes.c_bool(bool(transA)), _h(matB),
                                        ctypes.c_bool(bool(transB)), _h(matC), _s(stream), _p(profiler)))


# ---- Softmax / CE (gpu_links/SoftmaxLink.py, SoftmaxCrossEntropyLink.py:8,17) ----
def softmax(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuSoftmax(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def softmax_cross_entropy(in_arr_a, in_arr_b, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuSoftmaxCrossEntropy(_h(in_arr_a), _h(in_arr_b), _h(out_arr), _s(stream), _p(profiler)))


def softmax_cross_entropy_no_alloc(in_arr_a, in_arr_b, out_arr, stream=None):
    """The same loss from the entry point that allocates no device memory (no counterpart in the
    reference's gpu_links): at most 262144 rows, per-row losses in a fixed array of the library."""
    check_call(_LIB.TSplit_SoftmaxCrossEntropyNoAlloc(_h(in_arr_a), _h(in_arr_b), _h(out_arr), _s(stream)))


def softmax_cross_entropy_gradient(in_arr_a, in_arr_b, in_arr_c, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuSoftmaxCrossEntropy_Gradient(_h(in_arr_a), _h(in_arr_b), _h(in_arr_c), _h(out_arr),
                                                      _s(stream), _p(profiler)))


# ---- Conv2d (gpu_links/CudnnConv2d.py:8,21,33; gpu_links/Conv2dLink.py:8,24,35) ----
def CuDNN_conv2d(in_arr_x, in_arr_f, out_arr, padding=0, padding2=None, stride=1, stream=None, profiler=None):
    pad2 = padding if padding2 is None else padding2
    check_call(_LIB.CuDNN_DLGpuConv2d(_h(in_arr_x), _h(in_arr_f), _h(out_arr), int(padding), int(pad2),
                                      int(stride), _s(stream), _p(profiler)))


def CuDNN_conv2d_gradient_of_filter(in_arr_x, in_gradient_y, out_gradient_f, padding=0, padding2=None,
                                    stride=1, stream=None, profiler=None):
    pad2 = padding if padding2 is None else padding2
    check_call(_LIB.CuDNN_DLGpuConv2d_Gradient_of_Filter(_h(in_arr_x), _h(in_gradient_y), _h(out_gradient_f),
                                                         int(padding), int(pad2), int(stride),
                                                         _s(stream), _p(profiler)))


def CuDNN_conv2d_gradient_of_data(in_arr_f, in_gradient_y, out_gradient_x, padding=0, padding2=None,
                                  stride=1, stream=None, profiler=None):
    pad2 = padding if padding2 is None else padding2
    check_call(_LIB.CuDNN_DLGpuConv2d_Gradient_of_Data(_h(in_arr_f), _h(in_gradient_y), _h(out_gradient_x),
                                                       int(padding), int(pad2), int(stride),
                                                       _s(stream), _p(profiler)))


def conv2d(in_arr_x, in_arr_f, out_arr, workspace_arr, padding=0, stride=1, stream=None, profiler=None):
    check_call(_LIB.DLGpuConv2d(_h(in_arr_x), _h(in_arr_f), _h(out_arr), _h(workspace_arr),
                                int(padding), int(stride), _s(stream), _p(profiler)))


def conv2d_gradient_of_filter(in_arr_x, in_gradient_y, out_gradient_f, workspace_im2col,
                              workspace_batch_filter, padding=0, stride=1, stream=None, profiler=None):
    check_call(_LIB.DLGpuConv2d_Gradient_of_Filter(_h(in_arr_x), _h(in_gradient_y), _h(out_gradient_f),
                                                   _h(workspace_im2col), _h(workspace_batch_filter),
                                                   int(padding), int(stride), _s(stream), _p(profiler)))


def conv2d_gradient_of_data(in_arr_f, in_gradient_y, out_gradient_x, workspace_im2col, padding=0,
                            stride=1, stream=None, profiler=None):
    check_call(_LIB.DLGpuConv2d_Gradient_of_Data(_h(in_arr_f), _h(in_gradient_y), _h(out_gradient_x),
                                                 _h(workspace_im2col), int(padding), int(stride),
                                                 _s(stream), _p(profiler)))


# ---- BatchNorm (gpu_links/CudnnBnLink.py:8,17) ----
def CuDNN_Batch_Normalization(in_arr, bn_scale_arr, bn_bias_arr, out_arr, save_mean, save_var,
                              momentum=0.99, eps=0.001, stream=None, profiler=None):
    check_call(_LIB.CuDNN_DLGpuBatch_Normalization(
        _h(in_arr), _h(bn_scale_arr), _h(bn_bias_arr), _h(out_arr), ctypes.c_float(momentum),
        ctypes.c_float(eps), save_mean.handle if save_mean else None,
        save_var.handle if save_var else None, _s(stream), _p(profiler)))


def CuDNN_Batch_Normalization_gradient(in_gradient_y, in_arr_x, in_bn_scale, out_gradient_x,
                                       out_gradient_bn_scale, out_gradient_bn_bias, saved_mean, saved_var,
                                       eps=0.001, stream=None, profiler=None):
    check_call(_LIB.CuDNN_DLGpuBatch_Normalization_gradient(
        _h(in_gradient_y), _h(in_arr_x), _h(in_bn_scale), _h(out_gradient_x), _h(out_gradient_bn_scale),
        _h(out_gradient_bn_bias), ctypes.c_float(eps), saved_mean.handle if saved_mean else None,
        saved_var.handle if saved_var else None, _s(stream), _p(profiler)))


# ---- MaxPool (gpu_links/MaxPoolLink.py:8,15; gpu_links/CudnnMaxPoolLink.py:8,15) ----
def max_pooling2d(in_arr, kernel_H, kernel_W, pooled_layer, padding=0, stride=1, stream=None, profiler=None):
    check_call(_LIB.DLGpuMax_Pooling2d(_h(in_arr), int(kernel_H), int(kernel_W), _h(pooled_layer),
                                       int(padding), int(stride), _s(stream), _p(profiler)))


def max_pooling2d_gradient(in_arr, in_grad_arr, kernel_H, kernel_W, out_grad_arr, padding=0, stride=1,
                           stream=None, profiler=None):
    check_call(_LIB.DLGpuMax_Pooling2d_gradient(_h(in_arr), _h(in_grad_arr), int(kernel_H), int(kernel_W),
                                                _h(out_grad_arr), int(padding), int(stride),
                                                _s(stream), _p(profiler)))


def CuDNN_max_pooling2d(in_arr, kernel_H, kernel_W, pooled_layer, padding=0, stride=1, stream=None,
                        profiler=None):
    check_call(_LIB.CuDNN_DLGpuMax_Pooling2d(_h(in_arr), ctypes.c_size_t(kernel_H), ctypes.c_size_t(kernel_W),
                                             _h(pooled_layer), ctypes.c_size_t(padding),
                                             ctypes.c_size_t(stride), _s(stream), _p(profiler)))


def CuDNN_max_pooling2d_gradient(in_arr_y, in_gradient_y, in_arr_x, kernel_H, kernel_W, out_gradient_x,
                                 padding=0, stride=1, stream=None, profiler=None):
    check_call(_LIB.CuDNN_DLGpuMax_Pooling2d_gradient(
        _h(in_arr_y), _h(in_gradient_y), _h(in_arr_x), ctypes.c_size_t(kernel_H), ctypes.c_size_t(kernel_W),
        _h(out_gradient_x), ctypes.c_size_t(padding), ctypes.c_size_t(stride), _s(stream), _p(profiler)))


# ---- Concat / Slice (gpu_links/ConcatLink.py:8,14; gpu_links/SliceLink.py:8,16) ----
def concat(in_arr1, in_arr2, out_arr, axis=0, stream=None, profiler=None):
    check_call(_LIB.DLGpuConcat(_h(in_arr1), _h(in_arr2), _h(out_arr), int(axis), _s(stream), _p(profiler)))


def concat_gradient(out_grad_arr, in_arr, axis=0, idx=0, stream=None, profiler=None):
    check_call(_LIB.DLGpuConcat_gradient(_h(out_grad_arr), _h(in_arr), int(axis), int(idx),
                                         _s(stream), _p(profiler)))


def matrix_slice(in_arr, out_arr, begin_pos, stream=None, profiler=None):
    pos = (ctypes.c_int64 * len(begin_pos))(*list(begin_pos))
    check_call(_LIB.DLGpuSlice(_h(in_arr), _h(out_arr), pos, _s(stream), _p(profiler)))


def matrix_slice_gradient(in_arr, out_arr, begin_pos, stream=None, profiler=None):
    pos = (ctypes.c_int64 * len(begin_pos))(*list(begin_pos))
    check_call(_LIB.DLGpuSliceGradient(_h(in_arr), _h(out_arr), pos, _s(stream), _p(profiler)))


# ---- Optimizers (gpu_links/OptimizerLink.py:7-30) ----
def sgd_update(param, grad, lr, stream=None):
    check_call(_LIB.SGDOptimizerUpdate(_h(param), _h(grad), ctypes.c_float(lr), _s(stream)))


def momentum_update(param, grad, velocity, lr, momentum, nesterov, stream=None):
    check_call(_LIB.MomentumOptimizerUpdate(_h(param), _h(grad), _h(velocity), ctypes.c_float(lr),
                                            ctypes.c_float(momentum), ctypes.c_bool(bool(nesterov)), _s(stream)))


def optimizer_update_multi(params, grads, velocities, lr, momentum=0.0, nesterov=False, stream=None):
    """SGD (velocities None) or momentum update of a list of parameters in one launch."""
    n = len(params)
    table = lambda arrs: (_nd.DLArrayHandle * n)(*[_h(a) for a in arrs])
    check_call(_LIB.TSplit_OptimizerUpdateMulti(table(params), table(grads), table(velocities) if velocities is not None else None,
                                                n, ctypes.c_float(lr), ctypes.c_float(momentum), int(bool(nesterov)), _s(stream)))


def adagrad_update(param, grad, accumulation, lr, eps, stream=None):
    check_call(_LIB.AdaGradOptimizerUpdate(_h(param), _h(grad), _h(accumulation), ctypes.c_float(lr),
                                           ctypes.c_float(eps), _s(stream)))


def adam_update(param, grad, expavg, expavgsq, lr, beta1, beta2, beta1t, beta2t, eps, stream=None):
    check_call(_LIB.AdamOptimizerUpdate(_h(param), _h(grad), _h(expavg), _h(expavgsq), ctypes.c_float(lr),
                                        ctypes.c_float(beta1), ctypes.c_float(beta2), ctypes.c_float(beta1t),
                                        ctypes.c_float(beta2t), ctypes.c_float(eps), _s(stream)))


# ---- AvgPool (gpu_links/AvgPoolLink.py:8,15; gpu_links/CudnnAvgPoolLink.py:8,15) ----
def average_pooling2d(in_arr, kernel_H, kernel_W, pooled_layer, padding=0, stride=1, stream=None, profiler=None):
    check_call(_LIB.DLGpuAvgerage_Pooling2d(_h(in_arr), ctypes.c_size_t(kernel_H), ctypes.c_size_t(kernel_W),
                                            _h(pooled_layer), ctypes.c_size_t(padding), ctypes.c_size_t(stride),
                                            _s(stream), _p(profiler)))


def average_pooling2d_gradient(in_gradient_y, kernel_H, kernel_W, out_gradient_x, padding=0, stride=1,
                               stream=None, profiler=None):
    check_call(_LIB.DLGpuAvgerage_Pooling2d_gradient(
        _h(in_gradient_y), ctypes.c_size_t(kernel_H), ctypes.c_size_t(kernel_W), _h(out_gradient_x),
        ctypes.c_size_t(padding), ctypes.c_size_t(stride), _s(stream), _p(profiler)))


def CuDNN_average_pooling2d(in_arr, kernel_H, kernel_W, pooled_layer, padding=0, stride=1, stream=None,
                            profiler=None):
    check_call(_LIB.CuDNN_DLGpuAvgerage_Pooling2d(
        _h(in_arr), ctypes.c_size_t(kernel_H), ctypes.c_size_t(kernel_W), _h(pooled_layer),
        ctypes.c_size_t(padding), ctypes.c_size_t(stride), _s(stream), _p(profiler)))


def CuDNN_average_pooling2d_gradient(in_arr_y, in_gradient_y, in_arr_x, kernel_H, kernel_W, out_gradient_x,
                                     padding=0, stride=1, stream=None, profiler=None):
    check_call(_LIB.CuDNN_DLGpuAvgerage_Pooling2d_gradient(
        _h(in_arr_y), _h(in_gradient_y), _h(in_arr_x), ctypes.c_size_t(kernel_H), ctypes.c_size_t(kernel_W),
        _h(out_gradient_x), ctypes.c_size_t(padding), ctypes.c_size_t(stride), _s(stream), _p(profiler)))


# ---- Broadcast / reduce (gpu_links/BroadcastLink.py:8, ReduceSumAxisZeroLink.py:7,15,
#      Conv2dBroadcastLink.py:8, Conv2dReduceSumLink.py:8, BroadcastShapeLink.py:8, ReduceSumLink.py:7) ----
def broadcast_to(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuBroadcastTo(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def reduce_sum_axis_zero(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuReduceSumAxisZero(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def _reduce_sum_axis_zero(in_arr, out_arr, workspace_arr, stream=None, profiler=None):
    check_call(_LIB._DLGpuReduceSumAxisZero(_h(in_arr), _h(out_arr), _h(workspace_arr), _s(stream), _p(profiler)))


def conv2d_broadcast_to(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuConv2d_broadcast_to(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def conv2d_reduce_sum(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuConv2d_reduce_sum(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def broadcast_shape(in_arr, out_arr, add_axes=None, stream=None):
    pointer = (ctypes.c_int * len(add_axes))(*list(add_axes)) if add_axes else None
    check_call(_LIB.DLGpuBroadcastShape(_h(in_arr), _h(out_arr), pointer, _s(stream)))


def reduce_sum(in_arr, out_arr, axes, stream=None):
    pointer = (ctypes.c_int * len(axes))(*list(axes))
    check_call(_LIB.DLGpuReduceSum(_h(in_arr), _h(out_arr), pointer, ctypes.c_int(len(axes)), _s(stream)))


# ---- Pad (gpu_links/PadLink.py:8,30): paddings is a list of (before, after) pairs for the last axes ----
_PAD_MODES = {"CONSTANT": 0, "REFLECT": 1, "SYMMETRIC": 2}


def _pad_args(paddings, mode):
    flat = [int(v) for pair in paddings for v in pair]
    assert mode in _PAD_MODES
    return (ctypes.c_int * len(flat))(*flat), len(flat), ctypes.c_size_t(_PAD_MODES[mode])


def pad(in_arr, out_arr, paddings, mode="CONSTANT", constant_values=0, stream=None, profiler=None):
    arr, n, m = _pad_args(paddings, mode)
    check_call(_LIB.DLGpuPad(_h(in_arr), _h(out_arr), arr, n, m, ctypes.c_float(constant_values),
                             _s(stream), _p(profiler)))


def pad_gradient(out_grad_arr, in_grad_arr, paddings, mode="CONSTANT", stream=None, profiler=None):
    arr, n, m = _pad_args(paddings, mode)
    check_call(_LIB.DLGpuPad_gradient(_h(out_grad_arr), _h(in_grad_arr), arr, n, m, _s(stream), _p(profiler)))


# ---- Transpose / BatchMatMul (gpu_links/MatrixTransLink.py:8, BatchMatrixMultLink.py:7) ----
def matrix_transpose(in_mat, out_mat, perm, stream=None, profiler=None):
    pointer = (ctypes.c_int * len(perm))(*list(perm))
    check_call(_LIB.DLGpuTranspose(_h(in_mat), _h(out_mat), pointer, _s(stream), _p(profiler)))


def batch_matrix_multiply(matA, transA, matB, transB, matC, stream=None):
    check_call(_LIB.DLGpuBatchMatrixMultiply(_h(matA), ctypes.c_bool(bool(transA)), _h(matB),
                                             ctypes.c_bool(bool(transB)), _h(matC), _s(stream)))


# ---- OneHot / Where / Embedding (gpu_links/OneHotLink.py:8, WhereLink.py:8, EmbeddingLookUpLink.py:8,15) ----
def one_hot(in_arr, out_arr, stream=None):
    check_call(_LIB.DLGpuOneHot(_h(in_arr), _h(out_arr), _s(stream)))


def where(cond, arr1, arr2, out_arr, stream=None):
    check_call(_LIB.DLGpuWhere(_h(cond), _h(arr1), _h(arr2), _h(out_arr), _s(stream)))


def embedding_lookup(in_mat, ids, out_mat, stream=None, profiler=None):
    check_call(_LIB.DLGpuEmbeddingLookUp(_h(in_mat), _h(ids), _h(out_mat), _s(stream), _p(profiler)))


def embedding_lookup_gradient(grad_out, ids, grad_in, stream=None, profiler=None):
    check_call(_LIB.DLGpuEmbeddingLookUp_Gradient(_h(grad_out), _h(ids), _h(grad_in), _s(stream), _p(profiler)))


# ---- Dropout (gpu_links/CudnnDropoutLink.py:8,15).  reserve_size is a ctypes.c_int and
#      reserve_space a ctypes.c_void_p owned by the caller (one pair per dropout node); the first
#      forward call (firstTime == 1) fills both. ----
def CuDNN_Dropout(in_arr, dropout, out_arr, reserve_size, reserve_space, firstTime, stream=None, profiler=None):
    check_call(_LIB.CuDNN_DLGpuDropout(_h(in_arr), ctypes.c_float(dropout), _h(out_arr), ctypes.byref(reserve_size),
                                       ctypes.byref(reserve_space), ctypes.c_int(firstTime), _s(stream),
                                       _p(profiler)))


def CuDNN_Dropout_gradient(in_gradient_y, dropout, out_gradient_x, reserve_size, reserve_space, stream=None,
                           profiler=None):
    check_call(_LIB.CuDNN_DLGpuDropout_gradient(_h(in_gradient_y), ctypes.c_float(dropout), _h(out_gradient_x),
                                                ctypes.byref(reserve_size), ctypes.byref(reserve_space),
                                                _s(stream), _p(profiler)))


# ---- CSR sparse products (gpu_links/CuSparseLink.py:7,13) ----
def CuSparse_Csrmv(mat, trans, in_arr, out_arr, stream=None, profiler=None):
    assert isinstance(mat, _nd.ND_Sparse_Array)
    check_call(_LIB.CuSparse_DLGpuCsrmv(_h(mat.data), _h(mat.row), _h(mat.col), ctypes.c_int(mat.nrow),
                                        ctypes.c_int(mat.ncol), ctypes.c_bool(bool(trans)), _h(in_arr), _h(out_arr),
                                        _s(stream), _p(profiler)))


def CuSparse_Csrmm(matA, transA, matB, transB, matC, stream=None, profiler=None):
    assert isinstance(matA, _nd.ND_Sparse_Array)
    check_call(_LIB.CuSparse_DLGpuCsrmm(_h(matA.data), _h(matA.row), _h(matA.col), ctypes.c_int(matA.nrow),
                                        ctypes.c_int(matA.ncol), ctypes.c_bool(bool(transA)), _h(matB),
                                        ctypes.c_bool(bool(transB)), _h(matC), _s(stream), _p(profiler)))


# ---- Elementwise math (gpu_links/MatrixDivideLink.py:7, MatrixDivideConstLink.py:7, OppositeLink.py:8,
#      MatrixSqrtLink.py:8, MatrixRsqrtLink.py:8, TanhLink.py:8, SigmoidLink.py:7) ----
def matrix_elementwise_divide(matA, matB, matC, stream=None, profiler=None):
    check_call(_LIB.DLGpuMatrixElementwiseDivide(_h(matA), _h(matB), _h(matC), _s(stream), _p(profiler)))


def matrix_elementwise_divide_const(val, in_mat, out_mat, stream=None, profiler=None):
    check_call(_LIB.DLGpuMatrixDivConst(ctypes.c_float(val), _h(in_mat), _h(out_mat), _s(stream), _p(profiler)))


def matrix_opposite(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuOpposite(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def matrix_sqrt(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuSqrt(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def matrix_rsqrt(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuReciprocalSqrt(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def tanh(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuTanh(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


def sigmoid(in_arr, out_arr, stream=None, profiler=None):
    check_call(_LIB.DLGpuSigmoid(_h(in_arr), _h(out_arr), _s(stream), _p(profiler)))


# ---- Which routine a convolution takes (no counterpart in the reference's gpu_links) ----
def conv_takes_winograd(images, in_channels, out_channels, height, width, kernel=3, pad=1, stride=1, data_gradient=False,
                        filter_gradient=False):
    """True when the library runs this layer's forward pass (or, with `data_gradient` /
    `filter_gradient`, that gradient) through the Winograd F(4x4, 3x3) routine rather than the
    direct implicit GEMM."""
    which = 2 if filter_gradient else 1 if data_gradient else 0
    return bool(_LIB.TSplit_ConvTakesWinograd(int(images), int(in_channels), int(out_channels), int(height), int(width),
                                              int(kernel), int(kernel), int(pad), int(pad), int(stride), which))


def batch_norm_look_behind():
    """(BatchNorm calls that took their statistics from the sums the convolution in front of them left,
    whether such sums are pending right now)."""
    served, live = ctypes.c_longlong(0), ctypes.c_int(0)
    check_call(_LIB.TSplit_BatchNormLookBehind(ctypes.byref(served), ctypes.byref(live)))
    return int(served.value), bool(live.value)


def winograd_gemm_timing(on, kind=None):
    """Switch the event timing of the GEMM launches inside the Winograd routine on or off; with `kind`
    (see winograd_gemm_times) only the launches of that kind are timed."""
    check_call(_LIB.TSplit_WinogradGemmTiming(0 if not on else 1 if kind is None else 2 + int(kind)))


def split_bf16(on):
    """Switches the split-bf16 products of the Winograd routine's GEMMs on or off (off by default); returns
    the previous setting."""
    was = ctypes.c_int()
    check_call(_LIB.TSplit_SplitBf16(int(bool(on)), ctypes.byref(was)))
    return bool(was.value)


def winograd_gemm_times(filter_gradient=False, kind=None):
    """-> (launches, total ms, total executed FLOP, total algorithmic bytes) of the timed GEMM launches of
    kind 0 (forward / data gradient on 128 x 128 tiles), 1 (filter gradient), 2 (forward / data gradient
    of layers that produce at most 64 channels, on 64 x 256 tiles), 3 / 4 (forward and data gradient /
    filter gradient with split-bf16 products), 5 (forward / data gradient as one kernel), 6 (filter gradient as
    one kernel)."""
    which = int(bool(filter_gradient)) if kind is None else int(kind)
    n, ms, flop, nbytes = ctypes.c_double(), ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    check_call(_LIB.TSplit_WinogradGemmTimes(which, ctypes.byref(n), ctypes.byref(ms), ctypes.byref(flop)))
    check_call(_LIB.TSplit_WinogradGemmBytes(which, ctypes.byref(nbytes)))
    return int(n.value), ms.value, flop.value, nbytes.value


# ---- Fused BatchNorm + Relu (no counterpart in the reference's gpu_links) ----
def batch_norm_relu(in_arr, bn_scale_arr, bn_bias_arr, out_arr, save_mean, save_var, eps=0.01, stream=None,
                    profiler=None):
    check_call(_LIB.TSplit_BatchNormRelu(_h(in_arr), _h(bn_scale_arr), _h(bn_bias_arr), _h(out_arr),
                                         ctypes.c_float(eps), _h(save_mean), _h(save_var), _s(stream), _p(profiler)))


def batch_norm_relu_max_pool(in_arr, bn_scale_arr, bn_bias_arr, out_arr, save_mean, save_var, eps=0.01, stats=None, slots=0,
                             stream=None, profiler=None):
    """BatchNorm + Relu + 2x2 / stride 2 max pooling forward in one call: out_arr is the pooled tensor.  With
    `stats` (rows 0 .. slots-1 of a convolution's sums) the batch statistics come from there."""
    if stats is None:
        check_call(_LIB.TSplit_BatchNormReluMaxPool(_h(in_arr), _h(bn_scale_arr), _h(bn_bias_arr), _h(out_arr),
                                                    ctypes.c_float(eps), _h(save_mean), _h(save_var), _s(stream), _p(profiler)))
    else:
        check_call(_LIB.TSplit_BatchNormReluMaxPoolFromStats(_h(in_arr), _h(stats), int(slots), _h(bn_scale_arr),
                                                             _h(bn_bias_arr), _h(out_arr), ctypes.c_float(eps), _h(save_mean),
                                                             _h(save_var), _s(stream), _p(profiler)))


def batch_norm_relu_max_pool_gradient(gradient_pooled, in_arr, bn_scale_arr, bn_bias_arr, gradient_in, gradient_scale,
                                      gradient_bias, save_mean, save_var, eps=0.01, stream=None, profiler=None):
    check_call(_LIB.TSplit_BatchNormReluMaxPool_gradient(_h(gradient_pooled), _h(in_arr), _h(bn_scale_arr), _h(bn_bias_arr),
                                                         _h(gradient_in), _h(gradient_scale), _h(gradient_bias),
                                                         ctypes.c_float(eps), _h(save_mean), _h(save_var), _s(stream),
                                                         _p(profiler)))


def conv2d_batch_norm_stats(in_arr_x, in_arr_f, out_arr, stats, slot, padding=0, padding2=None, stride=1, stream=None,
                            profiler=None):
    """CuDNN_conv2d that also writes the per-channel (sum, sum of squares) of out_arr into row `slot` of
    `stats` (float32 array of at least (slot + 1) * out_channels * 4 elements, read as doubles)."""
    pad2 = padding if padding2 is None else padding2
    check_call(_LIB.TSplit_Conv2dBatchNormStats(_h(in_arr_x), _h(in_arr_f), _h(out_arr), int(padding), int(pad2),
                                                int(stride), _h(stats), int(slot), _s(stream), _p(profiler)))


def batch_norm_from_stats(in_arr, stats, slots, bn_scale_arr, bn_bias_arr, out_arr, save_mean, save_var, eps=0.01,
                          relu=False, stream=None, profiler=None):
    """BatchNorm (+ Relu) forward with the batch statistics taken from rows 0 .. slots-1 of `stats`."""
    check_call(_LIB.TSplit_BatchNormFromStats(_h(in_arr), _h(stats), int(slots), _h(bn_scale_arr), _h(bn_bias_arr),
                                              _h(out_arr), ctypes.c_float(eps), _h(save_mean) if save_mean else None,
                                              _h(save_var) if save_var else None, int(bool(relu)), _s(stream),
                                              _p(profiler)))


def batch_norm_relu_gradient(in_gradient_y, in_arr_x, in_bn_scale, in_bn_bias, out_gradient_x, out_gradient_bn_scale,
                             out_gradient_bn_bias, saved_mean, saved_var, eps=0.01, stream=None, profiler=None):
    check_call(_LIB.TSplit_BatchNormRelu_gradient(
        _h(in_gradient_y), _h(in_arr_x), _h(in_bn_scale), _h(in_bn_bias), _h(out_gradient_x),
        _h(out_gradient_bn_scale), _h(out_gradient_bn_bias), ctypes.c_float(eps), _h(saved_mean), _h(saved_var),
        _s(stream), _p(profiler)))
