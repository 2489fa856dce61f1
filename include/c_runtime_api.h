/*
 * C ABI of libc_runtime_api.so for MI355X (gfx950).
 *
 * Drop-in for the GPU operator layer of Athena/TSplit: every entry point below
 * has the name, argument order and argument meaning of the symbol the
 * reference's ctypes layer binds (python/athena/gpu_links/<Op>Link.py ->
 * _LIB.<symbol>), as declared in the reference's src/common/c_runtime_api.h
 * (cited per declaration as "ref:").  Where the reference's header and its
 * implementation disagree, the implementation -- i.e. what its Python call
 * sites really pass -- wins, and the comment says so.
 *
 * Conventions (ref: src/common/dlarray.h:22-63, src/common/runtime_base.h:13-47):
 *  - every tensor is dense, C-contiguous float32; 4-D tensors are NCHW, filters OIHW;
 *  - a DLStreamHandle of NULL means the default stream; all operator calls are
 *    asynchronous on their stream unless a non-NULL ProfilerHandle is given, in
 *    which case the call blocks and fills the Profiler (time in ms, sizes in MiB);
 *  - return 0 on success, -1 on failure (a message goes to stderr).
 */
#ifndef TSPLIT_AMD_C_RUNTIME_API_H_
#define TSPLIT_AMD_C_RUNTIME_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#else
#include <stdbool.h>
#endif

/* ---- types (ref: src/common/dlarray.h:22-63, src/common/profiler.h:13-22) ---- */
typedef enum { kCPU = 1, kGPU = 2 } DLDeviceType;

typedef struct {
  int device_id;
  DLDeviceType device_type;
} DLContext;

typedef struct {
  void *data;       /* device (kGPU) or host (kCPU) pointer; never owned by a micro-tensor view */
  DLContext ctx;
  int ndim;
  int64_t *shape;
} DLArray;          /* 32 bytes */

typedef struct {
  int device_id;
  void *handle;     /* points to a heap hipStream_t */
} DLStream;

typedef struct {
  int device_id;
  void *handle;     /* points to a heap hipEvent_t */
} DLEvent;

typedef struct Profiler {
  float time;              /* ms */
  float input_memory;      /* MiB */
  float output_memory;     /* MiB */
  float workspace_memory;  /* MiB */
} Profiler;

typedef int64_t index_t;
typedef DLArray *DLArrayHandle;
typedef DLStream *DLStreamHandle;
typedef DLEvent *DLEventHandle;
typedef Profiler *ProfilerHandle;

/* ---- runtime: profiler, streams, events (ref: c_runtime_api.h:33-52; impl
 *      src/common/c_runtime_api.cc:110-115, src/cuda_common/gpu_runtime.cc:64-126) ---- */
int ProfilerAlloc(ProfilerHandle *handle);            /* fields start at -1 */
int DLStreamCreate(size_t dev_id, DLStreamHandle *handle);
int DLStreamDestroy(DLStreamHandle handle);
int DLStreamSync(DLStreamHandle handle);
int DLEventCreate(size_t dev_id, DLEventHandle *handle);
int DLEventDestroy(DLEventHandle handle);
int DLEventRecord(DLStreamHandle stream_handle, DLEventHandle event_handle);
int DLEventSync(DLEventHandle handle);
/* ref declares `bool`; the ctypes caller reads an int, so a clean 0/1 int is exported. */
int DLEventQuery(DLEventHandle handle);

/* ---- runtime: library-handle hooks.  The reference creates cuDNN/cuBLAS/cuSPARSE
 *      handles here (gpu_runtime.h:100-105, gpu_runtime.cc:13-62); this library has
 *      no such handles, the calls only select the device. ---- */
void cudnn_init(size_t dev_id, DLStreamHandle stream);
void cublas_init(size_t dev_id, DLStreamHandle stream);
void cusp_init(size_t dev_id, DLStreamHandle stream);
void cuda_init(void);

/* ---- runtime: pooled allocator introspection (ref: c_runtime_api.h:49-51; impl
 *      c_runtime_api.cc:308-347 over src/cuda_common/gpu_memory_manager.cc:201-318) ---- */
void DLMemoryManager_PrintState(void *t, int type);   /* *(int*)t = number of free chunks; type!=0 prints */
void DLMemoryManager_Try_to_Malloc(size_t memory_size, void *p);  /* *(int*)p = 1 if it would succeed */
void DLMemoryManager_GPU_Usage(size_t *used_size, size_t *unused_unavailable_size,
                               size_t *unused_available_size);

/* ---- runtime: arrays (ref: c_runtime_api.h:64-106; impl c_runtime_api.cc:137-306).
 *      MEMORY_MANAGE_RULE 0 = raw device malloc/free per tensor, != 0 = pool. ---- */
int DLArrayAlloc(const index_t *shape, index_t ndim, DLContext ctx, DLArrayHandle *out,
                 int MEMORY_MANAGE_RULE);
int DLArrayAllocSelf(DLArrayHandle handle, int MEMORY_MANAGE_RULE);
int DLArrayFree(DLArrayHandle handle, int MEMORY_MANAGE_RULE);
int DLArrayFreeSelf(DLArrayHandle handle, int MEMORY_MANAGE_RULE);
int DLArrayCopyFromTo(DLArrayHandle from, DLArrayHandle to, DLStreamHandle stream);
/* One allocation holding an output (at the base) and an input (flush with the end) that
 * overlap by `overlap_pieces` of the input's `pieces` micro-tensors (impl c_runtime_api.cc:164-210). */
int DLArrayReuseAlloc(DLContext ctx, int MEMORY_MANAGE_RULE, const index_t *input_shape,
                      index_t input_ndim, DLArrayHandle *input, const index_t *output_shape,
                      index_t output_ndim, DLArrayHandle *output, int pieces, int overlap_pieces);
/* Zero-copy view of micro-tensor `index` of `total_number` along dimension 0 (batch) or 1
 * (impl c_runtime_api.cc:212-271).  The view owns its DLArray and shape, not the data. */
int DLArraySliceForMicroTensor(DLArrayHandle input, DLArrayHandle *output, int total_number,
                               int index, int dimension);

/* ---- graph-closure elementwise ops (ref: c_runtime_api.h:113,138-139,148-149,158-159,
 *      168-169,317; impl src/ops/ArraySet.cu:9, AddElewise.cu:9, AddConst.cu:9,
 *      MultiplyElewise.cu:9, MultiplyConst.cu:9, Reshape.cu:5) ---- */
int DLGpuArraySet(DLArrayHandle arr, float value, DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuMatrixElementwiseAdd(const DLArrayHandle matA, const DLArrayHandle matB,
                              DLArrayHandle output, DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuMatrixElementwiseAddByConst(const DLArrayHandle input, float val, DLArrayHandle output,
                                     DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuMatrixElementwiseMultiply(const DLArrayHandle matA, const DLArrayHandle matB,
                                   DLArrayHandle output, DLStreamHandle stream_handle,
                                   ProfilerHandle p);
int DLGpuMatrixMultiplyByConst(const DLArrayHandle input, float val, DLArrayHandle output,
                               DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuReshape(const DLArrayHandle in_arr, DLArrayHandle out_arr, DLStreamHandle stream_handle,
                 ProfilerHandle p);

/* ---- Relu (ref: c_runtime_api.h:234,243-244; impl src/ops/Relu.cu:9,82).
 *      Gradient is (sign(x)+1)*0.5*dy, i.e. 0.5*dy at x == 0. ---- */
int DLGpuRelu(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
              ProfilerHandle p);
int DLGpuReluGradient(const DLArrayHandle input, const DLArrayHandle in_grad, DLArrayHandle output,
                      DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- MatMul (ref: c_runtime_api.h:208-210; impl src/ops/MatrixMult.cu:4-72).
 *      Row-major 2-D C = op(A) op(B). ---- */
int DLGpuMatrixMultiply(const DLArrayHandle matA, bool transposeA, const DLArrayHandle matB,
                        bool transposeB, DLArrayHandle matC, DLStreamHandle stream_handle,
                        ProfilerHandle p);

/* ---- Softmax / SoftmaxCrossEntropy (ref: c_runtime_api.h:270,286-292; impl
 *      src/ops/Softmax.cu:24, src/ops/SoftmaxCrossEntropy.cu:44,106).  Rows = product of
 *      all but the last dimension; loss has one element = mean over rows; the gradient
 *      is (softmax(a) - b) * c[0] / a.shape[0]. ---- */
int DLGpuSoftmax(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
                 ProfilerHandle p);
int DLGpuSoftmaxCrossEntropy(const DLArrayHandle input_a, const DLArrayHandle input_b,
                             DLArrayHandle output, DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuSoftmaxCrossEntropy_Gradient(const DLArrayHandle input_a, const DLArrayHandle input_b,
                                      const DLArrayHandle input_c, DLArrayHandle output,
                                      DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- Softmax cross-entropy that allocates nothing.  NO counterpart in the reference.  For callers
 *      that cannot allocate device memory inside the call: code being captured into a HIP graph,
 *      tight serving loops, harnesses that forbid hipMalloc.  Same arguments, kernels and result
 *      (bit for bit) as DLGpuSoftmaxCrossEntropy without the profiler; the per-row losses live in
 *      a fixed 1 MiB array inside the library instead of its grow-on-demand scratch memory, so at
 *      most 262144 rows (product of all but the last dimension): more returns -1 with a message.
 *      Every GPU the library runs on holds its own copy of that array until the process ends; calls
 *      that overlap on one GPU (different streams) share it and race.  The array's address is
 *      looked up once per device, by cudnn_init(dev_id, ...) or else by the first call. ---- */
int TSplit_SoftmaxCrossEntropyNoAlloc(const DLArrayHandle input_a, const DLArrayHandle input_b,
                                      DLArrayHandle output, DLStreamHandle stream_handle);

/* ---- Conv2d, cross-correlation, no bias, square stride, dilation 1.
 *      `CuDNN_` symbols (ref: c_runtime_api.h:323-327; impl src/ops/CudnnConv2d.cu:6,207,410)
 *      take (pad_h, pad_w, stride); they are the ones the graph ops call
 *      (python/athena/gpu_ops/Conv2d.py:116-118).  Output/gradient shapes are taken from
 *      the pre-allocated output array. ---- */
int CuDNN_DLGpuConv2d(const DLArrayHandle input_x, const DLArrayHandle input_f,
                      DLArrayHandle output, const int padding, const int padding2,
                      const int stride, DLStreamHandle stream_handle, ProfilerHandle p);
int CuDNN_DLGpuConv2d_Gradient_of_Filter(const DLArrayHandle input_x,
                                         const DLArrayHandle gradient_y, DLArrayHandle gradient_f,
                                         const int padding, const int padding2, const int stride,
                                         DLStreamHandle stream_handle, ProfilerHandle p);
int CuDNN_DLGpuConv2d_Gradient_of_Data(const DLArrayHandle input_f, const DLArrayHandle gradient_y,
                                       DLArrayHandle gradient_x, const int padding,
                                       const int padding2, const int stride,
                                       DLStreamHandle stream_handle, ProfilerHandle p);
/*      Plain symbols: the reference header lists (padding1, padding2)
 *      (c_runtime_api.h:294-302) but its implementation and Python call sites pass ONE
 *      padding int (src/ops/Conv2d.cu:52,172,241; gpu_links/Conv2dLink.py:13-14,31-32,40-41):
 *      the implementation's signature is exported.  The caller-provided im2col workspaces
 *      are accepted and left untouched (the implicit-GEMM kernels need none). */
int DLGpuConv2d(const DLArrayHandle input_x, const DLArrayHandle input_f, DLArrayHandle output,
                DLArrayHandle workspace_arr, const int padding, const int stride,
                DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuConv2d_Gradient_of_Data(const DLArrayHandle input_f, const DLArrayHandle gradient_y,
                                 DLArrayHandle gradient_x, DLArrayHandle workspace_im2col,
                                 const int padding, const int stride,
                                 DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuConv2d_Gradient_of_Filter(const DLArrayHandle input_x, const DLArrayHandle gradient_y,
                                   DLArrayHandle gradient_f, DLArrayHandle workspace_im2col,
                                   DLArrayHandle workspace_batch_filter, const int padding,
                                   const int stride, DLStreamHandle stream_handle,
                                   ProfilerHandle p);

/* ---- BatchNorm, training mode, spatial, biased batch variance (ref: c_runtime_api.h:344-349;
 *      impl src/ops/CudnnBn.cu:12,212).  scale/bias/dscale/dbias/save_* hold C elements.
 *      save_mean_arr / save_var_arr may be NULL; when given, forward writes (batch mean,
 *      1/sqrt(var+eps)) and the gradient reads them instead of recomputing (the cuDNN
 *      convention the reference relies on).  `momentum` is accepted and unused: the
 *      reference computes running statistics into throw-away scratch (CudnnBn.cu:164-176). ---- */
int CuDNN_DLGpuBatch_Normalization(const DLArrayHandle input_X, const DLArrayHandle bn_scale,
                                   const DLArrayHandle bn_bias, DLArrayHandle output_Y,
                                   float momentum, float eps, DLArrayHandle save_mean_arr,
                                   DLArrayHandle save_var_arr, DLStreamHandle stream_handle,
                                   ProfilerHandle p);
int CuDNN_DLGpuBatch_Normalization_gradient(const DLArrayHandle gradient_Y,
                                            const DLArrayHandle input_X,
                                            const DLArrayHandle bn_scale, DLArrayHandle gradient_X,
                                            DLArrayHandle gradient_bn_scale,
                                            DLArrayHandle gradient_bn_bias, float eps,
                                            DLArrayHandle save_mean_arr,
                                            DLArrayHandle save_var_arr,
                                            DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- MaxPool (ref: c_runtime_api.h:311-315,340-342; impl src/ops/MaxPool.cu:45,138,
 *      src/ops/CudnnMaxPool.cu:3,103).  Windows are clipped to the image; the maximum is the
 *      first strict maximum in row-major scan; the gradient accumulates in window order and
 *      zero-fills the rest of gradient_X itself.  Note the differing argument orders and
 *      integer types of the two families. ---- */
int DLGpuMax_Pooling2d(const DLArrayHandle input, const int kernel_H, const int kernel_W,
                       DLArrayHandle output, const int padding, const int stride,
                       DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuMax_Pooling2d_gradient(const DLArrayHandle input, const DLArrayHandle output_grad,
                                const int kernel_H, const int kernel_W, DLArrayHandle input_grad,
                                const int padding, const int stride, DLStreamHandle stream_handle,
                                ProfilerHandle p);
int CuDNN_DLGpuMax_Pooling2d(const DLArrayHandle input, const size_t kernel_H,
                             const size_t kernel_W, DLArrayHandle output, const size_t padding,
                             const size_t stride, DLStreamHandle stream_handle, ProfilerHandle p);
int CuDNN_DLGpuMax_Pooling2d_gradient(const DLArrayHandle output_Y, const DLArrayHandle gradient_Y,
                                      const DLArrayHandle input_X, const size_t kernel_H,
                                      const size_t kernel_W, DLArrayHandle gradient_X,
                                      const size_t padding, const size_t stride,
                                      DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- Concat / Slice copies (ref: c_runtime_api.h:355-357,366-368; impl
 *      src/ops/Concat.cu:22,127, src/ops/Slice.cu:30,118).  begin_pos is a host array of
 *      ndim int64. ---- */
int DLGpuConcat(const DLArrayHandle input_x, const DLArrayHandle input_y, DLArrayHandle output,
                int axis, DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuConcat_gradient(const DLArrayHandle output_gradient, DLArrayHandle input_gradient,
                         int axis, int id, DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuSlice(const DLArrayHandle in_arr, DLArrayHandle out_arr, int64_t *begin_pos,
               DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuSliceGradient(const DLArrayHandle in_arr, DLArrayHandle out_arr, int64_t *begin_pos,
                       DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- Optimizer updates, in place, no ProfilerHandle (ref: c_runtime_api.h:371-380; impl
 *      src/ops/Optimizers.cu:9,48,87,122).  beta1t/beta2t are the host-accumulated powers.
 *      SGD and Momentum calls issued back to back are queued on their stream as ONE launch when the
 *      next call of any other kind reaches the library (DLStreamSync, DLEventRecord and copies
 *      included), so every effect visible through this interface keeps its order; environment
 *      TSPLIT_LAZY_UPDATES=0 issues each call at once. ---- */
int SGDOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, float lr,
                       DLStreamHandle stream_handle);
int MomentumOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, DLArrayHandle velocity,
                            float lr, float momentum, bool nesterov, DLStreamHandle stream_handle);
int AdaGradOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, DLArrayHandle acc,
                           float lr, float eps, DLStreamHandle stream_handle);
int AdamOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, DLArrayHandle expavg,
                        DLArrayHandle expavgsq, float lr, float beta1, float beta2, float beta1t,
                        float beta2t, float eps, DLStreamHandle stream_handle);

/* ==== Operators around the core path: needed by the ResNet / Inception-v4 / Transformer
 *      graphs of the reference's examples. ==== */

/* ---- AvgPool (ref: c_runtime_api.h:305-309,329-332; impl src/ops/AvgPool.cu,
 *      src/ops/CudnnAvgPool.cu).  Sum over the window clipped to the image divided by
 *      kernel_H*kernel_W whatever the clipping (python/athena/gpu_ops/AvgPool.py:27-50,
 *      139-161).  All four symbols take size_t geometry.  The `CuDNN_` gradient also
 *      receives output_Y and input_X, which the arithmetic does not need. ---- */
int DLGpuAvgerage_Pooling2d(const DLArrayHandle input, const size_t kernel_H,
                            const size_t kernel_W, DLArrayHandle output, const size_t padding,
                            const size_t stride, DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuAvgerage_Pooling2d_gradient(const DLArrayHandle gradient_Y, const size_t kernel_H,
                                     const size_t kernel_W, DLArrayHandle gradient_X,
                                     const size_t padding, const size_t stride,
                                     DLStreamHandle stream_handle, ProfilerHandle p);
int CuDNN_DLGpuAvgerage_Pooling2d(const DLArrayHandle input, const size_t kernel_H,
                                  const size_t kernel_W, DLArrayHandle output,
                                  const size_t padding, const size_t stride,
                                  DLStreamHandle stream_handle, ProfilerHandle p);
int CuDNN_DLGpuAvgerage_Pooling2d_gradient(const DLArrayHandle output_Y,
                                           const DLArrayHandle gradient_Y,
                                           const DLArrayHandle input_X, const size_t kernel_H,
                                           const size_t kernel_W, DLArrayHandle gradient_X,
                                           const size_t padding, const size_t stride,
                                           DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- Broadcast / reduce (ref: c_runtime_api.h:121,129-130,319,321,442,449; impl
 *      src/ops/Broadcast.cu:4-9 (out[i] = in[i % in_size]: new leading axes),
 *      src/ops/ReduceSumAxisZero.cu:27,98 (sum over axis 0; the `_` variant takes a
 *      caller workspace, which is accepted and left untouched),
 *      src/ops/Conv2dBroadcast.cu ([C] -> [N,C,H,W]), src/ops/Conv2dReduceSum.cu
 *      ([N,C,H,W] -> [C]), src/ops/BroadcastShape.cu:23 (add_axes: host int array of
 *      out.ndim - in.ndim new-axis positions, or NULL for alignment from the right),
 *      src/ops/ReduceSum.cu:3 (axes: host int array; out holds the kept elements, with or
 *      without the reduced axes as extent-1 axes)).  The last two have no ProfilerHandle. ---- */
int DLGpuBroadcastTo(const DLArrayHandle input, DLArrayHandle output,
                     DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuReduceSumAxisZero(const DLArrayHandle input, DLArrayHandle output,
                           DLStreamHandle stream_handle, ProfilerHandle p);
int _DLGpuReduceSumAxisZero(const DLArrayHandle input, DLArrayHandle output,
                            DLArrayHandle arr_workspace, DLStreamHandle stream_handle,
                            ProfilerHandle p);
int DLGpuConv2d_broadcast_to(const DLArrayHandle input_x, DLArrayHandle output_y,
                             DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuConv2d_reduce_sum(const DLArrayHandle input_x, DLArrayHandle output_y,
                           DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuBroadcastShape(const DLArrayHandle in_arr, DLArrayHandle out_arr, int *add_axes,
                        DLStreamHandle stream_handle);
int DLGpuReduceSum(const DLArrayHandle in_arr, DLArrayHandle out_arr, int *axes, int num_ax,
                   DLStreamHandle stream_handle);

/* ---- Pad, 4-D, mode 0 (CONSTANT) only (ref: c_runtime_api.h:351,353; impl
 *      src/ops/Pad.cu:23,76).  paddings: host array of pad_len ints, (before, after) pairs
 *      for the LAST pad_len/2 axes.  Unpadded leading axes are copied whole, as np.pad does
 *      (python/athena/gpu_ops/Pad.py:194-196); the reference's kernel keeps only their last
 *      index (src/ops/Pad.cu:29-31), which is not followed.  Modes 1/2 fail. ---- */
int DLGpuPad(const DLArrayHandle input_X, DLArrayHandle output_Y, int *paddings, int pad_len,
             size_t mode, float constant_values, DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuPad_gradient(const DLArrayHandle output_gradient_Y, DLArrayHandle input_gradient_X,
                      int *paddings, int pad_len, size_t mode, DLStreamHandle stream_handle,
                      ProfilerHandle p);

/* ---- Transpose (ref: c_runtime_api.h:360; impl src/ops/Transpose.cu).  perm: host array
 *      of ndim ints, output axis d is input axis perm[d]. ---- */
int DLGpuTranspose(const DLArrayHandle input, DLArrayHandle output, int *perm,
                   DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- BatchMatMul (ref: c_runtime_api.h:445-447; impl src/ops/BatchMatrixMult.cu).
 *      Row-major C[..., n, m] = op(A[...]) op(B[...]) for every leading index; no
 *      ProfilerHandle. ---- */
int DLGpuBatchMatrixMultiply(const DLArrayHandle matA, bool transposeA, const DLArrayHandle matB,
                             bool transposeB, DLArrayHandle matC, DLStreamHandle stream_handle);

/* ---- OneHot / Where / Embedding (ref: c_runtime_api.h:443,444,280-284; impl
 *      src/ops/OneHot.cu:16, src/ops/Where.cu:10, src/ops/EmbeddingLookup.cu:14,67).
 *      ids are float32 holding integers.  The embedding symbols honour ids as the numpy
 *      branch does (python/athena/gpu_ops/EmbeddingLookUp.py:41-42); the reference's CUDA
 *      kernels use the row number instead (src/ops/EmbeddingLookup.cu:6-7,59-60).  The
 *      gradient zero-fills input_grad and scatter-adds; an id outside the table fails. ---- */
int DLGpuOneHot(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle);
int DLGpuWhere(const DLArrayHandle cond, const DLArrayHandle arr1, const DLArrayHandle arr2,
               DLArrayHandle output, DLStreamHandle stream_handle);
int DLGpuEmbeddingLookUp(const DLArrayHandle input, const DLArrayHandle ids, DLArrayHandle output,
                         DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuEmbeddingLookUp_Gradient(const DLArrayHandle output_grad, const DLArrayHandle ids,
                                  DLArrayHandle input_grad, DLStreamHandle stream_handle,
                                  ProfilerHandle p);

/* ---- Elementwise math (ref: c_runtime_api.h:178-179,188-189,197,218,226,252,260; impl
 *      src/ops/DivideElewise.cu:6, DivideConst.cu:6 (val / input), Opposite.cu:6, Sqrt.cu:6,46,
 *      Tanh.cu:6, Sigmoid.cu:6) ---- */
int DLGpuMatrixElementwiseDivide(const DLArrayHandle matA, const DLArrayHandle matB,
                                 DLArrayHandle output, DLStreamHandle stream_handle,
                                 ProfilerHandle p);
int DLGpuMatrixDivConst(float val, const DLArrayHandle input, DLArrayHandle output,
                        DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuOpposite(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
                  ProfilerHandle p);
int DLGpuSqrt(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
              ProfilerHandle p);
int DLGpuReciprocalSqrt(const DLArrayHandle input, DLArrayHandle output,
                        DLStreamHandle stream_handle, ProfilerHandle p);
int DLGpuTanh(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
              ProfilerHandle p);
int DLGpuSigmoid(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
                 ProfilerHandle p);

/* ---- Dropout (ref: c_runtime_api.h:334-338; impl src/ops/CudnnDropout.cu:4-77, :79-151).
 *      `dropout` is the probability of zeroing an element, survivors are scaled by
 *      1/(1-dropout) (cuDNN's meaning of the argument).  The generator is re-seeded with the
 *      reference's constant before every call (CudnnDropout.cu:33,41), so equal element counts
 *      give equal masks.  With first_time == 1 the forward call allocates the reserve space (one
 *      bit per element) from the device pool and stores its byte size and address through the two
 *      pointers; later forward calls and the gradient reuse it.  Which elements are dropped is
 *      this library's generator (Philox-4x32-10), not cuDNN's.  In the gradient call output_Y is
 *      the incoming gradient and input_X receives the result. ---- */
int CuDNN_DLGpuDropout(const DLArrayHandle input_X, const float dropout, DLArrayHandle output_Y,
                       int *reserve_size, void **reserve_space, int first_time,
                       DLStreamHandle stream_handle, ProfilerHandle p);
int CuDNN_DLGpuDropout_gradient(const DLArrayHandle output_Y, const float dropout,
                                DLArrayHandle input_X, int *reserve_size, void **reserve_space,
                                DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- CSR sparse x dense products (ref: c_runtime_api.h:362-364; impl
 *      src/ops/CuSparseCsrmv.cu:3-64, src/ops/CuSparseCsrmm.cu:34-114).  data: fp32 values
 *      [nnz]; row: int32 row pointers [nrow+1]; col: int32 column indices [nnz], zero based
 *      (python/athena/ndarray.py:445-455).  Csrmv: output = A input, or A^T input.  Csrmm:
 *      matC = op(A) op(matB), dense operands row-major, all four transpose combinations. ---- */
int CuSparse_DLGpuCsrmv(const DLArrayHandle data_handle, const DLArrayHandle row_handle,
                        const DLArrayHandle col_handle, int nrow, int ncol, bool transpose,
                        const DLArrayHandle input_handle, DLArrayHandle output_handle,
                        DLStreamHandle stream_handle, ProfilerHandle p);
int CuSparse_DLGpuCsrmm(const DLArrayHandle data_handle, const DLArrayHandle row_handle,
                        const DLArrayHandle col_handle, int nrow, int ncol, bool transposeA,
                        const DLArrayHandle matB, bool transposeB, DLArrayHandle matC,
                        DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- Fused BatchNorm + Relu.  NO counterpart in the reference (its ABI has one symbol per graph
 *      node); for hosts that know the Relu follows the BatchNorm and want to skip its two passes
 *      over the activation.  Forward: output_Y = max(BN(input_X), 0); both save arrays are
 *      required and receive (batch mean, 1/sqrt(var+eps)).  Gradient: gradient_Y is the gradient
 *      behind the Relu; it is gated with the reference's Relu derivative (sign(z)+1)/2 of
 *      z = BN(input_X), rebuilt from input_X, bn_scale, bn_bias and the saved statistics of the
 *      fused forward call, then the BatchNorm gradient is taken.  Results equal the two-call
 *      sequence (same float expressions). ---- */
int TSplit_BatchNormRelu(const DLArrayHandle input_X, const DLArrayHandle bn_scale,
                         const DLArrayHandle bn_bias, DLArrayHandle output_Y, float eps,
                         DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                         DLStreamHandle stream_handle, ProfilerHandle p);
int TSplit_BatchNormRelu_gradient(const DLArrayHandle gradient_Y, const DLArrayHandle input_X,
                                  const DLArrayHandle bn_scale, const DLArrayHandle bn_bias,
                                  DLArrayHandle gradient_X, DLArrayHandle gradient_bn_scale,
                                  DLArrayHandle gradient_bn_bias, float eps,
                                  DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                  DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- Convolution that hands its output's batch statistics to the BatchNorm behind it.  NO counterpart
 *      in the reference, where the BatchNorm call (src/ops/CudnnBn.cu:12-210) reads the convolution's
 *      output (src/ops/CudnnConv2d.cu:6-206) once more to get them; for hosts that know a BatchNorm
 *      follows.  `stats` is float32 storage, 8-byte aligned, viewed as [slots][out_channels][2] doubles.
 *      TSplit_Conv2dBatchNormStats computes exactly what CuDNN_DLGpuConv2d computes (same kernels, same
 *      bits) and writes the per-channel (sum, sum of squares) of `output` into row `slot`; a host that
 *      runs the convolution on batch micro-tensors gives every piece its own row.
 *      TSplit_BatchNormFromStats adds rows 0 .. slots-1 in that order, derives the batch mean and
 *      variance over all of input_X, and applies the BatchNorm (relu == 0) or BatchNorm + Relu
 *      (relu != 0: both save arrays required, as for TSplit_BatchNormRelu) in one pass over input_X.
 *      The gradients are those of CuDNN_DLGpuBatch_Normalization_gradient /
 *      TSplit_BatchNormRelu_gradient with the saved statistics. ---- */
int TSplit_Conv2dBatchNormStats(const DLArrayHandle input_x, const DLArrayHandle input_f,
                                DLArrayHandle output, const int padding, const int padding2,
                                const int stride, DLArrayHandle stats, int slot,
                                DLStreamHandle stream_handle, ProfilerHandle p);
int TSplit_BatchNormFromStats(const DLArrayHandle input_X, const DLArrayHandle stats, int slots,
                              const DLArrayHandle bn_scale, const DLArrayHandle bn_bias,
                              DLArrayHandle output_Y, float eps, DLArrayHandle save_mean_arr,
                              DLArrayHandle save_var_arr, int relu, DLStreamHandle stream_handle,
                              ProfilerHandle p);

/* ---- BatchNorm + Relu + max pooling as one call each way.  NO counterpart in the reference, where the three
 *      nodes that end a VGG stage are three calls (src/ops/CudnnBn.cu:12-210, src/ops/Relu.cu,
 *      src/ops/CudnnMaxPool.cu:6-210) and the activation in front of the pooling is written, read back by
 *      the pooling and kept for its gradient; for hosts that know the three follow one another.  2x2
 *      windows, stride 2, no padding; H and W of input_X even.  The forward calls read input_X
 *      [N][C][H][W] once and write only output_Y [N][C][H/2][W/2] (values equal those of the three calls);
 *      TSplit_BatchNormReluMaxPool takes the batch statistics from input_X itself (one more read),
 *      TSplit_BatchNormReluMaxPoolFromStats from rows 0 .. slots-1 of `stats` as
 *      TSplit_BatchNormFromStats does.  Both save arrays are required.
 *      TSplit_BatchNormReluMaxPool_gradient takes the pooled tensor's gradient gradient_Y
 *      [N][C][H/2][W/2] and input_X: a window's gradient goes to the first maximum of Relu(BN(input_X))
 *      in row-major order (the tie rule of the pooling gradient), is gated with the reference's Relu
 *      derivative there, and the BatchNorm gradient is taken; gradient_X [N][C][H][W]. ---- */
int TSplit_BatchNormReluMaxPool(const DLArrayHandle input_X, const DLArrayHandle bn_scale,
                                const DLArrayHandle bn_bias, DLArrayHandle output_Y, float eps,
                                DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                DLStreamHandle stream_handle, ProfilerHandle p);
int TSplit_BatchNormReluMaxPoolFromStats(const DLArrayHandle input_X, const DLArrayHandle stats, int slots,
                                         const DLArrayHandle bn_scale, const DLArrayHandle bn_bias,
                                         DLArrayHandle output_Y, float eps, DLArrayHandle save_mean_arr,
                                         DLArrayHandle save_var_arr, DLStreamHandle stream_handle,
                                         ProfilerHandle p);
int TSplit_BatchNormReluMaxPool_gradient(const DLArrayHandle gradient_Y, const DLArrayHandle input_X,
                                         const DLArrayHandle bn_scale, const DLArrayHandle bn_bias,
                                         DLArrayHandle gradient_X, DLArrayHandle gradient_bn_scale,
                                         DLArrayHandle gradient_bn_bias, float eps,
                                         DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                         DLStreamHandle stream_handle, ProfilerHandle p);

/* ---- Optimizer update of a whole model in one launch.  NO counterpart in the reference, whose
 *      optimizer issues one SGDOptimizerUpdate / MomentumOptimizerUpdate per parameter
 *      (python/athena/optimizer.py:95-176): dozens of launches, most of them on BatchNorm vectors
 *      that cost a launch for nanoseconds of work.  params / grads / velocities are tables of `count`
 *      array handles; velocities == NULL selects plain SGD, otherwise momentum (nesterov != 0: the
 *      Nesterov form).  Per element the arithmetic is that of the single-parameter symbols (same
 *      bits).  The table is kept in device memory per stream and uploaded again only when it changes. ---- */
int TSplit_OptimizerUpdateMulti(DLArrayHandle *params, const DLArrayHandle *grads,
                                DLArrayHandle *velocities, int count, float lr, float momentum,
                                int nesterov, DLStreamHandle stream_handle);

/* ---- No counterpart in the reference: reports how CuDNN_DLGpuBatch_Normalization obtained its batch
 *      statistics.  A forward convolution whose epilogue sums its output per channel leaves those sums
 *      noted for the memory it wrote; a BatchNorm called next on exactly that tensor (the outputs of
 *      consecutive batch micro-tensors count as one tensor), on the same stream and with no other
 *      library call in between that could have written it, takes mean and variance from them and reads
 *      the tensor once instead of twice.  *calls_served: BatchNorm calls served that way since the
 *      library was loaded; *notes_live: non-zero while such a note is pending.  Either pointer may be
 *      NULL.  TSPLIT_BN_LOOKBEHIND=0 in the environment switches the mechanism off. ---- */
int TSplit_BatchNormLookBehind(long long *calls_served, int *notes_live);

/* ---- Which routine a convolution takes.  NO counterpart in the reference (cuDNN's choice is
 *      internal there, src/ops/CudnnConv2d.cu:66).  Returns 1 when CuDNN_DLGpuConv2d (pass 0),
 *      CuDNN_DLGpuConv2d_Gradient_of_Data (pass 1) or CuDNN_DLGpuConv2d_Gradient_of_Filter (pass 2)
 *      would run a layer of this shape through the Winograd F(4x4, 3x3) routine instead of the
 *      direct implicit GEMM, 0 otherwise; for benchmarks that label their timings.  in_channels /
 *      out_channels are the filter's C and O whatever the pass.  Environment:
 *      TSPLIT_CONV_WINOGRAD=0 never, =1 wherever the shape allows (3x3, stride 1, pad 1; for
 *      passes 0 and 1 the channel count that is summed over a multiple of 16). ---- */
int TSplit_ConvTakesWinograd(int images, int in_channels, int out_channels, int height, int width,
                             int kernel_h, int kernel_w, int pad_h, int pad_w, int stride, int pass);

/* ---- Timing of the GEMM launches inside the Winograd routine.  NO counterpart in the reference;
 *      for benchmarks that report a kernel's duration measured inside their own timed region.
 *      TSplit_WinogradGemmTiming(1) makes every such launch record an event pair on its stream
 *      (not while the stream is being recorded into a graph), (2 + k) only the launches of kind k, so
 *      that a timed region carries the events of the one kernel it reports; (0) stops and forgets them.
 *      TSplit_WinogradGemmTimes waits for the launches of kind `which` (0: forward and data
 *      gradient on 128 x 128 tiles, 1: filter gradient, 2: forward and data gradient of layers that
 *      produce at most 64 channels, which run on 64 x 256 tiles, 3 / 4: forward and data gradient /
 *      filter gradient with split-bf16 products, see TSplit_SplitBf16; 5: forward and data gradient of
 *      layers with at most 256 channels, which run as ONE kernel with the transforms inside, so that its
 *      milliseconds cover the whole call; 6: filter gradient of layers with at most 128 channels, one
 *      kernel with both transforms inside, followed by the filter's final 3x3 transform: one kernel per
 *      kind) and returns
 *      their count, summed milliseconds and summed executed FLOP (2 * 36 * rows * columns * depth
 *      per launch);
 *      TSplit_WinogradGemmBytes returns their summed algorithmic bytes (both operands read once,
 *      the result written once). ---- */
int TSplit_WinogradGemmTiming(int on);
int TSplit_WinogradGemmTimes(int which, double *launches, double *ms, double *flop);
int TSplit_WinogradGemmBytes(int which, double *bytes);

/* ---- Split-bf16 products in the Winograd routine's GEMMs and in DLGpuMatrixMultiply.  NO counterpart in
 *      the reference; opt-in, off by default (every product of the default path is an fp32 matrix
 *      instruction).  With TSplit_SplitBf16(1, NULL) the GEMMs of 3x3 layers with more than 64 channels on
 *      both sides and the matrix products whose depth is a multiple of 4 split each fp32 operand exactly
 *      into three bf16 terms, a = a1 + a2 + a3, and take a product as the six bf16 x bf16 products a_i b_j
 *      with i + j <= 4, accumulated in fp32 by the bf16 matrix instruction; what is left out is below
 *      2^-23 of the product, the rounding of one fp32 multiplication.  Operands and results stay fp32 in
 *      memory.  Affects calls issued afterwards, on every stream; `was` (may be NULL) receives the
 *      previous setting.  The environment variable TSPLIT_SPLIT_BF16=1 turns it on from the start. ---- */
int TSplit_SplitBf16(int on, int *was);

/* ---- Recorded steps.  NO counterpart in the reference (every step there is issued call by
 *      call from Python); for steps made of thousands of tiny kernels (recurrent nets, small
 *      MLPs) whose time is the host's launch rate.  Between TSplit_StreamBeginRecord and
 *      TSplit_StreamEndRecord every call of this library on `stream` is recorded into a HIP graph
 *      instead of being run; TSplit_GraphLaunch replays the recorded calls on a stream, with the
 *      arrays and scalar arguments they had when recorded (a step whose scalars change - Adam's
 *      bias-correction powers - cannot be replayed).  `stream` must be a created stream, not NULL.
 *      Run the step once before recording it: first-use set-up (tap tables, scratch growth) is
 *      refused while recording and the call that needs it returns -1, as TSplit_StreamEndRecord
 *      then does.  Host-visible calls (DLStreamSync, a copy with a NULL stream, an operator with
 *      a non-NULL profiler) are not allowed while recording.  The arrays a recorded step touches
 *      must stay allocated for as long as the graph is launched. ---- */
typedef struct {
  int device_id;
  void *handle;     /* an instantiated hipGraphExec_t */
} DLGraph;
typedef DLGraph *DLGraphHandle;
int TSplit_StreamBeginRecord(DLStreamHandle stream);
int TSplit_StreamEndRecord(DLStreamHandle stream, DLGraphHandle *graph);
int TSplit_GraphLaunch(DLGraphHandle graph, DLStreamHandle stream);
int TSplit_GraphDestroy(DLGraphHandle graph);

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* TSPLIT_AMD_C_RUNTIME_API_H_ */
