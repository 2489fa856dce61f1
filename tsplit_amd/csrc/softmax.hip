// Row softmax and softmax-cross-entropy (forward, gradient).
//
// One wavefront owns one row: max and sum are wave64 shuffle reductions, no LDS and no
// block barrier; a 256-thread block handles 4 rows.  The cross-entropy mean is a second,
// single-block deterministic reduction over the per-row losses (the reference does that
// mean serially in thread 0 of its only block: src/ops/SoftmaxCrossEntropy.cu:33-41).
// Long rows (a 32 000-word vocabulary) get a whole block per row instead: 16-byte loads,
// running (max, scaled sum) pairs so that the logits are read from memory once, and for the
// loss the label sums of the same pass: loss_r = (log s + m) * sum(l) - sum(l * y).
#include <mutex>

#include "common.h"
#include "reduce.h"

// Per-row losses of TSplit_SoftmaxCrossEntropyNoAlloc (below): a fixed array in the code object, so
// that call needs no device allocation.  No kernel names it: kernels get its address as an argument.
// The host code's reference to it (hipGetSymbolAddress below) is what makes the compiler give this
// static variable a symbol the runtime can find; it must NOT carry __attribute__((used)), which keeps
// the symbol local to the code object, and looking up a local symbol ends the process.
constexpr int kNoAllocMaxRows = 1 << 18;
static __device__ __align__(256) float scratch[kNoAllocMaxRows];

namespace tsplit {
namespace {

constexpr int kRowsPerBlock = 4;

__device__ __forceinline__ void row_max_sum(const float *row, int ncol, int lane, float &mx, float &sum) {
  float m = -INFINITY;
  for (int j = lane; j < ncol; j += kWave) m = fmaxf(m, row[j]);
  m = wave_max(m);
  float s = 0.f;
  for (int j = lane; j < ncol; j += kWave) s += expf(row[j] - m);
  mx = m;
  sum = wave_sum(s);
}

__global__ __launch_bounds__(256) void softmax_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                      int64_t nrow, int ncol) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / kWave;
  if (r >= nrow) return;
  const float *row = x + r * ncol;
  float m, s;
  row_max_sum(row, ncol, lane, m, s);
  const float inv = 1.f / s;
  float *out = y + r * ncol;
  for (int j = lane; j < ncol; j += kWave) out[j] = expf(row[j] - m) * inv;
}

// loss_r = sum_j label[j] * (log(sum) - (y[j] - max))
__global__ __launch_bounds__(256) void ce_rows_kernel(const float *__restrict__ y, const float *__restrict__ lab,
                                                      float *__restrict__ row_loss, int64_t nrow, int ncol) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / kWave;
  if (r >= nrow) return;
  const float *row = y + r * ncol;
  const float *l = lab + r * ncol;
  float m, s;
  row_max_sum(row, ncol, lane, m, s);
  const float lse = logf(s);
  float acc = 0.f;
  for (int j = lane; j < ncol; j += kWave) acc += l[j] * (lse - (row[j] - m));
  acc = wave_sum(acc);
  if (lane == 0) row_loss[r] = acc;
}

__global__ __launch_bounds__(256) void mean_kernel(const float *__restrict__ v, float *__restrict__ out, int64_t n) {
  __shared__ double sm[4];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += 256) acc += static_cast<double>(v[i]);
  acc = block_sum<double, 4>(acc, sm);
  if (threadIdx.x == 0) out[0] = static_cast<float>(acc / static_cast<double>(n));
}

__global__ __launch_bounds__(256) void ce_grad_kernel(const float *__restrict__ y, const float *__restrict__ lab,
                                                      const float *__restrict__ g, float *__restrict__ out,
                                                      int64_t nrow, int ncol, float inv_batch) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / kWave;
  if (r >= nrow) return;
  const float *row = y + r * ncol;
  const float *l = lab + r * ncol;
  float m, s;
  row_max_sum(row, ncol, lane, m, s);
  const float inv = 1.f / s;
  const float scale = g[0] * inv_batch;
  float *o = out + r * ncol;
  for (int j = lane; j < ncol; j += kWave) o[j] = (expf(row[j] - m) * inv - l[j]) * scale;
}

// ---- one 256-thread block per row ---------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kWideMinCols = 2048;

struct MaxSum {
  float m, s;     // s = sum of exp(x - m) over the elements seen so far
};

__device__ __forceinline__ void ms_add(MaxSum &a, float x) {
  if (x > a.m) {
    a.s = a.s * expf(a.m - x) + 1.f;      // expf(-inf) = 0 covers the first element
    a.m = x;
  } else {
    a.s += expf(x - a.m);
  }
}

__device__ __forceinline__ MaxSum ms_merge(MaxSum a, MaxSum b) {
  const float m = fmaxf(a.m, b.m);
  if (m == -INFINITY) return MaxSum{m, 0.f};
  return MaxSum{m, a.s * expf(a.m - m) + b.s * expf(b.m - m)};
}

__device__ __forceinline__ MaxSum ms_block(MaxSum v, float *smem /* 8 floats */) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) {
    MaxSum o{__shfl_xor(v.m, d, kWave), __shfl_xor(v.s, d, kWave)};
    v = ms_merge(v, o);
  }
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  if (lane == 0) {
    smem[2 * wave] = v.m;
    smem[2 * wave + 1] = v.s;
  }
  __syncthreads();
  MaxSum r{smem[0], smem[1]};
#pragma unroll
  for (int w = 1; w < 4; ++w) r = ms_merge(r, MaxSum{smem[2 * w], smem[2 * w + 1]});
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(256) void ce_rows_wide_kernel(const float *__restrict__ y, const float *__restrict__ lab,
                                                           float *__restrict__ row_loss, int ncol) {
  __shared__ float sm[8];
  __shared__ float sm2[8];
  const int64_t r = blockIdx.x;
  const f32x4 *row = reinterpret_cast<const f32x4 *>(y + r * ncol);
  const f32x4 *l = reinterpret_cast<const f32x4 *>(lab + r * ncol);
  MaxSum ms{-INFINITY, 0.f};
  float sl = 0.f, sly = 0.f;
  for (int j = threadIdx.x; j < ncol / 4; j += 256) {
    const f32x4 v = row[j], w = __builtin_nontemporal_load(l + j);
    ms_add(ms, v.x);
    ms_add(ms, v.y);
    ms_add(ms, v.z);
    ms_add(ms, v.w);
    sl += (w.x + w.y) + (w.z + w.w);
    sly += (w.x * v.x + w.y * v.y) + (w.z * v.z + w.w * v.w);
  }
  ms = ms_block(ms, sm);
  sl = block_sum<float, 4>(sl, sm2);
  __syncthreads();
  sly = block_sum<float, 4>(sly, sm2);
  if (threadIdx.x == 0) row_loss[r] = (logf(ms.s) + ms.m) * sl - sly;
}

__global__ __launch_bounds__(256) void ce_grad_wide_kernel(const float *__restrict__ y, const float *__restrict__ lab,
                                                           const float *__restrict__ g, float *__restrict__ out,
                                                           int ncol, float inv_batch) {
  __shared__ float sm[8];
  const int64_t r = blockIdx.x;
  const f32x4 *row = reinterpret_cast<const f32x4 *>(y + r * ncol);
  const f32x4 *l = reinterpret_cast<const f32x4 *>(lab + r * ncol);
  f32x4 *o = reinterpret_cast<f32x4 *>(out + r * ncol);
  MaxSum ms{-INFINITY, 0.f};
  for (int j = threadIdx.x; j < ncol / 4; j += 256) {
    const f32x4 v = row[j];
    ms_add(ms, v.x);
    ms_add(ms, v.y);
    ms_add(ms, v.z);
    ms_add(ms, v.w);
  }
  ms = ms_block(ms, sm);
  const float inv = 1.f / ms.s, scale = g[0] * inv_batch, m = ms.m;
  for (int j = threadIdx.x; j < ncol / 4; j += 256) {     // second read of the row: from L2
    const f32x4 v = row[j], w = __builtin_nontemporal_load(l + j);
    f32x4 q;
    q.x = (expf(v.x - m) * inv - w.x) * scale;
    q.y = (expf(v.y - m) * inv - w.y) * scale;
    q.z = (expf(v.z - m) * inv - w.z) * scale;
    q.w = (expf(v.w - m) * inv - w.w) * scale;
    __builtin_nontemporal_store(q, o + j);
  }
}

inline bool wide_rows(int ncol, const void *a, const void *b, const void *c) {
  return ncol >= kWideMinCols && ncol % 4 == 0 && aligned16(a) && aligned16(b) && (c == nullptr || aligned16(c));
}

inline bool rows_cols(const DLArray *a, int64_t &nrow, int &ncol) {
  if (a->ndim < 1) return false;
  nrow = 1;
  for (int i = 0; i + 1 < a->ndim; ++i) nrow *= a->shape[i];
  ncol = static_cast<int>(a->shape[a->ndim - 1]);
  return nrow > 0 && ncol > 0;
}

// ---------------------------------------------------------------- entry point that allocates nothing
// Each GPU holds its own copy of `scratch` (1 MiB) at its own address, from the time the library is
// loaded on it until the process ends.
constexpr int kNoAllocMaxDevices = 64;
std::mutex g_noalloc_mu;
float *g_noalloc_ptr[kNoAllocMaxDevices] = {};

}  // namespace

// Device address of `scratch` on device `dev`, looked up once per device with that device current.
// (In host code the array's name is only a handle for this lookup, never a device address.)
float *softmax_noalloc_scratch(int dev) {
  if (dev < 0 || dev >= kNoAllocMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lk(g_noalloc_mu);
  if (g_noalloc_ptr[dev]) return g_noalloc_ptr[dev];
  int caller_dev = -1;
  if (hipGetDevice(&caller_dev) != hipSuccess) {
    (void)hipGetLastError();
    caller_dev = -1;
  }
  if (hipSetDevice(dev) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  void *ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (caller_dev >= 0 && caller_dev != dev) (void)hipSetDevice(caller_dev);   // the caller's device stays current
  if (e != hipSuccess || ptr == nullptr) {
    (void)hipGetLastError();
    std::fprintf(stderr, "[libc_runtime_api] hipGetSymbolAddress(scratch) failed on device %d: %s\n", dev,
                 hipGetErrorString(e));
    return nullptr;
  }
  g_noalloc_ptr[dev] = static_cast<float *>(ptr);
  return g_noalloc_ptr[dev];
}

// Called from the library's per-device init call so that the first operator call finds the address.
void softmax_noalloc_setup(int dev) { (void)softmax_noalloc_scratch(dev); }

}  // namespace tsplit

using namespace tsplit;

extern "C" {

int TSplit_SoftmaxCrossEntropyNoAlloc(const DLArrayHandle input_a, const DLArrayHandle input_b, DLArrayHandle output,
                                      DLStreamHandle stream_handle) {
  const char *who = "TSplit_SoftmaxCrossEntropyNoAlloc";
  TS_REQUIRE(input_a && input_b && output, "%s: NULL array", who);
  TS_REQUIRE(numel(input_a) == numel(input_b), "%s: logits and labels differ in size", who);
  TS_REQUIRE(numel(output) >= 1, "%s: output must hold one element", who);
  int64_t nrow;
  int ncol;
  TS_REQUIRE(rows_cols(input_a, nrow, ncol), "%s: empty input", who);
  TS_REQUIRE(nrow <= kNoAllocMaxRows, "%s: %lld rows, the fixed scratch array holds %d; use DLGpuSoftmaxCrossEntropy", who,
             static_cast<long long>(nrow), kNoAllocMaxRows);
  float *row_loss = softmax_noalloc_scratch(input_a->ctx.device_id);
  TS_REQUIRE(row_loss, "%s: the scratch array of device %d could not be located", who, input_a->ctx.device_id);
  hipStream_t s = stream_of(stream_handle);
  // every row's entry is written by the first kernel before the second reads rows [0, nrow): nothing of
  // an earlier call's contents is read, so nothing has to be cleared
  const unsigned blocks = static_cast<unsigned>((nrow + kRowsPerBlock - 1) / kRowsPerBlock);
  if (wide_rows(ncol, input_a->data, input_b->data, nullptr))
    hipLaunchKernelGGL(ce_rows_wide_kernel, dim3(static_cast<unsigned>(nrow)), dim3(256), 0, s,
                       static_cast<const float *>(input_a->data), static_cast<const float *>(input_b->data), row_loss, ncol);
  else
    hipLaunchKernelGGL(ce_rows_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const float *>(input_a->data),
                       static_cast<const float *>(input_b->data), row_loss, nrow, ncol);
  hipLaunchKernelGGL(mean_kernel, dim3(1), dim3(256), 0, s, row_loss, static_cast<float *>(output->data), nrow);
  const hipError_t le = hipGetLastError();
  TS_REQUIRE(le == hipSuccess, "%s: kernel launch failed: %s", who, hipGetErrorString(le));
  return 0;
}

int DLGpuSoftmax(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input && output, "DLGpuSoftmax: NULL array");
  TS_REQUIRE(input->ndim == 2 && output->ndim == 2, "DLGpuSoftmax: 2-D arrays only");
  TS_REQUIRE(numel(input) == numel(output), "DLGpuSoftmax: sizes differ");
  int64_t nrow;
  int ncol;
  TS_REQUIRE(rows_cols(input, nrow, ncol), "DLGpuSoftmax: empty input");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input), numel(output), 0);
  const unsigned blocks = static_cast<unsigned>((nrow + kRowsPerBlock - 1) / kRowsPerBlock);
  hipLaunchKernelGGL(softmax_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const float *>(input->data),
                     static_cast<float *>(output->data), nrow, ncol);
  return ps.finish();
}

int DLGpuSoftmaxCrossEntropy(const DLArrayHandle input_a, const DLArrayHandle input_b, DLArrayHandle output,
                             DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input_a && input_b && output, "DLGpuSoftmaxCrossEntropy: NULL array");
  TS_REQUIRE(numel(input_a) == numel(input_b), "DLGpuSoftmaxCrossEntropy: logits and labels differ in size");
  TS_REQUIRE(numel(output) >= 1, "DLGpuSoftmaxCrossEntropy: output must hold one element");
  int64_t nrow;
  int ncol;
  TS_REQUIRE(rows_cols(input_a, nrow, ncol), "DLGpuSoftmaxCrossEntropy: empty input");
  hipStream_t s = stream_of(stream_handle);
  float *row_loss = static_cast<float *>(scratch_get(s, 0, static_cast<size_t>(nrow) * 4));
  TS_REQUIRE(row_loss, "DLGpuSoftmaxCrossEntropy: no scratch memory");
  ProfileScope ps(p, s, 2 * numel(input_a), 1, nrow);
  const unsigned blocks = static_cast<unsigned>((nrow + kRowsPerBlock - 1) / kRowsPerBlock);
  if (wide_rows(ncol, input_a->data, input_b->data, nullptr) && nrow < (1ll << 31))
    hipLaunchKernelGGL(ce_rows_wide_kernel, dim3(static_cast<unsigned>(nrow)), dim3(256), 0, s,
                       static_cast<const float *>(input_a->data), static_cast<const float *>(input_b->data), row_loss, ncol);
  else
    hipLaunchKernelGGL(ce_rows_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const float *>(input_a->data),
                       static_cast<const float *>(input_b->data), row_loss, nrow, ncol);
  hipLaunchKernelGGL(mean_kernel, dim3(1), dim3(256), 0, s, row_loss, static_cast<float *>(output->data), nrow);
  return ps.finish();
}

int DLGpuSoftmaxCrossEntropy_Gradient(const DLArrayHandle input_a, const DLArrayHandle input_b,
                                      const DLArrayHandle input_c, DLArrayHandle output,
                                      DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input_a && input_b && input_c && output, "DLGpuSoftmaxCrossEntropy_Gradient: NULL array");
  TS_REQUIRE(numel(input_a) == numel(input_b) && numel(input_a) == numel(output),
             "DLGpuSoftmaxCrossEntropy_Gradient: operand sizes differ");
  TS_REQUIRE(numel(input_c) >= 1, "DLGpuSoftmaxCrossEntropy_Gradient: upstream gradient is empty");
  int64_t nrow;
  int ncol;
  TS_REQUIRE(rows_cols(input_a, nrow, ncol), "DLGpuSoftmaxCrossEntropy_Gradient: empty input");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, 2 * numel(input_a) + 1, numel(output), 0);
  const unsigned blocks = static_cast<unsigned>((nrow + kRowsPerBlock - 1) / kRowsPerBlock);
  // scaled by 1/shape[0] (not 1/rows), as src/ops/SoftmaxCrossEntropy.cu:101,120 does
  const float inv_batch = 1.f / static_cast<float>(input_a->shape[0]);
  if (wide_rows(ncol, input_a->data, input_b->data, output->data) && nrow < (1ll << 31))
    hipLaunchKernelGGL(ce_grad_wide_kernel, dim3(static_cast<unsigned>(nrow)), dim3(256), 0, s,
                       static_cast<const float *>(input_a->data), static_cast<const float *>(input_b->data),
                       static_cast<const float *>(input_c->data), static_cast<float *>(output->data), ncol, inv_batch);
  else
    hipLaunchKernelGGL(ce_grad_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const float *>(input_a->data),
                       static_cast<const float *>(input_b->data), static_cast<const float *>(input_c->data),
                       static_cast<float *>(output->data), nrow, ncol, inv_batch);
  return ps.finish();
}

}  // extern "C"
