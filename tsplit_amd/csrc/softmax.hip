// Row softmax and softmax-cross-entropy (forward, gradient).
//
// One wavefront owns one row: max and sum are wave64 shuffle reductions, no LDS and no
// block barrier; a 256-thread block handles 4 rows.  The cross-entropy mean is a second,
// single-block deterministic reduction over the per-row losses (the reference does that
// mean serially in thread 0 of its only block: src/ops/SoftmaxCrossEntropy.cu:33-41).
#include "common.h"
#include "reduce.h"

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

inline bool rows_cols(const DLArray *a, int64_t &nrow, int &ncol) {
  if (a->ndim < 1) return false;
  nrow = 1;
  for (int i = 0; i + 1 < a->ndim; ++i) nrow *= a->shape[i];
  ncol = static_cast<int>(a->shape[a->ndim - 1]);
  return nrow > 0 && ncol > 0;
}

}  // namespace
}  // namespace tsplit

using namespace tsplit;

extern "C" {

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
  hipLaunchKernelGGL(ce_grad_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const float *>(input_a->data),
                     static_cast<const float *>(input_b->data), static_cast<const float *>(input_c->data),
                     static_cast<float *>(output->data), nrow, ncol, 1.f / static_cast<float>(input_a->shape[0]));
  return ps.finish();
}

}  // extern "C"
