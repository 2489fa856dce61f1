// Copying concat / slice kernels (the zero-copy batch split needs no kernel at all).
//
// Concat along `axis` of two tensors writes `outer` output rows, each the row of the first input
// (axis_extent * inner contiguous elements) followed by the row of the second, in one launch; the
// gradient copies one input's part of every row back.  Rows move as 16-byte words whenever lengths,
// strides, offsets and base pointers allow, else element-wise.  Slice is a general n-D
// window copy; shapes travel as kernel arguments (the reference stages them through three
// synchronous host-to-device copies per call: src/ops/Slice.cu:48-56).
#include "common.h"
#include "fastdiv.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;

template <typename W>
__global__ __launch_bounds__(kThreads) void rows_copy_kernel(const W *__restrict__ src, W *__restrict__ dst,
                                                             FastDiv len, uint32_t src_stride, uint32_t dst_stride,
                                                             int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  uint32_t r, j;
  if (total < (1ll << 32)) {
    r = len.div(static_cast<uint32_t>(idx));
    j = static_cast<uint32_t>(idx) - r * len.d;
  } else {
    r = static_cast<uint32_t>(idx / len.d);
    j = static_cast<uint32_t>(idx - static_cast<int64_t>(r) * len.d);
  }
  dst[static_cast<int64_t>(r) * dst_stride + j] = src[static_cast<int64_t>(r) * src_stride + j];
}

// copies `rows` rows of `len` floats; strides in floats
void rows_copy(const float *src, float *dst, int64_t rows, int64_t len, int64_t src_stride, int64_t dst_stride,
               hipStream_t s) {
  if (rows <= 0 || len <= 0) return;
  const bool vec = len % 4 == 0 && src_stride % 4 == 0 && dst_stride % 4 == 0 && aligned16(src) && aligned16(dst);
  if (vec) {
    const int64_t total = rows * (len / 4);
    hipLaunchKernelGGL(rows_copy_kernel<float4>, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                       dim3(kThreads), 0, s, reinterpret_cast<const float4 *>(src), reinterpret_cast<float4 *>(dst),
                       FastDiv(static_cast<uint32_t>(len / 4)), static_cast<uint32_t>(src_stride / 4),
                       static_cast<uint32_t>(dst_stride / 4), total);
  } else {
    const int64_t total = rows * len;
    hipLaunchKernelGGL(rows_copy_kernel<float>, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                       dim3(kThreads), 0, s, src, dst, FastDiv(static_cast<uint32_t>(len)),
                       static_cast<uint32_t>(src_stride), static_cast<uint32_t>(dst_stride), total);
  }
}

// Concat of two tensors in one launch: output row r = x row r (lx words) followed by y row r (ly words).
template <typename W>
__global__ __launch_bounds__(kThreads) void concat_rows_kernel(const W *__restrict__ x, const W *__restrict__ y,
                                                               W *__restrict__ dst, FastDiv row, uint32_t lx,
                                                               uint32_t ly, int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  uint32_t r, j;
  if (total < (1ll << 32)) {
    r = row.div(static_cast<uint32_t>(idx));
    j = static_cast<uint32_t>(idx) - r * row.d;
  } else {
    r = static_cast<uint32_t>(idx / row.d);
    j = static_cast<uint32_t>(idx - static_cast<int64_t>(r) * row.d);
  }
  dst[idx] = j < lx ? x[static_cast<int64_t>(r) * lx + j] : y[static_cast<int64_t>(r) * ly + (j - lx)];
}

void concat_rows(const float *x, const float *y, float *dst, int64_t rows, int64_t lx, int64_t ly, hipStream_t s) {
  if (rows <= 0 || lx + ly <= 0) return;
  const bool vec = lx % 4 == 0 && ly % 4 == 0 && aligned16(x) && aligned16(y) && aligned16(dst);
  if (vec) {
    const int64_t total = rows * ((lx + ly) / 4);
    hipLaunchKernelGGL(concat_rows_kernel<float4>, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                       dim3(kThreads), 0, s, reinterpret_cast<const float4 *>(x), reinterpret_cast<const float4 *>(y),
                       reinterpret_cast<float4 *>(dst), FastDiv(static_cast<uint32_t>((lx + ly) / 4)),
                       static_cast<uint32_t>(lx / 4), static_cast<uint32_t>(ly / 4), total);
  } else {
    const int64_t total = rows * (lx + ly);
    hipLaunchKernelGGL(concat_rows_kernel<float>, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                       dim3(kThreads), 0, s, x, y, dst, FastDiv(static_cast<uint32_t>(lx + ly)),
                       static_cast<uint32_t>(lx), static_cast<uint32_t>(ly), total);
  }
}

constexpr int kMaxDim = 8;
struct SliceGeo {
  int ndim;
  int64_t small[kMaxDim];   // shape of the window tensor
  int64_t big[kMaxDim];     // shape of the full tensor
  int64_t begin[kMaxDim];
};

// window[o] = full[begin + o]
__global__ __launch_bounds__(kThreads) void slice_kernel(const float *__restrict__ full, float *__restrict__ window,
                                                         SliceGeo g, int64_t total) {
  const int64_t o = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (o >= total) return;
  int64_t t = o, src = 0, mul = 1;
  for (int d = g.ndim - 1; d >= 0; --d) {
    const int64_t c = t % g.small[d];
    t /= g.small[d];
    src += (c + g.begin[d]) * mul;
    mul *= g.big[d];
  }
  window[o] = full[src];
}

// full[o] = inside the window ? window[o - begin] : 0
__global__ __launch_bounds__(kThreads) void slice_grad_kernel(const float *__restrict__ window,
                                                              float *__restrict__ full, SliceGeo g, int64_t total) {
  const int64_t o = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (o >= total) return;
  int64_t t = o, src = 0, mul = 1;
  bool inside = true;
  for (int d = g.ndim - 1; d >= 0; --d) {
    const int64_t c = t % g.big[d];
    t /= g.big[d];
    const int64_t w = c - g.begin[d];
    inside = inside && w >= 0 && w < g.small[d];
    src += w * mul;
    mul *= g.small[d];
  }
  full[o] = inside ? window[src] : 0.f;
}

int slice_geo(const char *who, const DLArray *full, const DLArray *window, const int64_t *begin, SliceGeo &g) {
  TS_REQUIRE(full && window && begin, "%s: NULL argument", who);
  TS_REQUIRE(full->ndim == window->ndim, "%s: ranks differ", who);
  TS_REQUIRE(full->ndim >= 1 && full->ndim <= kMaxDim, "%s: rank %d not supported", who, full->ndim);
  g.ndim = full->ndim;
  for (int d = 0; d < g.ndim; ++d) {
    g.small[d] = window->shape[d];
    g.big[d] = full->shape[d];
    g.begin[d] = begin[d];
    TS_REQUIRE(begin[d] >= 0 && begin[d] + window->shape[d] <= full->shape[d], "%s: window leaves the tensor on axis %d",
               who, d);
  }
  return 0;
}

inline const float *cf(const DLArray *a) { return static_cast<const float *>(a->data); }
inline float *mf(DLArray *a) { return static_cast<float *>(a->data); }

}  // namespace
}  // namespace tsplit

using namespace tsplit;

extern "C" {

int DLGpuConcat(const DLArrayHandle input_x, const DLArrayHandle input_y, DLArrayHandle output, int axis,
                DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input_x && input_y && output, "DLGpuConcat: NULL array");
  const int nd = input_x->ndim;
  TS_REQUIRE(input_y->ndim == nd && output->ndim == nd, "DLGpuConcat: ranks differ");
  TS_REQUIRE(axis >= 0 && axis < nd, "DLGpuConcat: axis %d out of range", axis);
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < nd; ++i) {
    if (i == axis) continue;
    TS_REQUIRE(input_x->shape[i] == input_y->shape[i] && input_x->shape[i] == output->shape[i],
               "DLGpuConcat: shapes differ on axis %d", i);
    (i < axis ? outer : inner) *= input_x->shape[i];
  }
  const int64_t ax = input_x->shape[axis], ay = input_y->shape[axis];
  TS_REQUIRE(output->shape[axis] == ax + ay, "DLGpuConcat: output extent on the axis must be %lld", (long long)(ax + ay));
  TS_REQUIRE((ax + ay) * inner < (1ll << 32), "DLGpuConcat: row too long");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input_x) + numel(input_y), numel(output), 0);
  concat_rows(cf(input_x), cf(input_y), mf(output), outer, ax * inner, ay * inner, s);
  return ps.finish();
}

int DLGpuConcat_gradient(const DLArrayHandle output_gradient, DLArrayHandle input_gradient, int axis, int id,
                         DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(output_gradient && input_gradient, "DLGpuConcat_gradient: NULL array");
  const int nd = output_gradient->ndim;
  TS_REQUIRE(input_gradient->ndim == nd, "DLGpuConcat_gradient: ranks differ");
  TS_REQUIRE(axis >= 0 && axis < nd, "DLGpuConcat_gradient: axis %d out of range", axis);
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < nd; ++i) {
    if (i == axis) continue;
    TS_REQUIRE(input_gradient->shape[i] == output_gradient->shape[i], "DLGpuConcat_gradient: shapes differ on axis %d", i);
    (i < axis ? outer : inner) *= output_gradient->shape[i];
  }
  const int64_t ai = input_gradient->shape[axis], ao = output_gradient->shape[axis];
  TS_REQUIRE(ai <= ao, "DLGpuConcat_gradient: input extent exceeds the output's");
  TS_REQUIRE(ao * inner < (1ll << 32), "DLGpuConcat_gradient: row too long");
  // id 0: leading part; id 1: trailing part (src/ops/Concat.cu:183-190)
  const int64_t offset = id == 1 ? (ao - ai) * inner : 0;
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(output_gradient), numel(input_gradient), 0);
  rows_copy(cf(output_gradient) + offset, mf(input_gradient), outer, ai * inner, ao * inner, ai * inner, s);
  return ps.finish();
}

int DLGpuSlice(const DLArrayHandle in_arr, DLArrayHandle out_arr, int64_t *begin_pos, DLStreamHandle stream_handle,
               ProfilerHandle p) {
  SliceGeo g;
  if (slice_geo("DLGpuSlice", in_arr, out_arr, begin_pos, g)) return -1;
  hipStream_t s = stream_of(stream_handle);
  const int64_t total = numel(out_arr);
  ProfileScope ps(p, s, numel(in_arr), total, 0);
  if (total > 0)
    hipLaunchKernelGGL(slice_kernel, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       s, cf(in_arr), mf(out_arr), g, total);
  return ps.finish();
}

int DLGpuSliceGradient(const DLArrayHandle in_arr, DLArrayHandle out_arr, int64_t *begin_pos,
                       DLStreamHandle stream_handle, ProfilerHandle p) {
  // in_arr is the gradient of the window, out_arr the (larger) gradient of the sliced tensor
  SliceGeo g;
  if (slice_geo("DLGpuSliceGradient", out_arr, in_arr, begin_pos, g)) return -1;
  hipStream_t s = stream_of(stream_handle);
  const int64_t total = numel(out_arr);
  ProfileScope ps(p, s, numel(in_arr), total, 0);
  if (total > 0)
    hipLaunchKernelGGL(slice_grad_kernel, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                       dim3(kThreads), 0, s, cf(in_arr), mf(out_arr), g, total);
  return ps.finish();
}

}  // extern "C"
