// AvgPool 2-D forward and backward, NCHW float32.
//
// Semantics (python/athena/gpu_ops/AvgPool.py:27-50,139-161; src/ops/AvgPool.cu): the window
// is clipped to the image and the clipped sum is divided by kH*kW, so padding counts as
// zeros in the mean.  Forward: one thread per output element, or -- when one window covers
// the whole plane (the global pools that end ResNet and Inception) -- one wavefront per
// plane, lanes striding over the plane and a shuffle reduction, so that reads stay
// coalesced.  Backward is a gather: one thread per input element sums the dy of the windows
// that contain it in ascending window order and divides once; no atomics, no zero-fill pass.
#include "common.h"
#include "reduce.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;

struct AvgGeo {
  int H, W, pH, pW, kH, kW, pad, stride;
  float area;
};

__global__ __launch_bounds__(kThreads) void avg_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, AvgGeo g,
                                                           int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int ow = static_cast<int>(idx % g.pW);
  const int64_t t = idx / g.pW;
  const int oh = static_cast<int>(t % g.pH);
  const int64_t nc = t / g.pH;
  const float *plane = x + nc * g.H * g.W;
  int hs = oh * g.stride - g.pad, ws = ow * g.stride - g.pad;
  const int he = min(hs + g.kH, g.H), we = min(ws + g.kW, g.W);
  hs = max(hs, 0);
  ws = max(ws, 0);
  float acc = 0.f;
  for (int i = hs; i < he; ++i)
    for (int j = ws; j < we; ++j) acc += plane[i * g.W + j];
  y[idx] = acc / g.area;
}

// one wavefront per plane; the window is the whole plane
__global__ __launch_bounds__(kThreads) void avg_global_kernel(const float *__restrict__ x, float *__restrict__ y, int hw,
                                                              float area, int64_t planes) {
  const int64_t plane = static_cast<int64_t>(blockIdx.x) * (kThreads / kWave) + threadIdx.x / kWave;
  if (plane >= planes) return;       // whole waves leave together
  const int lane = threadIdx.x & (kWave - 1);
  const float *p = x + plane * hw;
  float acc = 0.f;
  for (int i = lane; i < hw; i += kWave) acc += p[i];
  acc = wave_sum(acc);
  if (lane == 0) y[plane] = acc / area;
}

__global__ __launch_bounds__(kThreads) void avg_bwd_kernel(const float *__restrict__ dy, float *__restrict__ dx, AvgGeo g,
                                                           int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int w = static_cast<int>(idx % g.W);
  const int64_t t = idx / g.W;
  const int h = static_cast<int>(t % g.H);
  const int64_t nc = t / g.H;
  const float *dplane = dy + nc * g.pH * g.pW;
  // windows oh with oh*s - pad <= h < oh*s - pad + kH
  const int oh_lo = max(0, (h + g.pad - g.kH + g.stride) / g.stride);
  const int oh_hi = min(g.pH - 1, (h + g.pad) / g.stride);
  const int ow_lo = max(0, (w + g.pad - g.kW + g.stride) / g.stride);
  const int ow_hi = min(g.pW - 1, (w + g.pad) / g.stride);
  float acc = 0.f;
  for (int oh = oh_lo; oh <= oh_hi; ++oh)
    for (int ow = ow_lo; ow <= ow_hi; ++ow) acc += dplane[oh * g.pW + ow];
  dx[idx] = acc / g.area;
}

// x: the pooled tensor's input side (shape only), y: the output side (shape only)
int check_geo(const char *who, const DLArray *x, const DLArray *y, size_t kH, size_t kW, size_t pad, size_t stride,
              AvgGeo &g) {
  TS_REQUIRE(x && y && x->data && y->data, "%s: NULL array", who);
  TS_REQUIRE(x->ndim == 4 && y->ndim == 4, "%s: arrays must be 4-D NCHW", who);
  TS_REQUIRE(kH > 0 && kW > 0 && stride > 0 && kH < (1u << 15) && kW < (1u << 15) && stride < (1u << 15),
             "%s: bad kernel/stride", who);
  TS_REQUIRE(pad < kH && pad < kW, "%s: padding must be smaller than the kernel", who);
  TS_REQUIRE(x->shape[0] == y->shape[0] && x->shape[1] == y->shape[1], "%s: N,C of input and output differ", who);
  TS_REQUIRE(x->shape[2] < (1 << 30) && x->shape[3] < (1 << 30), "%s: image too large", who);
  g.H = static_cast<int>(x->shape[2]);
  g.W = static_cast<int>(x->shape[3]);
  g.pH = static_cast<int>(y->shape[2]);
  g.pW = static_cast<int>(y->shape[3]);
  g.kH = static_cast<int>(kH);
  g.kW = static_cast<int>(kW);
  g.pad = static_cast<int>(pad);
  g.stride = static_cast<int>(stride);
  g.area = static_cast<float>(kH * kW);
  TS_REQUIRE(g.H + 2 * g.pad >= g.kH && g.W + 2 * g.pad >= g.kW, "%s: kernel larger than the padded image", who);
  const int eh = (g.H + 2 * g.pad - g.kH) / g.stride + 1, ew = (g.W + 2 * g.pad - g.kW) / g.stride + 1;
  TS_REQUIRE(g.pH == eh && g.pW == ew, "%s: output is %dx%d, expected %dx%d", who, g.pH, g.pW, eh, ew);
  return 0;
}

int avg_forward(const char *who, const DLArray *x, DLArray *y, size_t kH, size_t kW, size_t pad, size_t stride,
                DLStreamHandle sh, ProfilerHandle p) {
  AvgGeo g;
  if (check_geo(who, x, y, kH, kW, pad, stride, g)) return -1;
  hipStream_t s = stream_of(sh);
  ProfileScope ps(p, s, numel(x), numel(y), 0);
  const int64_t total = numel(y);
  if (total > 0) {
    if (g.pH == 1 && g.pW == 1 && g.pad == 0 && g.kH == g.H && g.kW == g.W) {
      const int per_block = kThreads / kWave;
      hipLaunchKernelGGL(avg_global_kernel, dim3(static_cast<unsigned>((total + per_block - 1) / per_block)),
                         dim3(kThreads), 0, s, static_cast<const float *>(x->data), static_cast<float *>(y->data),
                         g.H * g.W, g.area, total);
    } else {
      hipLaunchKernelGGL(avg_fwd_kernel, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)), dim3(kThreads),
                         0, s, static_cast<const float *>(x->data), static_cast<float *>(y->data), g, total);
    }
  }
  return ps.finish();
}

int avg_backward(const char *who, const DLArray *dy, DLArray *dx, size_t kH, size_t kW, size_t pad, size_t stride,
                 DLStreamHandle sh, ProfilerHandle p) {
  AvgGeo g;
  if (check_geo(who, dx, dy, kH, kW, pad, stride, g)) return -1;
  hipStream_t s = stream_of(sh);
  ProfileScope ps(p, s, numel(dy), numel(dx), 0);
  const int64_t total = numel(dx);
  if (total > 0)
    hipLaunchKernelGGL(avg_bwd_kernel, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       s, static_cast<const float *>(dy->data), static_cast<float *>(dx->data), g, total);
  return ps.finish();
}

}  // namespace
}  // namespace tsplit

using namespace tsplit;

extern "C" {

int DLGpuAvgerage_Pooling2d(const DLArrayHandle input, const size_t kernel_H, const size_t kernel_W,
                            DLArrayHandle output, const size_t padding, const size_t stride,
                            DLStreamHandle stream_handle, ProfilerHandle p) {
  return avg_forward("DLGpuAvgerage_Pooling2d", input, output, kernel_H, kernel_W, padding, stride, stream_handle, p);
}

int DLGpuAvgerage_Pooling2d_gradient(const DLArrayHandle gradient_Y, const size_t kernel_H, const size_t kernel_W,
                                     DLArrayHandle gradient_X, const size_t padding, const size_t stride,
                                     DLStreamHandle stream_handle, ProfilerHandle p) {
  return avg_backward("DLGpuAvgerage_Pooling2d_gradient", gradient_Y, gradient_X, kernel_H, kernel_W, padding, stride,
                      stream_handle, p);
}

int CuDNN_DLGpuAvgerage_Pooling2d(const DLArrayHandle input, const size_t kernel_H, const size_t kernel_W,
                                  DLArrayHandle output, const size_t padding, const size_t stride,
                                  DLStreamHandle stream_handle, ProfilerHandle p) {
  return avg_forward("CuDNN_DLGpuAvgerage_Pooling2d", input, output, kernel_H, kernel_W, padding, stride, stream_handle,
                     p);
}

int CuDNN_DLGpuAvgerage_Pooling2d_gradient(const DLArrayHandle output_Y, const DLArrayHandle gradient_Y,
                                           const DLArrayHandle input_X, const size_t kernel_H, const size_t kernel_W,
                                           DLArrayHandle gradient_X, const size_t padding, const size_t stride,
                                           DLStreamHandle stream_handle, ProfilerHandle p) {
  // the mean's gradient depends on neither the pooled values nor the input values
  (void)output_Y;
  (void)input_X;
  return avg_backward("CuDNN_DLGpuAvgerage_Pooling2d_gradient", gradient_Y, gradient_X, kernel_H, kernel_W, padding,
                      stride, stream_handle, p);
}

}  // extern "C"
