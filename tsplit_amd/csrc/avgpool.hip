// AvgPool 2-D forward and backward, NCHW float32.
//
// Semantics (python/athena/gpu_ops/AvgPool.py:27-50,139-161; src/ops/AvgPool.cu): the window
// is clipped to the image and the clipped sum is divided by kH*kW, so padding counts as
// zeros in the mean.  Forward: one thread per output element, or -- when one window covers
// the whole plane (the global pools that end ResNet and Inception) -- one wavefront per
// plane, lanes striding over the plane and a shuffle reduction, so that reads stay
// coalesced.  Backward is a gather: one thread per input element sums the dy of the windows
// that contain it in ascending window order and divides once; no atomics, no zero-fill pass.
#include <algorithm>

#include "common.h"
#include "fastdiv.h"
#include "reduce.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;

struct AvgGeo {
  int H, W, pH, pW, kH, kW, pad, stride;
  float area;
  FastDiv div_pw, div_ph, div_w, div_h, div_stride;
};

// idx -> (plane, row, col) for rows of `w` elements and planes of `h` rows; 32-bit fast path
__device__ __forceinline__ void split3(int64_t idx, int64_t total, const FastDiv &w, const FastDiv &h, int64_t &plane,
                                       int &row, int &col) {
  if (total < (1ll << 32)) {
    const uint32_t i = static_cast<uint32_t>(idx);
    const uint32_t t = w.div(i);
    col = static_cast<int>(i - t * w.d);
    const uint32_t pl = h.div(t);
    row = static_cast<int>(t - pl * h.d);
    plane = pl;
  } else {
    col = static_cast<int>(idx % w.d);
    const int64_t t = idx / w.d;
    row = static_cast<int>(t % h.d);
    plane = t / h.d;
  }
}

// K: compile-time square window (all taps are fetched with predicated loads issued together),
// or 0 for run-time window sizes (a loop over the clipped window).
template <int K>
__global__ __launch_bounds__(kThreads) void avg_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, AvgGeo g,
                                                           int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  int ow, oh;
  int64_t nc;
  split3(idx, total, g.div_pw, g.div_ph, nc, oh, ow);
  const float *plane = x + nc * g.H * g.W;
  const int h0 = oh * g.stride - g.pad, w0 = ow * g.stride - g.pad;
  float acc = 0.f;
  if (K > 0) {
#pragma unroll
    for (int i = 0; i < K; ++i) {
      const int ih = h0 + i;
      const bool row_ok = static_cast<unsigned>(ih) < static_cast<unsigned>(g.H);
#pragma unroll
      for (int j = 0; j < K; ++j) {
        const int iw = w0 + j;
        const bool ok = row_ok && static_cast<unsigned>(iw) < static_cast<unsigned>(g.W);
        const float v = ok ? plane[ih * g.W + iw] : 0.f;
        acc += v;
      }
    }
  } else {
    const int he = min(h0 + g.kH, g.H), we = min(w0 + g.kW, g.W);
    const int hs = max(h0, 0), ws = max(w0, 0);
    for (int i = hs; i < he; ++i)
      for (int j = ws; j < we; ++j) acc += plane[i * g.W + j];
  }
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

// NW: compile-time bound on the windows per axis that can contain one element, ceil(k / stride)
// (predicated loads issued together), or 0 for a run-time loop.
template <int NW>
__global__ __launch_bounds__(kThreads) void avg_bwd_kernel(const float *__restrict__ dy, float *__restrict__ dx, AvgGeo g,
                                                           int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  int w, h;
  int64_t nc;
  split3(idx, total, g.div_w, g.div_h, nc, h, w);
  const float *dplane = dy + nc * g.pH * g.pW;
  // windows oh with oh*s - pad <= h < oh*s - pad + kH, i.e. ceil((h + pad - kH + 1) / s) <= oh <= (h + pad) / s
  const int th = h + g.pad - g.kH + g.stride, tw = w + g.pad - g.kW + g.stride;
  const int oh_lo = th > 0 ? static_cast<int>(g.div_stride.div(th)) : 0;
  const int oh_hi = min(g.pH - 1, static_cast<int>(g.div_stride.div(h + g.pad)));
  const int ow_lo = tw > 0 ? static_cast<int>(g.div_stride.div(tw)) : 0;
  const int ow_hi = min(g.pW - 1, static_cast<int>(g.div_stride.div(w + g.pad)));
  float acc = 0.f;
  if (NW > 0) {
#pragma unroll
    for (int a = 0; a < NW; ++a) {
      const int oh = oh_lo + a;
#pragma unroll
      for (int b = 0; b < NW; ++b) {
        const int ow = ow_lo + b;
        const float v = (oh <= oh_hi && ow <= ow_hi) ? dplane[oh * g.pW + ow] : 0.f;
        acc += v;
      }
    }
  } else {
    for (int oh = oh_lo; oh <= oh_hi; ++oh)
      for (int ow = ow_lo; ow <= ow_hi; ++ow) acc += dplane[oh * g.pW + ow];
  }
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
  g.div_pw = FastDiv(static_cast<uint32_t>(g.pW > 0 ? g.pW : 1));
  g.div_ph = FastDiv(static_cast<uint32_t>(g.pH > 0 ? g.pH : 1));
  g.div_w = FastDiv(static_cast<uint32_t>(g.W > 0 ? g.W : 1));
  g.div_h = FastDiv(static_cast<uint32_t>(g.H > 0 ? g.H : 1));
  g.div_stride = FastDiv(static_cast<uint32_t>(g.stride));
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
      const dim3 grid(static_cast<unsigned>((total + kThreads - 1) / kThreads)), block(kThreads);
      const float *xp = static_cast<const float *>(x->data);
      float *yp = static_cast<float *>(y->data);
      const int k = g.kH == g.kW ? g.kH : 0;
      if (k == 2)
        hipLaunchKernelGGL(avg_fwd_kernel<2>, grid, block, 0, s, xp, yp, g, total);
      else if (k == 3)
        hipLaunchKernelGGL(avg_fwd_kernel<3>, grid, block, 0, s, xp, yp, g, total);
      else
        hipLaunchKernelGGL(avg_fwd_kernel<0>, grid, block, 0, s, xp, yp, g, total);
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
  if (total > 0) {
    const dim3 grid(static_cast<unsigned>((total + kThreads - 1) / kThreads)), block(kThreads);
    const float *dyp = static_cast<const float *>(dy->data);
    float *dxp = static_cast<float *>(dx->data);
    const int nw = (std::max(g.kH, g.kW) + g.stride - 1) / g.stride;   // windows per axis over one element
    if (nw == 1)
      hipLaunchKernelGGL(avg_bwd_kernel<1>, grid, block, 0, s, dyp, dxp, g, total);
    else if (nw == 2)
      hipLaunchKernelGGL(avg_bwd_kernel<2>, grid, block, 0, s, dyp, dxp, g, total);
    else if (nw == 3)
      hipLaunchKernelGGL(avg_bwd_kernel<3>, grid, block, 0, s, dyp, dxp, g, total);
    else
      hipLaunchKernelGGL(avg_bwd_kernel<0>, grid, block, 0, s, dyp, dxp, g, total);
  }
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
