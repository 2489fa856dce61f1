// MaxPool 2-D forward and backward, NCHW float32.
//
// Semantics (src/ops/MaxPool.cu:3-43, python/athena/gpu_ops/MaxPool.py:8-68): the window is
// clipped to the image, the maximum is the first strict maximum in row-major scan order.
// The backward pass is a gather: one thread per input element looks at the (at most
// ceil(k/s)^2) windows that contain it and adds a window's dy when the window's argmax is
// this element -- in ascending window order, which is the accumulation order of the
// reference's scatter loop, without atomics and without a separate zero-fill pass (every dx
// element is written exactly once).  Non-overlapping windows recompute their argmax in the
// same kernel; overlapping 2x2 / 3x3 windows take their argmax from a first pass that stores
// one index per window in scratch.
// The 2x2 / stride 2 / no padding case (every VGG pool) has a vectorised path: a thread
// owns two adjacent windows, i.e. one 16-byte word from each of two input rows.
#include "common.h"
#include "fastdiv.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

struct PoolGeo {
  int H, W, pH, pW, kH, kW, pad, stride;
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

// Flat index (h*W + w) of the first strict maximum of window (oh, ow) in row-major scan order.
// K: compile-time square window -- every tap is fetched with a predicated load, so the loads
// issue together -- or 0 for run-time window sizes (a loop over the clipped window).
template <int K>
__device__ __forceinline__ int window_argmax(const float *__restrict__ plane, const PoolGeo &g, int oh, int ow) {
  const int h0 = oh * g.stride - g.pad, w0 = ow * g.stride - g.pad;
  if (K > 0) {
    constexpr int KK = K > 0 ? K : 1;
    float v[KK][KK];
    bool ok[KK][KK];
#pragma unroll
    for (int i = 0; i < K; ++i) {
      const int ih = h0 + i;
      const bool row_ok = static_cast<unsigned>(ih) < static_cast<unsigned>(g.H);
#pragma unroll
      for (int j = 0; j < K; ++j) {
        const int iw = w0 + j;
        ok[i][j] = row_ok && static_cast<unsigned>(iw) < static_cast<unsigned>(g.W);
        v[i][j] = ok[i][j] ? plane[ih * g.W + iw] : 0.f;
      }
    }
    int best = -1;
    float bv = 0.f;
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
      for (int j = 0; j < K; ++j)
        if (ok[i][j] && (best < 0 || v[i][j] > bv)) {
          bv = v[i][j];
          best = (h0 + i) * g.W + w0 + j;
        }
    return best;   // >= 0: padding is smaller than the window, so one tap is always inside
  }
  const int he = min(h0 + g.kH, g.H), we = min(w0 + g.kW, g.W);
  const int hs = max(h0, 0), ws = max(w0, 0);
  int best = hs * g.W + ws;
  float bv = plane[best];
  for (int i = hs; i < he; ++i)
    for (int j = ws; j < we; ++j) {
      const float v = plane[i * g.W + j];
      if (v > bv) {
        bv = v;
        best = i * g.W + j;
      }
    }
  return best;
}

template <int K>
__global__ __launch_bounds__(kThreads) void pool_fwd_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                            PoolGeo g, int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  int ow, oh;
  int64_t nc;
  split3(idx, total, g.div_pw, g.div_ph, nc, oh, ow);
  const float *plane = x + nc * g.H * g.W;
  y[idx] = plane[window_argmax<K>(plane, g, oh, ow)];
}

// NW: compile-time bound on the windows per axis that can contain one element (ceil(k / stride)),
// 0 for a run-time loop.
template <int K, int NW>
__global__ __launch_bounds__(kThreads) void pool_bwd_kernel(const float *__restrict__ x, const float *__restrict__ dy,
                                                            float *__restrict__ dx, PoolGeo g, int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  int w, h;
  int64_t nc;
  split3(idx, total, g.div_w, g.div_h, nc, h, w);
  const float *plane = x + nc * g.H * g.W;
  const float *dplane = dy + nc * g.pH * g.pW;
  // windows oh with oh*s - pad <= h < oh*s - pad + kH, i.e. ceil((h + pad - kH + 1) / s) <= oh <= (h + pad) / s
  const int th = h + g.pad - g.kH + g.stride, tw = w + g.pad - g.kW + g.stride;
  const int oh_lo = th > 0 ? static_cast<int>(g.div_stride.div(th)) : 0;
  const int oh_hi = min(g.pH - 1, static_cast<int>(g.div_stride.div(h + g.pad)));
  const int ow_lo = tw > 0 ? static_cast<int>(g.div_stride.div(tw)) : 0;
  const int ow_hi = min(g.pW - 1, static_cast<int>(g.div_stride.div(w + g.pad)));
  const int me = h * g.W + w;
  float acc = 0.f;
  if (NW > 0) {
#pragma unroll
    for (int a = 0; a < NW; ++a) {
#pragma unroll
      for (int b = 0; b < NW; ++b) {
        // a window beyond the last one is replaced by the last one and its result discarded
        const int oh = min(oh_lo + a, oh_hi), ow = min(ow_lo + b, ow_hi);
        const bool live = oh_lo + a <= oh_hi && ow_lo + b <= ow_hi;
        const bool mine = window_argmax<K>(plane, g, oh, ow) == me;
        const float gy = dplane[oh * g.pW + ow];
        if (live && mine) acc += gy;
      }
    }
  } else {
    for (int oh = oh_lo; oh <= oh_hi; ++oh)
      for (int ow = ow_lo; ow <= ow_hi; ++ow)
        if (window_argmax<K>(plane, g, oh, ow) == me) acc += dplane[oh * g.pW + ow];
  }
  dx[idx] = acc;
}

// Two-pass backward for overlapping windows: the argmax of every window is computed once into
// scratch (one thread per window), then every input element compares its own flat index with
// the stored argmax of the at most NW x NW windows over it.
template <int K>
__global__ __launch_bounds__(kThreads) void pool_argmax_kernel(const float *__restrict__ x, int *__restrict__ arg,
                                                               PoolGeo g, int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  int ow, oh;
  int64_t nc;
  split3(idx, total, g.div_pw, g.div_ph, nc, oh, ow);
  arg[idx] = window_argmax<K>(x + nc * g.H * g.W, g, oh, ow);
}

template <int NW>
__global__ __launch_bounds__(kThreads) void pool_bwd_from_argmax_kernel(const int *__restrict__ arg,
                                                                        const float *__restrict__ dy,
                                                                        float *__restrict__ dx, PoolGeo g,
                                                                        int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  int w, h;
  int64_t nc;
  split3(idx, total, g.div_w, g.div_h, nc, h, w);
  const int64_t wbase = nc * g.pH * g.pW;
  const int th = h + g.pad - g.kH + g.stride, tw = w + g.pad - g.kW + g.stride;
  const int oh_lo = th > 0 ? static_cast<int>(g.div_stride.div(th)) : 0;
  const int oh_hi = min(g.pH - 1, static_cast<int>(g.div_stride.div(h + g.pad)));
  const int ow_lo = tw > 0 ? static_cast<int>(g.div_stride.div(tw)) : 0;
  const int ow_hi = min(g.pW - 1, static_cast<int>(g.div_stride.div(w + g.pad)));
  const int me = h * g.W + w;
  float acc = 0.f;
#pragma unroll
  for (int a = 0; a < NW; ++a) {
#pragma unroll
    for (int b = 0; b < NW; ++b) {
      const int oh = min(oh_lo + a, oh_hi), ow = min(ow_lo + b, ow_hi);
      const bool live = oh_lo + a <= oh_hi && ow_lo + b <= ow_hi;
      const int64_t wi = wbase + oh * g.pW + ow;
      const int am = arg[wi];
      const float gy = dy[wi];
      if (live && am == me) acc += gy;
    }
  }
  dx[idx] = acc;
}

// ---- 2x2 stride 2 pad 0, W % 4 == 0, H % 2 == 0, 16-byte aligned x/dx and 8-byte aligned y/dy ----
// thread -> (plane, oh, q): input words (2oh, q) and (2oh+1, q), outputs (oh, 2q) and (oh, 2q+1)
__global__ __launch_bounds__(kThreads) void pool2x2_fwd_kernel(const f32x4 *__restrict__ x, f32x2 *__restrict__ y,
                                                               int W4, int pH, int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int q = static_cast<int>(idx % W4);
  const int64_t row = idx / W4;                 // plane * pH + oh
  const int64_t in = (row * 2) * W4 + q;        // (plane*H + 2*oh) * W4 + q, H = 2*pH
  const f32x4 a = __builtin_nontemporal_load(x + in), b = __builtin_nontemporal_load(x + in + W4);
  f32x2 o;
  // scan order: (0,0) (0,1) (1,0) (1,1); strict > keeps the first maximum
  float m = a.x;
  m = a.y > m ? a.y : m;
  m = b.x > m ? b.x : m;
  m = b.y > m ? b.y : m;
  o.x = m;
  m = a.z;
  m = a.w > m ? a.w : m;
  m = b.z > m ? b.z : m;
  m = b.w > m ? b.w : m;
  o.y = m;
  __builtin_nontemporal_store(o, y + idx);
}

__device__ __forceinline__ void route2x2(float v00, float v01, float v10, float v11, float g, float &o00, float &o01,
                                         float &o10, float &o11) {
  int k = 0;
  float m = v00;
  if (v01 > m) { m = v01; k = 1; }
  if (v10 > m) { m = v10; k = 2; }
  if (v11 > m) { m = v11; k = 3; }
  o00 = k == 0 ? g : 0.f;
  o01 = k == 1 ? g : 0.f;
  o10 = k == 2 ? g : 0.f;
  o11 = k == 3 ? g : 0.f;
}

__global__ __launch_bounds__(kThreads) void pool2x2_bwd_kernel(const f32x4 *__restrict__ x,
                                                               const f32x2 *__restrict__ dy, f32x4 *__restrict__ dx,
                                                               int W4, int64_t total) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int q = static_cast<int>(idx % W4);
  const int64_t row = idx / W4;
  const int64_t in = (row * 2) * W4 + q;
  const f32x4 a = __builtin_nontemporal_load(x + in), b = __builtin_nontemporal_load(x + in + W4);
  const f32x2 g = __builtin_nontemporal_load(dy + idx);
  float t[8];
  route2x2(a.x, a.y, b.x, b.y, g.x, t[0], t[1], t[4], t[5]);
  route2x2(a.z, a.w, b.z, b.w, g.y, t[2], t[3], t[6], t[7]);
  const f32x4 oa = {t[0], t[1], t[2], t[3]}, ob = {t[4], t[5], t[6], t[7]};
  __builtin_nontemporal_store(oa, dx + in);
  __builtin_nontemporal_store(ob, dx + in + W4);
}

inline bool aligned8(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 7) == 0; }

int check_geo(const char *who, const DLArray *x, const DLArray *y, int64_t kH, int64_t kW, int64_t pad, int64_t stride,
              PoolGeo &g) {
  TS_REQUIRE(x && y, "%s: NULL array", who);
  TS_REQUIRE(x->ndim == 4 && y->ndim == 4, "%s: arrays must be 4-D NCHW", who);
  TS_REQUIRE(kH > 0 && kW > 0 && stride > 0 && pad >= 0, "%s: bad kernel/stride/padding", who);
  TS_REQUIRE(pad < kH && pad < kW, "%s: padding must be smaller than the kernel", who);
  TS_REQUIRE(x->shape[0] == y->shape[0] && x->shape[1] == y->shape[1], "%s: N,C of input and output differ", who);
  g.H = static_cast<int>(x->shape[2]);
  g.W = static_cast<int>(x->shape[3]);
  g.pH = static_cast<int>(y->shape[2]);
  g.pW = static_cast<int>(y->shape[3]);
  g.kH = static_cast<int>(kH);
  g.kW = static_cast<int>(kW);
  g.pad = static_cast<int>(pad);
  g.stride = static_cast<int>(stride);
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

bool fast2x2(const PoolGeo &g, const void *x, const void *y, const void *dx) {
  return g.kH == 2 && g.kW == 2 && g.stride == 2 && g.pad == 0 && g.W % 4 == 0 && g.H % 2 == 0 && aligned16(x) &&
         aligned8(y) && (dx == nullptr || aligned16(dx));
}

int pool_forward(const char *who, const DLArray *x, DLArray *y, int64_t kH, int64_t kW, int64_t pad, int64_t stride,
                 DLStreamHandle sh, ProfilerHandle p) {
  PoolGeo g;
  if (check_geo(who, x, y, kH, kW, pad, stride, g)) return -1;
  hipStream_t s = stream_of(sh);
  ProfileScope ps(p, s, numel(x), numel(y), 0);
  const int64_t planes = x->shape[0] * x->shape[1];
  if (numel(y) > 0) {
    if (fast2x2(g, x->data, y->data, nullptr)) {
      const int64_t total = planes * g.pH * (g.W / 4);
      hipLaunchKernelGGL(pool2x2_fwd_kernel, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                         dim3(kThreads), 0, s, static_cast<const f32x4 *>(x->data), static_cast<f32x2 *>(y->data),
                         g.W / 4, g.pH, total);
    } else {
      const int64_t total = numel(y);
      const dim3 grid(static_cast<unsigned>((total + kThreads - 1) / kThreads)), block(kThreads);
      const float *xp = static_cast<const float *>(x->data);
      float *yp = static_cast<float *>(y->data);
      const int k = g.kH == g.kW ? g.kH : 0;
      if (k == 2)
        hipLaunchKernelGGL(pool_fwd_kernel<2>, grid, block, 0, s, xp, yp, g, total);
      else if (k == 3)
        hipLaunchKernelGGL(pool_fwd_kernel<3>, grid, block, 0, s, xp, yp, g, total);
      else
        hipLaunchKernelGGL(pool_fwd_kernel<0>, grid, block, 0, s, xp, yp, g, total);
    }
  }
  return ps.finish();
}

int pool_backward(const char *who, const DLArray *x, const DLArray *dy, DLArray *dx, int64_t kH, int64_t kW,
                  int64_t pad, int64_t stride, DLStreamHandle sh, ProfilerHandle p) {
  PoolGeo g;
  TS_REQUIRE(dx, "%s: NULL array", who);
  if (check_geo(who, x, dy, kH, kW, pad, stride, g)) return -1;
  TS_REQUIRE(dx->ndim == 4 && numel(dx) == numel(x), "%s: input gradient must have the input's shape", who);
  hipStream_t s = stream_of(sh);
  ProfileScope ps(p, s, numel(x) + numel(dy), numel(dx), 0);
  const int64_t planes = x->shape[0] * x->shape[1];
  if (numel(dx) > 0) {
    if (fast2x2(g, x->data, dy->data, dx->data)) {
      const int64_t total = planes * g.pH * (g.W / 4);
      hipLaunchKernelGGL(pool2x2_bwd_kernel, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                         dim3(kThreads), 0, s, static_cast<const f32x4 *>(x->data),
                         static_cast<const f32x2 *>(dy->data), static_cast<f32x4 *>(dx->data), g.W / 4, total);
    } else {
      const int64_t total = numel(dx);
      const dim3 grid(static_cast<unsigned>((total + kThreads - 1) / kThreads)), block(kThreads);
      const float *xp = static_cast<const float *>(x->data), *dyp = static_cast<const float *>(dy->data);
      float *dxp = static_cast<float *>(dx->data);
      const int k = g.kH == g.kW ? g.kH : 0;
      const int nw = k > 0 ? (k + g.stride - 1) / g.stride : 0;   // windows per axis over one element
      const int64_t windows = numel(dy);
      int *arg = nullptr;
      if ((k == 2 || k == 3) && (nw == 2 || nw == 3) && windows > 0) {
        arg = static_cast<int *>(scratch_get(s, 5, static_cast<size_t>(windows) * sizeof(int)));
        TS_REQUIRE(arg, "%s: out of device memory for %lld window indices", who, (long long)windows);
        if (p) p->workspace_memory = mib(windows);
        const dim3 wgrid(static_cast<unsigned>((windows + kThreads - 1) / kThreads));
        if (k == 2)
          hipLaunchKernelGGL(pool_argmax_kernel<2>, wgrid, block, 0, s, xp, arg, g, windows);
        else
          hipLaunchKernelGGL(pool_argmax_kernel<3>, wgrid, block, 0, s, xp, arg, g, windows);
        if (nw == 2)
          hipLaunchKernelGGL(pool_bwd_from_argmax_kernel<2>, grid, block, 0, s, arg, dyp, dxp, g, total);
        else
          hipLaunchKernelGGL(pool_bwd_from_argmax_kernel<3>, grid, block, 0, s, arg, dyp, dxp, g, total);
      } else if (k == 3 && nw == 1)
        hipLaunchKernelGGL((pool_bwd_kernel<3, 1>), grid, block, 0, s, xp, dyp, dxp, g, total);
      else if (k == 2 && nw == 1)
        hipLaunchKernelGGL((pool_bwd_kernel<2, 1>), grid, block, 0, s, xp, dyp, dxp, g, total);
      else
        hipLaunchKernelGGL((pool_bwd_kernel<0, 0>), grid, block, 0, s, xp, dyp, dxp, g, total);
    }
  }
  return ps.finish();
}

}  // namespace
}  // namespace tsplit

using namespace tsplit;

extern "C" {

int DLGpuMax_Pooling2d(const DLArrayHandle input, const int kernel_H, const int kernel_W, DLArrayHandle output,
                       const int padding, const int stride, DLStreamHandle stream_handle, ProfilerHandle p) {
  return pool_forward("DLGpuMax_Pooling2d", input, output, kernel_H, kernel_W, padding, stride, stream_handle, p);
}

int DLGpuMax_Pooling2d_gradient(const DLArrayHandle input, const DLArrayHandle output_grad, const int kernel_H,
                                const int kernel_W, DLArrayHandle input_grad, const int padding, const int stride,
                                DLStreamHandle stream_handle, ProfilerHandle p) {
  return pool_backward("DLGpuMax_Pooling2d_gradient", input, output_grad, input_grad, kernel_H, kernel_W, padding,
                       stride, stream_handle, p);
}

int CuDNN_DLGpuMax_Pooling2d(const DLArrayHandle input, const size_t kernel_H, const size_t kernel_W,
                             DLArrayHandle output, const size_t padding, const size_t stride,
                             DLStreamHandle stream_handle, ProfilerHandle p) {
  return pool_forward("CuDNN_DLGpuMax_Pooling2d", input, output, static_cast<int64_t>(kernel_H),
                      static_cast<int64_t>(kernel_W), static_cast<int64_t>(padding), static_cast<int64_t>(stride),
                      stream_handle, p);
}

int CuDNN_DLGpuMax_Pooling2d_gradient(const DLArrayHandle output_Y, const DLArrayHandle gradient_Y,
                                      const DLArrayHandle input_X, const size_t kernel_H, const size_t kernel_W,
                                      DLArrayHandle gradient_X, const size_t padding, const size_t stride,
                                      DLStreamHandle stream_handle, ProfilerHandle p) {
  // output_Y is not needed: the argmax is recomputed from input_X (first strict maximum), which
  // is what the plain symbol does and what the numpy reference defines.
  (void)output_Y;
  return pool_backward("CuDNN_DLGpuMax_Pooling2d_gradient", input_X, gradient_Y, gradient_X,
                       static_cast<int64_t>(kernel_H), static_cast<int64_t>(kernel_W), static_cast<int64_t>(padding),
                       static_cast<int64_t>(stride), stream_handle, p);
}

}  // extern "C"
