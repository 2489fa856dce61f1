// Training-mode spatial BatchNorm, forward and backward, NCHW float32.
//
// Per channel the N*H*W elements sit in N contiguous planes of H*W.  Both directions are
// two streaming passes over a (split, channel) grid:
//   forward : [stats]  partial (sum x, sum x^2) per block          -> scratch (double)
//             [apply]  every block folds the partials of its channel, then y = a*x + b
//   backward: [reduce] partial (sum dy, sum dy*x, sum x, sum x^2)   -> scratch (double)
//             [dx]     folds them, then dx = k1*dy + k2*x + k3; split 0 writes dgamma/dbeta
// Fused forms (TSplit_BatchNormRelu*): the apply pass stores max(a*x + b, 0) and the backward
// passes gate dy with relu'(a*x + b) recomputed from x, so the Relu costs no pass of its own.
// Threads walk a per-channel virtual index (in 16-byte words when H*W % 4 == 0) that is
// mapped to (plane, offset) with a multiply-shift division, so consecutive lanes read
// consecutive words of one plane.  Per-thread accumulation is float32 over a few hundred
// values; everything across threads and blocks is folded in double, which keeps
// E[x^2]-E[x]^2 and sum(dy*x)-mean*sum(dy) accurate.
// Algorithmic traffic is 8 B/elem forward and 12 B/elem backward; these kernels move
// 12 and 20 B/elem (x, and dy, are read by both passes).
// Small channels (N*H*W <= 16384: 14x14 and smaller planes at batch 64, 17x17 at batch 32) take
// one-pass kernels instead: one block per channel keeps the channel's values in registers, so
// x (and dy) are read once - the algorithmic 8 and 12 B/elem - in one launch per direction.
#include "common.h"
#include "fastdiv.h"
#include "reduce.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
// words a block of the read-only passes streams (four times as many ran a quarter slower on 56x56 planes)
constexpr uint32_t kStatsWords = 16 * kThreads;
constexpr int kReadAhead = 4;   // words per thread and array in flight in the read-only passes

struct Geo {
  FastDiv plane;      // divides by words per plane
  uint32_t wpp;       // words per plane (H*W / VEC)
  uint32_t words;     // words per channel (N * wpp)
  uint32_t chunk;     // words per block
  int C;
};

typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int VEC>
struct Word;
template <>
struct Word<4> {
  using T = f32x4;
};
template <>
struct Word<1> {
  using T = float;
};

template <int VEC>
__device__ __forceinline__ int64_t word_addr(const Geo &g, uint32_t i, int c) {
  const uint32_t n = g.plane.div(i);
  const uint32_t j = i - n * g.wpp;
  return (static_cast<int64_t>(n) * g.C + c) * g.wpp + j;
}

__device__ __forceinline__ void acc2(const f32x4 &v, float &s, float &q) {
  s += (v.x + v.y) + (v.z + v.w);
  q += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
}
__device__ __forceinline__ void acc2(const float &v, float &s, float &q) {
  s += v;
  q += v * v;
}
__device__ __forceinline__ void acc_dot(const f32x4 &a, const f32x4 &b, float &s, float &d) {
  s += (a.x + a.y) + (a.z + a.w);
  d += (a.x * b.x + a.y * b.y) + (a.z * b.z + a.w * b.w);
}
__device__ __forceinline__ void acc_dot(const float &a, const float &b, float &s, float &d) {
  s += a;
  d += a * b;
}
__device__ __forceinline__ f32x4 axpb(const f32x4 &x, float a, float b) {
  const f32x4 r = {a * x.x + b, a * x.y + b, a * x.z + b, a * x.w + b};
  return r;
}
__device__ __forceinline__ float axpb(const float &x, float a, float b) { return a * x + b; }
// Relu and its reference gradient factor (sign(z)+1)/2 (0.5 at z == 0)
__device__ __forceinline__ float relu1(float z) { return fmaxf(z, 0.f); }
__device__ __forceinline__ f32x4 relu_w(const f32x4 &z) {
  const f32x4 r = {relu1(z.x), relu1(z.y), relu1(z.z), relu1(z.w)};
  return r;
}
__device__ __forceinline__ float relu_w(const float &z) { return relu1(z); }
__device__ __forceinline__ float gate1(float z) { return z > 0.f ? 1.f : (z < 0.f ? 0.f : 0.5f); }
// dy * relu'(a*x + b)
__device__ __forceinline__ f32x4 gated(const f32x4 &dy, const f32x4 &x, float a, float b) {
  const f32x4 r = {dy.x * gate1(a * x.x + b), dy.y * gate1(a * x.y + b), dy.z * gate1(a * x.z + b),
                   dy.w * gate1(a * x.w + b)};
  return r;
}
__device__ __forceinline__ float gated(const float &dy, const float &x, float a, float b) {
  return dy * gate1(a * x + b);
}
__device__ __forceinline__ f32x4 lin2(const f32x4 &dy, const f32x4 &x, float k1, float k2, float k3) {
  const f32x4 r = {k1 * dy.x + k2 * x.x + k3, k1 * dy.y + k2 * x.y + k3, k1 * dy.z + k2 * x.z + k3,
                   k1 * dy.w + k2 * x.w + k3};
  return r;
}
__device__ __forceinline__ float lin2(const float &dy, const float &x, float k1, float k2, float k3) {
  return k1 * dy + k2 * x + k3;
}

// partial layout: [C][S][NQ] doubles
template <int VEC>
__global__ __launch_bounds__(kThreads) void bn_stats_kernel(const float *__restrict__ x, double *__restrict__ part,
                                                            Geo g, int S) {
  using W = typename Word<VEC>::T;
  __shared__ double sm[2 * kWaves];
  const int c = blockIdx.y, s = blockIdx.x;
  const uint32_t begin = s * g.chunk;
  const uint32_t end = min(begin + g.chunk, g.words);
  const W *xw = reinterpret_cast<const W *>(x);
  float sum = 0.f, sq = 0.f;
  uint32_t i = begin + threadIdx.x;
  // a read-only stream needs more bytes in flight than a read + write one: kReadAhead words per thread
  for (; i + (kReadAhead - 1) * kThreads < end; i += kReadAhead * kThreads) {
    W v[kReadAhead];
#pragma unroll
    for (int u = 0; u < kReadAhead; ++u) v[u] = __builtin_nontemporal_load(xw + word_addr<VEC>(g, i + u * kThreads, c));
#pragma unroll
    for (int u = 0; u < kReadAhead; ++u) acc2(v[u], sum, sq);
  }
  for (; i < end; i += kThreads) acc2(__builtin_nontemporal_load(xw + word_addr<VEC>(g, i, c)), sum, sq);
  // within a wave in float (a lane has summed a few hundred values), across the waves and beyond in
  // double; one barrier, so that the block's tail is short beside its stream
  sum = wave_sum(sum);
  sq = wave_sum(sq);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  if (lane == 0) {
    sm[w] = static_cast<double>(sum);
    sm[kWaves + w] = static_cast<double>(sq);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double ds = sm[0], dq = sm[kWaves];
#pragma unroll
    for (int j = 1; j < kWaves; ++j) {
      ds += sm[j];
      dq += sm[kWaves + j];
    }
    double *o = part + (static_cast<int64_t>(c) * S + s) * 2;
    o[0] = ds;
    o[1] = dq;
  }
}

// Folds the partials of channel c (the pair k at part[(c * part_c + k * part_k) * 2]; fixed order per
// thread, fixed tree: deterministic) into the coefficients of y = a*x + b, coef[2c] and coef[2c + 1],
// and the saved statistics.  One block per channel, so that the streaming pass behind it starts with
// two loads instead of a reduction in every block.
template <bool RELU>
__global__ __launch_bounds__(kThreads) void bn_coef_kernel(const double *__restrict__ part, int S, int64_t part_c,
                                                           int64_t part_k, const float *__restrict__ gamma,
                                                           const float *__restrict__ beta, float eps, double inv_m,
                                                           float *__restrict__ coef, float *__restrict__ save_mean,
                                                           float *__restrict__ save_istd) {
  __shared__ double sm[kWaves];
  const int c = blockIdx.x;
  double s = 0.0, q = 0.0;
  for (int k = threadIdx.x; k < S; k += kThreads) {
    s += part[(c * part_c + k * part_k) * 2];
    q += part[(c * part_c + k * part_k) * 2 + 1];
  }
  if (S > 1) {
    s = block_sum<double, kWaves>(s, sm);
    q = block_sum<double, kWaves>(q, sm);
  }
  if (threadIdx.x == 0) {
    const double mean = s * inv_m;
    double var = q * inv_m - mean * mean;
    if (var < 0.0) var = 0.0;
    double istd = 1.0 / sqrt(var + static_cast<double>(eps));
    double mean_used = mean;
    if (RELU) {
      // the fused backward pass rebuilds a and b from the saved float statistics and must see
      // the same sign of a*x + b: derive the coefficients from the rounded values here too
      mean_used = static_cast<double>(static_cast<float>(mean));
      istd = static_cast<double>(static_cast<float>(istd));
    }
    const double a = static_cast<double>(gamma[c]) * istd;
    coef[2 * c] = static_cast<float>(a);
    coef[2 * c + 1] = static_cast<float>(static_cast<double>(beta[c]) - mean_used * a);
    if (save_mean) save_mean[c] = static_cast<float>(mean);
    if (save_istd) save_istd[c] = static_cast<float>(istd);
  }
}

// y = a*x + b (then Relu) over a (split, channel) grid: for planes too short for the plane-major kernel
// and for arrays without 16-byte words
template <int VEC, bool RELU>
__global__ __launch_bounds__(kThreads) void bn_apply_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                            const float *__restrict__ coef, Geo g) {
  using W = typename Word<VEC>::T;
  const int c = blockIdx.y;
  const float a = coef[2 * c], b = coef[2 * c + 1];
  const uint32_t begin = blockIdx.x * g.chunk;
  const uint32_t end = min(begin + g.chunk, g.words);
  const W *xw = reinterpret_cast<const W *>(x);
  W *yw = reinterpret_cast<W *>(y);
  // second and last touch of x, only touch of y: non-temporal both ways
  uint32_t i = begin + threadIdx.x;
  for (; i + kThreads < end; i += 2 * kThreads) {
    const int64_t a0 = word_addr<VEC>(g, i, c), a1 = word_addr<VEC>(g, i + kThreads, c);
    const W v0 = __builtin_nontemporal_load(xw + a0), v1 = __builtin_nontemporal_load(xw + a1);
    __builtin_nontemporal_store(RELU ? relu_w(axpb(v0, a, b)) : axpb(v0, a, b), yw + a0);
    __builtin_nontemporal_store(RELU ? relu_w(axpb(v1, a, b)) : axpb(v1, a, b), yw + a1);
  }
  for (; i < end; i += kThreads) {
    const int64_t a0 = word_addr<VEC>(g, i, c);
    const W z = axpb(__builtin_nontemporal_load(xw + a0), a, b);
    __builtin_nontemporal_store(RELU ? relu_w(z) : z, yw + a0);
  }
}

// The same in the order the array lies in memory: thread -> one 16-byte word of the whole array, its
// channel from two multiply-shift divisions.  The blocks in flight then cover one contiguous window of
// the array, as an elementwise kernel's do, instead of a few hundred windows 4*C*H*W bytes apart:
// 6.3 - 6.5 TB/s against 5.3 - 5.5 for the (split, channel) order on the VGG shapes.
struct PlaneGeo {
  FastDiv wpp;      // divides by words per plane
  FastDiv chans;    // divides by C
  uint32_t words;   // words of the array
};
__device__ __forceinline__ uint32_t word_channel(const PlaneGeo &g, uint32_t i) {
  const uint32_t plane = g.wpp.div(i);
  return plane - g.chans.div(plane) * g.chans.d;
}
template <bool RELU>
__global__ __launch_bounds__(kThreads) void bn_apply_plane_kernel(const f32x4 *__restrict__ x, f32x4 *__restrict__ y,
                                                                  const float *__restrict__ coef, PlaneGeo g) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= g.words) return;
  const uint32_t c = word_channel(g, i);
  const float a = coef[2 * c], b = coef[2 * c + 1];
  const f32x4 z = axpb(__builtin_nontemporal_load(x + i), a, b);
  __builtin_nontemporal_store(RELU ? relu_w(z) : z, y + i);
}

// partials per block: sum dy, sum dy*x, sum x, sum x^2
// RELU: dy is the gradient behind a fused Relu; it is gated with relu'(a*x + b), a and b rebuilt
// from the saved statistics (gamma, beta, save_mean, save_istd must be given).
template <int VEC, bool STATS, bool RELU>
__global__ __launch_bounds__(kThreads) void bn_bwd_reduce_kernel(const float *__restrict__ dy,
                                                                 const float *__restrict__ x,
                                                                 double *__restrict__ part, Geo g, int S,
                                                                 const float *__restrict__ gamma,
                                                                 const float *__restrict__ beta,
                                                                 const float *__restrict__ save_mean,
                                                                 const float *__restrict__ save_istd) {
  using W = typename Word<VEC>::T;
  __shared__ double sm[4 * kWaves];
  const int c = blockIdx.y, s = blockIdx.x;
  float ga = 0.f, gb = 0.f;
  if (RELU) {
    // the same float expressions as the forward pass, so that the sign of a*x + b is the same
    const double a = static_cast<double>(gamma[c]) * static_cast<double>(save_istd[c]);
    ga = static_cast<float>(a);
    gb = static_cast<float>(static_cast<double>(beta[c]) - static_cast<double>(save_mean[c]) * a);
  }
  const uint32_t begin = s * g.chunk;
  const uint32_t end = min(begin + g.chunk, g.words);
  const W *xw = reinterpret_cast<const W *>(x);
  const W *dw = reinterpret_cast<const W *>(dy);
  float sdy = 0.f, sdx = 0.f, sx = 0.f, sq = 0.f;
  uint32_t i = begin + threadIdx.x;
  for (; i + (kReadAhead - 1) * kThreads < end; i += kReadAhead * kThreads) {
    W xv[kReadAhead], dv[kReadAhead];
#pragma unroll
    for (int u = 0; u < kReadAhead; ++u) {
      const int64_t at = word_addr<VEC>(g, i + u * kThreads, c);
      xv[u] = xw[at];
      dv[u] = dw[at];
    }
#pragma unroll
    for (int u = 0; u < kReadAhead; ++u) {
      if (RELU) dv[u] = gated(dv[u], xv[u], ga, gb);
      acc_dot(dv[u], xv[u], sdy, sdx);
      if (STATS) acc2(xv[u], sx, sq);
    }
  }
  for (; i < end; i += kThreads) {
    const int64_t a0 = word_addr<VEC>(g, i, c);
    W x0 = xw[a0], d0 = dw[a0];
    if (RELU) d0 = gated(d0, x0, ga, gb);
    acc_dot(d0, x0, sdy, sdx);
    if (STATS) acc2(x0, sx, sq);
  }
  // as in bn_stats_kernel: float within a wave, double from there on, one barrier
  sdy = wave_sum(sdy);
  sdx = wave_sum(sdx);
  if (STATS) {
    sx = wave_sum(sx);
    sq = wave_sum(sq);
  }
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  if (lane == 0) {
    sm[w] = static_cast<double>(sdy);
    sm[kWaves + w] = static_cast<double>(sdx);
    sm[2 * kWaves + w] = static_cast<double>(sx);
    sm[3 * kWaves + w] = static_cast<double>(sq);
  }
  __syncthreads();
  if (threadIdx.x < 4) {
    double r = sm[threadIdx.x * kWaves];
#pragma unroll
    for (int j = 1; j < kWaves; ++j) r += sm[threadIdx.x * kWaves + j];
    part[(static_cast<int64_t>(c) * S + s) * 4 + threadIdx.x] = r;
  }
}

// Folds the backward partials of channel c into the coefficients of dx = k1*dy + k2*x + k3 (coef[5c ..
// 5c+2]; with RELU also a and b of the gate, coef[5c+3], coef[5c+4]) and writes dgamma, dbeta.
template <bool RELU>
__global__ __launch_bounds__(kThreads) void bn_bwd_coef_kernel(const double *__restrict__ part, int S,
                                                               const float *__restrict__ gamma,
                                                               const float *__restrict__ beta, float eps, double inv_m,
                                                               const float *__restrict__ save_mean,
                                                               const float *__restrict__ save_istd,
                                                               float *__restrict__ coef, float *__restrict__ dgamma,
                                                               float *__restrict__ dbeta) {
  __shared__ double sm[kWaves];
  const int c = blockIdx.x;
  double sdy = 0.0, sdx = 0.0, sx = 0.0, sq = 0.0;
  for (int k = threadIdx.x; k < S; k += kThreads) {
    const double *o = part + (static_cast<int64_t>(c) * S + k) * 4;
    sdy += o[0];
    sdx += o[1];
    sx += o[2];
    sq += o[3];
  }
  if (S > 1) {
    sdy = block_sum<double, kWaves>(sdy, sm);
    sdx = block_sum<double, kWaves>(sdx, sm);
    sx = block_sum<double, kWaves>(sx, sm);
    sq = block_sum<double, kWaves>(sq, sm);
  }
  if (threadIdx.x == 0) {
    double mean, istd;
    if (save_mean && save_istd) {
      mean = static_cast<double>(save_mean[c]);
      istd = static_cast<double>(save_istd[c]);
    } else {
      mean = sx * inv_m;
      double var = sq * inv_m - mean * mean;
      if (var < 0.0) var = 0.0;
      istd = 1.0 / sqrt(var + static_cast<double>(eps));
    }
    const double dbias = sdy;
    const double dscale = (sdx - mean * sdy) * istd;
    const double k1 = static_cast<double>(gamma[c]) * istd;
    const double k2 = -k1 * istd * dscale * inv_m;
    const double k3 = -k1 * dbias * inv_m - k2 * mean;
    float *o = coef + 5 * c;
    o[0] = static_cast<float>(k1);
    o[1] = static_cast<float>(k2);
    o[2] = static_cast<float>(k3);
    if (RELU) {
      o[3] = static_cast<float>(k1);   // a = gamma * istd
      o[4] = static_cast<float>(static_cast<double>(beta[c]) - mean * k1);
    }
    if (dgamma) dgamma[c] = static_cast<float>(dscale);
    if (dbeta) dbeta[c] = static_cast<float>(dbias);
  }
}

template <int VEC, bool RELU>
__global__ __launch_bounds__(kThreads) void bn_bwd_dx_kernel(const float *__restrict__ dy, const float *__restrict__ x,
                                                             float *__restrict__ dx, const float *__restrict__ coef,
                                                             Geo g) {
  using W = typename Word<VEC>::T;
  const int c = blockIdx.y;
  const float k1 = coef[5 * c], k2 = coef[5 * c + 1], k3 = coef[5 * c + 2];
  const float ga = RELU ? coef[5 * c + 3] : 0.f, gb = RELU ? coef[5 * c + 4] : 0.f;
  const uint32_t begin = blockIdx.x * g.chunk;
  const uint32_t end = min(begin + g.chunk, g.words);
  const W *xw = reinterpret_cast<const W *>(x);
  const W *dw = reinterpret_cast<const W *>(dy);
  W *ow = reinterpret_cast<W *>(dx);
  uint32_t i = begin + threadIdx.x;
  for (; i + kThreads < end; i += 2 * kThreads) {
    const int64_t a0 = word_addr<VEC>(g, i, c), a1 = word_addr<VEC>(g, i + kThreads, c);
    const W x0 = __builtin_nontemporal_load(xw + a0), d0 = __builtin_nontemporal_load(dw + a0);
    const W x1 = __builtin_nontemporal_load(xw + a1), d1 = __builtin_nontemporal_load(dw + a1);
    __builtin_nontemporal_store(lin2(RELU ? gated(d0, x0, ga, gb) : d0, x0, k1, k2, k3), ow + a0);
    __builtin_nontemporal_store(lin2(RELU ? gated(d1, x1, ga, gb) : d1, x1, k1, k2, k3), ow + a1);
  }
  for (; i < end; i += kThreads) {
    const int64_t a0 = word_addr<VEC>(g, i, c);
    const W x0 = __builtin_nontemporal_load(xw + a0), d0 = __builtin_nontemporal_load(dw + a0);
    __builtin_nontemporal_store(lin2(RELU ? gated(d0, x0, ga, gb) : d0, x0, k1, k2, k3), ow + a0);
  }
}

// in the order of memory, as bn_apply_plane_kernel
template <bool RELU>
__global__ __launch_bounds__(kThreads) void bn_bwd_dx_plane_kernel(const f32x4 *__restrict__ dy, const f32x4 *__restrict__ x,
                                                                   f32x4 *__restrict__ dx, const float *__restrict__ coef,
                                                                   PlaneGeo g) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= g.words) return;
  const uint32_t c = word_channel(g, i);
  const float k1 = coef[5 * c], k2 = coef[5 * c + 1], k3 = coef[5 * c + 2];
  const float ga = RELU ? coef[5 * c + 3] : 0.f, gb = RELU ? coef[5 * c + 4] : 0.f;
  const f32x4 xv = __builtin_nontemporal_load(x + i), dv = __builtin_nontemporal_load(dy + i);
  __builtin_nontemporal_store(lin2(RELU ? gated(dv, xv, ga, gb) : dv, xv, k1, k2, k3), dx + i);
}

// ---- one block per channel, the channel in registers ------------------------------------
constexpr int kOnePassMax = 64 * kThreads;      // elements per channel

// element e of channel c: plane e / HW, offset e % HW
__device__ __forceinline__ int64_t chan_addr(const FastDiv &hw, uint32_t e, int c, int C) {
  const uint32_t n = hw.div(e);
  return (static_cast<int64_t>(n) * C + c) * hw.d + (e - n * hw.d);
}

// R: values per thread (compile-time bound of the register arrays)
template <int R, bool RELU>
__global__ __launch_bounds__(kThreads) void bn_fwd_onepass_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                  const float *__restrict__ gamma,
                                                                  const float *__restrict__ beta, FastDiv hw, int C,
                                                                  uint32_t m, float eps, double inv_m,
                                                                  float *__restrict__ save_mean,
                                                                  float *__restrict__ save_istd) {
  __shared__ double sm[kWaves];
  __shared__ float coef[2];
  const int c = blockIdx.x;
  float v[R];
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t e = r * kThreads + threadIdx.x;
    v[r] = e < m ? __builtin_nontemporal_load(x + chan_addr(hw, e, c, C)) : 0.f;
    s += v[r];
  }
  const double mean = block_sum<double, kWaves>(static_cast<double>(s), sm) * inv_m;
  // the values are at hand: the variance is the mean squared distance from the mean
  const float mf32 = static_cast<float>(mean);
  float q = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t e = r * kThreads + threadIdx.x;
    const float d = v[r] - mf32;
    q += e < m ? d * d : 0.f;
  }
  double var = block_sum<double, kWaves>(static_cast<double>(q), sm) * inv_m;
  // (x - float(mean)) leaves out mean - float(mean): var = E[(x - mf)^2] - (mean - mf)^2
  const double dm = mean - static_cast<double>(mf32);
  var -= dm * dm;
  if (var < 0.0) var = 0.0;
  if (threadIdx.x == 0) {
    double istd = 1.0 / sqrt(var + static_cast<double>(eps));
    double mean_used = mean;
    if (RELU) {      // as in bn_apply_kernel: coefficients from the rounded statistics the backward pass will read
      mean_used = static_cast<double>(static_cast<float>(mean));
      istd = static_cast<double>(static_cast<float>(istd));
    }
    const double a = static_cast<double>(gamma[c]) * istd;
    coef[0] = static_cast<float>(a);
    coef[1] = static_cast<float>(static_cast<double>(beta[c]) - mean_used * a);
    if (save_mean) save_mean[c] = static_cast<float>(mean);
    if (save_istd) save_istd[c] = static_cast<float>(istd);
  }
  __syncthreads();
  const float a = coef[0], b = coef[1];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t e = r * kThreads + threadIdx.x;
    if (e < m) {
      const float z = a * v[r] + b;
      __builtin_nontemporal_store(RELU ? relu1(z) : z, y + chan_addr(hw, e, c, C));
    }
  }
}

template <int R, bool STATS, bool RELU>
__global__ __launch_bounds__(kThreads) void bn_bwd_onepass_kernel(const float *__restrict__ dy, const float *__restrict__ x,
                                                                  float *__restrict__ dx, const float *__restrict__ gamma,
                                                                  const float *__restrict__ beta, FastDiv hw, int C,
                                                                  uint32_t m, float eps, double inv_m,
                                                                  const float *__restrict__ save_mean,
                                                                  const float *__restrict__ save_istd,
                                                                  float *__restrict__ dgamma, float *__restrict__ dbeta) {
  __shared__ double sm[kWaves];
  __shared__ float coef[3];
  const int c = blockIdx.x;
  float ga = 0.f, gb = 0.f;
  if (RELU) {
    const double a = static_cast<double>(gamma[c]) * static_cast<double>(save_istd[c]);
    ga = static_cast<float>(a);
    gb = static_cast<float>(static_cast<double>(beta[c]) - static_cast<double>(save_mean[c]) * a);
  }
  float xv[R], dv[R];
  float sdy = 0.f, sdx = 0.f, sx = 0.f, sq = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t e = r * kThreads + threadIdx.x;
    const bool ok = e < m;
    const int64_t at = ok ? chan_addr(hw, e, c, C) : 0;
    xv[r] = ok ? __builtin_nontemporal_load(x + at) : 0.f;
    dv[r] = ok ? __builtin_nontemporal_load(dy + at) : 0.f;
    if (RELU) dv[r] = gated(dv[r], xv[r], ga, gb);
    acc_dot(dv[r], xv[r], sdy, sdx);
    if (STATS) acc2(xv[r], sx, sq);
  }
  const double r0 = block_sum<double, kWaves>(static_cast<double>(sdy), sm);
  const double r1 = block_sum<double, kWaves>(static_cast<double>(sdx), sm);
  double r2 = 0.0, r3 = 0.0;
  if (STATS) {
    r2 = block_sum<double, kWaves>(static_cast<double>(sx), sm);
    r3 = block_sum<double, kWaves>(static_cast<double>(sq), sm);
  }
  if (threadIdx.x == 0) {
    double mean, istd;
    if (!STATS) {
      mean = static_cast<double>(save_mean[c]);
      istd = static_cast<double>(save_istd[c]);
    } else {
      mean = r2 * inv_m;
      double var = r3 * inv_m - mean * mean;
      if (var < 0.0) var = 0.0;
      istd = 1.0 / sqrt(var + static_cast<double>(eps));
    }
    const double dbias = r0;
    const double dscale = (r1 - mean * r0) * istd;
    const double k1 = static_cast<double>(gamma[c]) * istd;
    const double k2 = -k1 * istd * dscale * inv_m;
    const double k3 = -k1 * dbias * inv_m - k2 * mean;
    coef[0] = static_cast<float>(k1);
    coef[1] = static_cast<float>(k2);
    coef[2] = static_cast<float>(k3);
    if (dgamma) dgamma[c] = static_cast<float>(dscale);
    if (dbeta) dbeta[c] = static_cast<float>(dbias);
  }
  __syncthreads();
  const float k1 = coef[0], k2 = coef[1], k3 = coef[2];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t e = r * kThreads + threadIdx.x;
    if (e < m) __builtin_nontemporal_store(lin2(dv[r], xv[r], k1, k2, k3), dx + chan_addr(hw, e, c, C));
  }
}

inline bool one_pass_ok(const DLArray *x) {
  const int64_t m = x->shape[0] * x->shape[2] * x->shape[3];
  return m > 0 && m <= kOnePassMax && numel(x) < (1ll << 31);
}

struct Plan {
  Geo g;
  int S;
  int vec;
  int64_t m;
};

// words_per_block: how much of a channel one block streams
bool make_plan(const DLArray *x, bool all_aligned, uint32_t words_per_block, int max_blocks, Plan &pl) {
  if (x->ndim != 4) return false;
  const int64_t N = x->shape[0], C = x->shape[1], HW = x->shape[2] * x->shape[3];
  if (N <= 0 || C <= 0 || HW <= 0) return false;
  pl.m = N * HW;
  pl.vec = (HW % 4 == 0 && all_aligned) ? 4 : 1;
  const int64_t words = pl.m / pl.vec;
  if (words >= (1ll << 31) || C > 65535) return false;
  int64_t S = (words + words_per_block - 1) / words_per_block;
  const int64_t cap = max_blocks / C > 0 ? max_blocks / C : 1;
  if (S > cap) S = cap;
  if (S < 1) S = 1;
  int64_t chunk = (words + S - 1) / S;
  chunk = (chunk + kThreads - 1) / kThreads * kThreads;
  S = (words + chunk - 1) / chunk;
  pl.S = static_cast<int>(S);
  pl.g.wpp = static_cast<uint32_t>(HW / pl.vec);
  pl.g.plane = FastDiv(pl.g.wpp);
  pl.g.words = static_cast<uint32_t>(words);
  pl.g.chunk = static_cast<uint32_t>(chunk);
  pl.g.C = static_cast<int>(C);
  return true;
}

// dst[c * 2], dst[c * 2 + 1] = the sums of channel c's S partial pairs (one block per channel)
__global__ __launch_bounds__(kThreads) void bn_sums_fold_kernel(const double *__restrict__ part, int S,
                                                                double *__restrict__ dst) {
  __shared__ double sm[kWaves];
  const int c = blockIdx.x;
  double s = 0.0, q = 0.0;
  for (int k = threadIdx.x; k < S; k += kThreads) {
    s += part[(static_cast<int64_t>(c) * S + k) * 2];
    q += part[(static_cast<int64_t>(c) * S + k) * 2 + 1];
  }
  s = block_sum<double, kWaves>(s, sm);
  q = block_sum<double, kWaves>(q, sm);
  if (threadIdx.x == 0) {
    dst[c * 2] = s;
    dst[c * 2 + 1] = q;
  }
}

// The memory-order streaming kernels take arrays of 16-byte words, fewer than 2^32 of them.
inline bool plane_major_ok(const Plan &pl, const DLArray *x, PlaneGeo &pg, unsigned &blocks) {
  if (pl.vec != 4) return false;
  const int64_t words = x->shape[0] * x->shape[1] * static_cast<int64_t>(pl.g.wpp);
  if (words >= (1ll << 32) - kThreads) return false;
  pg.wpp = FastDiv(pl.g.wpp);
  pg.chans = FastDiv(static_cast<uint32_t>(x->shape[1]));
  pg.words = static_cast<uint32_t>(words);
  blocks = static_cast<unsigned>((words + kThreads - 1) / kThreads);
  return true;
}

// ---------------------------------------------------------------- BatchNorm + Relu + 2x2 / stride 2 max pooling
// One pass each way for the three nodes that end a VGG stage: the forward pass reads the BatchNorm's input and
// writes only the pooled tensor (the activation in front of the pooling is never written: 5 B per element
// instead of the 13 of BatchNorm+Relu and pooling on their own), the gradient reads that input and the
// pooled gradient twice and writes the input's gradient (14 B per element instead of 29).  A thread owns the
// 2x2 windows under VECW consecutive columns of two rows (VECW = 4: two windows, 16-byte loads; 2: one window).
// Element (plane, h, w) of x at x[(plane * H + h) * W + w], plane = image * C + channel; H and W even.
struct PoolGeo {
  FastDiv wq;       // words per row: W / VECW
  FastDiv rows;     // pooled rows per plane: H / 2
  FastDiv chans;    // C
  uint32_t words;   // words of the whole array: N * C * (H / 2) * (W / VECW)
  int H, W;
};
template <int VECW>
struct PoolWord;
template <>
struct PoolWord<4> {
  using In = f32x4;
  using Out = float __attribute__((ext_vector_type(2)));
};
template <>
struct PoolWord<2> {
  using In = float __attribute__((ext_vector_type(2)));
  using Out = float;
};
// word i -> its plane, channel and the offsets of its top row in x and of its pooled values
template <int VECW>
__device__ __forceinline__ void pool_locate(const PoolGeo &g, uint32_t i, uint32_t &c, int64_t &top, int64_t &pooled) {
  const uint32_t row = g.wq.div(i), q = i - row * g.wq.d;       // row = plane * (H / 2) + pooled row
  const uint32_t plane = g.rows.div(row), ph = row - plane * g.rows.d;
  c = plane - g.chans.div(plane) * g.chans.d;
  top = (static_cast<int64_t>(plane) * g.H + 2 * ph) * g.W + VECW * q;
  pooled = static_cast<int64_t>(row) * (g.W / 2) + (VECW / 2) * q;
}
__device__ __forceinline__ float max4(float a, float b, float c, float d) { return fmaxf(fmaxf(a, b), fmaxf(c, d)); }

template <int VECW>
__global__ __launch_bounds__(kThreads) void bn_relu_pool_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                const float *__restrict__ coef, PoolGeo g) {
  using In = typename PoolWord<VECW>::In;
  using Out = typename PoolWord<VECW>::Out;
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= g.words) return;
  uint32_t c;
  int64_t top, pooled;
  pool_locate<VECW>(g, i, c, top, pooled);
  const float a = coef[2 * c], b = coef[2 * c + 1];
  const In r0 = __builtin_nontemporal_load(reinterpret_cast<const In *>(x + top));
  const In r1 = __builtin_nontemporal_load(reinterpret_cast<const In *>(x + top + g.W));
  if constexpr (VECW == 4) {
    const f32x4 z0 = relu_w(axpb(r0, a, b)), z1 = relu_w(axpb(r1, a, b));
    const Out o = {max4(z0.x, z0.y, z1.x, z1.y), max4(z0.z, z0.w, z1.z, z1.w)};
    __builtin_nontemporal_store(o, reinterpret_cast<Out *>(y + pooled));
  } else {
    const float o = max4(relu1(a * r0.x + b), relu1(a * r0.y + b), relu1(a * r1.x + b), relu1(a * r1.y + b));
    __builtin_nontemporal_store(o, y + pooled);
  }
}

// The gradient that reaches the BatchNorm's output through pooling and Relu, for the 2x2 window with the
// BatchNorm outputs (z00 z01 / z10 z11): the pooled gradient goes to the first maximum of relu(z) in
// row-major order (the pooling gradient's tie rule), times the Relu gradient's factor there.
__device__ __forceinline__ void pool_route(float z00, float z01, float z10, float z11, float dyp, float &g00, float &g01,
                                           float &g10, float &g11) {
  const float r00 = relu1(z00), r01 = relu1(z01), r10 = relu1(z10), r11 = relu1(z11);
  const float m = max4(r00, r01, r10, r11);
  const int at = r00 == m ? 0 : r01 == m ? 1 : r10 == m ? 2 : 3;
  g00 = at == 0 ? dyp * gate1(z00) : 0.f;
  g01 = at == 1 ? dyp * gate1(z01) : 0.f;
  g10 = at == 2 ? dyp * gate1(z10) : 0.f;
  g11 = at == 3 ? dyp * gate1(z11) : 0.f;
}
// one word: the gradients g0 (top row), g1 (bottom row) behind the loaded rows r0, r1
template <int VECW>
__device__ __forceinline__ void pool_word_grads(const typename PoolWord<VECW>::In &r0, const typename PoolWord<VECW>::In &r1,
                                                const typename PoolWord<VECW>::Out &dyp, float a, float b,
                                                typename PoolWord<VECW>::In &g0, typename PoolWord<VECW>::In &g1) {
  float t[8];   // a vector's elements cannot be bound to references
  if constexpr (VECW == 4) {
    pool_route(a * r0.x + b, a * r0.y + b, a * r1.x + b, a * r1.y + b, dyp.x, t[0], t[1], t[4], t[5]);
    pool_route(a * r0.z + b, a * r0.w + b, a * r1.z + b, a * r1.w + b, dyp.y, t[2], t[3], t[6], t[7]);
    g0 = f32x4{t[0], t[1], t[2], t[3]};
    g1 = f32x4{t[4], t[5], t[6], t[7]};
  } else {
    pool_route(a * r0.x + b, a * r0.y + b, a * r1.x + b, a * r1.y + b, dyp, t[0], t[1], t[2], t[3]);
    g0 = typename PoolWord<VECW>::In{t[0], t[1]};
    g1 = typename PoolWord<VECW>::In{t[2], t[3]};
  }
}

// partials per block (split s of channel c): sum g, sum g*x, 0, 0 in the layout of bn_bwd_reduce_kernel;
// word j of a channel: image j / wpp, pooled row and column word from the rest
template <int VECW>
__global__ __launch_bounds__(kThreads) void bn_pool_bwd_reduce_kernel(const float *__restrict__ dyp, const float *__restrict__ x,
                                                                      double *__restrict__ part, PoolGeo g, FastDiv per_plane,
                                                                      uint32_t words_c, uint32_t chunk, int S,
                                                                      const float *__restrict__ gamma,
                                                                      const float *__restrict__ beta,
                                                                      const float *__restrict__ save_mean,
                                                                      const float *__restrict__ save_istd) {
  using In = typename PoolWord<VECW>::In;
  using Out = typename PoolWord<VECW>::Out;
  __shared__ double sm[2 * kWaves];
  const int c = blockIdx.y, s = blockIdx.x;
  // the same float expressions as the forward pass, so that the sign of a*x + b is the same
  const double ad = static_cast<double>(gamma[c]) * static_cast<double>(save_istd[c]);
  const float a = static_cast<float>(ad);
  const float b = static_cast<float>(static_cast<double>(beta[c]) - static_cast<double>(save_mean[c]) * ad);
  const uint32_t wpp = per_plane.d;
  const uint32_t begin = s * chunk, end = min(begin + chunk, words_c);
  float sg = 0.f, sgx = 0.f;
  for (uint32_t j = begin + threadIdx.x; j < end; j += kThreads) {
    const uint32_t n = per_plane.div(j), rest = j - n * wpp;
    const uint32_t ph = g.wq.div(rest), q = rest - ph * g.wq.d;
    const int64_t plane = static_cast<int64_t>(n) * g.chans.d + c;
    const int64_t top = (plane * g.H + 2 * ph) * g.W + VECW * q;
    const int64_t pooled = (plane * g.rows.d + ph) * (g.W / 2) + (VECW / 2) * q;
    const In r0 = *reinterpret_cast<const In *>(x + top), r1 = *reinterpret_cast<const In *>(x + top + g.W);
    const Out d = *reinterpret_cast<const Out *>(dyp + pooled);
    In g0, g1;
    pool_word_grads<VECW>(r0, r1, d, a, b, g0, g1);
    if constexpr (VECW == 4) {
      sg += (g0.x + g0.y) + (g0.z + g0.w) + (g1.x + g1.y) + (g1.z + g1.w);
      sgx += (g0.x * r0.x + g0.y * r0.y) + (g0.z * r0.z + g0.w * r0.w) + (g1.x * r1.x + g1.y * r1.y) + (g1.z * r1.z + g1.w * r1.w);
    } else {
      sg += (g0.x + g0.y) + (g1.x + g1.y);
      sgx += (g0.x * r0.x + g0.y * r0.y) + (g1.x * r1.x + g1.y * r1.y);
    }
  }
  sg = wave_sum(sg);
  sgx = wave_sum(sgx);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  if (lane == 0) {
    sm[w] = static_cast<double>(sg);
    sm[kWaves + w] = static_cast<double>(sgx);
  }
  __syncthreads();
  if (threadIdx.x < 4) {
    double r = 0.0;
    if (threadIdx.x < 2) {
      r = sm[threadIdx.x * kWaves];
#pragma unroll
      for (int k = 1; k < kWaves; ++k) r += sm[threadIdx.x * kWaves + k];
    }
    part[(static_cast<int64_t>(c) * S + s) * 4 + threadIdx.x] = r;
  }
}

// dx = k1*g + k2*x + k3 in the order of memory; coef[5c ..] as bn_bwd_coef_kernel<true> leaves them
template <int VECW>
__global__ __launch_bounds__(kThreads) void bn_pool_bwd_dx_kernel(const float *__restrict__ dyp, const float *__restrict__ x,
                                                                  float *__restrict__ dx, const float *__restrict__ coef,
                                                                  PoolGeo g) {
  using In = typename PoolWord<VECW>::In;
  using Out = typename PoolWord<VECW>::Out;
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= g.words) return;
  uint32_t c;
  int64_t top, pooled;
  pool_locate<VECW>(g, i, c, top, pooled);
  const float k1 = coef[5 * c], k2 = coef[5 * c + 1], k3 = coef[5 * c + 2], a = coef[5 * c + 3], b = coef[5 * c + 4];
  const In r0 = __builtin_nontemporal_load(reinterpret_cast<const In *>(x + top));
  const In r1 = __builtin_nontemporal_load(reinterpret_cast<const In *>(x + top + g.W));
  const Out d = __builtin_nontemporal_load(reinterpret_cast<const Out *>(dyp + pooled));
  In g0, g1;
  pool_word_grads<VECW>(r0, r1, d, a, b, g0, g1);
  In o0, o1;
  if constexpr (VECW == 4) {
    o0 = lin2(g0, r0, k1, k2, k3);
    o1 = lin2(g1, r1, k1, k2, k3);
  } else {
    o0 = In{k1 * g0.x + k2 * r0.x + k3, k1 * g0.y + k2 * r0.y + k3};
    o1 = In{k1 * g1.x + k2 * r1.x + k3, k1 * g1.y + k2 * r1.y + k3};
  }
  __builtin_nontemporal_store(o0, reinterpret_cast<In *>(dx + top));
  __builtin_nontemporal_store(o1, reinterpret_cast<In *>(dx + top + g.W));
}

// VECW and the geometry for x[N][C][H][W]; false when H or W is odd or the words do not fit 32 bits
inline bool make_pool_geo(const DLArray *x, bool aligned, int &vecw, PoolGeo &g) {
  if (x->ndim != 4) return false;
  const int64_t N = x->shape[0], C = x->shape[1], H = x->shape[2], W = x->shape[3];
  if (N <= 0 || C <= 0 || H < 2 || W < 2 || (H & 1) || (W & 1) || C > 65535) return false;
  vecw = (W % 4 == 0 && aligned) ? 4 : 2;
  const int64_t words = N * C * (H / 2) * (W / vecw);
  if (words >= (1ll << 32) - kThreads || N * (H / 2) * (W / vecw) >= (1ll << 31)) return false;
  g.wq = FastDiv(static_cast<uint32_t>(W / vecw));
  g.rows = FastDiv(static_cast<uint32_t>(H / 2));
  g.chans = FastDiv(static_cast<uint32_t>(C));
  g.words = static_cast<uint32_t>(words);
  g.H = static_cast<int>(H);
  g.W = static_cast<int>(W);
  return true;
}

inline const float *cf(const DLArray *a) { return static_cast<const float *>(a->data); }
inline float *mf(DLArray *a) { return static_cast<float *>(a->data); }

}  // namespace

int bn_channel_sums(const DLArray *y, double *dst, hipStream_t st) {
  Plan pl;
  TS_REQUIRE(make_plan(y, aligned16(y->data), kStatsWords, 16384, pl), "channel sums: unsupported shape");
  const int64_t C = y->shape[1];
  double *part = static_cast<double *>(scratch_get(st, 1, static_cast<size_t>(C) * pl.S * 2 * sizeof(double)));
  TS_REQUIRE(part, "channel sums: no scratch memory");
  const dim3 gs(pl.S, static_cast<unsigned>(C));
  if (pl.vec == 4)
    hipLaunchKernelGGL(bn_stats_kernel<4>, gs, dim3(kThreads), 0, st, cf(y), part, pl.g, pl.S);
  else
    hipLaunchKernelGGL(bn_stats_kernel<1>, gs, dim3(kThreads), 0, st, cf(y), part, pl.g, pl.S);
  hipLaunchKernelGGL(bn_sums_fold_kernel, dim3(static_cast<unsigned>(C)), dim3(kThreads), 0, st, part, pl.S, dst);
  return 0;
}

}  // namespace tsplit

using namespace tsplit;

// BatchNorm calls served from a convolution's note (TSplit_BatchNormLookBehind reports it)
static std::atomic<long long> g_bn_from_notes{0};

extern "C" {

int TSplit_BatchNormLookBehind(long long *calls_served, int *notes_live) {
  if (calls_served) *calls_served = g_bn_from_notes.load(std::memory_order_relaxed);
  if (notes_live) *notes_live = tsplit::g_conv_notes_live.load(std::memory_order_relaxed);
  return 0;
}

// coefficients from the partial sums (pair k of channel c at part[(c * part_c + k * part_k) * 2]), then
// the streaming pass y = a*x + b (+ Relu)
static void bn_apply_from(const double *part, int S, int64_t part_c, int64_t part_k, float *coef, const Plan &ap,
                          bool relu, const DLArray *x, const DLArray *scale, const DLArray *bias, DLArray *y,
                          float eps, DLArray *save_mean_arr, DLArray *save_var_arr, hipStream_t s) {
  const unsigned C = static_cast<unsigned>(x->shape[1]);
  const double inv_m = 1.0 / static_cast<double>(ap.m);
  float *sm = save_mean_arr ? mf(save_mean_arr) : nullptr;
  float *sv = save_var_arr ? mf(save_var_arr) : nullptr;
  if (relu)
    hipLaunchKernelGGL(bn_coef_kernel<true>, dim3(C), dim3(kThreads), 0, s, part, S, part_c, part_k, cf(scale), cf(bias),
                       eps, inv_m, coef, sm, sv);
  else
    hipLaunchKernelGGL(bn_coef_kernel<false>, dim3(C), dim3(kThreads), 0, s, part, S, part_c, part_k, cf(scale), cf(bias),
                       eps, inv_m, coef, sm, sv);
  PlaneGeo pg;
  unsigned blocks = 0;
  if (plane_major_ok(ap, x, pg, blocks)) {
    const f32x4 *xw = reinterpret_cast<const f32x4 *>(x->data);
    f32x4 *yw = reinterpret_cast<f32x4 *>(y->data);
    if (relu)
      hipLaunchKernelGGL(bn_apply_plane_kernel<true>, dim3(blocks), dim3(kThreads), 0, s, xw, yw, coef, pg);
    else
      hipLaunchKernelGGL(bn_apply_plane_kernel<false>, dim3(blocks), dim3(kThreads), 0, s, xw, yw, coef, pg);
    return;
  }
  const dim3 ga(ap.S, C);
#define BN_APPLY(V, R) \
  hipLaunchKernelGGL((bn_apply_kernel<V, R>), ga, dim3(kThreads), 0, s, cf(x), mf(y), static_cast<const float *>(coef), ap.g)
  if (ap.vec == 4) {
    if (relu)
      BN_APPLY(4, true);
    else
      BN_APPLY(4, false);
  } else {
    if (relu)
      BN_APPLY(1, true);
    else
      BN_APPLY(1, false);
  }
#undef BN_APPLY
}

static int bn_forward(const char *who, bool relu, const DLArrayHandle input_X, const DLArrayHandle bn_scale,
                      const DLArrayHandle bn_bias, DLArrayHandle output_Y, float eps, DLArrayHandle save_mean_arr,
                      DLArrayHandle save_var_arr, DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input_X && bn_scale && bn_bias && output_Y, "%s: NULL array", who);
  TS_REQUIRE(input_X->ndim == 4 && output_Y->ndim == 4, "%s: input and output must be 4-D NCHW", who);
  TS_REQUIRE(numel(input_X) == numel(output_Y), "%s: input/output sizes differ", who);
  const int64_t C = input_X->shape[1];
  TS_REQUIRE(numel(bn_scale) == C && numel(bn_bias) == C, "%s: scale/bias must hold C=%lld elements", who, (long long)C);
  TS_REQUIRE(!save_mean_arr || numel(save_mean_arr) == C, "%s: save_mean must hold C elements", who);
  TS_REQUIRE(!save_var_arr || numel(save_var_arr) == C, "%s: save_var must hold C elements", who);
  TS_REQUIRE(!relu || (save_mean_arr && save_var_arr), "%s: the fused form needs both save arrays", who);
  // sums a convolution left for exactly this tensor on this stream (common.h): looked up before
  // stream_of() ends all notes, since this call writes too
  const double *note_sums = nullptr;
  int note_slots = 0;
  if (numel(input_X) > 0 && !one_pass_ok(input_X) && C <= INT32_MAX && input_X->shape[2] * input_X->shape[3] <= INT32_MAX)
    note_slots = conv_notes_take(stream_keep_notes(stream_handle), input_X->data, static_cast<size_t>(numel(input_X)) * sizeof(float),
                                 static_cast<int>(C), static_cast<int>(input_X->shape[2] * input_X->shape[3]), &note_sums);
  hipStream_t s = stream_of(stream_handle);
  if (note_slots > 0) {
    // the later convolutions that reuse the sums' memory are ordered behind this call on its stream
    g_bn_from_notes.fetch_add(1, std::memory_order_relaxed);
    ProfileScope psn(p, s, numel(input_X) + 2 * C, numel(output_Y), 0);
    const bool aln = aligned16(input_X->data) && aligned16(output_Y->data);
    Plan apn;
    TS_REQUIRE(make_plan(input_X, aln, 4 * kThreads, 1 << 22, apn), "%s: unsupported shape", who);
    float *coefn = static_cast<float *>(scratch_get(s, 1, static_cast<size_t>(C) * 2 * sizeof(float)));
    TS_REQUIRE(coefn, "%s: no scratch memory", who);
    bn_apply_from(note_sums, note_slots, 1, C, coefn, apn, relu, input_X, bn_scale, bn_bias, output_Y, eps, save_mean_arr,
                  save_var_arr, s);
    return psn.finish();
  }
  if (one_pass_ok(input_X)) {
    const uint32_t hw = static_cast<uint32_t>(input_X->shape[2] * input_X->shape[3]);
    const uint32_t m = static_cast<uint32_t>(input_X->shape[0]) * hw;
    ProfileScope ps1(p, s, numel(input_X) + 2 * C, numel(output_Y), 0);
    float *sm1 = save_mean_arr ? mf(save_mean_arr) : nullptr;
    float *sv1 = save_var_arr ? mf(save_var_arr) : nullptr;
    const int per = static_cast<int>((m + kThreads - 1) / kThreads);
#define BN_FWD1(R, RL)                                                                                              \
  hipLaunchKernelGGL((bn_fwd_onepass_kernel<R, RL>), dim3(static_cast<unsigned>(C)), dim3(kThreads), 0, s,         \
                     cf(input_X), mf(output_Y), cf(bn_scale), cf(bn_bias), FastDiv(hw), static_cast<int>(C), m, eps, \
                     1.0 / static_cast<double>(m), sm1, sv1)
#define BN_FWD1_R(RL)   \
  do {                  \
    if (per <= 16)      \
      BN_FWD1(16, RL);  \
    else if (per <= 32) \
      BN_FWD1(32, RL);  \
    else                \
      BN_FWD1(64, RL);  \
  } while (0)
    if (relu)
      BN_FWD1_R(true);
    else
      BN_FWD1_R(false);
#undef BN_FWD1_R
#undef BN_FWD1
    return ps1.finish();
  }
  const bool al = aligned16(input_X->data) && aligned16(output_Y->data);
  Plan st, ap;
  TS_REQUIRE(make_plan(input_X, al, kStatsWords, 16384, st), "%s: unsupported shape", who);
  TS_REQUIRE(make_plan(input_X, al, 4 * kThreads, 1 << 22, ap), "%s: unsupported shape", who);
  // the partial sums, and behind them the two coefficients per channel
  const size_t part_bytes = static_cast<size_t>(C) * st.S * 2 * sizeof(double);
  double *part = static_cast<double *>(scratch_get(s, 1, part_bytes + static_cast<size_t>(C) * 2 * sizeof(float)));
  TS_REQUIRE(part, "%s: no scratch memory", who);
  float *coef = reinterpret_cast<float *>(part + static_cast<size_t>(C) * st.S * 2);
  ProfileScope ps(p, s, numel(input_X) + 2 * C, numel(output_Y), C * st.S * 4);
  const dim3 gs(st.S, static_cast<unsigned>(C));
  if (st.vec == 4)
    hipLaunchKernelGGL(bn_stats_kernel<4>, gs, dim3(kThreads), 0, s, cf(input_X), part, st.g, st.S);
  else
    hipLaunchKernelGGL(bn_stats_kernel<1>, gs, dim3(kThreads), 0, s, cf(input_X), part, st.g, st.S);
  bn_apply_from(part, st.S, static_cast<int64_t>(st.S), 1, coef, ap, relu, input_X, bn_scale, bn_bias, output_Y, eps,
                save_mean_arr, save_var_arr, s);
  return ps.finish();
}

int CuDNN_DLGpuBatch_Normalization(const DLArrayHandle input_X, const DLArrayHandle bn_scale,
                                   const DLArrayHandle bn_bias, DLArrayHandle output_Y, float momentum, float eps,
                                   DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                   DLStreamHandle stream_handle, ProfilerHandle p) {
  (void)momentum;
  return bn_forward("BatchNorm", false, input_X, bn_scale, bn_bias, output_Y, eps, save_mean_arr, save_var_arr,
                    stream_handle, p);
}

int TSplit_BatchNormRelu(const DLArrayHandle input_X, const DLArrayHandle bn_scale, const DLArrayHandle bn_bias,
                         DLArrayHandle output_Y, float eps, DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                         DLStreamHandle stream_handle, ProfilerHandle p) {
  return bn_forward("TSplit_BatchNormRelu", true, input_X, bn_scale, bn_bias, output_Y, eps, save_mean_arr,
                    save_var_arr, stream_handle, p);
}

// BatchNorm (relu == 0) or BatchNorm + Relu (relu != 0) forward whose batch statistics come from sums a
// producer left: `stats` is float32 storage viewed as [slots][C][2] doubles, row k holding the per-channel
// (sum, sum of squares) over one part of the batch (TSplit_Conv2dBatchNormStats writes such rows); the rows
// are added in ascending order.  One pass over x: 8 B per element.
int TSplit_BatchNormFromStats(const DLArrayHandle input_X, const DLArrayHandle stats, int slots,
                              const DLArrayHandle bn_scale, const DLArrayHandle bn_bias, DLArrayHandle output_Y,
                              float eps, DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr, int relu,
                              DLStreamHandle stream_handle, ProfilerHandle p) {
  const char *who = "TSplit_BatchNormFromStats";
  TS_REQUIRE(input_X && stats && bn_scale && bn_bias && output_Y, "%s: NULL array", who);
  TS_REQUIRE(input_X->ndim == 4 && output_Y->ndim == 4, "%s: input and output must be 4-D NCHW", who);
  TS_REQUIRE(numel(input_X) == numel(output_Y), "%s: input/output sizes differ", who);
  const int64_t C = input_X->shape[1];
  TS_REQUIRE(numel(bn_scale) == C && numel(bn_bias) == C, "%s: scale/bias must hold C=%lld elements", who, (long long)C);
  TS_REQUIRE(!save_mean_arr || numel(save_mean_arr) == C, "%s: save_mean must hold C elements", who);
  TS_REQUIRE(!save_var_arr || numel(save_var_arr) == C, "%s: save_var must hold C elements", who);
  TS_REQUIRE(!relu || (save_mean_arr && save_var_arr), "%s: the fused form needs both save arrays", who);
  TS_REQUIRE(slots >= 1 && numel(stats) >= static_cast<int64_t>(slots) * C * 4, "%s: stats must hold slots * C * 4 floats", who);
  TS_REQUIRE((reinterpret_cast<uintptr_t>(stats->data) & 7) == 0, "%s: stats must be 8-byte aligned", who);
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input_X) + 2 * C, numel(output_Y), 0);
  if (numel(input_X) == 0) return ps.finish();
  const bool al = aligned16(input_X->data) && aligned16(output_Y->data);
  Plan ap;
  TS_REQUIRE(make_plan(input_X, al, 4 * kThreads, 1 << 22, ap), "%s: unsupported shape", who);
  float *coef = static_cast<float *>(scratch_get(s, 1, static_cast<size_t>(C) * 2 * sizeof(float)));
  TS_REQUIRE(coef, "%s: no scratch memory", who);
  bn_apply_from(static_cast<const double *>(stats->data), slots, 1, C, coef, ap, relu != 0, input_X, bn_scale, bn_bias,
                output_Y, eps, save_mean_arr, save_var_arr, s);
  return ps.finish();
}

static int bn_backward(const char *who, bool relu, const DLArrayHandle gradient_Y, const DLArrayHandle input_X,
                       const DLArrayHandle bn_scale, const DLArrayHandle bn_bias, DLArrayHandle gradient_X,
                       DLArrayHandle gradient_bn_scale, DLArrayHandle gradient_bn_bias, float eps,
                       DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr, DLStreamHandle stream_handle,
                       ProfilerHandle p) {
  TS_REQUIRE(gradient_Y && input_X && bn_scale && gradient_X, "%s: NULL array", who);
  TS_REQUIRE(input_X->ndim == 4, "%s: input must be 4-D NCHW", who);
  TS_REQUIRE(numel(input_X) == numel(gradient_Y) && numel(input_X) == numel(gradient_X), "%s: x, dy, dx sizes differ", who);
  const int64_t C = input_X->shape[1];
  TS_REQUIRE(numel(bn_scale) == C, "%s: scale must hold C elements", who);
  TS_REQUIRE(!gradient_bn_scale || numel(gradient_bn_scale) == C, "%s: dscale must hold C elements", who);
  TS_REQUIRE(!gradient_bn_bias || numel(gradient_bn_bias) == C, "%s: dbias must hold C elements", who);
  const bool saved = save_mean_arr && save_var_arr;
  TS_REQUIRE(!saved || (numel(save_mean_arr) == C && numel(save_var_arr) == C),
             "%s: saved statistics must hold C elements", who);
  TS_REQUIRE(!relu || (saved && bn_bias && numel(bn_bias) == C),
             "%s: the fused form needs the bias and the statistics saved by the fused forward call", who);
  hipStream_t s = stream_of(stream_handle);
  if (one_pass_ok(input_X)) {
    const uint32_t hw = static_cast<uint32_t>(input_X->shape[2] * input_X->shape[3]);
    const uint32_t m = static_cast<uint32_t>(input_X->shape[0]) * hw;
    ProfileScope ps1(p, s, 2 * numel(input_X) + C, numel(gradient_X) + 2 * C, 0);
    const float *sm1 = saved ? cf(save_mean_arr) : nullptr;
    const float *sv1 = saved ? cf(save_var_arr) : nullptr;
    const float *bias1 = bn_bias ? cf(bn_bias) : nullptr;
    float *dg1 = gradient_bn_scale ? mf(gradient_bn_scale) : nullptr;
    float *db1 = gradient_bn_bias ? mf(gradient_bn_bias) : nullptr;
    const int per = static_cast<int>((m + kThreads - 1) / kThreads);
#define BN_BWD1(R, ST, RL)                                                                                          \
  hipLaunchKernelGGL((bn_bwd_onepass_kernel<R, ST, RL>), dim3(static_cast<unsigned>(C)), dim3(kThreads), 0, s,     \
                     cf(gradient_Y), cf(input_X), mf(gradient_X), cf(bn_scale), bias1, FastDiv(hw),                 \
                     static_cast<int>(C), m, eps, 1.0 / static_cast<double>(m), sm1, sv1, dg1, db1)
#define BN_BWD1_R(ST, RL)   \
  do {                      \
    if (per <= 16)          \
      BN_BWD1(16, ST, RL);  \
    else if (per <= 32)     \
      BN_BWD1(32, ST, RL);  \
    else                    \
      BN_BWD1(64, ST, RL);  \
  } while (0)
    if (relu)
      BN_BWD1_R(false, true);
    else if (saved)
      BN_BWD1_R(false, false);
    else
      BN_BWD1_R(true, false);
#undef BN_BWD1_R
#undef BN_BWD1
    return ps1.finish();
  }
  const bool al = aligned16(input_X->data) && aligned16(gradient_Y->data) && aligned16(gradient_X->data);
  Plan rd, dxp;
  TS_REQUIRE(make_plan(input_X, al, kStatsWords, 16384, rd), "%s: unsupported shape", who);
  TS_REQUIRE(make_plan(input_X, al, 4 * kThreads, 1 << 22, dxp), "%s: unsupported shape", who);
  // the partial sums, and behind them five coefficients per channel
  double *part = static_cast<double *>(scratch_get(s, 1, static_cast<size_t>(C) * rd.S * 4 * sizeof(double) +
                                                             static_cast<size_t>(C) * 5 * sizeof(float)));
  TS_REQUIRE(part, "%s: no scratch memory", who);
  float *coef = reinterpret_cast<float *>(part + static_cast<size_t>(C) * rd.S * 4);
  ProfileScope ps(p, s, 2 * numel(input_X) + C, numel(gradient_X) + 2 * C, C * rd.S * 8);
  const double inv_m = 1.0 / static_cast<double>(rd.m);
  const float *sm = saved ? cf(save_mean_arr) : nullptr;
  const float *sv = saved ? cf(save_var_arr) : nullptr;
  const float *bias = bn_bias ? cf(bn_bias) : nullptr;
  float *dg = gradient_bn_scale ? mf(gradient_bn_scale) : nullptr;
  float *db = gradient_bn_bias ? mf(gradient_bn_bias) : nullptr;
  const unsigned Cu = static_cast<unsigned>(C);
  dim3 gr(rd.S, Cu), gd(dxp.S, Cu);
  PlaneGeo pg;
  unsigned blocks = 0;
  const bool plane_major = plane_major_ok(dxp, input_X, pg, blocks);
  const f32x4 *xw = reinterpret_cast<const f32x4 *>(input_X->data), *dyw = reinterpret_cast<const f32x4 *>(gradient_Y->data);
  f32x4 *dxw = reinterpret_cast<f32x4 *>(gradient_X->data);
#define BN_BWD(V, ST, R)                                                                                            \
  do {                                                                                                              \
    hipLaunchKernelGGL((bn_bwd_reduce_kernel<V, ST, R>), gr, dim3(kThreads), 0, s, cf(gradient_Y), cf(input_X),     \
                       part, rd.g, rd.S, cf(bn_scale), bias, sm, sv);                                               \
    hipLaunchKernelGGL((bn_bwd_coef_kernel<R>), dim3(Cu), dim3(kThreads), 0, s, static_cast<const double *>(part),  \
                       rd.S, cf(bn_scale), bias, eps, inv_m, sm, sv, coef, dg, db);                                 \
    if (V == 4 && plane_major)                                                                                      \
      hipLaunchKernelGGL((bn_bwd_dx_plane_kernel<R>), dim3(blocks), dim3(kThreads), 0, s, dyw, xw, dxw,             \
                         static_cast<const float *>(coef), pg);                                                     \
    else                                                                                                            \
      hipLaunchKernelGGL((bn_bwd_dx_kernel<V, R>), gd, dim3(kThreads), 0, s, cf(gradient_Y), cf(input_X),           \
                         mf(gradient_X), static_cast<const float *>(coef), dxp.g);                                  \
  } while (0)
  if (rd.vec == 4) {
    if (relu)
      BN_BWD(4, false, true);
    else if (saved)
      BN_BWD(4, false, false);
    else
      BN_BWD(4, true, false);
  } else {
    if (relu)
      BN_BWD(1, false, true);
    else if (saved)
      BN_BWD(1, false, false);
    else
      BN_BWD(1, true, false);
  }
#undef BN_BWD
  return ps.finish();
}

int CuDNN_DLGpuBatch_Normalization_gradient(const DLArrayHandle gradient_Y, const DLArrayHandle input_X,
                                            const DLArrayHandle bn_scale, DLArrayHandle gradient_X,
                                            DLArrayHandle gradient_bn_scale, DLArrayHandle gradient_bn_bias,
                                            float eps, DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                            DLStreamHandle stream_handle, ProfilerHandle p) {
  return bn_backward("BatchNorm gradient", false, gradient_Y, input_X, bn_scale, nullptr, gradient_X, gradient_bn_scale,
                     gradient_bn_bias, eps, save_mean_arr, save_var_arr, stream_handle, p);
}

int TSplit_BatchNormRelu_gradient(const DLArrayHandle gradient_Y, const DLArrayHandle input_X,
                                  const DLArrayHandle bn_scale, const DLArrayHandle bn_bias, DLArrayHandle gradient_X,
                                  DLArrayHandle gradient_bn_scale, DLArrayHandle gradient_bn_bias, float eps,
                                  DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                  DLStreamHandle stream_handle, ProfilerHandle p) {
  return bn_backward("TSplit_BatchNormRelu_gradient", true, gradient_Y, input_X, bn_scale, bn_bias, gradient_X,
                     gradient_bn_scale, gradient_bn_bias, eps, save_mean_arr, save_var_arr, stream_handle, p);
}

// ---- BatchNorm + Relu + 2x2 / stride 2 max pooling as one call each way (outside the reference's ABI) ----
static int bn_relu_pool_forward(const char *who, const DLArrayHandle input_X, const DLArrayHandle stats, int slots,
                                const DLArrayHandle bn_scale, const DLArrayHandle bn_bias, DLArrayHandle output_Y, float eps,
                                DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr, DLStreamHandle stream_handle,
                                ProfilerHandle p) {
  TS_REQUIRE(input_X && bn_scale && bn_bias && output_Y && save_mean_arr && save_var_arr, "%s: NULL array", who);
  TS_REQUIRE(input_X->ndim == 4 && output_Y->ndim == 4, "%s: input and output must be 4-D NCHW", who);
  const int64_t N = input_X->shape[0], C = input_X->shape[1], H = input_X->shape[2], W = input_X->shape[3];
  TS_REQUIRE(H % 2 == 0 && W % 2 == 0, "%s: height and width must be even, got %lld x %lld", who, (long long)H, (long long)W);
  TS_REQUIRE(output_Y->shape[0] == N && output_Y->shape[1] == C && output_Y->shape[2] == H / 2 && output_Y->shape[3] == W / 2,
             "%s: the output must be [N][C][H/2][W/2]", who);
  TS_REQUIRE(numel(bn_scale) == C && numel(bn_bias) == C, "%s: scale/bias must hold C=%lld elements", who, (long long)C);
  TS_REQUIRE(numel(save_mean_arr) == C && numel(save_var_arr) == C, "%s: the save arrays must hold C elements", who);
  if (stats) {
    TS_REQUIRE(slots >= 1 && numel(stats) >= static_cast<int64_t>(slots) * C * 4, "%s: stats must hold slots * C * 4 floats", who);
    TS_REQUIRE((reinterpret_cast<uintptr_t>(stats->data) & 7) == 0, "%s: stats must be 8-byte aligned", who);
  }
  TS_REQUIRE(numel(input_X) > 0, "%s: batch statistics of an empty tensor", who);
  TS_REQUIRE((reinterpret_cast<uintptr_t>(input_X->data) & 7) == 0, "%s: the input must be 8-byte aligned", who);
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input_X) + 2 * C, numel(output_Y), 0);
  int vecw = 2;
  PoolGeo pg;
  TS_REQUIRE(make_pool_geo(input_X, aligned16(input_X->data) && (reinterpret_cast<uintptr_t>(output_Y->data) & 7) == 0, vecw, pg),
             "%s: unsupported shape", who);
  const double inv_m = 1.0 / static_cast<double>(N * H * W);
  const unsigned Cu = static_cast<unsigned>(C);
  float *coef = nullptr;
  if (stats) {
    coef = static_cast<float *>(scratch_get(s, 1, static_cast<size_t>(C) * 2 * sizeof(float)));
    TS_REQUIRE(coef, "%s: no scratch memory", who);
    hipLaunchKernelGGL(bn_coef_kernel<true>, dim3(Cu), dim3(kThreads), 0, s, static_cast<const double *>(stats->data), slots,
                       static_cast<int64_t>(1), C, cf(bn_scale), cf(bn_bias), eps, inv_m, coef, mf(save_mean_arr),
                       mf(save_var_arr));
  } else {
    Plan st;
    TS_REQUIRE(make_plan(input_X, aligned16(input_X->data), kStatsWords, 16384, st), "%s: unsupported shape", who);
    double *part = static_cast<double *>(scratch_get(s, 1, static_cast<size_t>(C) * st.S * 2 * sizeof(double) +
                                                               static_cast<size_t>(C) * 2 * sizeof(float)));
    TS_REQUIRE(part, "%s: no scratch memory", who);
    coef = reinterpret_cast<float *>(part + static_cast<size_t>(C) * st.S * 2);
    const dim3 gs(st.S, Cu);
    if (st.vec == 4)
      hipLaunchKernelGGL(bn_stats_kernel<4>, gs, dim3(kThreads), 0, s, cf(input_X), part, st.g, st.S);
    else
      hipLaunchKernelGGL(bn_stats_kernel<1>, gs, dim3(kThreads), 0, s, cf(input_X), part, st.g, st.S);
    hipLaunchKernelGGL(bn_coef_kernel<true>, dim3(Cu), dim3(kThreads), 0, s, static_cast<const double *>(part), st.S,
                       static_cast<int64_t>(st.S), static_cast<int64_t>(1), cf(bn_scale), cf(bn_bias), eps, inv_m, coef,
                       mf(save_mean_arr), mf(save_var_arr));
  }
  const unsigned blocks = (pg.words + kThreads - 1) / kThreads;
  if (vecw == 4)
    hipLaunchKernelGGL(bn_relu_pool_kernel<4>, dim3(blocks), dim3(kThreads), 0, s, cf(input_X), mf(output_Y),
                       static_cast<const float *>(coef), pg);
  else
    hipLaunchKernelGGL(bn_relu_pool_kernel<2>, dim3(blocks), dim3(kThreads), 0, s, cf(input_X), mf(output_Y),
                       static_cast<const float *>(coef), pg);
  return ps.finish();
}

// BatchNorm + Relu + max pooling (2x2 windows, stride 2, no padding) forward: output_Y [N][C][H/2][W/2] from
// input_X [N][C][H][W] (H, W even); the save arrays as TSplit_BatchNormRelu leaves them.
int TSplit_BatchNormReluMaxPool(const DLArrayHandle input_X, const DLArrayHandle bn_scale, const DLArrayHandle bn_bias,
                                DLArrayHandle output_Y, float eps, DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                DLStreamHandle stream_handle, ProfilerHandle p) {
  return bn_relu_pool_forward("TSplit_BatchNormReluMaxPool", input_X, nullptr, 0, bn_scale, bn_bias, output_Y, eps,
                              save_mean_arr, save_var_arr, stream_handle, p);
}

// The same with the batch statistics taken from rows 0 .. slots-1 of `stats` (as TSplit_BatchNormFromStats).
int TSplit_BatchNormReluMaxPoolFromStats(const DLArrayHandle input_X, const DLArrayHandle stats, int slots,
                                         const DLArrayHandle bn_scale, const DLArrayHandle bn_bias, DLArrayHandle output_Y,
                                         float eps, DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                         DLStreamHandle stream_handle, ProfilerHandle p) {
  const char *who = "TSplit_BatchNormReluMaxPoolFromStats";
  TS_REQUIRE(stats, "%s: NULL array", who);
  return bn_relu_pool_forward(who, input_X, stats, slots, bn_scale, bn_bias, output_Y, eps, save_mean_arr, save_var_arr,
                              stream_handle, p);
}

// Their gradient: gradient_Y is the pooled tensor's gradient [N][C][H/2][W/2], input_X the BatchNorm's input,
// gradient_X its gradient; the statistics are those the forward call saved.
int TSplit_BatchNormReluMaxPool_gradient(const DLArrayHandle gradient_Y, const DLArrayHandle input_X,
                                         const DLArrayHandle bn_scale, const DLArrayHandle bn_bias, DLArrayHandle gradient_X,
                                         DLArrayHandle gradient_bn_scale, DLArrayHandle gradient_bn_bias, float eps,
                                         DLArrayHandle save_mean_arr, DLArrayHandle save_var_arr,
                                         DLStreamHandle stream_handle, ProfilerHandle p) {
  const char *who = "TSplit_BatchNormReluMaxPool_gradient";
  TS_REQUIRE(gradient_Y && input_X && bn_scale && bn_bias && gradient_X && save_mean_arr && save_var_arr, "%s: NULL array", who);
  TS_REQUIRE(input_X->ndim == 4 && gradient_Y->ndim == 4, "%s: arrays must be 4-D NCHW", who);
  const int64_t N = input_X->shape[0], C = input_X->shape[1], H = input_X->shape[2], W = input_X->shape[3];
  TS_REQUIRE(H % 2 == 0 && W % 2 == 0, "%s: height and width must be even, got %lld x %lld", who, (long long)H, (long long)W);
  TS_REQUIRE(gradient_Y->shape[0] == N && gradient_Y->shape[1] == C && gradient_Y->shape[2] == H / 2 &&
                 gradient_Y->shape[3] == W / 2, "%s: the pooled gradient must be [N][C][H/2][W/2]", who);
  TS_REQUIRE(numel(gradient_X) == numel(input_X), "%s: x and dx sizes differ", who);
  TS_REQUIRE(numel(bn_scale) == C && numel(bn_bias) == C && numel(save_mean_arr) == C && numel(save_var_arr) == C,
             "%s: scale, bias and the saved statistics must hold C elements", who);
  TS_REQUIRE(!gradient_bn_scale || numel(gradient_bn_scale) == C, "%s: dscale must hold C elements", who);
  TS_REQUIRE(!gradient_bn_bias || numel(gradient_bn_bias) == C, "%s: dbias must hold C elements", who);
  TS_REQUIRE(numel(input_X) > 0, "%s: batch statistics of an empty tensor", who);
  hipStream_t s = stream_of(stream_handle);
  TS_REQUIRE(((reinterpret_cast<uintptr_t>(input_X->data) | reinterpret_cast<uintptr_t>(gradient_X->data)) & 7) == 0,
             "%s: x and dx must be 8-byte aligned", who);
  int vecw = 2;
  PoolGeo pg;
  const bool al = aligned16(input_X->data) && aligned16(gradient_X->data) && (reinterpret_cast<uintptr_t>(gradient_Y->data) & 7) == 0;
  TS_REQUIRE(make_pool_geo(input_X, al, vecw, pg), "%s: unsupported shape", who);
  // a channel's words, cut into S ranges of whole blocks' worth
  const uint32_t wpp = static_cast<uint32_t>((H / 2) * (W / vecw));
  const uint32_t words_c = static_cast<uint32_t>(N) * wpp;
  int64_t S = (words_c + kStatsWords / 2 - 1) / (kStatsWords / 2);
  const int64_t cap = 16384 / C > 0 ? 16384 / C : 1;
  if (S > cap) S = cap;
  if (S < 1) S = 1;
  uint32_t chunk = static_cast<uint32_t>((words_c + S - 1) / S);
  chunk = (chunk + kThreads - 1) / kThreads * kThreads;
  S = (words_c + chunk - 1) / chunk;
  double *part = static_cast<double *>(scratch_get(s, 1, static_cast<size_t>(C) * S * 4 * sizeof(double) +
                                                             static_cast<size_t>(C) * 5 * sizeof(float)));
  TS_REQUIRE(part, "%s: no scratch memory", who);
  float *coef = reinterpret_cast<float *>(part + static_cast<size_t>(C) * S * 4);
  ProfileScope ps(p, s, 2 * numel(input_X) + 2 * numel(gradient_Y) + C, numel(gradient_X) + 2 * C, C * S * 8);
  const double inv_m = 1.0 / static_cast<double>(N * H * W);
  const unsigned Cu = static_cast<unsigned>(C);
  const dim3 gr(static_cast<unsigned>(S), Cu);
  const unsigned blocks = (pg.words + kThreads - 1) / kThreads;
  float *dg = gradient_bn_scale ? mf(gradient_bn_scale) : nullptr;
  float *db = gradient_bn_bias ? mf(gradient_bn_bias) : nullptr;
#define BN_POOL_BWD(V)                                                                                               \
  do {                                                                                                               \
    hipLaunchKernelGGL(bn_pool_bwd_reduce_kernel<V>, gr, dim3(kThreads), 0, s, cf(gradient_Y), cf(input_X), part, pg, \
                       FastDiv(wpp), words_c, chunk, static_cast<int>(S), cf(bn_scale), cf(bn_bias),                 \
                       cf(save_mean_arr), cf(save_var_arr));                                                         \
    hipLaunchKernelGGL(bn_bwd_coef_kernel<true>, dim3(Cu), dim3(kThreads), 0, s, static_cast<const double *>(part),  \
                       static_cast<int>(S), cf(bn_scale), cf(bn_bias), eps, inv_m, cf(save_mean_arr),                \
                       cf(save_var_arr), coef, dg, db);                                                              \
    hipLaunchKernelGGL(bn_pool_bwd_dx_kernel<V>, dim3(blocks), dim3(kThreads), 0, s, cf(gradient_Y), cf(input_X),    \
                       mf(gradient_X), static_cast<const float *>(coef), pg);                                        \
  } while (0)
  if (vecw == 4)
    BN_POOL_BWD(4);
  else
    BN_POOL_BWD(2);
#undef BN_POOL_BWD
  return ps.finish();
}

}  // extern "C"
