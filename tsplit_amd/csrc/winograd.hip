// 3x3, stride-1, pad-1 convolution by the Winograd minimal-filtering algorithm F(4x4, 3x3)
// (Lavin & Gray, "Fast Algorithms for Convolutional Neural Networks", 2015), for layers wide
// enough that the direct implicit GEMM is bound by fp32 MFMA throughput: 36 multiplications per
// 4x4 output tile and channel pair instead of 144.
//
//   U[xi][o][c] = (G g G^T)[xi]          filter transform, once per call (36 planes of O x C)
//   V[xi][c][t] = (B^T d B)[xi]          input transform of the 6x6 patch d of tile t, channel c
//   M[xi][o][t] = sum_c U[xi][o][c] V[xi][c][t]      36 independent GEMMs on the MFMA tile engine
//   y tile      = A^T M[.][o][t] A       output transform, 4x4 outputs per tile
//
// Tiles are numbered image-major (t = (n * tiles_h + th) * tiles_w + tw), so consecutive lanes of
// the transform kernels touch consecutive tiles: V and M accesses are contiguous and the 16-byte
// output rows of neighbouring tiles join up.  The batch is processed in runs of whole images so that
// V and M, 2.25 times the size of the activations they stand for, stay within a scratch allowance
// (1 GiB unless TSPLIT_WINOGRAD_RUN_MIB says otherwise; longer runs mean larger, better-filled GEMMs).
//
// The same routine gives the data gradient: dx = conv(dy, w rotated by 180 degrees with its channel
// axes exchanged), which only changes the index the filter transform reads from.
//
// Arithmetic is fp32 throughout; the transforms' constants (up to 8 and 1/24) make the result
// differ from the directly summed one by a few 1e-6 of the output's magnitude.
#include <algorithm>
#include <cstdlib>
#include <atomic>
#include <mutex>
#include <vector>

#include "common.h"
#include "mfma_gemm.h"
#include "reduce.h"
#include "wino_gemm_split.h"

namespace tsplit {
using namespace mg;
namespace {

constexpr int kXi = 36;   // 6 x 6 transformed points

// ---------------------------------------------------------------- filter transform
// rows of G applied to (g0, g1, g2)
__device__ __forceinline__ void g_rows(float g0, float g1, float g2, float u[6]) {
  u[0] = 0.25f * g0;
  u[1] = (g0 + g1 + g2) * (-1.0f / 6.0f);
  u[2] = (g1 - g0 - g2) * (1.0f / 6.0f);
  u[3] = g0 * (1.0f / 24.0f) + g1 * (1.0f / 12.0f) + g2 * (1.0f / 6.0f);
  u[4] = g0 * (1.0f / 24.0f) - g1 * (1.0f / 12.0f) + g2 * (1.0f / 6.0f);
  u[5] = g2;
}

// U[xi][o][c], o over the produced channels, c over the gathered ones.  Forward: the filter is
// stored [o][c][3][3].  Data gradient: stored [c][o][3][3] and read rotated by 180 degrees.
__device__ __forceinline__ void wino_filter_block(const float *__restrict__ w, float *__restrict__ U, int produced, int gathered,
                                                  bool rotated, int bx) {
  const int i = bx * 256 + threadIdx.x;
  if (i >= produced * gathered) return;
  const int o = i / gathered, c = i - o * gathered;
  const float *g = w + (rotated ? static_cast<int64_t>(c) * produced + o : static_cast<int64_t>(o) * gathered + c) * 9;
  float k[9];
#pragma unroll
  for (int j = 0; j < 9; ++j) k[j] = rotated ? g[8 - j] : g[j];
  float t[3][6];   // G applied down the columns
#pragma unroll
  for (int col = 0; col < 3; ++col) g_rows(k[col], k[3 + col], k[6 + col], t[col]);
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    float u[6];
    g_rows(t[0][r], t[1][r], t[2][r], u);
#pragma unroll
    for (int q = 0; q < 6; ++q) U[static_cast<int64_t>(r * 6 + q) * produced * gathered + i] = u[q];
  }
}
__global__ __launch_bounds__(256) void wino_filter_kernel(const float *__restrict__ w, float *__restrict__ U, int produced,
                                                          int gathered, bool rotated) {
  wino_filter_block(w, U, produced, gathered, rotated, blockIdx.x);
}
// A filter transform that rides in the first rows of another kernel's grid (the input transform of a call's
// first run: neither depends on the other, and a launch of its own would cost its ramp and tail).
struct FilterJob {
  const float *w;
  float *U;
  int produced, gathered;
  bool rotated;
  int blocks;   // blocks of 256 filter elements; 0: nothing to do
  int rows;     // grid rows (of the host kernel's width) they take
};

// ---------------------------------------------------------------- input transform
// rows of B^T applied to (d0 .. d5)
__device__ __forceinline__ void bt_rows(const float d[6], float t[6]) {
  t[0] = 4.0f * d[0] - 5.0f * d[2] + d[4];
  t[1] = d[3] + d[4] - 4.0f * (d[1] + d[2]);
  t[2] = 4.0f * (d[1] - d[2]) - d[3] + d[4];
  t[3] = 2.0f * (d[3] - d[1]) - d[2] + d[4];
  t[4] = 2.0f * (d[1] - d[3]) - d[2] + d[4];
  t[5] = 4.0f * d[1] - 5.0f * d[3] + d[5];
}

struct WinoGeo {
  int chans;      // channels of the tensor this kernel touches
  int H, W;       // plane size (input and output planes are equal: stride 1, pad 1)
  int th, tw;     // tiles per plane
  int tiles;      // tiles of the run (images * th * tw)
  int ld;         // tiles rounded up to a multiple of 4: row pitch of V and M
  bool quads;     // output rows may be stored as aligned 16-byte quads
};

// one thread per (channel, tile).  With QUADS (W a multiple of 4, planes
// 16-byte aligned) a thread loads the aligned quad of each of its six rows and takes the two columns
// beside it from the neighbouring lanes, which hold the neighbouring tiles of the same tile row; at
// a wave's ends those come from memory, at the plane's edges they are the zero padding.
template <bool QUADS>
__device__ __forceinline__ void wino_input_block(const float *__restrict__ x, float *__restrict__ V, const WinoGeo &g, int c) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.ld) return;
  float *out = V + static_cast<int64_t>(c) * g.ld + t;
  const int64_t plane_stride = static_cast<int64_t>(g.chans) * g.ld;
  if (t >= g.tiles) {   // padding columns of the GEMMs: defined, and never read back
#pragma unroll
    for (int xi = 0; xi < kXi; ++xi) out[xi * plane_stride] = 0.0f;
    return;
  }
  const int per_img = g.th * g.tw;
  const int n = t / per_img, rem = t - n * per_img;
  const int ty = rem / g.tw, tx = rem - ty * g.tw;
  const int h0 = 4 * ty - 1, w0 = 4 * tx - 1;
  const float *plane = x + (static_cast<int64_t>(n) * g.chans + c) * g.H * g.W;
  float d[6][6];
  if constexpr (QUADS) {
    const int lane = threadIdx.x & 63;
    const bool from_left = tx > 0 && lane == 0, from_right = tx < g.tw - 1 && lane == 63;
#pragma unroll
    for (int r = 0; r < 6; ++r) {
      const int h = h0 + r;
      const bool row_ok = h >= 0 && h < g.H;
      const float *row = plane + (row_ok ? h : 0) * g.W + 4 * tx;
      float4 v = *reinterpret_cast<const float4 *>(row);
      if (!row_ok) v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      float left = __shfl_up(v.w, 1), right = __shfl_down(v.x, 1);
      if (from_left) left = row_ok ? row[-1] : 0.0f;
      if (from_right) right = row_ok ? row[4] : 0.0f;
      d[r][0] = tx > 0 ? left : 0.0f;
      d[r][1] = v.x;
      d[r][2] = v.y;
      d[r][3] = v.z;
      d[r][4] = v.w;
      d[r][5] = tx < g.tw - 1 ? right : 0.0f;
    }
  } else {
#pragma unroll
    for (int r = 0; r < 6; ++r) {
      const int h = h0 + r;
      const bool row_ok = h >= 0 && h < g.H;
#pragma unroll
      for (int q = 0; q < 6; ++q) {
        const int w = w0 + q;
        d[r][q] = row_ok && w >= 0 && w < g.W ? plane[h * g.W + w] : 0.0f;
      }
    }
  }
  float tmp[6][6];   // tmp[q][.] = B^T applied down column q
#pragma unroll
  for (int q = 0; q < 6; ++q) {
    const float col[6] = {d[0][q], d[1][q], d[2][q], d[3][q], d[4][q], d[5][q]};
    bt_rows(col, tmp[q]);
  }
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    const float row[6] = {tmp[0][r], tmp[1][r], tmp[2][r], tmp[3][r], tmp[4][r], tmp[5][r]};
    float v[6];
    bt_rows(row, v);
#pragma unroll
    for (int q = 0; q < 6; ++q) out[(r * 6 + q) * plane_stride] = v[q];
  }
}
// grid (ceil(ld / 256), job.rows + chans): the first job.rows rows are the filter transform's
template <bool QUADS>
__global__ __launch_bounds__(256) void wino_input_kernel(const float *__restrict__ x, float *__restrict__ V, WinoGeo g,
                                                         FilterJob job) {
  const int row = blockIdx.y;
  if (row < job.rows) {
    const int fb = row * gridDim.x + blockIdx.x;
    if (fb < job.blocks) wino_filter_block(job.w, job.U, job.produced, job.gathered, job.rotated, fb);
    return;
  }
  wino_input_block<QUADS>(x, V, g, row - job.rows);
}

// ---------------------------------------------------------------- output transform
// rows of A^T applied to (m0 .. m5)
__device__ __forceinline__ void at_rows(const float m[6], float o[4]) {
  const float s12 = m[1] + m[2], d12 = m[1] - m[2], s34 = m[3] + m[4], d34 = m[3] - m[4];
  o[0] = m[0] + s12 + s34;
  o[1] = d12 + 2.0f * d34;
  o[2] = s12 + 4.0f * s34;
  o[3] = d12 + 8.0f * d34 + m[5];
}

// one thread per (channel, tile): grid (ceil(tiles / 256), chans).  With STATS the block also leaves the
// sum and the sum of squares of the outputs it stored (the values are at hand; the kernel is bound by
// memory) at stats[(blockIdx.x * chans + channel) * 2]: partial sums for a BatchNorm that follows.
template <bool STATS>
__global__ __launch_bounds__(256) void wino_output_kernel(const float *__restrict__ M, float *__restrict__ y, WinoGeo g,
                                                          float *__restrict__ stats) {
  __shared__ float sm[8];
  const int t = blockIdx.x * 256 + threadIdx.x;
  const int o = blockIdx.y;
  float sum = 0.0f, sq = 0.0f;
  if (t < g.tiles) {
    const float *in = M + static_cast<int64_t>(o) * g.ld + t;
    const int64_t plane_stride = static_cast<int64_t>(g.chans) * g.ld;
    float tmp[6][4];   // tmp[q][.] = A^T applied down column q
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      float col[6];
#pragma unroll
      for (int r = 0; r < 6; ++r) col[r] = in[(r * 6 + q) * plane_stride];
      at_rows(col, tmp[q]);
    }
    const int per_img = g.th * g.tw;
    const int n = t / per_img, rem = t - n * per_img;
    const int ty = rem / g.tw, tx = rem - ty * g.tw;
    float *plane = y + (static_cast<int64_t>(n) * g.chans + o) * g.H * g.W;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int h = 4 * ty + r;
      if (h >= g.H) break;
      const float row[6] = {tmp[0][r], tmp[1][r], tmp[2][r], tmp[3][r], tmp[4][r], tmp[5][r]};
      float v[4];
      at_rows(row, v);
      float *dst = plane + static_cast<int64_t>(h) * g.W + 4 * tx;
      if (g.quads) {
        *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        if (STATS) {
          sum += (v[0] + v[1]) + (v[2] + v[3]);
          sq += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (4 * tx + q < g.W) {
            dst[q] = v[q];
            if (STATS) {
              sum += v[q];
              sq += v[q] * v[q];
            }
          }
      }
    }
  }
  if (STATS) {
    sum = wave_sum(sum);
    sq = wave_sum(sq);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
      sm[wave] = sum;
      sm[4 + wave] = sq;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      float *dst = stats + (static_cast<int64_t>(blockIdx.x) * g.chans + o) * 2;
      dst[0] = (sm[0] + sm[1]) + (sm[2] + sm[3]);
      dst[1] = (sm[4] + sm[5]) + (sm[6] + sm[7]);
    }
  }
}

}  // namespace
}  // namespace tsplit
namespace tsplit {
namespace {
#include "wino_fused.h"

// ---------------------------------------------------------------- filter gradient
// The forward map is linear in the filter, y = A^T [(G g G^T) . (B^T d B)] A per tile, so the filter
// gradient is its adjoint: dg = G^T [ sum over tiles (A dy A^T) . (B^T d B) ] G.
//
// rows of A applied to (d0 .. d3)
__device__ __forceinline__ void a_rows(const float d[4], float o[6]) {
  const float e = d[0] + d[2], f = d[1] + d[3], p = d[0] + 4.0f * d[2], q = 2.0f * d[1] + 8.0f * d[3];
  o[0] = d[0];
  o[1] = e + f;
  o[2] = e - f;
  o[3] = p + q;
  o[4] = p - q;
  o[5] = d[3];
}

// Y[xi][o][t] = (A dy A^T)[xi] of the 4x4 output tile t, channel o (zero beyond the plane's edge)
template <bool QUADS>
__device__ __forceinline__ void wino_grad_block(const float *__restrict__ dy, float *__restrict__ Y, const WinoGeo &g, int o) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.ld) return;
  float *out = Y + static_cast<int64_t>(o) * g.ld + t;
  const int64_t plane_stride = static_cast<int64_t>(g.chans) * g.ld;
  if (t >= g.tiles) {   // padding of the reduction: contributes nothing
#pragma unroll
    for (int xi = 0; xi < kXi; ++xi) out[xi * plane_stride] = 0.0f;
    return;
  }
  const int per_img = g.th * g.tw;
  const int n = t / per_img, rem = t - n * per_img;
  const int ty = rem / g.tw, tx = rem - ty * g.tw;
  const float *plane = dy + (static_cast<int64_t>(n) * g.chans + o) * g.H * g.W;
  float tmp[4][6];   // tmp[q][.] = A applied down column q
  {
    float d[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int h = 4 * ty + r;
      const bool row_ok = h < g.H;
      const float *row = plane + static_cast<int64_t>(row_ok ? h : 0) * g.W + 4 * tx;
      if constexpr (QUADS) {
        float4 v = *reinterpret_cast<const float4 *>(row);
        if (!row_ok) v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        d[r][0] = v.x;
        d[r][1] = v.y;
        d[r][2] = v.z;
        d[r][3] = v.w;
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) d[r][q] = row_ok && 4 * tx + q < g.W ? row[q] : 0.0f;
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float col[4] = {d[0][q], d[1][q], d[2][q], d[3][q]};
      a_rows(col, tmp[q]);
    }
  }
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    const float row[4] = {tmp[0][r], tmp[1][r], tmp[2][r], tmp[3][r]};
    float v[6];
    a_rows(row, v);
#pragma unroll
    for (int q = 0; q < 6; ++q) out[(r * 6 + q) * plane_stride] = v[q];
  }
}
#include "wino_fgrad_fused.h"

// Both transforms of a filter-gradient run in one launch, grid (ceil(ld / 256), gx.chans + gy.chans): rows
// below gx.chans transform a channel of x, the others a channel of dy (the two share nothing but the tiling)
template <bool QUADS_X, bool QUADS_Y>
__global__ __launch_bounds__(256) void wino_grad_pair_kernel(const float *__restrict__ x, float *__restrict__ V, WinoGeo gx,
                                                             const float *__restrict__ dy, float *__restrict__ Y, WinoGeo gy) {
  const int row = blockIdx.y;
  if (row < gx.chans)
    wino_input_block<QUADS_X>(x, V, gx, row);
  else
    wino_grad_block<QUADS_Y>(dy, Y, gy, row - gx.chans);
}

// rows of G^T applied to (u0 .. u5)
__device__ __forceinline__ void gt_rows(const float u[6], float w[3]) {
  const float s12 = u[1] + u[2], s34 = u[3] + u[4];
  w[0] = 0.25f * u[0] - s12 * (1.0f / 6.0f) + s34 * (1.0f / 24.0f);
  w[1] = (u[2] - u[1]) * (1.0f / 6.0f) + (u[3] - u[4]) * (1.0f / 12.0f);
  w[2] = (s34 - s12) * (1.0f / 6.0f) + u[5];
}

// dw[o][c][3][3] = G^T (sum of the partial dU) G; part[(p * 36 + xi) * O * C + o * C + c].
// A block of 1024 threads takes 64 filter elements (o, c): wave w sums nine of the 36 points (w % 4) over a
// quarter of the parts (w / 4: contiguous stretches, each in ascending order; consecutive lanes read consecutive
// elements), the quarters are added in ascending order in LDS, and the first wave applies G^T . G and stores the
// 64 x 9 results, which are contiguous in dw, as whole lines.  (One wave per nine points over all parts took
// 19 us with the 85 parts of a one-kernel filter gradient.)
constexpr int kPartSlices = 4;
__global__ __launch_bounds__(256 * kPartSlices) void wino_filter_grad_kernel(const float *__restrict__ part, float *__restrict__ dw,
                                                                             int oc, int parts) {
  __shared__ float slices[kPartSlices][kXi][64 + 1];
  __shared__ float sums[kXi][64 + 1];
  __shared__ float outs[64 * 9];
  const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3, slice = threadIdx.x >> 8;
  const int i0 = blockIdx.x * 64, i = i0 + lane;
  if (i < oc) {
    const int64_t step = static_cast<int64_t>(kXi) * oc;
    const int per = (parts + kPartSlices - 1) / kPartSlices;
    const int p0 = slice * per, p1 = min(parts, p0 + per);
    float sum[9];
#pragma unroll
    for (int j = 0; j < 9; ++j) sum[j] = 0.0f;
    for (int p = p0; p < p1; ++p) {
#pragma unroll
      for (int j = 0; j < 9; ++j) sum[j] += part[p * step + static_cast<int64_t>(9 * wave + j) * oc + i];
    }
#pragma unroll
    for (int j = 0; j < 9; ++j) slices[slice][9 * wave + j][lane] = sum[j];
  }
  __syncthreads();
  if (slice == 0 && i < oc) {
#pragma unroll
    for (int j = 0; j < 9; ++j) {
      float total = slices[0][9 * wave + j][lane];
#pragma unroll
      for (int q = 1; q < kPartSlices; ++q) total += slices[q][9 * wave + j][lane];
      sums[9 * wave + j][lane] = total;
    }
  }
  __syncthreads();
  if (threadIdx.x < 64 && i < oc) {
    float t[6][3];   // t[q][.] = G^T applied down column q
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      float col[6];
#pragma unroll
      for (int r = 0; r < 6; ++r) col[r] = sums[r * 6 + q][lane];
      gt_rows(col, t[q]);
    }
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const float row[6] = {t[0][r], t[1][r], t[2][r], t[3][r], t[4][r], t[5][r]};
      float w[3];
      gt_rows(row, w);
#pragma unroll
      for (int q = 0; q < 3; ++q) outs[lane * 9 + r * 3 + q] = w[q];
    }
  }
  __syncthreads();
  const int n = min(64, oc - i0) * 9;
  float *dst = dw + static_cast<int64_t>(i0) * 9;
  for (int k = threadIdx.x; k < n; k += 256 * kPartSlices) dst[k] = outs[k];
}

// ---------------------------------------------------------------- GEMM launch timing (opt-in)
// With TSplit_WinogradGemmTiming(1) every GEMM launch below is bracketed by two events on its own
// stream, so a benchmark can read the duration of these kernels inside its timed region.
struct TimedLaunch {
  hipEvent_t begin, end;
  int which;       // 0: forward / data-gradient GEMMs on 128 x 128 tiles, 1: filter-gradient GEMMs,
                   // 2: forward / data-gradient GEMMs on 64 x 256 tiles (at most 64 channels produced),
                   // 3 / 4: forward / data-gradient and filter-gradient GEMMs in split bf16,
                   // 5 / 6: forward / data gradient and filter gradient as one kernel each (wino_fused.h, wino_fgrad_fused.h)
  double flop, bytes;
};
std::mutex g_timing_mu;
unsigned g_timing_kinds = 0;   // bit k: launches of kind k are timed
std::vector<TimedLaunch> g_timed;

class GemmTiming {
 public:
  GemmTiming(hipStream_t st, int which, double flop, double bytes) : st_(st) {
    std::lock_guard<std::mutex> lk(g_timing_mu);
    if (!((g_timing_kinds >> which) & 1u)) return;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return;
    if (hipEventCreate(&t_.begin) != hipSuccess) return;
    if (hipEventCreate(&t_.end) != hipSuccess) {
      (void)hipEventDestroy(t_.begin);
      return;
    }
    t_.which = which;
    t_.flop = flop;
    t_.bytes = bytes;
    on_ = hipEventRecord(t_.begin, st) == hipSuccess;
  }
  ~GemmTiming() {
    if (!on_) return;
    (void)hipEventRecord(t_.end, st_);
    std::lock_guard<std::mutex> lk(g_timing_mu);
    g_timed.push_back(t_);
  }

 private:
  hipStream_t st_;
  TimedLaunch t_{};
  bool on_ = false;
};

// compute units of the current device and resident blocks of the GEMM kernel on each, asked once
inline int compute_units() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus < 1) {
      (void)hipGetLastError();
      cus = 256;
    }
    return cus;
  }();
  return n;
}

// How the filter-gradient GEMMs of one run are cut: tile shape, depth per range, and (128 x 128 tiles) the
// persistent grid.  Narrow layers (64 produced or gathered channels) take 64-wide tiles whose idle waves
// share the depth, one tile per block, with as many ranges as give three blocks per compute unit.  The
// others run on the persistent kernel: the number of ranges is chosen so that the units (tiles x ranges x
// 36) fill one, two or three rounds of the grid as fully as possible, fewer rounds winning unless more
// rounds fill at least 7 % better; a range keeps at least 12 k-steps.
struct GradPlan {
  int tile_m, tile_n;   // block tile
  int tm, tn;           // tiles
  int kchunk;           // depth per range
  int grid;             // persistent grid (128 x 128 tiles), else 0
};
constexpr int kGradBlocksPerCu = 3;

inline GradPlan plan_grad_gemm(int O, int C, int ld, int cus) {
  GradPlan g{};
  const int slots = cus * kGradBlocksPerCu / 8 * 8;
  if (O <= 64 || C <= 64) {
    g.tile_m = O <= 64 ? 64 : 128;
    g.tile_n = (g.tile_m == 128 || C <= 64) ? 64 : 128;
    g.tm = (O + g.tile_m - 1) / g.tile_m;
    g.tn = (C + g.tile_n - 1) / g.tile_n;
    const int per = kXi * g.tm * g.tn;
    int ranges = std::max(1, (slots + per / 2) / per);
    ranges = std::min(ranges, std::max(1, ld / 1024));
    g.kchunk = ((ld + ranges - 1) / ranges + 63) / 64 * 64;
    g.grid = 0;
    return g;
  }
  g.tile_m = g.tile_n = 128;
  g.tm = (O + 127) / 128;
  g.tn = (C + 127) / 128;
  const int per = kXi * g.tm * g.tn;
  const int max_ranges = std::max(1, ld / (12 * BK));
  int best_ranges = 1;
  double best_fill = 0.0;
  for (int rounds = 1; rounds <= 3; ++rounds) {
    const int ranges = std::min(max_ranges, std::max(1, rounds * slots / per));
    const int units = per * ranges;
    const double fill = static_cast<double>(units) / (static_cast<double>((units + slots - 1) / slots) * slots);
    if (fill > best_fill + 0.07 || (rounds == 1)) {
      best_fill = fill;
      best_ranges = ranges;
    }
  }
  g.kchunk = ((ld + best_ranges - 1) / best_ranges + BK - 1) / BK * BK;
  g.grid = slots;
  return g;
}

// `here` ranges of p.kchunk cover p.ld; partial sum z = range * 36 + xi goes to p.out + z * rows * cols
inline void launch_grad_gemm(const GradPlan &g, wg::GradProblem p, int here, hipStream_t st, bool split) {
  p.tm = g.tm;
  p.tn = g.tn;
  const int units = g.tm * g.tn * kXi * here;
  if (g.grid > 0) {
    const int grid = std::min(g.grid, (units + 7) / 8 * 8);
    if (split)
      hipLaunchKernelGGL((wg::wino_grad_gemm_split_kernel<kGradBlocksPerCu>), dim3(grid), dim3(kThreads), 0, st, p, units);
    else
      hipLaunchKernelGGL((wg::wino_grad_gemm_kernel<kGradBlocksPerCu>), dim3(grid), dim3(kThreads), 0, st, p, units);
    return;
  }
  const TileGrid tg{g.tm, g.tn, units};
  const dim3 grid(grid_blocks(g.tm, g.tn, kXi * here));
  if (g.tile_m == 64 && g.tile_n == 64)
    hipLaunchKernelGGL((wg::wino_grad_gemm_narrow_kernel<64, 64>), grid, dim3(kThreads), 0, st, p, tg);
  else if (g.tile_m == 128)
    hipLaunchKernelGGL((wg::wino_grad_gemm_narrow_kernel<128, 64>), grid, dim3(kThreads), 0, st, p, tg);
  else
    hipLaunchKernelGGL((wg::wino_grad_gemm_narrow_kernel<64, 128>), grid, dim3(kThreads), 0, st, p, tg);
}

// bytes of V and M one run of images may take together
inline int64_t run_bytes() {
  const char *e = std::getenv("TSPLIT_WINOGRAD_RUN_MIB");
  const long mibs = e ? std::atol(e) : 0;
  return static_cast<int64_t>(mibs > 0 ? mibs : 1024) << 20;
}

// images per run: what the scratch allowance holds of both transformed tensors, within reach of the GEMM
// loaders' 32-bit byte offsets (one transformed plane set is channels x tiles floats), in equal runs
inline int run_images(int imgs, int per_img, int chans_a, int chans_b) {
  const int64_t img_bytes = static_cast<int64_t>(chans_a + chans_b) * kXi * 4 * per_img;
  const int64_t reach = ((1ll << 31) - 64) / (4ll * std::max(chans_a, chans_b)) / per_img;
  int64_t run = std::min<int64_t>(std::max<int64_t>(1, run_bytes() / img_bytes), reach);
  if (run < 1) return 0;
  run = std::min<int64_t>(run, imgs);
  const int64_t runs = (imgs + run - 1) / run;
  return static_cast<int>((imgs + runs - 1) / runs);
}

}  // namespace

// Opt-in: the Winograd GEMMs of layers with more than 64 channels on both sides and the matrix products take
// their products in split bf16 (wino_gemm_split.h, gemm_split.h).  -1 until asked: the environment variable
// TSPLIT_SPLIT_BF16 then gives the first value.
std::atomic<int> g_split_bf16{-1};
bool split_bf16_enabled() {
  int v = g_split_bf16.load(std::memory_order_relaxed);
  if (v < 0) {
    const char *e = std::getenv("TSPLIT_SPLIT_BF16");
    v = e && std::atoi(e) != 0 ? 1 : 0;
    g_split_bf16.store(v, std::memory_order_relaxed);
  }
  return v != 0;
}

// Which layers take the one-kernel form: up to 256 channels on either side (in bands of 64 produced channels and
// chunks of 16 gathered ones).  Measured per 16- or 64-image call against the three-kernel routine: 64 -> 64 at
// 224 x 224 forward 467 -> 251 us, 128 -> 128 at 112 x 112 284 -> 232, 128 -> 256 at 56 x 56 486 -> 382, 256 -> 256
// at 56 x 56 778 -> 708; beyond that the three-kernel routine's GEMM, which runs at 120 TFLOP/s against 90 here,
// outweighs the transforms it pays for.  TSPLIT_WINOGRAD_FUSED=0 switches the form off, =2 lifts the limit.
namespace {
// 0: not this layer; otherwise the value of TSPLIT_WINOGRAD_FUSED (1 unless set)
inline int fused_form(int gathered, int produced) {
  static const int mode = [] {
    const char *e = std::getenv("TSPLIT_WINOGRAD_FUSED");
    return e ? std::atoi(e) : 1;
  }();
  if (mode == 0 || produced % fused::kBand || gathered % fused::kChunk) return 0;
  return (mode == 2 || std::max(gathered, produced) <= 256) ? mode : 0;
}
}  // namespace

// y[n][produced][H][W] = conv3x3(x[n][gathered][H][W], filter), stride 1, pad 1.  `rotated` selects
// the data-gradient reading of the filter (stored [gathered][produced][3][3], rotated 180 degrees).
// With a sink, every block of the output transform adds one partial (sum, sum of squares) per channel.
int conv_winograd_3x3(const float *x, const float *w, float *y, int imgs, int gathered, int produced, int H, int W,
                      bool rotated, hipStream_t st, StatsSink *sink) {
  const int th = (H + 3) / 4, tw = (W + 3) / 4;
  const int per_img = th * tw;
  {
    // few channels: the one-kernel form, whose transformed tensors never leave the chip (wino_fused.h)
    int gw = 0, gh = 0;
    // (with the opt-in split-bf16 products the layers they cover keep the three-kernel routine, whose GEMM takes them)
    const bool split_products = produced > 64 && (gathered & 7) == 0 && split_bf16_enabled();
    const int form = fused_form(gathered, produced);
    if (!split_products && form && (H & 3) == 0 && (W & 3) == 0 && aligned16(x) && aligned16(y) &&
        static_cast<int64_t>(imgs) * std::max(gathered, produced) * H * W < (1ll << 31)) {
      int groups = 0;
      if (fused::fused_group(tw, th, gw, gh, groups)) {
        const int items = imgs * groups * (produced / fused::kBand);
        const fused::FusedGeo fg{gathered, produced, H, W, tw, th, gw, gh, gw ? tw / gw : 0, groups, items};
        float *Uf = static_cast<float *>(scratch_get(st, 3, fused::fused_filter_floats(produced, gathered) * 4));
        TS_REQUIRE(Uf, "conv (Winograd): no scratch memory");
        hipLaunchKernelGGL(fused::wino_filter_fused_kernel, dim3((produced * gathered + 255) / 256), dim3(256), 0, st, w, Uf, produced,
                           gathered, rotated, fused::kAhead);
        const unsigned blocks = static_cast<unsigned>((items + 7) / 8 * 8);
        const double flop = 2.0 * kXi * produced * static_cast<double>(imgs) * per_img * gathered;
        const double bytes = 4.0 * (static_cast<double>(gathered + produced) * imgs * H * W + static_cast<double>(kXi) * produced * gathered);
        GemmTiming timed(st, 5, flop, bytes);
        const bool runs = gw == 0;
        if (sink) {
          const int parts = imgs * fg.groups;
          TS_REQUIRE(sink->used + parts <= sink->capacity, "conv (Winograd): statistics buffer too small");
          float *stats = sink->part + static_cast<int64_t>(sink->used) * produced * 2;
          if (runs)
            hipLaunchKernelGGL((fused::wino_fused_kernel<true, true>), dim3(blocks), dim3(fused::kThreadsF), 0, st, x, Uf, y, fg, stats);
          else
            hipLaunchKernelGGL((fused::wino_fused_kernel<true, false>), dim3(blocks), dim3(fused::kThreadsF), 0, st, x, Uf, y, fg, stats);
          sink->used += parts;
        } else if (runs) {
          hipLaunchKernelGGL((fused::wino_fused_kernel<false, true>), dim3(blocks), dim3(fused::kThreadsF), 0, st, x, Uf, y, fg,
                             static_cast<float *>(nullptr));
        } else {
          hipLaunchKernelGGL((fused::wino_fused_kernel<false, false>), dim3(blocks), dim3(fused::kThreadsF), 0, st, x, Uf, y, fg,
                             static_cast<float *>(nullptr));
        }
        return 0;
      }
    }
  }
  const int run = run_images(imgs, per_img, gathered, produced);
  TS_REQUIRE(run > 0, "conv (Winograd): one image's tiles do not fit 32-bit offsets");
  const int ld_max = (run * per_img + 3) / 4 * 4;
  float *U = static_cast<float *>(scratch_get(st, 3, static_cast<size_t>(kXi) * produced * gathered * 4));
  float *VM = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(kXi) * (gathered + produced) * ld_max * 4));
  TS_REQUIRE(U && VM, "conv (Winograd): no scratch memory");
  float *V = VM, *M = VM + static_cast<int64_t>(kXi) * gathered * ld_max;
  for (int first = 0; first < imgs; first += run) {
    const int n = std::min(run, imgs - first);
    WinoGeo gi{gathered, H, W, th, tw, n * per_img, (n * per_img + 3) / 4 * 4,
               (W & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0};
    WinoGeo go = gi;
    go.chans = produced;
    const float *xr = x + static_cast<int64_t>(first) * gathered * H * W;
    // the filter transform rides in the first rows of the first run's input transform
    const int nbx = (gi.ld + 255) / 256;
    FilterJob job{w, U, produced, gathered, rotated, 0, 0};
    if (first == 0) {
      job.blocks = (produced * gathered + 255) / 256;
      job.rows = (job.blocks + nbx - 1) / nbx;
      if (job.rows + gathered > 65535) {   // a huge filter beside a narrow grid: a launch of its own
        hipLaunchKernelGGL(wino_filter_kernel, dim3(job.blocks), dim3(256), 0, st, w, U, produced, gathered, rotated);
        job.blocks = job.rows = 0;
      }
    }
    const dim3 grid_in(nbx, job.rows + gathered);
    if ((W & 3) == 0 && (reinterpret_cast<uintptr_t>(xr) & 15) == 0)
      hipLaunchKernelGGL(wino_input_kernel<true>, grid_in, dim3(256), 0, st, xr, V, gi, job);
    else
      hipLaunchKernelGGL(wino_input_kernel<false>, grid_in, dim3(256), 0, st, xr, V, gi, job);
    {
      // every operand read once, the result written once
      const double flop = 2.0 * kXi * produced * static_cast<double>(gi.ld) * gathered;
      const double bytes = 4.0 * kXi * (static_cast<double>(produced) * gathered + static_cast<double>(gathered + produced) * gi.ld);
      const bool split = produced > 64 && (gathered & 7) == 0 && split_bf16_enabled();
      GemmTiming timed(st, split ? 3 : produced <= 64 ? 2 : 0, flop, bytes);
      const wg::Problem gemm{U, V, M, produced, gathered, gi.ld, 0, 0};
      if (split)
        wg::launch_split(gemm, st, compute_units());
      else
        wg::launch(gemm, st, compute_units());
    }
    const dim3 grid_out((go.tiles + 255) / 256, produced);
    float *yr = y + static_cast<int64_t>(first) * produced * H * W;
    if (sink) {
      TS_REQUIRE(sink->used + static_cast<int>(grid_out.x) <= sink->capacity, "conv (Winograd): statistics buffer too small");
      hipLaunchKernelGGL(wino_output_kernel<true>, grid_out, dim3(256), 0, st, M, yr, go,
                         sink->part + static_cast<int64_t>(sink->used) * produced * 2);
      sink->used += static_cast<int>(grid_out.x);
    } else {
      hipLaunchKernelGGL(wino_output_kernel<false>, grid_out, dim3(256), 0, st, M, yr, go, static_cast<float *>(nullptr));
    }
  }
  return 0;
}

// dw[O][C][3][3] = filter gradient of the 3x3 / stride 1 / pad 1 convolution of x[n][C][H][W] whose output
// gradient is dy[n][O][H][W]
int conv_winograd_3x3_filter_grad(const float *x, const float *dy, float *dw, int imgs, int C, int O, int H, int W,
                                  hipStream_t st) {
  const int th = (H + 3) / 4, tw = (W + 3) / 4;
  const int per_img = th * tw;
  const int64_t oc = static_cast<int64_t>(O) * C;
  {
    // few channels: the one-kernel form, whose transformed tensors never leave the chip (wino_fgrad_fused.h)
    const bool split_products = O > 64 && C > 64 && split_bf16_enabled();
    // Taken where it was measured faster than the three-kernel routine: at most 128 channels on both sides (with more
    // bands every band pair reads the activations again, and the routine's deep GEMMs run at three quarters of the
    // matrix peak) and at least 4096 tiles (below, its launch of ranges and their partial sums weigh more than the
    // transformed tensors' way through memory).  TSPLIT_WINOGRAD_FGRAD_FUSED: 0 never, 2 wherever the kernel can run.
    static const int fgrad_mode = [] {
      const char *e = std::getenv("TSPLIT_WINOGRAD_FGRAD_FUSED");
      return e ? std::atoi(e) : 1;
    }();
    const int64_t tiles = static_cast<int64_t>(imgs) * per_img;
    const bool pays = fgrad_mode == 2 ? tiles >= 16 * fgrad::kStep : (std::max(C, O) <= 128 && tiles >= 4096);
    if (fgrad_mode != 0 && pays && !split_products && fused_form(C, O) && (C % fgrad::kBandF) == 0 && (H & 3) == 0 && (W & 3) == 0 &&
        aligned16(x) && aligned16(dy) && static_cast<int64_t>(imgs) * std::max(C, O) * H * W < (1ll << 29)) {
      fgrad::FGradGeo fg{C, O, H, W, tw, th, imgs * per_img, 0, 0, C / fgrad::kBandF, O / fgrad::kBandF, 0};
      fgrad::fgrad_plan(fg, compute_units());
      float *part = static_cast<float *>(scratch_get(st, 3, static_cast<size_t>(fg.ranges) * kXi * oc * 4));
      TS_REQUIRE(part, "conv (Winograd): no scratch memory");
      {
        const double flop = 2.0 * kXi * O * static_cast<double>(fg.tiles) * C;
        const double bytes = 4.0 * (static_cast<double>(C + O) * imgs * H * W + static_cast<double>(kXi) * oc * fg.ranges);
        GemmTiming timed(st, 6, flop, bytes);
        hipLaunchKernelGGL(fgrad::wino_fgrad_fused_kernel, dim3(static_cast<unsigned>((fg.items + 7) / 8 * 8)), dim3(256), 0, st, x, dy, part,
                           fg);
      }
      hipLaunchKernelGGL(wino_filter_grad_kernel, dim3(static_cast<unsigned>((oc + 63) / 64)), dim3(256 * kPartSlices), 0, st, part, dw,
                         static_cast<int>(oc), fg.ranges);
      return 0;
    }
  }
  const int run = run_images(imgs, per_img, C, O);
  TS_REQUIRE(run > 0, "conv (Winograd): one image's tiles do not fit 32-bit offsets");
  const int runs = (imgs + run - 1) / run;
  const int ld_max = (run * per_img + 3) / 4 * 4;
  const GradPlan plan = plan_grad_gemm(O, C, ld_max, compute_units());
  const int kchunk = plan.kchunk;
  const int parts_max = runs * ((ld_max + kchunk - 1) / kchunk);
  float *VY = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(kXi) * (C + O) * ld_max * 4));
  float *part = static_cast<float *>(scratch_get(st, 3, static_cast<size_t>(parts_max) * kXi * oc * 4));
  TS_REQUIRE(VY && part, "conv (Winograd): no scratch memory");
  float *V = VY, *Y = VY + static_cast<int64_t>(kXi) * C * ld_max;
  int parts = 0;
  for (int first = 0; first < imgs; first += run) {
    const int n = std::min(run, imgs - first);
    const float *xr = x + static_cast<int64_t>(first) * C * H * W, *dyr = dy + static_cast<int64_t>(first) * O * H * W;
    WinoGeo gx{C, H, W, th, tw, n * per_img, (n * per_img + 3) / 4 * 4, false};
    WinoGeo gy = gx;
    gy.chans = O;
    const dim3 grid_xy((gx.ld + 255) / 256, C + O);
    const bool qx = (W & 3) == 0 && (reinterpret_cast<uintptr_t>(xr) & 15) == 0;
    const bool qy = (W & 3) == 0 && (reinterpret_cast<uintptr_t>(dyr) & 15) == 0;
    if (qx && qy)
      hipLaunchKernelGGL((wino_grad_pair_kernel<true, true>), grid_xy, dim3(256), 0, st, xr, V, gx, dyr, Y, gy);
    else if (qx)
      hipLaunchKernelGGL((wino_grad_pair_kernel<true, false>), grid_xy, dim3(256), 0, st, xr, V, gx, dyr, Y, gy);
    else if (qy)
      hipLaunchKernelGGL((wino_grad_pair_kernel<false, true>), grid_xy, dim3(256), 0, st, xr, V, gx, dyr, Y, gy);
    else
      hipLaunchKernelGGL((wino_grad_pair_kernel<false, false>), grid_xy, dim3(256), 0, st, xr, V, gx, dyr, Y, gy);
    const int here = (gx.ld + kchunk - 1) / kchunk;
    {
      const bool split = plan.grid > 0 && split_bf16_enabled();
      GemmTiming timed(st, split ? 4 : 1, 2.0 * kXi * O * static_cast<double>(gx.ld) * C,
                       4.0 * kXi * (static_cast<double>(O) * C * here + static_cast<double>(O + C) * gx.ld));
      launch_grad_gemm(plan, wg::GradProblem{Y, V, part + static_cast<int64_t>(parts) * kXi * oc, O, C, gx.ld, kchunk, 0, 0},
                       here, st, split);
    }
    parts += here;
  }
  hipLaunchKernelGGL(wino_filter_grad_kernel, dim3(static_cast<unsigned>((oc + 63) / 64)), dim3(256 * kPartSlices), 0, st, part, dw,
                     static_cast<int>(oc), parts);
  return 0;
}

}  // namespace tsplit

// Switches the split-bf16 products of the Winograd routine's GEMMs and of the matrix products on or off (off unless the environment
// variable TSPLIT_SPLIT_BF16 says otherwise); `was`, if given, receives the previous setting.
extern "C" int TSplit_SplitBf16(int on, int *was) {
  const bool before = tsplit::split_bf16_enabled();
  tsplit::g_split_bf16.store(on != 0 ? 1 : 0, std::memory_order_relaxed);
  if (was) *was = before ? 1 : 0;
  return 0;
}

// Switches the timing of the Winograd routine's GEMM launches on (1: every kind, 2 + k: kind k only) or off (0),
// and forgets what was recorded.
extern "C" int TSplit_WinogradGemmTiming(int on) {
  using namespace tsplit;
  std::lock_guard<std::mutex> lk(g_timing_mu);
  for (TimedLaunch &t : g_timed) {
    (void)hipEventDestroy(t.begin);
    (void)hipEventDestroy(t.end);
  }
  g_timed.clear();
  g_timing_kinds = on == 1 ? ~0u : (on >= 2 && on < 34) ? 1u << (on - 2) : 0u;
  return 0;
}

// The summed algorithmic bytes (every operand read once, the result written once) of the recorded launches
// of kind `which`.
extern "C" int TSplit_WinogradGemmBytes(int which, double *bytes) {
  using namespace tsplit;
  std::lock_guard<std::mutex> lk(g_timing_mu);
  double total = 0;
  for (const TimedLaunch &t : g_timed)
    if (t.which == which) total += t.bytes;
  if (bytes) *bytes = total;
  return 0;
}

// Waits for the recorded launches of kind `which` and reports their number, summed duration in
// milliseconds and summed GEMM FLOP (2 * 36 * rows * columns * depth per launch); -1 on a HIP error.
extern "C" int TSplit_WinogradGemmTimes(int which, double *launches, double *ms, double *flop) {
  using namespace tsplit;
  std::lock_guard<std::mutex> lk(g_timing_mu);
  double n = 0, total = 0, work = 0;
  for (const TimedLaunch &t : g_timed) {
    if (t.which != which) continue;
    float one = 0.0f;
    TS_HIP(hipEventSynchronize(t.end));
    TS_HIP(hipEventElapsedTime(&one, t.begin, t.end));
    n += 1;
    total += one;
    work += t.flop;
  }
  if (launches) *launches = n;
  if (ms) *ms = total;
  if (flop) *flop = work;
  return 0;
}
