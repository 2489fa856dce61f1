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

#include "common.h"
#include "mfma_gemm.h"

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
__global__ __launch_bounds__(256) void wino_filter_kernel(const float *__restrict__ w, float *__restrict__ U, int produced,
                                                          int gathered, bool rotated) {
  const int i = blockIdx.x * 256 + threadIdx.x;
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

// one thread per (channel, tile): grid (ceil(ld / 256), chans).  With QUADS (W a multiple of 4, planes
// 16-byte aligned) a thread loads the aligned quad of each of its six rows and takes the two columns
// beside it from the neighbouring lanes, which hold the neighbouring tiles of the same tile row; at
// a wave's ends those come from memory, at the plane's edges they are the zero padding.
template <bool QUADS>
__global__ __launch_bounds__(256) void wino_input_kernel(const float *__restrict__ x, float *__restrict__ V, WinoGeo g) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.ld) return;
  const int c = blockIdx.y;
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

// ---------------------------------------------------------------- output transform
// rows of A^T applied to (m0 .. m5)
__device__ __forceinline__ void at_rows(const float m[6], float o[4]) {
  const float s12 = m[1] + m[2], d12 = m[1] - m[2], s34 = m[3] + m[4], d34 = m[3] - m[4];
  o[0] = m[0] + s12 + s34;
  o[1] = d12 + 2.0f * d34;
  o[2] = s12 + 4.0f * s34;
  o[3] = d12 + 8.0f * d34 + m[5];
}

// one thread per (channel, tile): grid (ceil(tiles / 256), chans)
__global__ __launch_bounds__(256) void wino_output_kernel(const float *__restrict__ M, float *__restrict__ y, WinoGeo g) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.tiles) return;
  const int o = blockIdx.y;
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
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (4 * tx + q < g.W) dst[q] = v[q];
    }
  }
}

// bytes of V and M one run of images may take together
inline int64_t run_bytes() {
  const char *e = std::getenv("TSPLIT_WINOGRAD_RUN_MIB");
  const long mibs = e ? std::atol(e) : 0;
  return static_cast<int64_t>(mibs > 0 ? mibs : 1024) << 20;
}

}  // namespace

// y[n][produced][H][W] = conv3x3(x[n][gathered][H][W], filter), stride 1, pad 1.  `rotated` selects
// the data-gradient reading of the filter (stored [gathered][produced][3][3], rotated 180 degrees).
int conv_winograd_3x3(const float *x, const float *w, float *y, int imgs, int gathered, int produced, int H, int W,
                      bool rotated, hipStream_t st) {
  const int th = (H + 3) / 4, tw = (W + 3) / 4;
  const int per_img = th * tw;
  const int64_t img_bytes = static_cast<int64_t>(gathered + produced) * kXi * 4 * per_img;
  int run = static_cast<int>(std::max<int64_t>(1, run_bytes() / img_bytes));
  run = std::min(run, imgs);
  const int runs = (imgs + run - 1) / run;
  run = (imgs + runs - 1) / runs;   // equal runs
  const int ld_max = (run * per_img + 3) / 4 * 4;
  TS_REQUIRE(static_cast<int64_t>(std::max(gathered, produced)) * ld_max * 4 < (1ll << 31),
             "conv (Winograd): a run of %d images does not fit 32-bit offsets", run);
  float *U = static_cast<float *>(scratch_get(st, 3, static_cast<size_t>(kXi) * produced * gathered * 4));
  float *VM = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(kXi) * (gathered + produced) * ld_max * 4));
  TS_REQUIRE(U && VM, "conv (Winograd): no scratch memory");
  float *V = VM, *M = VM + static_cast<int64_t>(kXi) * gathered * ld_max;
  hipLaunchKernelGGL(wino_filter_kernel, dim3((produced * gathered + 255) / 256), dim3(256), 0, st, w, U, produced,
                     gathered, rotated);
  using AL = KContigBufLoader<128>;
  using BL = MnContigBufLoader<128>;
  for (int first = 0; first < imgs; first += run) {
    const int n = std::min(run, imgs - first);
    WinoGeo gi{gathered, H, W, th, tw, n * per_img, (n * per_img + 3) / 4 * 4,
               (W & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0};
    WinoGeo go = gi;
    go.chans = produced;
    const float *xr = x + static_cast<int64_t>(first) * gathered * H * W;
    if ((W & 3) == 0 && (reinterpret_cast<uintptr_t>(xr) & 15) == 0)
      hipLaunchKernelGGL(wino_input_kernel<true>, dim3((gi.ld + 255) / 256, gathered), dim3(256), 0, st, xr, V, gi);
    else
      hipLaunchKernelGGL(wino_input_kernel<false>, dim3((gi.ld + 255) / 256, gathered), dim3(256), 0, st, xr, V, gi);
    const int tm = (produced + 127) / 128, tn = (gi.ld + 127) / 128;
    typename AL::Params ap{U, gathered, produced, gathered};
    typename BL::Params bp{V, gi.ld, gi.ld, gathered};
    hipLaunchKernelGGL((mfma_batched_gemm_kernel<128, 128, 2, 2, AL, BL>), dim3(grid_blocks(tm, tn, kXi)), dim3(kThreads),
                       0, st, ap, bp, M, static_cast<int64_t>(produced) * gathered, static_cast<int64_t>(gathered) * gi.ld,
                       static_cast<int64_t>(produced) * gi.ld, produced, gi.ld, gathered, TileGrid{tm, tn, tm * tn * kXi});
    hipLaunchKernelGGL(wino_output_kernel, dim3((go.tiles + 255) / 256, produced), dim3(256), 0, st, M,
                       y + static_cast<int64_t>(first) * produced * H * W, go);
  }
  return 0;
}

}  // namespace tsplit
