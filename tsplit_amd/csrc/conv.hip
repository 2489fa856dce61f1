// Conv2d forward, backward-data and backward-filter as implicit GEMMs on the fp32 MFMA tile
// engine.  NCHW activations, OIHW filters, cross-correlation, no bias, square stride,
// dilation 1, separate (pad_h, pad_w).  No im2col buffer is ever materialised: the gather
// loaders below compute im2col addresses on the fly while staging tiles into LDS.
//
//   forward     y[img,o,p]  : M = O,  N = imgs*oH*oW, K = C*kH*kW
//                 A = filter [O][K] as it lies in memory (K contiguous)
//                 B = gather of x: (k=(c,kh,kw), n=(img,oh,ow)) -> x[img,c,oh*s-ph+kh,ow*s-pw+kw]
//   bwd-data    dx[img,c,q] : M = C,  N = imgs*H*W,   K = O*kH*kW
//                 A = filter re-laid as [C][O*kH*kW] by a small kernel (<= 9.4 MB per VGG layer)
//                 B = gather of dy: (k=(o,kh,kw), n=(img,h,w)) -> dy[img,o,(h+ph-kh)/s,(w+pw-kw)/s]
//   bwd-filter  dw[o,j]     : M = O,  N = C*kH*kW,    K = imgs*oH*oW   (split-K, folded in order)
//                 A = dy: (m=o, k=(img,p)) -> dy[img,o,p]       (K contiguous inside an image)
//                 B = gather of x: (k=(img,oh,ow), j=(c,kh,kw)) -> x[img,c,oh*s-ph+kh,ow*s-pw+kw]
//
// The (c,kh,kw) -> offset decomposition is a per-geometry table built once on the host and
// cached on the device; the (img,oh,ow) decomposition uses multiply-shift division and is
// done once per thread (forward, bwd-data: a thread's columns never change) or once per
// k-step (bwd-filter).
#include <algorithm>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>
#include <type_traits>
#include <vector>

#include "common.h"
#include "fastdiv.h"
#include "mfma_gemm.h"

namespace tsplit {
// winograd.hip
int conv_winograd_3x3(const float *x, const float *w, float *y, int imgs, int gathered, int produced, int H, int W,
                      bool rotated, hipStream_t st, StatsSink *sink = nullptr);
int conv_winograd_3x3_filter_grad(const float *x, const float *dy, float *dw, int imgs, int C, int O, int H, int W,
                                  hipStream_t st);
namespace {

using namespace mg;

struct ConvGeo {
  int imgs, C, H, W, O, kH, kW, ph, pw, s, oH, oW;
};

// one entry per reduction index (c|o, kh, kw)
struct Tap {
  int off;      // offset of the tap inside one image of the gathered tensor
  short kh, kw;
};

// ------------------------------------------------------------------ tap tables (host cache)
struct TapKey {
  int chans, kH, kW, plane_w, plane_hw, sign;
  bool operator<(const TapKey &o) const {
    return std::tie(chans, kH, kW, plane_w, plane_hw, sign) <
           std::tie(o.chans, o.kH, o.kW, o.plane_w, o.plane_hw, o.sign);
  }
};
std::map<TapKey, Tap *> g_taps;
std::mutex g_taps_mu;

// off = ch*plane_hw + sign*(kh*plane_w + kw)
const Tap *tap_table(int chans, int kH, int kW, int plane_w, int plane_hw, int sign) {
  std::lock_guard<std::mutex> lk(g_taps_mu);
  TapKey key{chans, kH, kW, plane_w, plane_hw, sign};
  auto it = g_taps.find(key);
  if (it != g_taps.end()) return it->second;
  std::vector<Tap> h(static_cast<size_t>(chans) * kH * kW);
  size_t i = 0;
  for (int c = 0; c < chans; ++c)
    for (int a = 0; a < kH; ++a)
      for (int b = 0; b < kW; ++b, ++i) {
        h[i].off = c * plane_hw + sign * (a * plane_w + b);
        h[i].kh = static_cast<short>(a);
        h[i].kw = static_cast<short>(b);
      }
  Tap *d = nullptr;
  if (hipMalloc(&d, h.size() * sizeof(Tap)) != hipSuccess) return nullptr;
  if (hipMemcpy(d, h.data(), h.size() * sizeof(Tap), hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipFree(d);
    return nullptr;
  }
  g_taps[key] = d;
  return d;
}

// ------------------------------------------------------------------ gather loader, k-major
// Serves forward (gathers x) and bwd-data (gathers dy).  Column n = (img, r, c) of the GEMM
// output; reduction index k = (ch, kh, kw).
//   forward : src row = r*s - ph + kh           (always "divisible")
//   bwd-data: src row = (r + ph - kh) / s       valid only when divisible and inside
template <int BN, bool BWD_DATA>
struct GatherColsLoader {
  using Lds = KMajorLds<BN>;
  struct Params {
    const float *src;     // x (forward) or dy (bwd-data)
    const Tap *taps;
    FastDiv plane;        // columns per image: oH*oW (forward) or H*W (bwd-data)
    FastDiv width;        // oW (forward) or W (bwd-data)
    int64_t img_stride;   // elements per image of src
    int src_h, src_w;     // extent of one plane of src
    int ph, pw, s;
    int n_total;
  };
  static constexpr int kPerThread = BN / 16;          // 16 * BN / 256
  static constexpr int kKStep = kThreads / BN;        // 2 (BN=128) or 1 (BN=256)
  float r[kPerThread];
  const float *base;
  const Tap *taps;
  int r0, c0;            // forward: oh*s-ph, ow*s-pw ; bwd-data: h+ph, w+pw
  int src_h, src_w, s, kfirst;
  bool col_ok;

  __device__ __forceinline__ void init(const Params &P, int n0, int tid) {
    const int n = n0 + tid % BN;
    kfirst = tid / BN;
    col_ok = n < P.n_total;
    const uint32_t nn = col_ok ? n : 0;
    const uint32_t img = P.plane.div(nn);
    const uint32_t p = nn - img * P.plane.d;
    const uint32_t row = P.width.div(p);
    const uint32_t col = p - row * P.width.d;
    taps = P.taps;
    src_h = P.src_h;
    src_w = P.src_w;
    s = P.s;
    if (BWD_DATA) {
      r0 = static_cast<int>(row) + P.ph;
      c0 = static_cast<int>(col) + P.pw;
      base = P.src + static_cast<int64_t>(img) * P.img_stride;
    } else {
      r0 = static_cast<int>(row) * P.s - P.ph;
      c0 = static_cast<int>(col) * P.s - P.pw;
      base = P.src + static_cast<int64_t>(img) * P.img_stride + static_cast<int64_t>(r0) * P.src_w + c0;
    }
  }
  __device__ __forceinline__ void load(int k0, int kend) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int k = k0 + kfirst + kKStep * i;
      float v = 0.f;
      if (col_ok && k < kend) {
        const Tap t = taps[k];
        if (BWD_DATA) {
          int rr = r0 - t.kh, cc = c0 - t.kw;
          bool ok = rr >= 0 && cc >= 0;
          if (s != 1) {
            ok = ok && (rr % s == 0) && (cc % s == 0);
            rr /= s;
            cc /= s;
          }
          // tap offset already holds the channel part; the spatial part is recomputed here
          if (ok && rr < src_h && cc < src_w)
            v = base[static_cast<int64_t>(t.off) + static_cast<int64_t>(rr) * src_w + cc];
        } else {
          const int rr = r0 + t.kh, cc = c0 + t.kw;
          if (static_cast<unsigned>(rr) < static_cast<unsigned>(src_h) &&
              static_cast<unsigned>(cc) < static_cast<unsigned>(src_w))
            v = base[t.off];
        }
      }
      r[i] = v;
    }
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) lds[(kfirst + kKStep * i) * Lds::kStride + tid % BN] = r[i];
  }
};


// ------------------------------------------------------------------ tap-major gather loader
// Fast path of forward and (stride 1) bwd-data when the channel count is a multiple of 16.
// The reduction index is re-ordered k' = ((ch/16)*kH*kW + tap)*16 + ch%16, so one 16-wide
// k-step covers 16 consecutive channels of ONE filter tap, and the kH*kW steps that follow
// each other gather from the same 16 channel planes (L1 hits): the padding test is done once per
// step and thread instead of once per element, there is no tap table, and a thread's 8 (or
// 16) values are consecutive in k', so they go to an mn-major LDS tile with 16-byte writes
// and are read back with 16-byte reads.  The filter is re-laid to match by a small kernel.
template <int BN, bool BWD_DATA>
struct TapMajorColsLoader {
  using Lds = MnMajorLds<BN>;
  struct Params {
    const float *src;     // x (forward) or dy (bwd-data)
    FastDiv plane;        // columns per image
    FastDiv width;
    int64_t img_stride;   // elements per image of src
    int chan_stride;      // elements per channel plane of src
    int src_h, src_w;
    int ph, pw, s;
    int chans, kW, taps_total;
    int n_total;
  };
  static constexpr int kPerThread = BN / 16;      // 8 or 16 consecutive k'
  static constexpr int kQuads = kPerThread / 4;
  float4 r[kQuads];
  const float *base;      // image base
  int r0, c0;             // forward: oh*s-ph, ow*s-pw ; bwd-data: h+ph, w+pw
  int src_h, src_w, chan_stride, kW, taps_total;
  int klocal0;            // first k' (within a step) of this thread
  int tap, ch0;           // running position of the current step: tap index and first channel
  bool col_ok, started;

  __device__ __forceinline__ void init(const Params &P, int n0, int tid) {
    const int n = n0 + tid % BN;
    klocal0 = (tid / BN) * kPerThread;
    col_ok = n < P.n_total;
    const uint32_t nn = col_ok ? n : 0;
    const uint32_t img = P.plane.div(nn);
    const uint32_t p = nn - img * P.plane.d;
    const uint32_t row = P.width.div(p);
    const uint32_t col = p - row * P.width.d;
    src_h = P.src_h;
    src_w = P.src_w;
    chan_stride = P.chan_stride;
    kW = P.kW;
    taps_total = P.taps_total;
    base = P.src + static_cast<int64_t>(img) * P.img_stride;
    if (BWD_DATA) {
      r0 = static_cast<int>(row) + P.ph;
      c0 = static_cast<int>(col) + P.pw;
    } else {
      r0 = static_cast<int>(row) * P.s - P.ph;
      c0 = static_cast<int>(col) * P.s - P.pw;
    }
    started = false;
  }
  __device__ __forceinline__ void load(int k0, int /*kend*/) {
    if (!started) {            // steps arrive in order; only the first needs a division
      const int step = k0 / BK;
      ch0 = (step / taps_total) * BK;
      tap = step % taps_total;
      started = true;
    }
    const int kh = tap / kW, kw = tap - kh * kW;
    const int rr = BWD_DATA ? r0 - kh : r0 + kh;
    const int cc = BWD_DATA ? c0 - kw : c0 + kw;
    const bool ok = col_ok && static_cast<unsigned>(rr) < static_cast<unsigned>(src_h) &&
                    static_cast<unsigned>(cc) < static_cast<unsigned>(src_w);
    const float *p = base + static_cast<int64_t>(ch0 + klocal0) * chan_stride + rr * src_w + cc;
#pragma unroll
    for (int q = 0; q < kQuads; ++q) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (ok) {
        v.x = p[(4 * q + 0) * chan_stride];
        v.y = p[(4 * q + 1) * chan_stride];
        v.z = p[(4 * q + 2) * chan_stride];
        v.w = p[(4 * q + 3) * chan_stride];
      }
      r[q] = v;
    }
    if (++tap == taps_total) {   // all taps of these 16 channels first: the gathers of
      tap = 0;                   // consecutive steps then hit the same cache lines
      ch0 += BK;
    }
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int q = 0; q < kQuads; ++q)
      *reinterpret_cast<float4 *>(lds + (tid % BN) * Lds::kStride + klocal0 + 4 * q) = r[q];
  }
};


// ------------------------------------------------------------------ the tap-major conv kernel
// Forward and stride-1 backward-data for channel counts that are multiples of 16: the same
// tiling, LDS layout and MFMA schedule as mfma_gemm_kernel with both operands mn-major, but
// with the k-loop written so that it needs almost no vector-ALU work.  On this chip a VALU
// instruction issued while the matrix pipe is saturated costs MFMA issue time, so address
// arithmetic in the loop is what separates 63 % from the clock-limited rate.  Here:
//   * all global reads are buffer loads: per-thread byte offsets are loop constants, the part
//     that changes per step (filter tap, channel block, k position) is wave-uniform and
//     travels in the scalar offset, computed on the scalar unit;
//   * a thread's padding test for all taps is one bit mask built before the loop; a lane
//     whose tap falls into the padding gets an out-of-range offset, for which a buffer load
//     returns 0 - no zero-fill, no divergent branch.
struct TapConvParams {
  // filter re-laid as [M][K], k' = ((ch/16)*taps + tap)*16 + ch%16 - or, for the RAW kernels, the
  // filter as it lies in memory, [O][C][taps]: element (row m, channel ch, tap) at
  // m*raw_row + ch*raw_ch + tap (forward: rows are O, channels C; backward-data: the other way)
  const float *wf;
  int raw_row, raw_ch;
  const float *src;     // x (forward) or dy (backward-data)
  unsigned wf_bytes, src_bytes;
  FastDiv plane, width; // output columns per image / per row
  int img_stride;       // elements per image of src
  int chan_stride;      // elements per channel plane of src
  int src_h, src_w, ph, pw, s, kW, taps;
  int M, N, K;
  int out_plane;        // elements per channel plane of the output
  int64_t out_img_stride;
  // Column (i, j) of an image goes to element (out_a0 + out_s*i)*out_w + out_b0 + out_s*j of its
  // output plane.  out_s == 1 with out_a0 = out_b0 = 0 and out_w = the column width: linear.
  int out_s, out_a0, out_b0, out_w;
  // STATS kernels: partial (sum, sum of squares) of output row m over the 32 columns [32 g, 32 g + 32)
  // goes to stats[(g * M + m) * 2]
  float *stats;
};

// Sums over the 32 lanes of each half of a wave for NR registers at once, NR = 32 or 16: in step b the
// lanes whose bit b is clear keep the lower half of the registers and the others the upper half, each
// adding what its partner held of that half, so that NR + NR/2 + ... shuffles do the work of 5 NR.
// Afterwards r[0] of lane l is the sum of register (l % 32) for NR = 32, of register (l % 32) / 2 for
// NR = 16 (both lanes of a pair hold it).
template <int NR>
__device__ __forceinline__ void half_wave_sums(float (&r)[NR], int lane) {
  static_assert(NR == 32 || NR == 16, "one or two registers per lane and row");
  constexpr int kTop = NR == 32 ? 4 : 3;   // register halving runs over lane bits 4..0 or 4..1
#pragma unroll
  for (int step = 0; step <= kTop; ++step) {
    const int h = NR >> (step + 1);
    const int bit = 4 - step;
    const bool up = (lane >> bit) & 1;
#pragma unroll
    for (int i = 0; i < h; ++i) {
      const float send = up ? r[i] : r[i + h], keep = up ? r[i + h] : r[i];
      r[i] = keep + __shfl_xor(send, 1 << bit, 64);
    }
  }
  if (NR == 16) r[0] += __shfl_xor(r[0], 1, 64);
}

// offset of output column n (without the row term)
__device__ __forceinline__ int64_t tap_out_col(const TapConvParams &P, int n) {
  const uint32_t img = P.plane.div(n);
  const uint32_t p = n - img * P.plane.d;
  if (P.out_s == 1) return static_cast<int64_t>(img) * P.out_img_stride + p;
  const uint32_t i = P.width.div(p), j = p - i * P.width.d;
  return static_cast<int64_t>(img) * P.out_img_stride +
         static_cast<int64_t>(P.out_a0 + P.out_s * static_cast<int>(i)) * P.out_w + (P.out_b0 + P.out_s * static_cast<int>(j));
}


// Work distribution.  The tiles of one M row (tile_m fixed) form a chain; block `logical`
// works on row logical % tm, so the tm blocks with consecutive ids sit on the tiles that share
// one set of gathered columns, at the same k-step at about the same time, in one XCD (ids are
// transposed so that an XCD owns consecutive ids): the gathered operand comes from HBM once
// and from that XCD's L2 for the other tm - 1 tiles.  The grid is one full wave of resident
// blocks.  A row's tiles are first taken whole, one per block and wave of blocks - all blocks
// of an XCD then walk k together and share each step's filter words in its L2 as well - and
// the tiles left over (fewer than there are blocks; all of them in a layer with few tiles) are
// cut "stream-K" fashion: the unit of work is one 16-wide k-step, every block takes an equal
// contiguous range of the leftover chain, so 3.06 tiles per slot cost 3.06 tile-times, not 4,
// and 392 tiles keep 512 slots busy.  A range is shorter than a tile; a block parks the
// accumulators of its (at most two) partial pieces in scratch - slot 0 for a piece that is
// the first segment of its range, slot 1 for a partial last segment - and a second kernel
// adds the pieces of each cut tile in ascending block order and writes the tile.  Nothing
// depends on scheduling; results do depend on where the cuts fall, i.e. on the problem shape.
struct StreamK {
  int ksteps;            // k-steps per tile
  int total;             // k-steps of the cut part of one M row's chain
  int iters_per_block;
  int tm;                // M tiles (tile index = tile_n * tm + tile_m)
  int ranges;            // blocks per M row
  int whole_waves;       // tiles every block takes whole before its range of the cut part
  int cut_first;         // tile_n of the first tile of the cut part (= whole_waves * ranges)
};

// RAW: the filter operand is read from the [O][C][taps] filter itself with four 4-byte loads per
// 16-byte word of the re-laid form; for small backward-data passes, where a re-lay kernel in
// front of every call costs more than the extra loads.
// MINB: resident blocks per CU the register budget is cut for.  2 leaves every value in registers;
// 3 spills a dozen set-up values but keeps a third block resident, which pays on layers with
// thousands of tiles (+1-4 % on the VGG layers) and costs on small ones (finer pieces, -1-3 % on
// the ResNet-50 / Inception-v4 steps), so the launcher picks by tile count.
// STATS: a block that stores a whole tile also leaves the per-row sums and sums of squares of each
// 32-column group of it (partial sums for a BatchNorm that follows; columns beyond N are zeros).
template <int BM, int BN, int WM, int WN, bool BWD_DATA, bool RAW, int MINB, bool STATS = false>
__global__ __launch_bounds__(kThreads, MINB) void conv_tap_kernel(TapConvParams P, float *__restrict__ out,
                                                               float *__restrict__ pieces, StreamK sk) {
  static_assert(WM * WN == 4 && BM / WM == 64 && BN / WN == 64, "each of the 4 waves owns a 64x64 sub-tile");
  using ALds = MnMajorLds<BM>;
  using BLds = MnMajorLds<BN>;
  constexpr int PA = BM / 64;        // 16-byte filter words per thread and step
  constexpr int KPT = BN / 16;       // gathered values per thread and step (consecutive k')
  // one array: the STATS epilogue borrows the stages (4 waves x 32 x 68 floats) for its transposition
  __shared__ __attribute__((aligned(16))) float lds_all[2 * (ALds::kFloats + BLds::kFloats)];
  static_assert(!STATS || 4 * 32 * 68 <= 2 * (ALds::kFloats + BLds::kFloats), "the operand stages hold the staging areas");
  float(*lds_a)[ALds::kFloats] = reinterpret_cast<float(*)[ALds::kFloats]>(lds_all);
  float(*lds_b)[BLds::kFloats] = reinterpret_cast<float(*)[BLds::kFloats]>(lds_all + 2 * ALds::kFloats);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WN) * 64, wn0 = (wave % WN) * 64;
  // consecutive workgroup ids go to different XCDs: transpose so that an XCD owns a contiguous
  // eighth of the work (neighbouring tiles share gathered activations in its L2)
  const int logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int range = logical / sk.tm, tile_m = logical - range * sk.tm;
  const int it_begin = range * sk.iters_per_block;
  int it = it_begin;
  const int it_end = min(sk.total, it + sk.iters_per_block);

  // uniform bias so that every per-thread offset is non-negative and every scalar offset too
  const int bias = BWD_DATA ? (P.taps / P.kW - 1) * P.src_w + (P.kW - 1) : P.ph * P.src_w + P.pw;
  const __amdgpu_buffer_rsrc_t ra =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.wf), 0, static_cast<int>(P.wf_bytes), kBufFlags);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(P.src) - bias, 0, static_cast<int>(P.src_bytes + 4u * bias), kBufFlags);
  const int klocal0 = (tid / BN) * KPT;

  int wave_no = 0;
  while (wave_no < sk.whole_waves || it < it_end) {
    int tile_n, ks0, ks1;
    if (wave_no < sk.whole_waves) {
      tile_n = wave_no * sk.ranges + range;
      ks0 = 0;
      ks1 = sk.ksteps;
      ++wave_no;
    } else {
      const int t = it / sk.ksteps;
      tile_n = sk.cut_first + t;
      ks0 = it - t * sk.ksteps;
      ks1 = min(sk.ksteps, ks0 + (it_end - it));
      it += ks1 - ks0;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // ---- filter operand: thread -> (row tid/4 + 64 s, 16-byte word tid%4); rows clamped
    unsigned a_voff[PA];
#pragma unroll
    for (int s = 0; s < PA; ++s) {
      const int row = min(m0 + (tid >> 2) + 64 * s, P.M - 1);
      a_voff[s] = RAW ? (static_cast<unsigned>(row) * P.raw_row + 4u * (tid & 3) * P.raw_ch) * 4u
                      : (static_cast<unsigned>(row) * P.K + 4u * (tid & 3)) * 4u;
    }
    const unsigned a_next = static_cast<unsigned>(P.raw_ch) * 4u;    // RAW: bytes between two channels
    // ---- gathered operand: thread -> (column tid % BN, KPT consecutive k' starting at klocal0)
    unsigned b_voff, vmask = 0;
    {
      const int n = n0 + tid % BN;
      const bool col_ok = n < P.N;
      const uint32_t nn = col_ok ? n : 0;
      const uint32_t img = P.plane.div(nn);
      const uint32_t p = nn - img * P.plane.d;
      const uint32_t row = P.width.div(p);
      const uint32_t col = p - row * P.width.d;
      const int r0 = BWD_DATA ? static_cast<int>(row) + P.ph : static_cast<int>(row) * P.s - P.ph;
      const int c0 = BWD_DATA ? static_cast<int>(col) + P.pw : static_cast<int>(col) * P.s - P.pw;
      if (col_ok) {
        for (int t = 0; t < P.taps; ++t) {
          const int kh = t / P.kW, kw = t - kh * P.kW;
          const int rr = BWD_DATA ? r0 - kh : r0 + kh, cc = BWD_DATA ? c0 - kw : c0 + kw;
          if (static_cast<unsigned>(rr) < static_cast<unsigned>(P.src_h) &&
              static_cast<unsigned>(cc) < static_cast<unsigned>(P.src_w))
            vmask |= 1u << t;
        }
      }
      // forward : src offset = thread part + (kh*W + kw)       with the bias ph*W + pw folded in
      // bwd-data: src offset = thread part - (kh*W + kw)       with the bias (kH-1)*W + kW-1 folded in
      const int thread_part = BWD_DATA ? r0 * P.src_w + c0 : (r0 + P.ph) * P.src_w + (c0 + P.pw);
      b_voff =
          static_cast<unsigned>(static_cast<int>(img) * P.img_stride + klocal0 * P.chan_stride + thread_part) * 4u;
    }

    acc16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    u32x4 ra_regs[PA];
    unsigned rb_regs[KPT];
    // position of the NEXT step to load: step ks covers channels [16*(ks/taps), +16) of tap ks%taps
    int tap = ks0 % P.taps, ch0 = (ks0 / P.taps) * BK;

    auto load_step = [&](int step) {
      // filter words: scalar offset = k position of the step
      if (RAW) {
        const int soff_a = (ch0 * P.raw_ch + tap) * 4;
#pragma unroll
        for (int s = 0; s < PA; ++s) {
          ra_regs[s].x = __builtin_amdgcn_raw_buffer_load_b32(ra, a_voff[s], soff_a, 0);
          ra_regs[s].y = __builtin_amdgcn_raw_buffer_load_b32(ra, a_voff[s] + a_next, soff_a, 0);
          ra_regs[s].z = __builtin_amdgcn_raw_buffer_load_b32(ra, a_voff[s] + 2u * a_next, soff_a, 0);
          ra_regs[s].w = __builtin_amdgcn_raw_buffer_load_b32(ra, a_voff[s] + 3u * a_next, soff_a, 0);
        }
      } else {
        const int soff_a = step * (BK * 4);
#pragma unroll
        for (int s = 0; s < PA; ++s) ra_regs[s] = __builtin_amdgcn_raw_buffer_load_b128(ra, a_voff[s], soff_a, 0);
      }
      // gathered values: scalar offset = channel block + tap displacement
      const int kh = tap / P.kW, kw = tap - kh * P.kW;
      const int disp = BWD_DATA ? bias - (kh * P.src_w + kw) : kh * P.src_w + kw;
      const int soff_b = (ch0 * P.chan_stride + disp) * 4;
      const unsigned voff = (vmask >> tap) & 1u ? b_voff : kOobOffset;
#pragma unroll
      for (int i = 0; i < KPT; ++i)
        rb_regs[i] = __builtin_amdgcn_raw_buffer_load_b32(rb, voff, soff_b + i * P.chan_stride * 4, 0);
      if (++tap == P.taps) {
        tap = 0;
        ch0 += BK;
      }
    };
    auto store_step = [&](float *sa, float *sb) {
#pragma unroll
      for (int s = 0; s < PA; ++s)
        *reinterpret_cast<u32x4 *>(sa + ((tid >> 2) + 64 * s) * ALds::kStride + 4 * (tid & 3)) = ra_regs[s];
#pragma unroll
      for (int q = 0; q < KPT / 4; ++q) {
        u32x4 v = {rb_regs[4 * q], rb_regs[4 * q + 1], rb_regs[4 * q + 2], rb_regs[4 * q + 3]};
        *reinterpret_cast<u32x4 *>(sb + (tid % BN) * BLds::kStride + klocal0 + 4 * q) = v;
      }
    };
    auto mma_step = [&](const float *sa, const float *sb) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        float fa[2][4], fb[2][4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          ALds::frag(sa, wm0 + 32 * i, j, lane, fa[i]);
          BLds::frag(sb, wn0 + 32 * i, j, lane, fb[i]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
              acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[mi][e], fb[ni][e], acc[mi][ni], 0, 0, 0);
      }
    };

    load_step(ks0);
    store_step(lds_a[0], lds_b[0]);
    __syncthreads();
    int stage = 0;
    for (int st = ks0; st < ks1; ++st) {
      const bool more = st + 1 < ks1;
      if (more) load_step(st + 1);
      mma_step(lds_a[stage], lds_b[stage]);
      if (more) store_step(lds_a[stage ^ 1], lds_b[stage ^ 1]);
      __syncthreads();   // also fences the LDS stages against the next tile of this block
      stage ^= 1;
    }

    // epilogue: accumulator register e of a 32x32 block holds row 8*(e/4) + 4*(lane/32) + e%4, column
    // lane%32; out[img][m][p] with column n = img*plane + p
    const bool whole = ks0 == 0 && ks1 == sk.ksteps;
    if (whole) {
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const int n = n0 + wn0 + 32 * ni + (lane & 31);
        if (n >= P.N) continue;
        const int64_t coff = tap_out_col(P, n);
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) {
          const int mb = m0 + wm0 + 32 * mi + 4 * (lane >> 5);
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int m = mb + 8 * (e >> 2) + (e & 3);
            if (m < P.M) out[static_cast<int64_t>(m) * P.out_plane + coff] = acc[mi][ni][e];
          }
        }
      }
      if (STATS) {
        // Row sums through LDS (the k-loop ended with a barrier: the stages are free).  A wave lays a
        // 64 x 32 half of its sub-tile down as [column][row] - a lane's four consecutive rows are one
        // 16-byte word - and then every lane sums one row over the 32 columns: pitch 68 keeps both the
        // words and the column walks free of bank conflicts, and the 64 lanes store 64 neighbouring
        // channels' pairs.
        constexpr int kPitch = 68;
        float *mine = lds_all + wave * (32 * kPitch);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
#pragma unroll
          for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              typedef float f32x4 __attribute__((ext_vector_type(4)));
              const f32x4 v = {acc[mi][ni][4 * g4], acc[mi][ni][4 * g4 + 1], acc[mi][ni][4 * g4 + 2], acc[mi][ni][4 * g4 + 3]};
              *reinterpret_cast<f32x4 *>(mine + (lane & 31) * kPitch + 32 * mi + 8 * g4 + 4 * (lane >> 5)) = v;
            }
          __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): a wave's own staging area needs no block barrier
          __builtin_amdgcn_wave_barrier();
          float sum = 0.f, sq = 0.f;
#pragma unroll
          for (int col = 0; col < 32; ++col) {
            const float v = mine[col * kPitch + lane];
            sum += v;
            sq += v * v;
          }
          const int m = m0 + wm0 + lane, col0 = n0 + wn0 + 32 * ni;
          if (m < P.M && col0 < P.N) {
            float2 *dst = reinterpret_cast<float2 *>(P.stats + (static_cast<int64_t>(col0 >> 5) * P.M + m) * 2);
            *dst = make_float2(sum, sq);
          }
          __builtin_amdgcn_s_waitcnt(0xc07f);
          __builtin_amdgcn_wave_barrier();
        }
        __syncthreads();   // the next tile's first step is staged into this memory
      }
    } else {
      // a piece of a cut tile: registers go to scratch as they are, [register][thread]
      const int slot = (it - (ks1 - ks0)) == it_begin ? 0 : 1;
      float *pc = pieces + (static_cast<int64_t>(logical) * 2 + slot) * (BM * BN) + tid;
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
          for (int e = 0; e < 16; ++e) pc[((mi * 2 + ni) * 16 + e) * kThreads] = acc[mi][ni][e];
    }
  }
}

// Assembles the tiles that block ranges cut into pieces.  Four blocks per tile, one per 32x32
// accumulator block of every wave (registers 16q .. 16q+15): each adds the pieces in ascending
// block order and stores its share of the tile.  Thread and register layout are those of
// conv_tap_kernel's epilogue.
template <int BM, int BN, int WM, int WN, bool STATS = false>
__global__ __launch_bounds__(kThreads) void conv_tap_assemble_kernel(TapConvParams P, float *__restrict__ out,
                                                                     const float *__restrict__ pieces, StreamK sk) {
  const int tile = blockIdx.x >> 2, q = blockIdx.x & 3;
  const int mi = q >> 1, ni = q & 1;
  const int t = tile / sk.tm, tile_m = tile - t * sk.tm;                  // t: tile of the cut part
  const int tile_n = sk.cut_first + t;
  const int first = t * sk.ksteps, last = first + sk.ksteps - 1;          // within the cut part of row tile_m
  const int b0 = first / sk.iters_per_block, b1 = last / sk.iters_per_block;
  if (b0 == b1) return;   // computed and stored by one block
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WN) * 64, wn0 = (wave % WN) * 64;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  float acc[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  for (int b = b0; b <= b1; ++b) {
    const int slot = b * sk.iters_per_block >= first ? 0 : 1;
    const float *pc =
        pieces + (static_cast<int64_t>(b * sk.tm + tile_m) * 2 + slot) * (BM * BN) + (q * 16) * kThreads + tid;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] += __builtin_nontemporal_load(pc + e * kThreads);
  }
  const int n = n0 + wn0 + 32 * ni + (lane & 31);
  if (STATS) {
    // the pieces of columns beyond N are zeros: every lane takes part in the sums
    float r[16], q[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      r[e] = acc[e];
      q[e] = acc[e] * acc[e];
    }
    half_wave_sums<16>(r, lane);
    half_wave_sums<16>(q, lane);
    const int e = (lane & 31) >> 1;
    const int m = m0 + wm0 + 32 * mi + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
    const int col0 = n0 + wn0 + 32 * ni;
    if ((lane & 1) == 0 && m < P.M && col0 < P.N) {
      float *dst = P.stats + (static_cast<int64_t>(col0 >> 5) * P.M + m) * 2;
      dst[0] = r[0];
      dst[1] = q[0];
    }
  }
  if (n >= P.N) return;
  const int64_t coff = tap_out_col(P, n);
  const int mb = m0 + wm0 + 32 * mi + 4 * (lane >> 5);
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int m = mb + 8 * (e >> 2) + (e & 3);
    if (m < P.M) out[static_cast<int64_t>(m) * P.out_plane + coff] = acc[e];
  }
}

// ------------------------------------------------------------------ the tap-major filter-gradient kernel
// Backward-filter for convolutions with C % 16 == 0, written like conv_tap_kernel so that the
// k-loop does almost no vector-ALU work.  First the "same" stride-1 case (oH = H, oW = W):
// The reduction runs over positions k = (img, p); because the convolution is "same", the
// gathered element of tap (dr, dc) for output position p is x[img][c][p + dr*W + dc] - linear
// in p - so the per-thread byte offset is a loop constant and the step's (img, p0) travels in
// the scalar offset.  A 16-wide step never straddles two images (H*W % 16 == 0, or the TAIL
// variant pads every image to that).  The padding
// test needs the column of p, kept incrementally, and one range test on the linear index.
// GEN (any stride, padding and output size): the gathered element of output position (oh, ow)
// is x[c][oh*s - ph + kh][ow*s - pw + kw], no longer linear in p, so every thread keeps the
// (oh, ow) of its position incrementally and rebuilds its byte offset each step: two
// multiply-adds and two range tests more than the "same" case.
struct TapWgradParams {
  const float *dy, *x;
  int64_t dy_bytes, x_bytes;   // whole tensors; a block addresses from the first image of its k range
  int O, C, HW, W, kW, taps;
  int ph, pw;
  int M, N, K;           // O, C*taps, imgs*HWp
  int kchunk;            // k range per split (multiple of 16)
  int HWp;               // HW rounded up to a multiple of 16: the reduction runs over imgs*HWp positions
  // GEN only (HW and W above are then the OUTPUT plane oH*oW and width oW)
  int s, xH, xW, xHW;    // stride, input height, width and plane
};

// TAIL: H*W is not a multiple of 16.  Every image's positions are padded to HWp; the padded ones
// read as zeros (a compare per operand and step, three selects per dy word).  When H*W is not a
// multiple of 4 either, the 16-byte dy words start on 4-byte boundaries.
template <int BM, int BN, int WM, int WN, bool TAIL, bool GEN>
__global__ __launch_bounds__(kThreads, (BM == 128 ? 4 : 1)) void conv_wgrad_tap_kernel(TapWgradParams P, float *__restrict__ part,
                                                                  TileGrid tg) {
  static_assert(WM * WN == 4 && BM / WM == 64 && BN / WN == 64, "each of the 4 waves owns a 64x64 sub-tile");
  using ALds = MnMajorLds<BM>;
  using BLds = MnMajorLds<BN>;
  constexpr int PA = BM / 64;
  constexpr int KCOLS = BN / 16;     // consecutive columns (channels of one tap) per thread
  __shared__ __attribute__((aligned(16))) float lds_a[2][ALds::kFloats];
  __shared__ __attribute__((aligned(16))) float lds_b[2][BLds::kFloats];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (logical >= tg.total) return;
  const int per_split = tg.tm * tg.tn;
  const int zsplit = logical / per_split;
  const int rem = logical - zsplit * per_split;
  const int tile_n = rem / tg.tm, tile_m = rem - tile_n * tg.tm;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int wm0 = (wave / WN) * 64, wn0 = (wave % WN) * 64;
  const int kbegin = zsplit * P.kchunk;
  const int kend = min(P.K, kbegin + P.kchunk);

  // 32-bit offsets count from the first image of this block's k range, so only the images of one
  // split have to lie within 2 GiB of each other, not the whole tensors
  const int bias = GEN ? 0 : P.ph * P.W + P.pw;
  const int x_plane = GEN ? P.xHW : P.HW;
  const int img_first = kbegin / P.HWp;
  const int64_t a_base = static_cast<int64_t>(img_first) * P.O * P.HW, b_base = static_cast<int64_t>(img_first) * P.C * x_plane;
  const int64_t a_left = P.dy_bytes - 4 * a_base, b_left = P.x_bytes - 4 * b_base + 4 * bias;
  const int a_records = static_cast<int>(a_left < 0 ? 0 : (a_left < 0x7fffffffll ? a_left : 0x7fffffffll));
  const int b_records = static_cast<int>(b_left < 0 ? 0 : (b_left < 0x7fffffffll ? b_left : 0x7fffffffll));
  const __amdgpu_buffer_rsrc_t ra =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.dy) + a_base, 0, a_records, kBufFlags);
  const __amdgpu_buffer_rsrc_t rb =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.x) + b_base - bias, 0, b_records, kBufFlags);

  // ---- dy operand: thread -> (row tid/4 + 64 s, 4 consecutive positions tid%4)
  unsigned a_voff[PA];
#pragma unroll
  for (int s = 0; s < PA; ++s) {
    const int row = min(m0 + (tid >> 2) + 64 * s, P.O - 1);
    a_voff[s] = (static_cast<unsigned>(row) * P.HW + 4u * (tid & 3)) * 4u;
  }
  // ---- x operand: thread -> (position tid%16 of the step, KCOLS consecutive channels of one tap)
  const int klocal = tid & 15;
  const int jlocal0 = KCOLS * (tid >> 4);
  const int j = n0 + jlocal0;
  const bool cols_ok = j < P.N;                   // C % KCOLS == 0: all of a thread's columns or none
  const int jj = cols_ok ? j : 0;
  const int tap = jj / P.C, c_first = jj - tap * P.C;
  const int kh = tap / P.kW, kw = tap - kh * P.kW;
  const int dr = kh - P.ph, dc = kw - P.pw;
  const int shift = dr * P.W + dc;                // x index = p + shift
  const unsigned b_voff = GEN ? static_cast<unsigned>(c_first * x_plane) * 4u
                              : static_cast<unsigned>(c_first * P.HW + klocal + shift + bias) * 4u;

  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int jx = 0; jx < 2; ++jx)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][jx][e] = 0.f;

  // uniform position of the NEXT step to load, and this thread's column within the image row
  int img = 0, p0 = kbegin - img_first * P.HWp;   // img counts from img_first
  int ow = (p0 + klocal) % P.W;
  const int ow_first = klocal % P.W;   // column of this thread's position in the first step of an image
  int oh = (p0 + klocal) / P.W;        // GEN: its row
  const int oh_first = klocal / P.W;

  u32x4 ra_regs[PA];
  unsigned rb_regs[KCOLS];
  int a_cnt = 4;

  auto load_step = [&]() {
    const int soff_a = (img * P.O * P.HW + p0) * 4;
    if (TAIL) a_cnt = P.HW - (p0 + 4 * (tid & 3));               // positions of this thread's word inside the image
#pragma unroll
    for (int s = 0; s < PA; ++s)
      ra_regs[s] = __builtin_amdgcn_raw_buffer_load_b128(ra, a_cnt > 0 ? a_voff[s] : kOobOffset, soff_a, 0);
    const int p = p0 + klocal;
    if (GEN) {
      const int ih = oh * P.s + dr, iw = ow * P.s + dc;
      const bool ok = cols_ok && (!TAIL || p < P.HW) && static_cast<unsigned>(ih) < static_cast<unsigned>(P.xH) &&
                      static_cast<unsigned>(iw) < static_cast<unsigned>(P.xW);
      const unsigned voff = ok ? b_voff + static_cast<unsigned>(ih * P.xW + iw) * 4u : kOobOffset;
      const int soff_b = img * P.C * x_plane * 4;
#pragma unroll
      for (int i = 0; i < KCOLS; ++i)
        rb_regs[i] = __builtin_amdgcn_raw_buffer_load_b32(rb, voff, soff_b + i * x_plane * 4, 0);
    } else {
      const bool ok = cols_ok && (!TAIL || p < P.HW) &&
                      static_cast<unsigned>(p + dr * P.W) < static_cast<unsigned>(P.HW) &&
                      static_cast<unsigned>(ow + dc) < static_cast<unsigned>(P.W);
      const unsigned voff = ok ? b_voff : kOobOffset;
      const int soff_b = (img * P.C * P.HW + p0) * 4;
#pragma unroll
      for (int i = 0; i < KCOLS; ++i)
        rb_regs[i] = __builtin_amdgcn_raw_buffer_load_b32(rb, voff, soff_b + i * P.HW * 4, 0);
    }
    p0 += BK;
    ow += BK;                      // BK may exceed W for tiny images: reduce until in range
    while (ow >= P.W) {
      ow -= P.W;
      if (GEN) ++oh;
    }
    if (p0 >= P.HWp) {
      p0 = 0;
      ++img;
      if (TAIL) ow = ow_first;     // positions do not continue across the padded tail
      if (GEN) oh = oh_first;
    }
  };
  auto store_step = [&](float *sa, float *sb) {
#pragma unroll
    for (int s = 0; s < PA; ++s) {
      u32x4 r = ra_regs[s];
      if (TAIL) {        // a word that straddles the end of the image carries the next row's first values
        r.y = a_cnt >= 2 ? r.y : 0u;
        r.z = a_cnt >= 3 ? r.z : 0u;
        r.w = a_cnt >= 4 ? r.w : 0u;
      }
      *reinterpret_cast<u32x4 *>(sa + ((tid >> 2) + 64 * s) * ALds::kStride + 4 * (tid & 3)) = r;
    }
#pragma unroll
    for (int i = 0; i < KCOLS; ++i)
      reinterpret_cast<unsigned *>(sb)[(jlocal0 + i) * BLds::kStride + klocal] = rb_regs[i];
  };
  auto mma_step = [&](const float *sa, const float *sb) {
#pragma unroll
    for (int jg = 0; jg < 2; ++jg) {
      float fa[2][4], fb[2][4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        ALds::frag(sa, wm0 + 32 * i, jg, lane, fa[i]);
        BLds::frag(sb, wn0 + 32 * i, jg, lane, fb[i]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
          for (int ni = 0; ni < 2; ++ni)
            acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[mi][e], fb[ni][e], acc[mi][ni], 0, 0, 0);
    }
  };

  const int steps = (kend - kbegin) / BK;    // K and kchunk are multiples of 16
  if (steps > 0) {
    load_step();
    store_step(lds_a[0], lds_b[0]);
  }
  __syncthreads();
  // A wave whose 64x64 sub-tile lies outside the matrix (ragged last N tile: 576 columns = 2.25
  // tiles of 256) only helps with the staging and leaves the matrix pipe to other blocks.  Two
  // copies of the loop, chosen once: a test inside the loop costs the full tiles 20 %.
  auto k_loop = [&](auto with_mma) {
    int stage = 0;
    for (int st = 0; st < steps; ++st) {
      const bool more = st + 1 < steps;
      if (more) load_step();
      if (decltype(with_mma)::value) mma_step(lds_a[stage], lds_b[stage]);
      if (more) store_step(lds_a[stage ^ 1], lds_b[stage ^ 1]);
      __syncthreads();
      stage ^= 1;
    }
  };
  if (m0 + wm0 < P.M && n0 + wn0 < P.N)
    k_loop(std::true_type{});
  else
    k_loop(std::false_type{});

  float *o = part + static_cast<int64_t>(zsplit) * P.M * P.N;
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int n = n0 + wn0 + 32 * ni + (lane & 31);
    if (n >= P.N) continue;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
      const int mb = m0 + wm0 + 32 * mi + 4 * (lane >> 5);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = mb + 8 * (e >> 2) + (e & 3);
        if (m < P.M) o[static_cast<int64_t>(m) * P.N + n] = acc[mi][ni][e];
      }
    }
  }
}

// ------------------------------------------------------------------ bwd-filter loaders, mn-major
// A = dy: row m = output channel, k = (img, p); K contiguous inside an image.
template <int BM>
struct DyRowsLoader {
  using Lds = MnMajorLds<BM>;
  struct Params {
    const float *dy;
    FastDiv plane;     // oH*oW
    int O;
    bool vec;          // oH*oW % 4 == 0 and dy 16-byte aligned
  };
  static constexpr int kPasses = BM / 64;
  float4 r[kPasses];
  const float *dy;
  FastDiv plane;
  int O, row0, kq;
  bool vec;

  __device__ __forceinline__ void init(const Params &P, int m0, int tid) {
    dy = P.dy;
    plane = P.plane;
    O = P.O;
    vec = P.vec;
    row0 = m0 + (tid >> 2);
    kq = tid & 3;
  }
  __device__ __forceinline__ float one(int k, int row, int kend) const {
    if (k >= kend) return 0.f;
    const uint32_t img = plane.div(k);
    const uint32_t p = k - img * plane.d;
    return dy[(static_cast<int64_t>(img) * O + row) * plane.d + p];
  }
  __device__ __forceinline__ void load(int k0, int kend) {
    const int k = k0 + 4 * kq;
    const uint32_t img = plane.div(k);
    const uint32_t p = k - img * plane.d;
#pragma unroll
    for (int s = 0; s < kPasses; ++s) {
      const int row = row0 + 64 * s;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (row < O) {
        if (vec && k + 3 < kend) {
          v = *reinterpret_cast<const float4 *>(dy + (static_cast<int64_t>(img) * O + row) * plane.d + p);
        } else {
          v.x = one(k, row, kend);
          v.y = one(k + 1, row, kend);
          v.z = one(k + 2, row, kend);
          v.w = one(k + 3, row, kend);
        }
      }
      r[s] = v;
    }
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int s = 0; s < kPasses; ++s)
      *reinterpret_cast<float4 *>(lds + ((tid >> 2) + 64 * s) * Lds::kStride + 4 * kq) = r[s];
  }
};

// B = gather of x: column j = (c, kh, kw) (fixed per thread), k = (img, oh, ow).
template <int BN>
struct GatherRowsLoader {
  using Lds = MnMajorLds<BN>;
  struct Params {
    const float *x;
    const Tap *taps;
    FastDiv plane;        // oH*oW
    FastDiv width;        // oW
    int64_t img_stride;   // C*H*W
    int H, W, ph, pw, s;
    int j_total;
  };
  static constexpr int kCols = BN / 16;   // columns per thread
  float r[kCols];
  int off[kCols];
  short kh[kCols], kw[kCols];
  const float *x;
  FastDiv plane, width;
  int64_t img_stride;
  int H, W, ph, pw, s, klocal;

  __device__ __forceinline__ void init(const Params &P, int j0, int tid) {
    x = P.x;
    plane = P.plane;
    width = P.width;
    img_stride = P.img_stride;
    H = P.H;
    W = P.W;
    ph = P.ph;
    pw = P.pw;
    s = P.s;
    klocal = tid & 15;
#pragma unroll
    for (int i = 0; i < kCols; ++i) {
      const int j = j0 + (tid >> 4) + 16 * i;
      if (j < P.j_total) {
        const Tap t = P.taps[j];
        off[i] = t.off;
        kh[i] = t.kh;
        kw[i] = t.kw;
      } else {
        off[i] = 0;
        kh[i] = -20000;   // fails the range test below for any row
        kw[i] = 0;
      }
    }
  }
  __device__ __forceinline__ void load(int k0, int kend) {
    const int k = k0 + klocal;
    const bool k_ok = k < kend;
    const uint32_t kk = k_ok ? k : 0;
    const uint32_t img = plane.div(kk);
    const uint32_t p = kk - img * plane.d;
    const uint32_t oh = width.div(p);
    const uint32_t ow = p - oh * width.d;
    const int r0 = static_cast<int>(oh) * s - ph, c0 = static_cast<int>(ow) * s - pw;
    const float *base = x + static_cast<int64_t>(img) * img_stride + static_cast<int64_t>(r0) * W + c0;
#pragma unroll
    for (int i = 0; i < kCols; ++i) {
      const int rr = r0 + kh[i], cc = c0 + kw[i];
      float v = 0.f;
      if (k_ok && static_cast<unsigned>(rr) < static_cast<unsigned>(H) &&
          static_cast<unsigned>(cc) < static_cast<unsigned>(W))
        v = base[off[i]];
      r[i] = v;
    }
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int i = 0; i < kCols; ++i) lds[((tid >> 4) + 16 * i) * Lds::kStride + klocal] = r[i];
  }
};


// Tap-major variant of the bwd-filter gather: columns are ordered j' = (kh*kW + kw)*C + c and
// a thread owns BN/16 CONSECUTIVE columns, i.e. consecutive channels of one filter tap, so
// the padding test is done once per step and the loads differ only by a channel stride.
// The result comes out as dw'[o][tap][c]; the split-K fold writes it back as [o][c][tap].
template <int BN>
struct TapMajorRowsLoader {
  using Lds = MnMajorLds<BN>;
  struct Params {
    const float *x;
    FastDiv plane;        // oH*oW
    FastDiv width;        // oW
    int64_t img_stride;   // C*H*W
    int chan_stride;      // H*W
    int H, W, ph, pw, s;
    int C, kW;
    int j_total;
  };
  static constexpr int kCols = BN / 16;
  float r[kCols];
  const float *x;
  FastDiv plane, width;
  int64_t img_stride, col_off;
  int chan_stride, H, W, s, klocal, jlocal0, dr, dc;   // dr = kh - ph, dc = kw - pw
  bool cols_ok;

  __device__ __forceinline__ void init(const Params &P, int j0, int tid) {
    x = P.x;
    plane = P.plane;
    width = P.width;
    img_stride = P.img_stride;
    chan_stride = P.chan_stride;
    H = P.H;
    W = P.W;
    s = P.s;
    klocal = tid & 15;
    jlocal0 = kCols * (tid >> 4);
    const int j = j0 + jlocal0;
    cols_ok = j < P.j_total;           // C % kCols == 0: a thread's columns are all valid or none
    const int jj = cols_ok ? j : 0;
    const int tap = jj / P.C, c = jj - tap * P.C;
    const int kh = tap / P.kW, kw = tap - kh * P.kW;
    dr = kh - P.ph;
    dc = kw - P.pw;
    col_off = static_cast<int64_t>(c) * P.chan_stride;
  }
  __device__ __forceinline__ void load(int k0, int kend) {
    const int k = k0 + klocal;
    const bool k_ok = cols_ok && k < kend;
    const uint32_t kk = k_ok ? k : 0;
    const uint32_t img = plane.div(kk);
    const uint32_t p = kk - img * plane.d;
    const uint32_t oh = width.div(p);
    const uint32_t ow = p - oh * width.d;
    const int rr = static_cast<int>(oh) * s + dr, cc = static_cast<int>(ow) * s + dc;
    const bool ok = k_ok && static_cast<unsigned>(rr) < static_cast<unsigned>(H) &&
                    static_cast<unsigned>(cc) < static_cast<unsigned>(W);
    const float *q = x + static_cast<int64_t>(img) * img_stride + col_off + rr * W + cc;
#pragma unroll
    for (int i = 0; i < kCols; ++i) r[i] = ok ? q[i * chan_stride] : 0.f;
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int i = 0; i < kCols; ++i) lds[(jlocal0 + i) * Lds::kStride + klocal] = r[i];
  }
};

// ------------------------------------------------------------------ NCHW output columns
struct NchwCols {   // out[img][m][p]: column n = img*plane + p -> img*img_stride + p ; row stride = plane
  FastDiv plane;
  int64_t img_stride;
  __device__ __forceinline__ int64_t operator()(int n) const {
    const uint32_t img = plane.div(n);
    return static_cast<int64_t>(img) * img_stride + (n - img * plane.d);
  }
};

// filter [O][C][kHW] -> [C][O][kHW]
__global__ __launch_bounds__(256) void filter_oc_swap_kernel(const float *__restrict__ w, float *__restrict__ wt,
                                                             int O, int C, int kHW) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= O * C * kHW) return;
  const int r = idx % kHW;
  const int t = idx / kHW;
  const int o = t % O, c = t / O;
  wt[idx] = w[(o * C + c) * kHW + r];
}

// re-lays of the filter [O][C][kHW] for the tap-major loaders, reduction index
// k' = ((ch/16)*kHW + tap)*16 + ch%16:
//   forward : out[o][k'] with ch = c     bwd-data: out[c][k'] with ch = o
__global__ __launch_bounds__(256) void filter_tap_major_kernel(const float *__restrict__ w, float *__restrict__ out,
                                                               int O, int C, int kHW, bool for_bwd_data) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= O * C * kHW) return;
  const int K = (for_bwd_data ? O : C) * kHW;
  const int row = idx / K, kp = idx - row * K;
  const int lo = kp & 15;
  const int t = kp >> 4;
  const int tap = t % kHW, blk = t / kHW;
  const int ch = blk * 16 + lo;
  const int o = for_bwd_data ? ch : row, c = for_bwd_data ? row : ch;
  out[idx] = w[(o * C + c) * kHW + tap];
}

// split-K fold for the tap-major bwd-filter: part[z][o][tap][c] summed over z (ascending, so the
// result does not depend on scheduling) and written as dw[o][c][tap]
// A block folds 64 outputs with 4 slice-lanes each (lane l adds slices l, l + 4, ...), combined
// through LDS in a fixed order.
__global__ __launch_bounds__(256) void fold_tap_major_kernel(const float *__restrict__ part, float *__restrict__ dw,
                                                             int O, int C, int kHW, int64_t stride, int S) {
  __shared__ float sm[3][64];
  const int cx = threadIdx.x & 63, ry = threadIdx.x >> 6;
  const int idx = blockIdx.x * 64 + cx;                // index into one partial: (o*kHW + tap)*C + c
  const bool live = idx < O * C * kHW;
  float acc = 0.f;
  if (live) {
#pragma unroll 4
    for (int z = ry; z < S; z += 4) acc += part[z * stride + idx];
  }
  if (ry > 0) sm[ry - 1][cx] = acc;
  __syncthreads();
  if (ry == 0 && live) {
    acc = ((acc + sm[0][cx]) + sm[1][cx]) + sm[2][cx];
    const int c = idx % C;
    const int t = idx / C;
    const int tap = t % kHW, o = t / kHW;
    dw[(o * C + c) * kHW + tap] = acc;
  }
}

// ------------------------------------------------------------------ host side
int geo_from(const char *who, const DLArray *x, const DLArray *w, const DLArray *y, int ph, int pw, int s,
             ConvGeo &g) {
  TS_REQUIRE(x && w && y, "%s: NULL array", who);
  TS_REQUIRE(x->ndim == 4 && w->ndim == 4 && y->ndim == 4, "%s: arrays must be 4-D", who);
  TS_REQUIRE(s >= 1 && ph >= 0 && pw >= 0, "%s: bad stride/padding", who);
  g.imgs = static_cast<int>(x->shape[0]);
  g.C = static_cast<int>(x->shape[1]);
  g.H = static_cast<int>(x->shape[2]);
  g.W = static_cast<int>(x->shape[3]);
  g.O = static_cast<int>(w->shape[0]);
  g.kH = static_cast<int>(w->shape[2]);
  g.kW = static_cast<int>(w->shape[3]);
  g.ph = ph;
  g.pw = pw;
  g.s = s;
  g.oH = static_cast<int>(y->shape[2]);
  g.oW = static_cast<int>(y->shape[3]);
  TS_REQUIRE(w->shape[1] == g.C, "%s: filter has %lld input channels, input has %d", who, (long long)w->shape[1], g.C);
  TS_REQUIRE(y->shape[0] == g.imgs && y->shape[1] == g.O, "%s: output N,C must be %d,%d", who, g.imgs, g.O);
  TS_REQUIRE(g.H + 2 * ph >= g.kH && g.W + 2 * pw >= g.kW, "%s: filter larger than the padded image", who);
  const int eh = (g.H + 2 * ph - g.kH) / s + 1, ew = (g.W + 2 * pw - g.kW) / s + 1;
  TS_REQUIRE(g.oH == eh && g.oW == ew, "%s: output is %dx%d, expected %dx%d", who, g.oH, g.oW, eh, ew);
  TS_REQUIRE(numel(x) < (1ll << 31) && numel(y) < (1ll << 31) && numel(w) < (1ll << 31), "%s: tensor too large", who);
  TS_REQUIRE(g.kH < 20000 && g.kW < 20000, "%s: filter too large", who);
  return 0;
}

inline const float *cf(const DLArray *a) { return static_cast<const float *>(a->data); }
inline float *mf(DLArray *a) { return static_cast<float *>(a->data); }

template <int BM, int BN, int WM, int WN>
void launch_fwd(const ConvGeo &g, const float *x, const float *w, float *y, const Tap *taps, hipStream_t st) {
  using AL = KContigLoader<BM>;
  using BL = GatherColsLoader<BN, false>;
  const int K = g.C * g.kH * g.kW, N = g.imgs * g.oH * g.oW, M = g.O;
  typename AL::Params ap{w, K, M, K % 4 == 0 && aligned16(w)};
  typename BL::Params bp{x, taps, FastDiv(g.oH * g.oW), FastDiv(g.oW), static_cast<int64_t>(g.C) * g.H * g.W,
                         g.H, g.W, g.ph, g.pw, g.s, N};
  NchwCols cm{FastDiv(g.oH * g.oW), static_cast<int64_t>(g.O) * g.oH * g.oW};
  const int tn = (N + BN - 1) / BN, tm = (M + BM - 1) / BM;
  dim3 grid(grid_blocks(tm, tn, 1));
  hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, NchwCols>), grid, dim3(kThreads), 0, st, ap, bp, y,
                     int64_t(0), static_cast<int64_t>(g.oH) * g.oW, cm, M, N, K, (K + BK - 1) / BK * BK, TileGrid{tm, tn, tm * tn});
}

// forward with the tap-major reduction order; wf is the filter re-laid as [O][kHW][C]
template <int BM, int BN, int WM, int WN>
void launch_fwd_tap_major(const ConvGeo &g, const float *x, const float *wf, float *y, hipStream_t st) {
  using AL = KContigLoader<BM>;
  using BL = TapMajorColsLoader<BN, false>;
  const int K = g.C * g.kH * g.kW, N = g.imgs * g.oH * g.oW, M = g.O;
  typename AL::Params ap{wf, K, M, true};
  typename BL::Params bp{x, FastDiv(g.oH * g.oW), FastDiv(g.oW), static_cast<int64_t>(g.C) * g.H * g.W, g.H * g.W,
                         g.H, g.W, g.ph, g.pw, g.s, g.C, g.kW, g.kH * g.kW, N};
  NchwCols cm{FastDiv(g.oH * g.oW), static_cast<int64_t>(g.O) * g.oH * g.oW};
  const int tn = (N + BN - 1) / BN, tm = (M + BM - 1) / BM;
  dim3 grid(grid_blocks(tm, tn, 1));
  hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, NchwCols>), grid, dim3(kThreads), 0, st, ap, bp, y,
                     int64_t(0), static_cast<int64_t>(g.oH) * g.oW, cm, M, N, K, K, TileGrid{tm, tn, tm * tn});
}

template <int BM, int BN, int WM, int WN>
void launch_bwd_data(const ConvGeo &g, const float *wt, const float *dy, float *dx, const Tap *taps,
                     hipStream_t st) {
  using AL = KContigLoader<BM>;
  using BL = GatherColsLoader<BN, true>;
  const int K = g.O * g.kH * g.kW, N = g.imgs * g.H * g.W, M = g.C;
  typename AL::Params ap{wt, K, M, K % 4 == 0 && aligned16(wt)};
  typename BL::Params bp{dy, taps, FastDiv(g.H * g.W), FastDiv(g.W), static_cast<int64_t>(g.O) * g.oH * g.oW,
                         g.oH, g.oW, g.ph, g.pw, g.s, N};
  NchwCols cm{FastDiv(g.H * g.W), static_cast<int64_t>(g.C) * g.H * g.W};
  const int tn = (N + BN - 1) / BN, tm = (M + BM - 1) / BM;
  dim3 grid(grid_blocks(tm, tn, 1));
  hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, NchwCols>), grid, dim3(kThreads), 0, st, ap, bp, dx,
                     int64_t(0), static_cast<int64_t>(g.H) * g.W, cm, M, N, K, (K + BK - 1) / BK * BK, TileGrid{tm, tn, tm * tn});
}

// ------------------------------------------------------------------ strided bwd-data by phases
// With stride s an input position (h, w) only receives the taps kh = (h + ph) mod s (mod s),
// kw likewise: 1 - 1/s^2 of the taps of the plain formulation multiply nothing.  The positions
// are therefore split into s*s phases (a, b) = ((h + ph) mod s, (w + pw) mod s).  Within a
// phase, h = a' + s*i and the tap kh = a + s*u reads dy row i + (a' + ph - kh)/s: a stride-1
// correlation of dy with the sub-filter {kh = a (mod s)} x {kw = b (mod s)}, whose outputs are
// scattered with stride s.  Each phase is one GEMM with K = O * |taps of the phase| and
// N = imgs * Hp * Wp on the forward gather loader; phases without taps (a 1x1 filter with
// stride 2 has one phase with a tap and three without) are zero-filled.
struct PhaseCols {   // column n = (img, i, j) of a phase -> img*img_stride + (a + s*i)*W + (b + s*j)
  FastDiv plane, width;
  int64_t img_stride;
  int a, b, s, W;
  __device__ __forceinline__ int64_t operator()(int n) const {
    const uint32_t img = plane.div(n);
    const uint32_t p = n - img * plane.d;
    const uint32_t i = width.div(p);
    const uint32_t j = p - i * width.d;
    return static_cast<int64_t>(img) * img_stride + static_cast<int64_t>(a + s * static_cast<int>(i)) * W + (b + s * static_cast<int>(j));
  }
};

struct PhasePlan {
  const Tap *taps = nullptr;   // device table of the phase's (o, u, v) in order
  int nu = 0, nv = 0;          // taps of the phase along each axis
  int a0 = 0, b0 = 0;          // first input row / column of the phase
  int hp = 0, wp = 0;          // positions of the phase along each axis
  int shift_r = 0, shift_c = 0;   // the loader's padding: dy row = i - shift_r + tap.kh
};

struct PhaseKey {
  int O, kH, kW, oH, oW, H, W, ph, pw, s, a, b;
  bool operator<(const PhaseKey &o) const {
    return std::tie(O, kH, kW, oH, oW, H, W, ph, pw, s, a, b) <
           std::tie(o.O, o.kH, o.kW, o.oH, o.oW, o.H, o.W, o.ph, o.pw, o.s, o.a, o.b);
  }
};
std::map<PhaseKey, PhasePlan> g_phase_plans;

// floor division for possibly negative numerators
inline int floor_div(int x, int d) { return x >= 0 ? x / d : -((-x + d - 1) / d); }

bool phase_plan(const ConvGeo &g, int a, int b, PhasePlan &out) {
  std::lock_guard<std::mutex> lk(g_taps_mu);
  const PhaseKey key{g.O, g.kH, g.kW, g.oH, g.oW, g.H, g.W, g.ph, g.pw, g.s, a, b};
  auto it = g_phase_plans.find(key);
  if (it != g_phase_plans.end()) {
    out = it->second;
    return true;
  }
  PhasePlan pl;
  const int s = g.s;
  pl.a0 = ((a - g.ph) % s + s) % s;
  pl.b0 = ((b - g.pw) % s + s) % s;
  pl.hp = pl.a0 < g.H ? (g.H - pl.a0 + s - 1) / s : 0;
  pl.wp = pl.b0 < g.W ? (g.W - pl.b0 + s - 1) / s : 0;
  pl.nu = a < g.kH ? (g.kH - a + s - 1) / s : 0;
  pl.nv = b < g.kW ? (g.kW - b + s - 1) / s : 0;
  if (pl.nu > 0 && pl.nv > 0 && pl.hp > 0 && pl.wp > 0) {
    // dy row of tap u for position i: i + dr(u), dr(u) = (a0 + ph - (a + s*u)) / s (exact); the
    // smallest dr belongs to the last tap
    pl.shift_r = -floor_div(pl.a0 + g.ph - (a + s * (pl.nu - 1)), s);
    pl.shift_c = -floor_div(pl.b0 + g.pw - (b + s * (pl.nv - 1)), s);
    std::vector<Tap> h(static_cast<size_t>(g.O) * pl.nu * pl.nv);
    size_t i = 0;
    for (int o = 0; o < g.O; ++o)
      for (int u = 0; u < pl.nu; ++u)
        for (int v = 0; v < pl.nv; ++v, ++i) {
          const int dr = floor_div(pl.a0 + g.ph - (a + s * u), s), dc = floor_div(pl.b0 + g.pw - (b + s * v), s);
          h[i].kh = static_cast<short>(dr + pl.shift_r);   // >= 0
          h[i].kw = static_cast<short>(dc + pl.shift_c);
          h[i].off = o * g.oH * g.oW + h[i].kh * g.oW + h[i].kw;
        }
    Tap *d = nullptr;
    if (hipMalloc(&d, h.size() * sizeof(Tap)) != hipSuccess) return false;
    if (hipMemcpy(d, h.data(), h.size() * sizeof(Tap), hipMemcpyHostToDevice) != hipSuccess) return false;
    pl.taps = d;
  }
  g_phase_plans[key] = pl;
  out = pl;
  return true;
}

// sub-filter of a phase: out[c][(o, u, v)] = w[o][c][a + s*u][b + s*v]
__global__ __launch_bounds__(256) void filter_phase_kernel(const float *__restrict__ w, float *__restrict__ out, int O,
                                                           int C, int kH, int kW, int a, int b, int s, int nu, int nv) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int kp = O * nu * nv;
  if (idx >= C * kp) return;
  const int c = idx / kp;
  int r = idx - c * kp;
  const int o = r / (nu * nv);
  r -= o * nu * nv;
  const int u = r / nv, v = r - u * nv;
  out[idx] = w[((o * C + c) * kH + (a + s * u)) * kW + (b + s * v)];
}

__global__ __launch_bounds__(256) void zero_fill_kernel(float *__restrict__ p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

template <int BM, int BN, int WM, int WN>
int launch_bwd_data_phases(const ConvGeo &g, const float *w, const float *dy, float *dx, float *wscratch,
                           hipStream_t st) {
  using AL = KContigLoader<BM>;
  using BL = GatherColsLoader<BN, false>;
  const int s = g.s;
  PhasePlan plans[64];
  TS_REQUIRE(s * s <= 64, "conv bwd-data: stride %d not supported", s);
  bool any_empty = false;
  for (int a = 0; a < s; ++a)
    for (int b = 0; b < s; ++b) {
      PhasePlan &pl = plans[a * s + b];
      TS_REQUIRE(phase_plan(g, a, b, pl), "conv bwd-data: could not build a phase table");
      if (pl.hp > 0 && pl.wp > 0 && (pl.nu == 0 || pl.nv == 0)) any_empty = true;
    }
  if (any_empty) {
    const int64_t n = static_cast<int64_t>(g.imgs) * g.C * g.H * g.W;
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, dx, n);
  }
  int64_t woff = 0;
  for (int a = 0; a < s; ++a)
    for (int b = 0; b < s; ++b) {
      const PhasePlan &pl = plans[a * s + b];
      if (!pl.taps) continue;
      const int K = g.O * pl.nu * pl.nv, N = g.imgs * pl.hp * pl.wp, M = g.C;
      float *wp = wscratch + woff;          // every phase uses its own part of the re-laid filter
      woff += static_cast<int64_t>(M) * K;
      hipLaunchKernelGGL(filter_phase_kernel, dim3((M * K + 255) / 256), dim3(256), 0, st, w, wp, g.O, g.C, g.kH, g.kW,
                         a, b, s, pl.nu, pl.nv);
      typename AL::Params ap{wp, K, M, K % 4 == 0 && aligned16(wp)};
      typename BL::Params bp{dy, pl.taps, FastDiv(pl.hp * pl.wp), FastDiv(pl.wp), static_cast<int64_t>(g.O) * g.oH * g.oW,
                             g.oH, g.oW, pl.shift_r, pl.shift_c, 1, N};
      PhaseCols cm{FastDiv(pl.hp * pl.wp), FastDiv(pl.wp), static_cast<int64_t>(g.C) * g.H * g.W, pl.a0, pl.b0, s, g.W};
      const int tn = (N + BN - 1) / BN, tm = (M + BM - 1) / BM;
      hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, PhaseCols>), dim3(grid_blocks(tm, tn, 1)),
                         dim3(kThreads), 0, st, ap, bp, dx, int64_t(0), static_cast<int64_t>(g.H) * g.W, cm, M, N, K,
                         (K + BK - 1) / BK * BK, TileGrid{tm, tn, tm * tn});
    }
  return 0;
}

// stride-1 bwd-data with the tap-major reduction order; wt is the filter re-laid as [C][kHW][O]
template <int BM, int BN, int WM, int WN>
void launch_bwd_data_tap_major(const ConvGeo &g, const float *wt, const float *dy, float *dx, hipStream_t st) {
  using AL = KContigLoader<BM>;
  using BL = TapMajorColsLoader<BN, true>;
  const int K = g.O * g.kH * g.kW, N = g.imgs * g.H * g.W, M = g.C;
  typename AL::Params ap{wt, K, M, true};
  typename BL::Params bp{dy, FastDiv(g.H * g.W), FastDiv(g.W), static_cast<int64_t>(g.O) * g.oH * g.oW, g.oH * g.oW,
                         g.oH, g.oW, g.ph, g.pw, 1, g.O, g.kW, g.kH * g.kW, N};
  NchwCols cm{FastDiv(g.H * g.W), static_cast<int64_t>(g.C) * g.H * g.W};
  const int tn = (N + BN - 1) / BN, tm = (M + BM - 1) / BM;
  dim3 grid(grid_blocks(tm, tn, 1));
  hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, NchwCols>), grid, dim3(kThreads), 0, st, ap, bp, dx,
                     int64_t(0), static_cast<int64_t>(g.H) * g.W, cm, M, N, K, K, TileGrid{tm, tn, tm * tn});
}

template <int BM, int BN, int WM, int WN>
int launch_bwd_filter(const ConvGeo &g, const float *x, const float *dy, float *dw, const Tap *taps, hipStream_t st,
                      int64_t *ws_elems) {
  using AL = DyRowsLoader<BM>;
  using BL = GatherRowsLoader<BN>;
  const int K = g.imgs * g.oH * g.oW, N = g.C * g.kH * g.kW, M = g.O;
  typename AL::Params ap{dy, FastDiv(g.oH * g.oW), g.O, (g.oH * g.oW) % 4 == 0 && aligned16(dy)};
  typename BL::Params bp{x, taps, FastDiv(g.oH * g.oW), FastDiv(g.oW), static_cast<int64_t>(g.C) * g.H * g.W,
                         g.H, g.W, g.ph, g.pw, g.s, N};
  const int tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
  int S, kchunk;
  static const int occ = blocks_per_cu(mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, RowMajorCols>);
  plan_splitk(tm * tn, K, 1024, occ, S, kchunk);
  const int64_t mn = static_cast<int64_t>(M) * N;
  float *out = dw;
  if (S > 1) {
    out = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(S) * mn * 4));
    TS_REQUIRE(out, "conv bwd-filter: no scratch memory for split-K");
    *ws_elems = S * mn;
  }
  hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, RowMajorCols>), dim3(grid_blocks(tm, tn, S)),
                     dim3(kThreads), 0, st, ap, bp, out, mn, static_cast<int64_t>(N), RowMajorCols{}, M, N, K, kchunk,
                     TileGrid{tm, tn, tm * tn * S});
  if (S > 1)
    hipLaunchKernelGGL(splitk_fold_kernel, dim3(static_cast<unsigned>((mn + 255) / 256)), dim3(256), 0, st, out, dw,
                       mn, mn, S);
  return 0;
}

// bwd-filter with tap-major columns; always goes through the fold kernel, which also restores
// the OIHW layout
template <int BM, int BN, int WM, int WN>
int launch_bwd_filter_tap_major(const ConvGeo &g, const float *x, const float *dy, float *dw, hipStream_t st,
                                int64_t *ws_elems) {
  using AL = DyRowsLoader<BM>;
  using BL = TapMajorRowsLoader<BN>;
  const int K = g.imgs * g.oH * g.oW, N = g.C * g.kH * g.kW, M = g.O;
  typename AL::Params ap{dy, FastDiv(g.oH * g.oW), g.O, (g.oH * g.oW) % 4 == 0 && aligned16(dy)};
  typename BL::Params bp{x, FastDiv(g.oH * g.oW), FastDiv(g.oW), static_cast<int64_t>(g.C) * g.H * g.W, g.H * g.W,
                         g.H, g.W, g.ph, g.pw, g.s, g.C, g.kW, N};
  const int tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
  int S, kchunk;
  static const int occ = blocks_per_cu(mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, RowMajorCols>);
  plan_splitk(tm * tn, K, 1024, occ, S, kchunk);
  const int64_t mn = static_cast<int64_t>(M) * N;
  float *part = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(S) * mn * 4));
  TS_REQUIRE(part, "conv bwd-filter: no scratch memory for split-K");
  *ws_elems = S * mn;
  hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, RowMajorCols>), dim3(grid_blocks(tm, tn, S)),
                     dim3(kThreads), 0, st, ap, bp, part, mn, static_cast<int64_t>(N), RowMajorCols{}, M, N, K, kchunk,
                     TileGrid{tm, tn, tm * tn * S});
  hipLaunchKernelGGL(fold_tap_major_kernel, dim3(static_cast<unsigned>((mn + 63) / 64)), dim3(256), 0, st, part, dw,
                     g.O, g.C, g.kH * g.kW, mn, S);
  return 0;
}

// launches conv_tap_kernel; `w_relaid` is [M][K] in the tap-major order
// One stride phase of a strided backward-data pass, seen as a stride-1 backward-data problem:
// dx[a0 + s*i][b0 + s*j] = sum over (o, u, v) of w[o][c][a + s*u][b + s*v] * dy[o][i + pad_r - u][j + pad_c - v].
struct TapPhase {
  int a, b;          // first filter row / column of the phase
  int nu, nv;        // filter taps of the phase along each axis
  int a0, b0;        // first input row / column of the phase
  int hp, wp;        // positions of the phase along each axis
  int pad_r, pad_c;  // (a0 + ph - a) / s, (b0 + pw - b) / s
};

// sub-filter of a phase in the tap-major order of conv_tap_kernel:
// out[c][((o/16)*T + t)*16 + o%16] = w[o][c][a + s*u][b + s*v],  t = u*nv + v, T = nu*nv
__global__ __launch_bounds__(256) void filter_phase_tap_major_kernel(const float *__restrict__ w, float *__restrict__ out,
                                                                     int O, int C, int kH, int kW, int a, int b, int s,
                                                                     int nu, int nv) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int T = nu * nv, K = O * T;
  if (idx >= C * K) return;
  const int c = idx / K, kp = idx - c * K;
  const int lo = kp & 15, q = kp >> 4;
  const int t = q % T, o = (q / T) * 16 + lo;
  const int u = t / nv, v = t - u * nv;
  out[idx] = w[((o * C + c) * kH + (a + s * u)) * kW + (b + s * v)];
}

constexpr int kManyTiles = 1024;

template <int BM, int BN, int WM, int WN, bool BWD_DATA, bool RAW = false>
int launch_conv_tap(const ConvGeo &g, const float *src, const float *w_relaid, float *out, hipStream_t st,
                    const TapPhase *phase = nullptr, StatsSink *sink = nullptr) {
  TapConvParams P;
  int taps = g.kH * g.kW;
  P.out_s = 1;
  P.out_a0 = P.out_b0 = 0;
  if (BWD_DATA) {   // out = dx [imgs][C][H][W], src = dy [imgs][O][oH][oW]
    P.M = g.C;
    P.N = g.imgs * g.H * g.W;
    P.K = g.O * taps;
    P.plane = FastDiv(g.H * g.W);
    P.width = FastDiv(g.W);
    P.img_stride = g.O * g.oH * g.oW;
    P.chan_stride = g.oH * g.oW;
    P.src_h = g.oH;
    P.src_w = g.oW;
    P.out_plane = g.H * g.W;
    P.out_img_stride = static_cast<int64_t>(g.C) * g.H * g.W;
    P.src_bytes = static_cast<unsigned>(static_cast<int64_t>(g.imgs) * g.O * g.oH * g.oW * 4);
  } else {          // out = y [imgs][O][oH][oW], src = x [imgs][C][H][W]
    P.M = g.O;
    P.N = g.imgs * g.oH * g.oW;
    P.K = g.C * taps;
    P.plane = FastDiv(g.oH * g.oW);
    P.width = FastDiv(g.oW);
    P.img_stride = g.C * g.H * g.W;
    P.chan_stride = g.H * g.W;
    P.src_h = g.H;
    P.src_w = g.W;
    P.out_plane = g.oH * g.oW;
    P.out_img_stride = static_cast<int64_t>(g.O) * g.oH * g.oW;
    P.src_bytes = static_cast<unsigned>(static_cast<int64_t>(g.imgs) * g.C * g.H * g.W * 4);
  }
  P.ph = g.ph;
  P.pw = g.pw;
  P.s = g.s;
  P.kW = g.kW;
  P.out_w = BWD_DATA ? g.W : g.oW;
  if (phase) {      // one stride phase of a backward-data pass: a stride-1 problem on a sub-grid of dx
    taps = phase->nu * phase->nv;
    P.N = g.imgs * phase->hp * phase->wp;
    P.K = g.O * taps;
    P.plane = FastDiv(phase->hp * phase->wp);
    P.width = FastDiv(phase->wp);
    P.ph = phase->pad_r;
    P.pw = phase->pad_c;
    P.s = 1;
    P.kW = phase->nv;
    P.out_s = g.s;
    P.out_a0 = phase->a0;
    P.out_b0 = phase->b0;
  }
  P.stats = nullptr;
  if (sink) {     // forward passes only: one partial per channel and 32 output columns
    const int groups = (P.N + 31) / 32;
    TS_REQUIRE(!BWD_DATA && !RAW && !phase && sink->used + groups <= sink->capacity, "conv: statistics buffer too small");
    P.stats = sink->part + static_cast<int64_t>(sink->used) * P.M * 2;
    sink->used += groups;
  }
  P.wf = w_relaid;
  P.raw_row = BWD_DATA ? taps : g.C * taps;      // (only read by the RAW kernels; never with stride phases)
  P.raw_ch = BWD_DATA ? g.C * taps : taps;
  P.src = src;
  P.wf_bytes = static_cast<unsigned>(static_cast<int64_t>(P.M) * P.K * 4);
  P.taps = taps;
  const int tn = (P.N + BN - 1) / BN, tm = (P.M + BM - 1) / BM;
  const int tiles = tm * tn;
  StreamK sk;
  sk.ksteps = P.K / BK;
  sk.total = tn * sk.ksteps;
  sk.tm = tm;
  // many tiles: the variant with three resident blocks per CU (never with RAW, which is for small layers)
  const bool many = !RAW && tiles >= kManyTiles;
  static const int occ2 = blocks_per_cu(conv_tap_kernel<BM, BN, WM, WN, BWD_DATA, RAW, 2>);
  static const int occ3 = RAW ? occ2 : blocks_per_cu(conv_tap_kernel<BM, BN, WM, WN, BWD_DATA, false, 3>);
  const int slots = 256 * (many ? occ3 : occ2);
  unsigned grid;
  float *pieces = nullptr;
  sk.whole_waves = 0;
  sk.cut_first = 0;
  int cut_tiles = tiles;         // tiles the assemble kernel looks at
  // With little work, pieces stay at least kMinPiece k-steps long (shorter ones are all prologue and
  // assembly), and nothing is cut unless that at least halves the longest block's work.
  constexpr int kMinPiece = 8;
  const bool little = static_cast<int64_t>(tiles) * sk.ksteps < slots * kMinPiece;
  const bool cut_little = little && tiles * 2 <= slots && sk.ksteps >= 2 * kMinPiece && sk.total / kMinPiece >= 8;
  if (tiles % slots == 0 || (little && !cut_little)) {
    // whole tiles fill whole waves of blocks, or there is too little work to cut: one tile per block
    sk.iters_per_block = sk.ksteps;
    sk.ranges = tn;
    grid = (tiles + 7) / 8 * 8;
  } else {                       // one full wave of blocks (fewer when the work is little)
    // ranges per row: a multiple of 8, so that the tm blocks of one range share an XCD
    sk.ranges = std::max(8, slots / tm / 8 * 8);
    if (cut_little) sk.ranges = std::max(8, std::min(sk.ranges, sk.total / kMinPiece / 8 * 8));
    grid = static_cast<unsigned>(sk.ranges) * tm;
    const int full = tn / sk.ranges;
    sk.whole_waves = full;
    sk.cut_first = sk.whole_waves * sk.ranges;
    sk.total = (tn - sk.cut_first) * sk.ksteps;
    cut_tiles = (tn - sk.cut_first) * tm;
    sk.iters_per_block = std::max(1, (sk.total + sk.ranges - 1) / sk.ranges);
    if (sk.total > 0) {          // (whole waves may cover every row exactly: then nothing is cut)
      pieces = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(grid) * 2 * BM * BN * sizeof(float)));
      TS_REQUIRE(pieces, "conv: no scratch memory for the pieces of cut tiles");
    }
  }
  if constexpr (!BWD_DATA && !RAW) {
    if (sink) {
      if (many)
        hipLaunchKernelGGL((conv_tap_kernel<BM, BN, WM, WN, false, false, 3, true>), dim3(grid), dim3(kThreads), 0, st, P,
                           out, pieces, sk);
      else
        hipLaunchKernelGGL((conv_tap_kernel<BM, BN, WM, WN, false, false, 2, true>), dim3(grid), dim3(kThreads), 0, st, P,
                           out, pieces, sk);
      if (pieces)
        hipLaunchKernelGGL((conv_tap_assemble_kernel<BM, BN, WM, WN, true>), dim3(cut_tiles * 4), dim3(kThreads), 0, st, P,
                           out, pieces, sk);
      return 0;
    }
  }
  if (many)
    hipLaunchKernelGGL((conv_tap_kernel<BM, BN, WM, WN, BWD_DATA, false, 3>), dim3(grid), dim3(kThreads), 0, st, P, out,
                       pieces, sk);
  else
    hipLaunchKernelGGL((conv_tap_kernel<BM, BN, WM, WN, BWD_DATA, RAW, 2>), dim3(grid), dim3(kThreads), 0, st, P, out,
                       pieces, sk);
  if (pieces)
    hipLaunchKernelGGL((conv_tap_assemble_kernel<BM, BN, WM, WN>), dim3(cut_tiles * 4), dim3(kThreads), 0, st, P, out,
                       pieces, sk);
  return 0;
}

// Strided backward-data on conv_tap_kernel: one launch per stride phase (O % 16 == 0).
template <int BM, int BN, int WM, int WN>
int launch_bwd_data_phases_tap(const ConvGeo &g, const float *w, const float *dy, float *dx, float *wscratch,
                               hipStream_t st) {
  const int s = g.s;
  TS_REQUIRE(s * s <= 64, "conv bwd-data: stride %d not supported", s);
  TapPhase ph[64];
  int count = 0;
  bool any_empty = false;
  for (int a = 0; a < s; ++a)
    for (int b = 0; b < s; ++b) {
      TapPhase t;
      t.a = a;
      t.b = b;
      t.a0 = ((a - g.ph) % s + s) % s;
      t.b0 = ((b - g.pw) % s + s) % s;
      t.hp = t.a0 < g.H ? (g.H - t.a0 + s - 1) / s : 0;
      t.wp = t.b0 < g.W ? (g.W - t.b0 + s - 1) / s : 0;
      t.nu = a < g.kH ? (g.kH - a + s - 1) / s : 0;
      t.nv = b < g.kW ? (g.kW - b + s - 1) / s : 0;
      t.pad_r = (t.a0 + g.ph - a) / s;
      t.pad_c = (t.b0 + g.pw - b) / s;
      if (t.hp <= 0 || t.wp <= 0) continue;
      if (t.nu == 0 || t.nv == 0) {
        any_empty = true;        // positions no filter tap reaches: their gradient is zero
        continue;
      }
      ph[count++] = t;
    }
  if (any_empty) {
    const int64_t n = static_cast<int64_t>(g.imgs) * g.C * g.H * g.W;
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, dx, n);
  }
  int64_t woff = 0;
  for (int i = 0; i < count; ++i) {
    const TapPhase &t = ph[i];
    const int K = g.O * t.nu * t.nv;
    float *wp = wscratch + woff;          // every phase uses its own part of the re-laid filter
    woff += static_cast<int64_t>(g.C) * K;
    hipLaunchKernelGGL(filter_phase_tap_major_kernel, dim3((g.C * K + 255) / 256), dim3(256), 0, st, w, wp, g.O, g.C,
                       g.kH, g.kW, t.a, t.b, s, t.nu, t.nv);
    const int rc = launch_conv_tap<BM, BN, WM, WN, true>(g, dy, wp, dx, st, &t);
    if (rc) return rc;
  }
  return 0;
}

// Bytes a block may address from its base pointer: 2 GiB - 1 (offsets are signed 32-bit and the
// out-of-range marker is 0x80000000).  TSPLIT_CONV_REACH_BYTES lowers it, which makes small tensors
// take the paths of tensors beyond 2 GiB (for tests of those paths against a CPU result).
inline int64_t conv_reach_bytes() {
  const int64_t full = (1ll << 31) - 1;
  if (const char *e = std::getenv("TSPLIT_CONV_REACH_BYTES")) {
    const long long v = std::atoll(e);
    if (v > 0 && v < full) return v;
  }
  return full;
}

// The buffer-load path addresses with 32-bit byte offsets and a 32-tap bit mask.  A gathered
// tensor beyond 2 GiB is taken in runs of whole images, one launch each (images are independent
// in the forward and backward-data passes): -> images per launch, 0 if the path cannot be used.
inline int tap_kernel_images(const ConvGeo &g, int64_t src_elems_per_img, int64_t w_elems) {
  if (g.kH * g.kW > 32 || w_elems * 4 >= (1ll << 31) || g.imgs <= 0) return 0;
  const int64_t room = conv_reach_bytes() - 4 * (static_cast<int64_t>(g.kH) * g.W + g.kW + g.ph * g.W + g.pw);
  const int64_t fit = room / (src_elems_per_img * 4);
  if (fit < 1) return 0;
  if (fit >= g.imgs) return g.imgs;
  const int64_t launches = (g.imgs + fit - 1) / fit;          // equal runs rather than a short last one
  return static_cast<int>((g.imgs + launches - 1) / launches);
}

// 64-row tiles (64x256) instead of 128-row ones (128x128): always for up to 64 rows; beyond that when
// the rows would fill 128-row tiles a quarter worse than 64-row ones (192 rows = 1.5 tiles of 128 but
// exactly 3 of 64), which outweighs the ~10 % the 64x256 tiles lose on their gathers.
inline bool short_tiles(int rows) {
  if (rows <= 64) return true;
  const int by128 = (rows + 127) / 128 * 128, by64 = (rows + 63) / 64 * 64;
  return by128 * 4 >= by64 * 5;
}

// Small backward-data passes read the filter where it lies instead of re-laying it first (RAW
// kernels): in that pass neighbouring rows of the operand are neighbours in memory (4*taps bytes
// apart), so the four 4-byte loads cost less than a re-lay kernel in front of every call.  The
// forward pass reads rows C*taps apart with taps between the words of a row and loses more than
// the re-lay costs (measured), so it keeps it.
// TSPLIT_CONV_RAW=0 / 1 forces the choice (tests run both kernels on the same shapes).
inline bool raw_filter_pays(const ConvGeo &g) {
  if (const char *e = std::getenv("TSPLIT_CONV_RAW")) return e[0] == '1';
  return 2.0 * g.imgs * g.O * g.oH * g.oW * g.C * g.kH * g.kW < 12e9;
}

// Runs f(geometry of the run, first image) over runs of `per` images.
template <class F>
inline int for_image_runs(const ConvGeo &g, int per, F f) {
  for (int first = 0; first < g.imgs; first += per) {
    ConvGeo run = g;
    run.imgs = std::min(per, g.imgs - first);
    const int rc = f(run, static_cast<int64_t>(first));
    if (rc) return rc;
  }
  return 0;
}

// Images that fit into the 2 GiB a block of conv_wgrad_tap_kernel addresses from the first image of
// its k range, in the larger of x and dy.  A split of kchunk positions touches at most
// kchunk / HWp + 2 images.
inline int wgrad_tap_span_images(const ConvGeo &g) {
  const int64_t img_bytes = std::max(static_cast<int64_t>(g.C) * g.H * g.W, static_cast<int64_t>(g.O) * g.oH * g.oW) * 4;
  const int64_t room = conv_reach_bytes() - 8 * (static_cast<int64_t>(g.ph) * g.W + g.pw) - 64;
  return static_cast<int>(std::min<int64_t>(room / img_bytes, 1 << 20));
}

template <int BM, int BN, int WM, int WN, bool TAIL, bool GEN>
int wgrad_tap_occupancy() {
  static const int occ = blocks_per_cu(conv_wgrad_tap_kernel<BM, BN, WM, WN, TAIL, GEN>);
  return occ;
}

// bwd-filter on conv_wgrad_tap_kernel
template <int BM, int BN, int WM, int WN>
int launch_wgrad_tap(const ConvGeo &g, const float *x, const float *dy, float *dw, hipStream_t st, int64_t *ws_elems) {
  const bool gen = !(g.s == 1 && g.oH == g.H && g.oW == g.W);
  TapWgradParams P;
  P.dy = dy;
  P.x = x;
  P.dy_bytes = static_cast<int64_t>(g.imgs) * g.O * g.oH * g.oW * 4;
  P.x_bytes = static_cast<int64_t>(g.imgs) * g.C * g.H * g.W * 4;
  P.O = g.O;
  P.C = g.C;
  P.HW = g.oH * g.oW;
  P.W = g.oW;
  P.s = g.s;
  P.xH = g.H;
  P.xW = g.W;
  P.xHW = g.H * g.W;
  P.kW = g.kW;
  P.taps = g.kH * g.kW;
  P.ph = g.ph;
  P.pw = g.pw;
  P.M = g.O;
  P.N = g.C * g.kH * g.kW;
  P.HWp = (P.HW + BK - 1) / BK * BK;
  P.K = g.imgs * P.HWp;
  const bool tail = P.HWp != P.HW;
  const int tm = (P.M + BM - 1) / BM, tn = (P.N + BN - 1) / BN;
  int S;
  // resident blocks per CU of the variant that will run (the padded-tail and general-geometry
  // variants need a few more registers and may fit one block fewer): the K split aims at exactly
  // one full wave of resident blocks
  const int occ = gen ? (tail ? wgrad_tap_occupancy<BM, BN, WM, WN, true, true>() : wgrad_tap_occupancy<BM, BN, WM, WN, false, true>())
                      : (tail ? wgrad_tap_occupancy<BM, BN, WM, WN, true, false>() : wgrad_tap_occupancy<BM, BN, WM, WN, false, false>());
  plan_splitk(tm * tn, P.K, 1024, occ, S, P.kchunk);
  // the images one split touches must lie within 2 GiB in both tensors: shorten the splits until they do
  const int span = wgrad_tap_span_images(g);
  if (P.kchunk / P.HWp + 2 > span) {
    P.kchunk = std::max(BK, (span - 2) * P.HWp / BK * BK);
    S = (P.K + P.kchunk - 1) / P.kchunk;
  }
  const int64_t mn = static_cast<int64_t>(P.M) * P.N;
  float *part = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(S) * mn * 4));
  TS_REQUIRE(part, "conv bwd-filter: no scratch memory for split-K");
  *ws_elems = S * mn;
  const dim3 grid(grid_blocks(tm, tn, S));
  const TileGrid tg{tm, tn, tm * tn * S};
  if (gen && tail)
    hipLaunchKernelGGL((conv_wgrad_tap_kernel<BM, BN, WM, WN, true, true>), grid, dim3(kThreads), 0, st, P, part, tg);
  else if (gen)
    hipLaunchKernelGGL((conv_wgrad_tap_kernel<BM, BN, WM, WN, false, true>), grid, dim3(kThreads), 0, st, P, part, tg);
  else if (tail)
    hipLaunchKernelGGL((conv_wgrad_tap_kernel<BM, BN, WM, WN, true, false>), grid, dim3(kThreads), 0, st, P, part, tg);
  else
    hipLaunchKernelGGL((conv_wgrad_tap_kernel<BM, BN, WM, WN, false, false>), grid, dim3(kThreads), 0, st, P, part, tg);
  hipLaunchKernelGGL(fold_tap_major_kernel, dim3(static_cast<unsigned>((mn + 63) / 64)), dim3(256), 0, st, part, dw,
                     g.O, g.C, g.kH * g.kW, mn, S);
  return 0;
}

// ------------------------------------------------------------------ bwd-filter, few columns
// dw[O, N] with N = C*kH*kW <= 32 (the first layer of an image network: 3 input channels).  The
// 64x64-per-wave tiling would spend 7/8 of its MFMAs on padding, and the reduction
// (K = imgs*oH*oW, hundreds of thousands) is what has to be streamed: dy is read exactly
// once.  A block owns 64 rows x 32 columns and a slice of K; steps are 32 k wide; the four
// waves split every step's k four ways (8 k each = 4 MFMAs per 32x32 block), so the whole
// block advances one step per barrier, and their accumulators are added through LDS at the
// end.  Slice sums go to scratch and are folded in slice order.
constexpr int NK = 32;                 // k per step
constexpr int kNStride = NK + 4;       // LDS row stride (floats), keeps 16-byte alignment
constexpr int kNarrowCols = 32;
struct NarrowWgradParams {
  const float *dy, *x;
  const Tap *taps;
  FastDiv plane, width;    // oH*oW, oW
  int64_t img_stride;      // C*H*W
  int O, N, K, H, W, ph, pw, s, steps_per_slice;
  bool vec;                // oH*oW % 4 == 0 and dy 16-byte aligned
};

__global__ __launch_bounds__(kThreads) void conv_wgrad_narrow_kernel(NarrowWgradParams P, float *__restrict__ part) {
  constexpr int kAFloats = 64 * kNStride, kBFloats = kNarrowCols * kNStride;
  __shared__ __attribute__((aligned(16))) float lds_all[2 * kAFloats + 2 * kBFloats];
  float(*lds_a)[kAFloats] = reinterpret_cast<float(*)[kAFloats]>(lds_all);
  float(*lds_b)[kBFloats] = reinterpret_cast<float(*)[kBFloats]>(lds_all + 2 * kAFloats);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * 64;
  const int kbegin = blockIdx.x * P.steps_per_slice * NK;
  const int kend = min(P.K, kbegin + P.steps_per_slice * NK);

  // A (dy rows): thread -> rows tid/8 and tid/8 + 32, k quad tid%8
  const int arow = tid >> 3, akq = tid & 7;
  // B (gathered x): thread -> k = tid%32, columns tid/32 + 8*i
  const int bk = tid & 31, bcol = tid >> 5;
  int toff[4];
  short tkh[4], tkw[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int j = bcol + 8 * i;
    if (j < P.N) {
      const Tap t = P.taps[j];
      toff[i] = t.off;
      tkh[i] = t.kh;
      tkw[i] = t.kw;
    } else {
      toff[i] = 0;
      tkh[i] = -20000;   // fails the range test for any row
      tkw[i] = 0;
    }
  }
  float4 ra[2];
  float rb[4];
  auto dy_one = [&](int k, int row) -> float {
    if (k >= kend) return 0.f;
    const uint32_t img = P.plane.div(k);
    const uint32_t px = k - img * P.plane.d;
    return P.dy[(static_cast<int64_t>(img) * P.O + row) * P.plane.d + px];
  };
  auto load = [&](int k0) {
    {
      const int k = k0 + 4 * akq;
      const uint32_t img = P.plane.div(k);
      const uint32_t px = k - img * P.plane.d;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = m0 + arow + 32 * h;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (row < P.O) {
          if (P.vec && k + 3 < kend) {
            v = *reinterpret_cast<const float4 *>(P.dy + (static_cast<int64_t>(img) * P.O + row) * P.plane.d + px);
          } else {
            v.x = dy_one(k, row);
            v.y = dy_one(k + 1, row);
            v.z = dy_one(k + 2, row);
            v.w = dy_one(k + 3, row);
          }
        }
        ra[h] = v;
      }
    }
    {
      const int k = k0 + bk;
      const bool k_ok = k < kend;
      const uint32_t kk = k_ok ? k : 0;
      const uint32_t img = P.plane.div(kk);
      const uint32_t px = kk - img * P.plane.d;
      const uint32_t oh = P.width.div(px);
      const uint32_t ow = px - oh * P.width.d;
      const int r0 = static_cast<int>(oh) * P.s - P.ph, c0 = static_cast<int>(ow) * P.s - P.pw;
      const float *base = P.x + static_cast<int64_t>(img) * P.img_stride + static_cast<int64_t>(r0) * P.W + c0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int rr = r0 + tkh[i], cc = c0 + tkw[i];
        float v = 0.f;
        if (k_ok && static_cast<unsigned>(rr) < static_cast<unsigned>(P.H) &&
            static_cast<unsigned>(cc) < static_cast<unsigned>(P.W))
          v = base[toff[i]];
        rb[i] = v;
      }
    }
  };
  auto store = [&](int stage) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
      *reinterpret_cast<float4 *>(&lds_a[stage][(arow + 32 * h) * kNStride + 4 * akq]) = ra[h];
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_b[stage][(bcol + 8 * i) * kNStride + bk] = rb[i];
  };

  acc16 acc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;

  if (kbegin < kend) {
    load(kbegin);
    store(0);
  }
  __syncthreads();
  int stage = 0;
  for (int k0 = kbegin; k0 < kend; k0 += NK) {
    const bool more = k0 + NK < kend;
    if (more) load(k0 + NK);
    // this wave's 8 k of the step: lanes 0-31 supply k = 8*wave + e, lanes 32-63 k = 8*wave + 4 + e
    const int kofs = 8 * wave + 4 * (lane >> 5);
    const float4 fb = *reinterpret_cast<const float4 *>(&lds_b[stage][(lane & 31) * kNStride + kofs]);
    const float4 fa0 = *reinterpret_cast<const float4 *>(&lds_a[stage][(lane & 31) * kNStride + kofs]);
    const float4 fa1 = *reinterpret_cast<const float4 *>(&lds_a[stage][(32 + (lane & 31)) * kNStride + kofs]);
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa0.x, fb.x, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa1.x, fb.x, acc[1], 0, 0, 0);
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa0.y, fb.y, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa1.y, fb.y, acc[1], 0, 0, 0);
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa0.z, fb.z, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa1.z, fb.z, acc[1], 0, 0, 0);
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa0.w, fb.w, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa1.w, fb.w, acc[1], 0, 0, 0);
    if (more) store(stage ^ 1);
    __syncthreads();
    stage ^= 1;
  }

  // add the four waves' accumulators: waves 1-3 park theirs in LDS (the staging buffers are
  // free now: the loop ended with a barrier), wave 0 adds them to its own in a fixed order and
  // writes the block's 64 x N slice sum.  red[wave - 1][row][col], row stride 33.
  float *red = lds_all;
  static_assert(3 * 64 * 33 <= 2 * kAFloats + 2 * kBFloats, "reduction buffer fits in the staging LDS");
  if (wave > 0) {
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = 32 * mi + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        red[((wave - 1) * 64 + row) * 33 + (lane & 31)] = acc[mi][e];
      }
  }
  __syncthreads();
  if (wave == 0) {
    float *o = part + static_cast<int64_t>(blockIdx.x) * P.O * P.N;
    const int col = lane & 31;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = 32 * mi + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        const float v = ((acc[mi][e] + red[row * 33 + col]) + red[(64 + row) * 33 + col]) + red[(128 + row) * 33 + col];
        if (m0 + row < P.O && col < P.N) o[static_cast<int64_t>(m0 + row) * P.N + col] = v;
      }
  }
}

// out[i] = sum over slices of part[slice][i]: 64 outputs x 4 slice-lanes per block, slice-lane l
// adds slices l, l + 4, ... and the four sums are combined through LDS in a fixed order.
__global__ __launch_bounds__(kThreads) void fold_many_slices_kernel(const float *__restrict__ part,
                                                                    float *__restrict__ out, int n, int slices) {
  __shared__ float sm[3][64];
  const int cx = threadIdx.x & 63, ry = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + cx;
  float acc = 0.f;
  if (i < n) {
#pragma unroll 8
    for (int s = ry; s < slices; s += 4) acc += part[static_cast<int64_t>(s) * n + i];
  }
  if (ry > 0) sm[ry - 1][cx] = acc;
  __syncthreads();
  if (ry == 0 && i < n) out[i] = ((acc + sm[0][cx]) + sm[1][cx]) + sm[2][cx];
}

inline bool wgrad_narrow_ok(const ConvGeo &g) {
  return g.C * g.kH * g.kW <= kNarrowCols && static_cast<int64_t>(g.imgs) * g.oH * g.oW < (1ll << 31) - 64;
}

int launch_wgrad_narrow(const ConvGeo &g, const float *x, const float *dy, float *dw, hipStream_t st,
                        int64_t *ws_elems) {
  NarrowWgradParams P;
  P.dy = dy;
  P.x = x;
  P.taps = tap_table(g.C, g.kH, g.kW, g.W, g.H * g.W, +1);
  TS_REQUIRE(P.taps, "conv bwd-filter: could not build the tap table");
  P.plane = FastDiv(g.oH * g.oW);
  P.width = FastDiv(g.oW);
  P.img_stride = static_cast<int64_t>(g.C) * g.H * g.W;
  P.O = g.O;
  P.N = g.C * g.kH * g.kW;
  P.K = g.imgs * g.oH * g.oW;
  P.H = g.H;
  P.W = g.W;
  P.ph = g.ph;
  P.pw = g.pw;
  P.s = g.s;
  P.vec = (g.oH * g.oW) % 4 == 0 && aligned16(dy);
  const int tm = (g.O + 63) / 64;
  const int steps = (P.K + NK - 1) / NK;
  // about four blocks per CU, at least 8 steps each
  int slices = std::max(1, std::min(1024 / tm, steps / 8));
  P.steps_per_slice = (steps + slices - 1) / slices;
  slices = (steps + P.steps_per_slice - 1) / P.steps_per_slice;
  const int mn = g.O * P.N;
  float *part = dw;
  if (slices > 1) {
    part = static_cast<float *>(scratch_get(st, 2, static_cast<size_t>(slices) * mn * 4));
    TS_REQUIRE(part, "conv bwd-filter: no scratch memory for split-K");
    *ws_elems = static_cast<int64_t>(slices) * mn;
  }
  hipLaunchKernelGGL(conv_wgrad_narrow_kernel, dim3(slices, tm), dim3(kThreads), 0, st, P, part);
  if (slices > 1)
    hipLaunchKernelGGL(fold_many_slices_kernel, dim3((mn + 63) / 64), dim3(kThreads), 0, st, part, dw, mn, slices);
  return 0;
}

inline bool wgrad_tap_ok(const ConvGeo &g) {
  // three images within a block's reach: a split of at least one image's positions stays addressable
  return g.C % BK == 0 && wgrad_tap_span_images(g) >= 3 &&
         static_cast<int64_t>(g.imgs) * ((g.oH * g.oW + BK - 1) / BK * BK) < (1ll << 31) - BK;
}

// ------------------------------------------------------------------ thin forward (first layer)
// Forward pass with at most 32 reduction indices (Cin*kH*kW: a first layer on 3 channels).  Two
// 16-wide k-steps cannot amortise a tile's gather set-up and the layer is bound by writing its
// output, so it runs on the vector ALU: a wave takes 64 consecutive output positions and 32
// output channels (measured best of 16 / 32 / 64: more channels per thread repeat the gather of
// the <= 32 inputs less often but leave fewer waves to hide its latency); the filter, re-laid
// [k][Cout], is wave-uniform and feeds the multiply-adds from scalar registers; every output
// plane gets 256-byte stores.  Algorithmic bytes =
// 4 * (x + w + y), almost all of it y.
constexpr int kThinMaxK = 32;

struct ThinParams {
  int C, H, W, O, Opad, kH, kW, ph, pw, s, oH, oW, K;   // Opad: O rounded up to the channels per thread
  FastDiv plane, width;              // oH*oW, oW
  int64_t n_total;                   // imgs * oH * oW
  int64_t x_bytes;
};

__global__ __launch_bounds__(256) void filter_thin_kernel(const float *__restrict__ w, float *__restrict__ out, int O,
                                                          int Opad, int K) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= K * Opad) return;
  const int k = idx / Opad, o = idx - k * Opad;
  out[idx] = o < O ? w[o * K + k] : 0.f;
}

// wt: the filter as [K][Opad]; kThinChans: output channels per thread
template <int kThinChans>
__global__ __launch_bounds__(256) void conv_thin_fwd_kernel(ThinParams P, const float *__restrict__ x,
                                                            const float *__restrict__ wt, float *__restrict__ y) {
  __shared__ int tab[kThinMaxK][4];     // per reduction index: kh, kw, offset inside one image of x
  if (threadIdx.x < P.K) {
    const int taps = P.kH * P.kW;
    const int c = threadIdx.x / taps, t = threadIdx.x - c * taps;
    const int kh = t / P.kW, kw = t - kh * P.kW;
    tab[threadIdx.x][0] = kh;
    tab[threadIdx.x][1] = kw;
    tab[threadIdx.x][2] = (c * P.H + kh) * P.W + kw;
    tab[threadIdx.x][3] = 0;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const int og = __builtin_amdgcn_readfirstlane(blockIdx.y * 4 + (threadIdx.x >> 6));   // channel group of this wave
  if (og * kThinChans >= P.O) return;
  const int64_t n = static_cast<int64_t>(blockIdx.x) * 64 + lane;
  const bool ok = n < P.n_total;
  const uint32_t nn = ok ? static_cast<uint32_t>(n) : 0u;
  const uint32_t img = P.plane.div(nn);
  const uint32_t p = nn - img * P.plane.d;
  const uint32_t oh = P.width.div(p), ow = p - oh * P.width.d;
  const int ih0 = static_cast<int>(oh) * P.s - P.ph, iw0 = static_cast<int>(ow) * P.s - P.pw;
  const float *xi = x + static_cast<int64_t>(img) * P.C * P.H * P.W + ih0 * P.W + iw0;
  const float *wg = wt + og * kThinChans;
  // all gathered values first (independent loads, all in flight), then the multiply-adds
  float xv[kThinMaxK];
#pragma unroll
  for (int k = 0; k < kThinMaxK; ++k) {
    xv[k] = 0.f;
    if (k < P.K) {
      const int kh = tab[k][0], kw = tab[k][1], off = tab[k][2];
      const bool in = ok && static_cast<unsigned>(ih0 + kh) < static_cast<unsigned>(P.H) &&
                      static_cast<unsigned>(iw0 + kw) < static_cast<unsigned>(P.W);
      if (in) xv[k] = xi[off];
    }
  }
  float acc[kThinChans];
#pragma unroll
  for (int o = 0; o < kThinChans; ++o) acc[o] = 0.f;
#pragma unroll
  for (int k = 0; k < kThinMaxK; ++k) {
    if (k < P.K) {
      const float *wk = wg + k * P.Opad;         // wave-uniform: scalar loads
#pragma unroll
      for (int o = 0; o < kThinChans; ++o) acc[o] += xv[k] * wk[o];
    }
  }
  if (!ok) return;
  float *yo = y + (static_cast<int64_t>(img) * P.O + og * kThinChans) * P.plane.d + p;
#pragma unroll
  for (int o = 0; o < kThinChans; ++o)
    if (og * kThinChans + o < P.O) __builtin_nontemporal_store(acc[o], yo + static_cast<int64_t>(o) * P.plane.d);
}

// The same layer class on the matrix pipes, without LDS staging and without barriers: y[oc][pos] = sum over k of
// w[oc][k] patch[k][pos] as 32 x 32 x 2 MFMAs whose operands come straight from memory in the instruction's
// own layout.  A wave takes 64 consecutive output positions (two column tiles) and 64 output channels (two
// row tiles).  Lane l supplies, for MFMA j, the filter value w[32 t + l % 32][2 j + l / 32] (kept in
// registers for the whole wave: the filter is 64 x 27 numbers) and the input value of position l % 32 under
// reduction index 2 j + l / 32 (a gather from x, which stays in L2: 32 consecutive positions are 128
// consecutive bytes of an image row); the result's lanes 0 - 31 hold 32 consecutive positions of one output
// channel, so every store instruction writes two whole 128-byte lines.  The multiplications take a quarter
// of the time it takes to write y: the kernel is bound by that write.
template <int kRowTiles, int kSteps, bool kAllRows>
__global__ __launch_bounds__(256) void conv_thin_mfma_kernel(ThinParams P, const float *__restrict__ x,
                                                             const float *__restrict__ w, float *__restrict__ y) {
  __shared__ int tab[2 * kSteps][4];     // per reduction index: kh, kw, offset inside one image of x
  if (threadIdx.x < 2 * kSteps) {
    const int k = threadIdx.x < P.K ? threadIdx.x : 0;
    const int taps = P.kH * P.kW;
    const int c = k / taps, t = k - c * taps;
    const int kh = t / P.kW, kw = t - kh * P.kW;
    tab[threadIdx.x][0] = kh;
    tab[threadIdx.x][1] = kw;
    tab[threadIdx.x][2] = (c * P.H + kh) * P.W + kw;
    tab[threadIdx.x][3] = threadIdx.x < P.K ? 1 : 0;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5;
  const int oc0 = blockIdx.y * (32 * kRowTiles);
  // Both operands come through buffer loads: an element that does not exist (a channel beyond O, an index
  // beyond K, a tap outside the image, a position beyond the last one) gets an offset beyond the buffer and
  // reads as zero, without a branch.
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(w), 0, P.O * P.K * 4, mg::kBufFlags);
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(x), 0, static_cast<int>(P.x_bytes), mg::kBufFlags);
  float wa[kRowTiles][kSteps];
#pragma unroll
  for (int t = 0; t < kRowTiles; ++t)
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const int oc = oc0 + 32 * t + col, k = 2 * j + half;
      const unsigned off = oc < P.O && k < P.K ? static_cast<unsigned>(oc * P.K + k) * 4u : mg::kOobOffset;
      wa[t][j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rw, off, 0, 0));
    }
  const int64_t n0 = (static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6)) * 64;
  if (n0 >= P.n_total) return;
  // the gathered inputs of this lane's two positions, all loads in flight together
  float xb[2][kSteps];
  uint32_t img[2], pos[2];
  bool ok[2];
#pragma unroll
  for (int pt = 0; pt < 2; ++pt) {
    const int64_t n = n0 + 32 * pt + col;
    ok[pt] = n < P.n_total;
    const uint32_t nn = ok[pt] ? static_cast<uint32_t>(n) : 0u;
    img[pt] = P.plane.div(nn);
    pos[pt] = nn - img[pt] * P.plane.d;
    const uint32_t oh = P.width.div(pos[pt]), ow = pos[pt] - oh * P.width.d;
    const int ih0 = static_cast<int>(oh) * P.s - P.ph, iw0 = static_cast<int>(ow) * P.s - P.pw;
    const int base = static_cast<int>(img[pt]) * (P.C * P.H * P.W) + ih0 * P.W + iw0;   // below 2^29 elements
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const int4 e = *reinterpret_cast<const int4 *>(tab[2 * j + half]);
      const bool in = ok[pt] && e.w != 0 && static_cast<unsigned>(ih0 + e.x) < static_cast<unsigned>(P.H) &&
                      static_cast<unsigned>(iw0 + e.y) < static_cast<unsigned>(P.W);
      const unsigned off = in ? static_cast<unsigned>(base + e.z) * 4u : mg::kOobOffset;
      xb[pt][j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rx, off, 0, 0));
    }
  }
  mg::acc16 acc[kRowTiles][2];
#pragma unroll
  for (int t = 0; t < kRowTiles; ++t)
#pragma unroll
    for (int pt = 0; pt < 2; ++pt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[t][pt][e] = 0.f;
#pragma unroll
  for (int j = 0; j < kSteps; ++j)
#pragma unroll
    for (int t = 0; t < kRowTiles; ++t)
#pragma unroll
      for (int pt = 0; pt < 2; ++pt)
        acc[t][pt] = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[t][j], xb[pt][j], acc[t][pt], 0, 0, 0);
  // element e of a lane: output channel 32 t + 8 (e / 4) + 4 (lane / 32) + e % 4, position of the lane
#pragma unroll
  for (int pt = 0; pt < 2; ++pt) {
    if (!ok[pt]) continue;
    float *yo = y + static_cast<int64_t>(img[pt]) * P.O * P.plane.d + pos[pt];
#pragma unroll
    for (int t = 0; t < kRowTiles; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int oc = oc0 + 32 * t + 8 * (e >> 2) + 4 * half + (e & 3);
        if (kAllRows || oc < P.O) __builtin_nontemporal_store(acc[t][pt][e], yo + static_cast<int64_t>(oc) * P.plane.d);
      }
  }
}

// from 32 output channels on, the matrix-pipe form (TSPLIT_CONV_THIN_MFMA=0 keeps the vector-ALU kernel)
inline bool thin_on_matrix_pipes(const ConvGeo &g) {
  const char *e = std::getenv("TSPLIT_CONV_THIN_MFMA");
  return g.O >= 32 && static_cast<int64_t>(g.imgs) * g.C * g.H * g.W < (1ll << 29) && !(e && e[0] == '0');
}

inline bool thin_fwd_ok(const ConvGeo &g) {
  return g.C * g.kH * g.kW <= kThinMaxK && static_cast<int64_t>(g.imgs) * g.oH * g.oW < (1ll << 31);
}

int launch_conv_thin_fwd(const ConvGeo &g, const float *x, const float *w, float *y, hipStream_t st) {
  ThinParams P;
  P.K = g.C * g.kH * g.kW;
  const int chans = g.O > 16 ? 32 : 16;
  P.Opad = (g.O + chans - 1) / chans * chans;
  const bool mfma = thin_on_matrix_pipes(g);
  float *wt = nullptr;
  if (!mfma) {
    wt = static_cast<float *>(scratch_get(st, 3, static_cast<size_t>(P.K) * P.Opad * 4));
    TS_REQUIRE(wt, "conv: no scratch memory for the re-laid filter");
    hipLaunchKernelGGL(filter_thin_kernel, dim3((P.K * P.Opad + 255) / 256), dim3(256), 0, st, w, wt, g.O, P.Opad, P.K);
  }
  P.C = g.C;
  P.H = g.H;
  P.W = g.W;
  P.O = g.O;
  P.kH = g.kH;
  P.kW = g.kW;
  P.ph = g.ph;
  P.pw = g.pw;
  P.s = g.s;
  P.oH = g.oH;
  P.oW = g.oW;
  P.plane = FastDiv(g.oH * g.oW);
  P.width = FastDiv(g.oW);
  P.n_total = static_cast<int64_t>(g.imgs) * g.oH * g.oW;
  if (mfma) {
    const dim3 grid_m(static_cast<unsigned>((P.n_total + 255) / 256), static_cast<unsigned>((g.O + 63) / 64));
    P.x_bytes = static_cast<int64_t>(g.imgs) * g.C * g.H * g.W * 4;
    const bool all = g.O % 64 == 0;   // every row tile is whole: the stores need no channel check
    if (P.K <= 28 && all)
      hipLaunchKernelGGL((conv_thin_mfma_kernel<2, 14, true>), grid_m, dim3(256), 0, st, P, x, w, y);
    else if (P.K <= 28)
      hipLaunchKernelGGL((conv_thin_mfma_kernel<2, 14, false>), grid_m, dim3(256), 0, st, P, x, w, y);
    else if (all)
      hipLaunchKernelGGL((conv_thin_mfma_kernel<2, 16, true>), grid_m, dim3(256), 0, st, P, x, w, y);
    else
      hipLaunchKernelGGL((conv_thin_mfma_kernel<2, 16, false>), grid_m, dim3(256), 0, st, P, x, w, y);
    return 0;
  }
  const unsigned groups = static_cast<unsigned>(P.Opad / chans);
  const dim3 grid(static_cast<unsigned>((P.n_total + 63) / 64), (groups + 3) / 4);
  if (chans == 32)
    hipLaunchKernelGGL(conv_thin_fwd_kernel<32>, grid, dim3(256), 0, st, P, x, wt, y);
  else
    hipLaunchKernelGGL(conv_thin_fwd_kernel<16>, grid, dim3(256), 0, st, P, x, wt, y);
  return 0;
}

// 3x3 / stride 1 / pad 1 layers wide enough to be bound by MFMA throughput go through the Winograd
// F(4x4, 3x3) routine (winograd.hip): a quarter of the multiplications for 2.25x the activation
// traffic.  TSPLIT_CONV_WINOGRAD=0 switches it off, =1 takes it wherever the shape allows.

inline int winograd_forced() {
  const char *e = std::getenv("TSPLIT_CONV_WINOGRAD");
  return e ? (e[0] == '1' ? 1 : 0) : -1;
}

inline bool winograd_shape(const ConvGeo &g) {
  // channels are a dimension of the transform kernels' grids (both tensors' together in the filter gradient)
  return g.kH == 3 && g.kW == 3 && g.s == 1 && g.ph == 1 && g.pw == 1 && g.oH == g.H && g.oW == g.W &&
         static_cast<int64_t>(std::max(g.C, g.O)) * g.H * g.W < (1ll << 29) && g.C + g.O <= 32768;
}

// wide enough for the 36 GEMMs to outweigh the transforms (64 channels on both sides: with tiles as
// wide as the produced channels even the 64 -> 64 layer at 224 x 224 runs a quarter faster than on the
// direct kernels, forward and data gradient), little of the 4x4 tiling hanging over the plane's edge,
// and enough tiles to fill the chip
inline bool winograd_wide(const ConvGeo &g) {
  const int64_t covered = static_cast<int64_t>((g.H + 3) / 4) * ((g.W + 3) / 4) * 16;
  return std::min(g.C, g.O) >= 64 && covered * 3 <= static_cast<int64_t>(g.H) * g.W * 4 &&
         static_cast<int64_t>(g.imgs) * covered >= 16 * 1024;
}

// forward and data gradient: the channels summed over are the GEMMs' K
inline bool winograd_pays(const ConvGeo &g, int gathered) {
  const int forced = winograd_forced();
  if (!winograd_shape(g) || gathered % BK != 0 || forced == 0) return false;
  return forced == 1 || winograd_wide(g);
}

inline bool winograd_filter_grad_pays(const ConvGeo &g) {
  const int forced = winograd_forced();
  if (!winograd_shape(g) || forced == 0) return false;
  return forced == 1 || winograd_wide(g);
}

// ------------------------------------------------------------------ statistics of the output
// Folds the partial (sum, sum of squares) pairs the forward kernels leave, part[(k * C + c) * 2], k < used,
// in two steps with a fixed order: `slices` blocks per group of 32 channels each sum a contiguous range
// of k in double (lanes of a wave read neighbouring channels), then one thread per channel adds the
// slices in ascending order and writes dst[c * 2], dst[c * 2 + 1] as doubles.
constexpr int kFoldRows = 32;      // partials a block of 32 x kFoldRows threads reads at a time
__global__ __launch_bounds__(32 * kFoldRows) void conv_stats_fold_kernel(const float *__restrict__ part, int used, int C,
                                                                         double *__restrict__ tmp, int chunk) {
  __shared__ double sm[kFoldRows][32][2];
  const int cc = threadIdx.x & 31, kk = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + cc, slice = blockIdx.y;
  const int kend = min(used, (slice + 1) * chunk);
  double s = 0.0, q = 0.0;
  if (c < C)
    for (int k = slice * chunk + kk; k < kend; k += kFoldRows) {
      const float2 v = *reinterpret_cast<const float2 *>(part + (static_cast<int64_t>(k) * C + c) * 2);
      s += static_cast<double>(v.x);
      q += static_cast<double>(v.y);
    }
  sm[kk][cc][0] = s;
  sm[kk][cc][1] = q;
  __syncthreads();
  if (kk == 0 && c < C) {
#pragma unroll
    for (int j = 1; j < kFoldRows; ++j) {
      s += sm[j][cc][0];
      q += sm[j][cc][1];
    }
    tmp[(static_cast<int64_t>(slice) * C + c) * 2] = s;
    tmp[(static_cast<int64_t>(slice) * C + c) * 2 + 1] = q;
  }
}
__global__ __launch_bounds__(256) void conv_stats_final_kernel(const double *__restrict__ tmp, int slices, int C,
                                                               double *__restrict__ dst) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  double s = 0.0, q = 0.0;
  for (int j = 0; j < slices; ++j) {
    s += tmp[(static_cast<int64_t>(j) * C + c) * 2];
    q += tmp[(static_cast<int64_t>(j) * C + c) * 2 + 1];
  }
  dst[c * 2] = s;
  dst[c * 2 + 1] = q;
}

constexpr int kStatsSlices = 64;

// `stats_dst` (optional): per-channel (sum, sum of squares) of y as doubles, [O][2], for a BatchNorm that
// follows.  The Winograd routine and the tap-major kernels produce them in their epilogues; the other
// routes by a pass over y.
int conv_forward(const char *who, const DLArray *x, const DLArray *w, DLArray *y, int ph, int pw, int s,
                 DLStreamHandle sh, ProfilerHandle p, double *stats_dst = nullptr) {
  ConvGeo g;
  if (geo_from(who, x, w, y, ph, pw, s, g)) return -1;
  // Without a caller's array for the sums this call may leave a note for the BatchNorm that follows (see
  // common.h): it then keeps the notes of other ranges (earlier micro-tensors of the same tensor) and
  // drops those of the range it writes.
  const bool may_note = !stats_dst && conv_notes_enabled() && numel(y) > 0;
  hipStream_t st = may_note ? stream_keep_notes(sh) : stream_of(sh);
  if (may_note) conv_notes_drop_overlapping(y->data, static_cast<size_t>(numel(y)) * sizeof(float));
  ProfileScope ps(p, st, numel(x) + numel(w), numel(y), 0);
  StatsSink sink{nullptr, g.O, 0, 0};
  StatsSink *sk = nullptr;
  // routes whose epilogue sums the output per channel at (almost) no cost
  const bool sums_in_epilogue = numel(y) > 0 && !thin_fwd_ok(g) &&
      (winograd_pays(g, g.C) ||
       (g.C % BK == 0 && tap_kernel_images(g, static_cast<int64_t>(g.C) * g.H * g.W, numel(w)) > 0));
  double *note_dst = nullptr;
  // (a BatchNorm over at most 16384 values per channel holds them in registers and reads its input once
  // anyway, so an output that small gets no note: the fold launch behind the epilogue would be paid for
  // nothing, and networks of many small layers have hundreds of such calls a step.  For the same reason an
  // output below 32 MiB gets none: the pass over it that the note saves takes about as long as that launch)
  if (may_note && sums_in_epilogue && static_cast<int64_t>(g.imgs) * g.oH * g.oW > 16384 && g.O <= 4096 &&
      numel(y) >= (8ll << 20) && numel(y) < (1ll << 31)) {
    note_dst = conv_note_sums(st, g.O);
    stats_dst = note_dst;
  }
  if (stats_dst && sums_in_epilogue) {
    // one partial per 32 output positions at most, and a ragged group per run of images
    sink.capacity = static_cast<int>((static_cast<int64_t>(g.imgs) * g.oH * g.oW + 31) / 32) + g.imgs;
    const size_t bytes = static_cast<size_t>(sink.capacity) * g.O * 2 * sizeof(float) +
                         static_cast<size_t>(kStatsSlices) * g.O * 2 * sizeof(double);
    sink.part = static_cast<float *>(scratch_get(st, 7, bytes));
    TS_REQUIRE(sink.part, "%s: no scratch memory", who);
    sk = &sink;
  }
  if (numel(y) > 0) {
    if (thin_fwd_ok(g)) {
      const int rc = launch_conv_thin_fwd(g, cf(x), cf(w), mf(y), st);
      if (rc) return rc;
    } else if (winograd_pays(g, g.C)) {
      const int rc = conv_winograd_3x3(cf(x), cf(w), mf(y), g.imgs, g.C, g.O, g.H, g.W, false, st, sk);
      if (rc) return rc;
    } else if (g.C % BK == 0) {
      // a 1x1 filter [O][C] already is tap-major: used where it lies
      const float *wf = cf(w);
      const int64_t x_img = static_cast<int64_t>(g.C) * g.H * g.W, y_img = static_cast<int64_t>(g.O) * g.oH * g.oW;
      const int per = tap_kernel_images(g, x_img, numel(w));
      if (g.kH * g.kW != 1 || !aligned16(wf)) {
        float *relaid = static_cast<float *>(scratch_get(st, 3, static_cast<size_t>(numel(w)) * 4));
        TS_REQUIRE(relaid, "%s: no scratch memory", who);
        const int total = static_cast<int>(numel(w));
        hipLaunchKernelGGL(filter_tap_major_kernel, dim3((total + 255) / 256), dim3(256), 0, st, cf(w), relaid, g.O,
                           g.C, g.kH * g.kW, false);
        wf = relaid;
      }
      if (per) {
        const int rc = for_image_runs(g, per, [&](const ConvGeo &run, int64_t first) {
          const float *xr = cf(x) + first * x_img;
          float *yr = mf(y) + first * y_img;
          return short_tiles(g.O) ? launch_conv_tap<64, 256, 1, 4, false>(run, xr, wf, yr, st, nullptr, sk)
                           : launch_conv_tap<128, 128, 2, 2, false>(run, xr, wf, yr, st, nullptr, sk);
        });
        if (rc) return rc;
      } else if (g.O <= 64) {
        launch_fwd_tap_major<64, 256, 1, 4>(g, cf(x), wf, mf(y), st);
      } else {
        launch_fwd_tap_major<128, 128, 2, 2>(g, cf(x), wf, mf(y), st);
      }
    } else {
      const Tap *taps = tap_table(g.C, g.kH, g.kW, g.W, g.H * g.W, +1);
      TS_REQUIRE(taps, "%s: could not build the tap table", who);
      if (g.O <= 64)
        launch_fwd<64, 256, 1, 4>(g, cf(x), cf(w), mf(y), taps, st);
      else
        launch_fwd<128, 128, 2, 2>(g, cf(x), cf(w), mf(y), taps, st);
    }
  }
  if (stats_dst) {
    if (sk) {
      // the slices' sums live behind the partials in the same scratch buffer (8-byte aligned: the
      // partials are pairs of floats)
      double *tmp = reinterpret_cast<double *>(sink.part + static_cast<int64_t>(sink.capacity) * g.O * 2);
      // (one slice per 512 partials: the second kernel walks the slices one after the other)
      const int slices = std::max(1, std::min(kStatsSlices, (sink.used + 511) / 512));
      const int chunk = (sink.used + slices - 1) / slices;
      // one slice: its sums are the result (slice 0 of tmp has dst's layout), no second launch
      hipLaunchKernelGGL(conv_stats_fold_kernel, dim3((g.O + 31) / 32, slices), dim3(32 * kFoldRows), 0, st, sink.part, sink.used, g.O,
                         slices == 1 ? stats_dst : tmp, chunk);
      if (slices > 1)
        hipLaunchKernelGGL(conv_stats_final_kernel, dim3((g.O + 255) / 256), dim3(256), 0, st, tmp, slices, g.O, stats_dst);
    } else if (numel(y) > 0) {
      if (bn_channel_sums(y, stats_dst, st)) return -1;
    } else {
      hipLaunchKernelGGL(conv_stats_final_kernel, dim3((g.O + 255) / 256), dim3(256), 0, st,
                         static_cast<const double *>(nullptr), 0, g.O, stats_dst);
    }
  }
  if (note_dst)
    conv_note_add(ConvNote{st, static_cast<const char *>(y->data), static_cast<size_t>(numel(y)) * sizeof(float), g.imgs, g.O,
                           g.oH * g.oW, note_dst});
  return ps.finish();
}

int conv_bwd_data(const char *who, const DLArray *w, const DLArray *dy, DLArray *dx, int ph, int pw, int s,
                  DLStreamHandle sh, ProfilerHandle p) {
  ConvGeo g;
  if (geo_from(who, dx, w, dy, ph, pw, s, g)) return -1;
  hipStream_t st = stream_of(sh);
  ProfileScope ps(p, st, numel(dy) + numel(w), numel(dx), numel(w));
  if (numel(dx) > 0 && winograd_pays(g, g.O)) {
    const int rc = conv_winograd_3x3(cf(dy), cf(w), mf(dx), g.imgs, g.O, g.C, g.H, g.W, true, st);
    if (rc) return rc;
  } else if (numel(dx) > 0) {
    float *wt = static_cast<float *>(scratch_get(st, 3, static_cast<size_t>(numel(w)) * 4));
    TS_REQUIRE(wt, "%s: no scratch memory", who);
    const int total = static_cast<int>(numel(w));
    const int64_t dy_img = static_cast<int64_t>(g.O) * g.oH * g.oW, dx_img = static_cast<int64_t>(g.C) * g.H * g.W;
    const int per = tap_kernel_images(g, dy_img, numel(w));
    if (g.s == 1 && g.O % BK == 0) {
      const bool raw = per && raw_filter_pays(g);
      if (!raw)
        hipLaunchKernelGGL(filter_tap_major_kernel, dim3((total + 255) / 256), dim3(256), 0, st, cf(w), wt, g.O, g.C,
                           g.kH * g.kW, true);
      if (per) {
        const int rc = for_image_runs(g, per, [&](const ConvGeo &run, int64_t first) {
          const float *dyr = cf(dy) + first * dy_img;
          float *dxr = mf(dx) + first * dx_img;
          if (raw)
            return short_tiles(g.C) ? launch_conv_tap<64, 256, 1, 4, true, true>(run, dyr, cf(w), dxr, st)
                             : launch_conv_tap<128, 128, 2, 2, true, true>(run, dyr, cf(w), dxr, st);
          return short_tiles(g.C) ? launch_conv_tap<64, 256, 1, 4, true>(run, dyr, wt, dxr, st)
                           : launch_conv_tap<128, 128, 2, 2, true>(run, dyr, wt, dxr, st);
        });
        if (rc) return rc;
      } else if (g.C <= 64) {
        launch_bwd_data_tap_major<64, 256, 1, 4>(g, wt, cf(dy), mf(dx), st);
      } else {
        launch_bwd_data_tap_major<128, 128, 2, 2>(g, wt, cf(dy), mf(dx), st);
      }
    } else {
      if (g.s > 1) {
        // the sub-filters of all phases together hold every filter element once
        int rc;
        if (g.O % BK == 0 && per)
          rc = for_image_runs(g, per, [&](const ConvGeo &run, int64_t first) {
            return g.C <= 64 ? launch_bwd_data_phases_tap<64, 256, 1, 4>(run, cf(w), cf(dy) + first * dy_img,
                                                                        mf(dx) + first * dx_img, wt, st)
                             : launch_bwd_data_phases_tap<128, 128, 2, 2>(run, cf(w), cf(dy) + first * dy_img,
                                                                          mf(dx) + first * dx_img, wt, st);
          });
        else
          rc = g.C <= 64 ? launch_bwd_data_phases<64, 256, 1, 4>(g, cf(w), cf(dy), mf(dx), wt, st)
                         : launch_bwd_data_phases<128, 128, 2, 2>(g, cf(w), cf(dy), mf(dx), wt, st);
        if (rc) return rc;
      } else {
        // taps index dy: off = o*oH*oW (the spatial part is recomputed because of the stride test)
        const Tap *taps = tap_table(g.O, g.kH, g.kW, 0, g.oH * g.oW, 0);
        TS_REQUIRE(taps, "%s: could not build the tap table", who);
        hipLaunchKernelGGL(filter_oc_swap_kernel, dim3((total + 255) / 256), dim3(256), 0, st, cf(w), wt, g.O, g.C,
                           g.kH * g.kW);
        if (g.C <= 64)
          launch_bwd_data<64, 256, 1, 4>(g, wt, cf(dy), mf(dx), taps, st);
        else
          launch_bwd_data<128, 128, 2, 2>(g, wt, cf(dy), mf(dx), taps, st);
      }
    }
  }
  return ps.finish();
}

int conv_bwd_filter(const char *who, const DLArray *x, const DLArray *dy, DLArray *dw, int ph, int pw, int s,
                    DLStreamHandle sh, ProfilerHandle p) {
  ConvGeo g;
  if (geo_from(who, x, dw, dy, ph, pw, s, g)) return -1;
  hipStream_t st = stream_of(sh);
  int64_t ws = 0;
  ProfileScope ps(p, st, numel(x) + numel(dy), numel(dw), 0);
  int rc = 0;
  if (numel(dw) > 0 && (numel(x) == 0 || numel(dy) == 0)) {
    // a sum over no positions (an empty batch: the last of more micro-tensors than there are images)
    const int64_t n = numel(dw);
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, mf(dw), n);
  } else if (numel(dw) > 0) {
    if (wgrad_narrow_ok(g)) {
      rc = launch_wgrad_narrow(g, cf(x), cf(dy), mf(dw), st, &ws);
    } else if (winograd_filter_grad_pays(g)) {
      rc = conv_winograd_3x3_filter_grad(cf(x), cf(dy), mf(dw), g.imgs, g.C, g.O, g.H, g.W, st);
    } else if (wgrad_tap_ok(g)) {
      if (short_tiles(g.O))
        rc = launch_wgrad_tap<64, 256, 1, 4>(g, cf(x), cf(dy), mf(dw), st, &ws);
      else
        rc = launch_wgrad_tap<128, 128, 2, 2>(g, cf(x), cf(dy), mf(dw), st, &ws);
    } else if (g.C % BK == 0) {
      if (g.O <= 64)
        rc = launch_bwd_filter_tap_major<64, 256, 1, 4>(g, cf(x), cf(dy), mf(dw), st, &ws);
      else
        rc = launch_bwd_filter_tap_major<128, 128, 2, 2>(g, cf(x), cf(dy), mf(dw), st, &ws);
    } else {
      const Tap *taps = tap_table(g.C, g.kH, g.kW, g.W, g.H * g.W, +1);
      TS_REQUIRE(taps, "%s: could not build the tap table", who);
      if (g.O <= 64)
        rc = launch_bwd_filter<64, 256, 1, 4>(g, cf(x), cf(dy), mf(dw), taps, st, &ws);
      else
        rc = launch_bwd_filter<128, 128, 2, 2>(g, cf(x), cf(dy), mf(dw), taps, st, &ws);
    }
  }
  if (p) p->workspace_memory = mib(ws);
  if (rc) return rc;
  return ps.finish();
}

}  // namespace

}  // namespace tsplit

using namespace tsplit;

extern "C" {

int TSplit_ConvTakesWinograd(int images, int in_channels, int out_channels, int height, int width, int kernel_h,
                             int kernel_w, int pad_h, int pad_w, int stride, int pass) {
  if (images <= 0 || in_channels <= 0 || out_channels <= 0 || height <= 0 || width <= 0 || stride <= 0) return 0;
  ConvGeo g{images, in_channels, height, width, out_channels, kernel_h, kernel_w, pad_h, pad_w, stride,
            (height + 2 * pad_h - kernel_h) / stride + 1, (width + 2 * pad_w - kernel_w) / stride + 1};
  if (pass == 2) return winograd_filter_grad_pays(g) && !wgrad_narrow_ok(g);
  return winograd_pays(g, pass == 1 ? out_channels : in_channels);
}

int CuDNN_DLGpuConv2d(const DLArrayHandle input_x, const DLArrayHandle input_f, DLArrayHandle output,
                      const int padding, const int padding2, const int stride, DLStreamHandle stream_handle,
                      ProfilerHandle p) {
  return conv_forward("CuDNN_DLGpuConv2d", input_x, input_f, output, padding, padding2, stride, stream_handle, p);
}

// Convolution that also leaves the per-channel sum and sum of squares of its output, as doubles, in row
// `slot` of `stats` (float32 storage viewed as [slots][C][2] doubles): the statistics pass of a BatchNorm
// that follows (TSplit_BatchNormFromStats) then need not read the output again.
int TSplit_Conv2dBatchNormStats(const DLArrayHandle input_x, const DLArrayHandle input_f, DLArrayHandle output,
                                const int padding, const int padding2, const int stride, DLArrayHandle stats,
                                int slot, DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input_x && input_f && output && stats, "Conv2dBatchNormStats: NULL array");
  TS_REQUIRE(input_f->ndim == 4, "Conv2dBatchNormStats: filter must be 4-D");
  const int64_t C = input_f->shape[0];
  TS_REQUIRE(slot >= 0 && numel(stats) >= (static_cast<int64_t>(slot) + 1) * C * 4,
             "Conv2dBatchNormStats: stats must hold (slot + 1) * out_channels * 4 floats");
  TS_REQUIRE((reinterpret_cast<uintptr_t>(stats->data) & 7) == 0, "Conv2dBatchNormStats: stats must be 8-byte aligned");
  double *dst = static_cast<double *>(stats->data) + static_cast<int64_t>(slot) * C * 2;
  return conv_forward("Conv2dBatchNormStats", input_x, input_f, output, padding, padding2, stride, stream_handle, p, dst);
}

int CuDNN_DLGpuConv2d_Gradient_of_Filter(const DLArrayHandle input_x, const DLArrayHandle gradient_y,
                                         DLArrayHandle gradient_f, const int padding, const int padding2,
                                         const int stride, DLStreamHandle stream_handle, ProfilerHandle p) {
  return conv_bwd_filter("CuDNN_DLGpuConv2d_Gradient_of_Filter", input_x, gradient_y, gradient_f, padding, padding2,
                         stride, stream_handle, p);
}

int CuDNN_DLGpuConv2d_Gradient_of_Data(const DLArrayHandle input_f, const DLArrayHandle gradient_y,
                                       DLArrayHandle gradient_x, const int padding, const int padding2,
                                       const int stride, DLStreamHandle stream_handle, ProfilerHandle p) {
  return conv_bwd_data("CuDNN_DLGpuConv2d_Gradient_of_Data", input_f, gradient_y, gradient_x, padding, padding2,
                       stride, stream_handle, p);
}

// The plain symbols take one padding int and caller-provided im2col workspaces
// (src/ops/Conv2d.cu:52,172,241).  The workspaces are not needed and are left untouched.
int DLGpuConv2d(const DLArrayHandle input_x, const DLArrayHandle input_f, DLArrayHandle output,
                DLArrayHandle workspace_arr, const int padding, const int stride, DLStreamHandle stream_handle,
                ProfilerHandle p) {
  (void)workspace_arr;
  return conv_forward("DLGpuConv2d", input_x, input_f, output, padding, padding, stride, stream_handle, p);
}

int DLGpuConv2d_Gradient_of_Data(const DLArrayHandle input_f, const DLArrayHandle gradient_y,
                                 DLArrayHandle gradient_x, DLArrayHandle workspace_im2col, const int padding,
                                 const int stride, DLStreamHandle stream_handle, ProfilerHandle p) {
  (void)workspace_im2col;
  return conv_bwd_data("DLGpuConv2d_Gradient_of_Data", input_f, gradient_y, gradient_x, padding, padding, stride,
                       stream_handle, p);
}

int DLGpuConv2d_Gradient_of_Filter(const DLArrayHandle input_x, const DLArrayHandle gradient_y,
                                   DLArrayHandle gradient_f, DLArrayHandle workspace_im2col,
                                   DLArrayHandle workspace_batch_filter, const int padding, const int stride,
                                   DLStreamHandle stream_handle, ProfilerHandle p) {
  (void)workspace_im2col;
  (void)workspace_batch_filter;
  return conv_bwd_filter("DLGpuConv2d_Gradient_of_Filter", input_x, gradient_y, gradient_f, padding, padding, stride,
                         stream_handle, p);
}

}  // extern "C"
