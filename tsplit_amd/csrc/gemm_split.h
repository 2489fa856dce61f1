// Row-major C = op(A) op(B) with split-bf16 products (opt-in, see wino_gemm_split.h for the method): 128 x 128
// tiles, 16 k values per step, split-K as in the fp32 engine.  The operands stay fp32 in memory; a loader
// reads them as fp32, splits them in registers and leaves three bf16 planes per operand in LDS, laid out
// plane[k / 8][index][k % 8] so that a lane's 8 consecutive k of one row or column are one 16-byte word.
#pragma once
#include "wino_gemm_split.h"

namespace tsplit {
namespace mg {

using wg::bf16x8;
using wg::kSplitPlane;
using wg::kSplitStage;
using wg::split8;
using wg::split_products;

// element (mn, k) at p[mn * ld + k]: a thread takes 8 consecutive k of one row as two 16-byte words, each of
// which must lie wholly inside or outside the k range (K and the range bounds are multiples of 4)
struct SplitKContigLoader {
  using Params = DenseParams;
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned voff;
  int row, half;
  float r[8];
  __device__ __forceinline__ void init(const Params &P, int mn0, int tid) {
    row = tid >> 1;
    half = tid & 1;
    const int rows_left = P.mn_total - mn0;
    const int64_t bytes = static_cast<int64_t>(rows_left) * P.ld * 4;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.p) + static_cast<int64_t>(mn0) * P.ld, 0,
                                             static_cast<int>(bytes < 0x7fffffffll ? bytes : 0x7fffffffll), kBufFlags);
    voff = row < rows_left ? (static_cast<unsigned>(row) * static_cast<unsigned>(P.ld) + 8u * half) * 4u : kOobOffset;
  }
  __device__ __forceinline__ void load(int k0, int kend) {
    const int k = k0 + 8 * half;
    const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(rsrc, k < kend ? voff : kOobOffset, k0 * 4, 0);
    const u32x4 hi = __builtin_amdgcn_raw_buffer_load_b128(rsrc, k + 4 < kend ? voff : kOobOffset, k0 * 4 + 16, 0);
    const unsigned w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = __uint_as_float(w[j]);
  }
  __device__ __forceinline__ void store(__bf16 *planes) const {
    u32x4 s[3];
    split8(r, s);
#pragma unroll
    for (int t = 0; t < 3; ++t) *reinterpret_cast<u32x4 *>(planes + t * kSplitPlane + (half * 128 + row) * 8) = s[t];
  }
};

// element (k, mn) at p[k * ld + mn]: a thread takes 8 rows of one column as eight 4-byte loads (256 contiguous
// bytes per wave each); rows at or beyond the range's end read as zeros
struct SplitMnContigLoader {
  using Params = DenseParams;
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned voff;
  int col, half, row_bytes;
  float r[8];
  __device__ __forceinline__ void init(const Params &P, int mn0, int tid) {
    col = tid & 127;
    half = __builtin_amdgcn_readfirstlane(tid >> 7);
    row_bytes = static_cast<int>(P.ld) * 4;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.p), 0,
                                             static_cast<int>(static_cast<int64_t>(P.k_total) * P.ld * 4), kBufFlags);
    voff = mn0 + col < P.mn_total ? static_cast<unsigned>(mn0 + col) * 4u : kOobOffset;
  }
  __device__ __forceinline__ void load(int k0, int kend) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = k0 + 8 * half + j;
      r[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, k < kend ? voff : kOobOffset, k * row_bytes, 0));
    }
  }
  __device__ __forceinline__ void store(__bf16 *planes) const {
    u32x4 s[3];
    split8(r, s);
#pragma unroll
    for (int t = 0; t < 3; ++t) *reinterpret_cast<u32x4 *>(planes + t * kSplitPlane + (half * 128 + col) * 8) = s[t];
  }
};

// split z covers k in [z * kchunk, (z + 1) * kchunk) and writes to out + z * z_stride; one tile per block
template <class ALoader, class BLoader>
__global__ __launch_bounds__(kThreads, 3) void mfma_gemm_split_kernel(typename ALoader::Params ap, typename BLoader::Params bp,
                                                                      float *__restrict__ out, int64_t z_stride, int M, int N,
                                                                      int K, int kchunk, TileGrid tg) {
  __shared__ __attribute__((aligned(16))) __bf16 lds_h[2 * kSplitStage];   // 48 KB
  int z, tile_m, tile_n;
  if (!block_tile(tg, z, tile_m, tile_n)) return;
  const int kbegin = z * kchunk, kend = min(K, kbegin + kchunk);
  const int m0 = tile_m * 128, n0 = tile_n * 128;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;

  ALoader la;
  BLoader lb;
  la.init(ap, m0, tid);
  lb.init(bp, n0, tid);
  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  if (kbegin < kend) {
    la.load(kbegin, kend);
    lb.load(kbegin, kend);
    la.store(lds_h);
    lb.store(lds_h + 3 * kSplitPlane);
  }
  __syncthreads();
  const bool live = m0 + wm0 < M && n0 + wn0 < N;
  const int frag = ((lane >> 5) * 128 + (lane & 31)) * 8;
  int stage = 0;
  for (int k0 = kbegin; k0 < kend; k0 += BK) {
    const bool more = k0 + BK < kend;
    if (more) {
      la.load(k0 + BK, kend);
      lb.load(k0 + BK, kend);
    }
    if (live) {
      const __bf16 *s = lds_h + stage * kSplitStage;
      bf16x8 fa[2][3], fb[2][3];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int t = 0; t < 3; ++t) {
          fa[i][t] = *reinterpret_cast<const bf16x8 *>(s + t * kSplitPlane + frag + (wm0 + 32 * i) * 8);
          fb[i][t] = *reinterpret_cast<const bf16x8 *>(s + (3 + t) * kSplitPlane + frag + (wn0 + 32 * i) * 8);
        }
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = split_products(fa[mi], fb[ni], acc[mi][ni]);
    }
    if (more) {
      __bf16 *next = lds_h + (stage ^ 1) * kSplitStage;
      la.store(next);
      lb.store(next + 3 * kSplitPlane);
    }
    __syncthreads();
    stage ^= 1;
  }
  if (!live) return;
  float *__restrict__ o = out + static_cast<int64_t>(z) * z_stride;
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int n = n0 + wn0 + 32 * ni + (lane & 31);
    if (n >= N) continue;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
      const int mb = m0 + wm0 + 32 * mi + 4 * (lane >> 5);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = mb + 8 * (e >> 2) + (e & 3);
        if (m < M) o[static_cast<int64_t>(m) * N + n] = acc[mi][ni][e];
      }
    }
  }
}

}  // namespace mg
}  // namespace tsplit
