// The 36 GEMMs of the Winograd routine, M[xi] (rows x cols) = U[xi] (rows x depth) V[xi] (depth x cols),
// on the fp32 MFMA tile engine of mfma_gemm.h: U is depth-contiguous, V and M are column-contiguous.
//
// Their depth is the layer's channel count (64 ... 512: 4 ... 32 k-steps per 128x128 tile), far less
// than in the direct convolutions, and they write as many bytes as they read, so what happens around a
// tile's k-loop weighs more: with one tile per block, a block holds its slot on the CU until its 64 KB
// of stores are acknowledged, and the kernel ran at the speed of "multiply, then write" (a version that
// computed the tiles and stored nothing was 15 - 40 % faster, most for the shallow layers).
#pragma once
#include "mfma_gemm.h"

namespace tsplit {
namespace wg {
using namespace mg;

constexpr int kXi = 36;

struct Problem {
  const float *U;   // [36][rows][depth]
  const float *V;   // [36][depth][ld]
  float *M;         // [36][rows][ld]
  int rows, depth, ld;
  int tm, tn;       // tiles of 128 rows / 128 columns
};

// Persistent form: the grid is one resident round of blocks (blocks_per_cu on each CU) and every block
// walks its own list of tiles.  A tile's result leaves through LDS as 16-byte words, and the loads of
// the NEXT tile's first k-step are issued before those stores: the memory counter of this architecture
// counts loads and stores in issue order, so waiting for these loads does not wait for the stores, and
// the block multiplies its next tile while the previous one is still on its way to memory.  (A block
// that ends after its one tile holds its slot until the last store is acknowledged.)  The stores are
// marked non-temporal: M is read next by another kernel, after the whole of it has been written.
// Summation order is that of the one-tile-per-block engine: the results are the same bits.
static __global__ __launch_bounds__(kThreads, 4) void wino_gemm_kernel(Problem p, int total) {
  using ALoader = KContigBufLoader<128>;
  using BLoader = MnContigBufLoader<128>;
  using ALds = typename ALoader::Lds;
  using BLds = typename BLoader::Lds;
  constexpr int kStage = ALds::kFloats + BLds::kFloats;
  __shared__ __attribute__((aligned(16))) float lds[2 * kStage];
  constexpr int kPitch = 64 + 4;
  static_assert(4 * 32 * kPitch <= 2 * kStage, "staging areas fit the operand stages");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
  const int M = p.rows, N = p.ld, K = p.depth;
  const int per_xi = p.tm * p.tn;
  // XCD-aware order: the dispatcher deals consecutive block ids to the 8 XCDs in turn, so XCD x owns
  // the x-th eighth of the logical order and its blocks walk it side by side
  const int per_xcd = (total + 7) / 8, local_blocks = gridDim.x >> 3;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int chunk_end = min(total, (xcd + 1) * per_xcd);
  int logical = xcd * per_xcd + local;
  if (logical >= chunk_end) return;

  auto locate = [&](int l, int &z, int &m0, int &n0) {
    z = l / per_xi;
    const int rem = l - z * per_xi;
    const int tile_n = rem / p.tm;
    m0 = (rem - tile_n * p.tm) * 128;
    n0 = tile_n * 128;
  };

  ALoader la;
  BLoader lb;
  int z, m0, n0;
  locate(logical, z, m0, n0);
  {
    typename ALoader::Params ap{p.U + static_cast<int64_t>(z) * M * K, K, M, K};
    typename BLoader::Params bp{p.V + static_cast<int64_t>(z) * K * N, N, N, K};
    la.init(ap, m0, tid);
    lb.init(bp, n0, tid);
    la.load(0, K);
    lb.load(0, K);
  }
  float *mine = lds + wave * (32 * kPitch);
  const int r4 = lane >> 4, c4 = (lane & 15) * 4;

  for (;;) {
    acc16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    __syncthreads();   // the staging areas of the previous tile's epilogue are the operand stages
    la.store(lds, tid);
    lb.store(lds + ALds::kFloats, tid);
    __syncthreads();

    const bool live = m0 + wm0 < M && n0 + wn0 < N;
    int stage = 0;
    for (int k0 = 0; k0 < K; k0 += BK) {
      const bool more = k0 + BK < K;
      if (more) {
        la.load(k0 + BK, K);
        lb.load(k0 + BK, K);
      }
      if (live) {
        const float *sa = lds + stage * kStage, *sb = sa + ALds::kFloats;
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
      }
      if (more) {
        float *sa = lds + (stage ^ 1) * kStage;
        la.store(sa, tid);
        lb.store(sa + ALds::kFloats, tid);
      }
      __syncthreads();
      stage ^= 1;
    }

    // this tile's place in M, then the next tile's first loads, then this tile's stores
    float *__restrict__ o = p.M + static_cast<int64_t>(z) * M * N;
    const int om0 = m0 + wm0, on = n0 + wn0 + c4;
    logical += local_blocks;
    const bool again = logical < chunk_end;
    if (again) {
      locate(logical, z, m0, n0);
      typename ALoader::Params ap{p.U + static_cast<int64_t>(z) * M * K, K, M, K};
      typename BLoader::Params bp{p.V + static_cast<int64_t>(z) * K * N, N, N, K};
      la.init(ap, m0, tid);
      lb.init(bp, n0, tid);
      la.load(0, K);
      lb.load(0, K);
    }
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          mine[(8 * (e >> 2) + 4 * (lane >> 5) + (e & 3)) * kPitch + 32 * ni + (lane & 31)] = acc[mi][ni][e];
      __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): a wave's own staging area needs no barrier
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int row = it * 4 + r4;
        const int m = om0 + 32 * mi + row;
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const f32x4 v = *reinterpret_cast<const f32x4 *>(mine + row * kPitch + c4);
        if (m < M && on < N) {   // N is a multiple of 4
          f32x4 *dst = reinterpret_cast<f32x4 *>(o + static_cast<int64_t>(m) * N + on);
          __builtin_nontemporal_store(v, dst);
        }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
    }
    if (!again) break;
  }
}

// One resident round of blocks: `blocks_per_cu` (what hipOccupancyMaxActiveBlocksPerMultiprocessor reports for
// the kernel) on each of `cus` compute units, never more blocks than tiles.
inline void launch(const Problem &p, hipStream_t st, int blocks_per_cu, int cus) {
  const int total = p.tm * p.tn * kXi;
  int grid = cus * blocks_per_cu / 8 * 8;
  if (grid > (total + 7) / 8 * 8) grid = (total + 7) / 8 * 8;
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(wino_gemm_kernel, dim3(grid), dim3(kThreads), 0, st, p, total);
}

}  // namespace wg
}  // namespace tsplit
