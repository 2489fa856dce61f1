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
  int tm, tn;       // tiles of BM rows / BN columns
};

// Persistent form: the grid is one resident round of blocks (blocks_per_cu on each CU) and every block
// walks its own list of tiles.  A tile's result leaves through LDS as 16-byte words, and the loads of
// the NEXT tile's first k-step are issued before those stores: the memory counter of this architecture
// counts loads and stores in issue order, so waiting for these loads does not wait for the stores, and
// the block multiplies its next tile while the previous one is still on its way to memory.  (A block
// that ends after its one tile holds its slot until the last store is acknowledged.)  The stores are
// marked non-temporal: M is read next by another kernel, after the whole of it has been written.
// Summation order is that of the one-tile-per-block engine: the results are the same bits.
// Tiles are 128 x 128 (2 x 2 waves; four resident blocks per compute unit: registers and 4 x 40 KB of LDS
// allow exactly four) or, for layers that produce at most 64 channels, 64 x 256 (1 x 4 waves, so that no
// wave idles on rows that do not exist; 44 KB of LDS, three blocks).
template <int BM, int BN>
constexpr int gemm_blocks_per_cu() {
  return BM == 128 ? 4 : 3;
}
template <int BM, int BN>
static __global__ __launch_bounds__(kThreads, (gemm_blocks_per_cu<BM, BN>())) void wino_gemm_kernel(Problem p, int total) {
  static_assert((BM == 128 && BN == 128) || (BM == 64 && BN == 256), "each of the 4 waves owns a 64x64 sub-tile");
  constexpr int WN = BN / 64;
  using ALoader = KContigBufLoader<BM>;
  using BLoader = MnContigBufLoader<BN>;
  using ALds = typename ALoader::Lds;
  using BLds = typename BLoader::Lds;
  constexpr int kStage = ALds::kFloats + BLds::kFloats;
  __shared__ __attribute__((aligned(16))) float lds[2 * kStage];
  constexpr int kPitch = 64 + 4;
  static_assert(4 * 32 * kPitch <= 2 * kStage, "staging areas fit the operand stages");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WN) * 64, wn0 = (wave % WN) * 64;
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
    m0 = (rem - tile_n * p.tm) * BM;
    n0 = tile_n * BN;
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

// ---------------------------------------------------------------- filter-gradient GEMMs of narrow layers
// dU[xi] (rows x cols) = Y[xi] (rows x depth) V[xi]^T (cols x depth), both operands depth-contiguous, cut along
// the depth (the tiles of the layer) into ranges; block group z = range * 36 + xi writes its partial sum
// to out + z * rows * cols.  With 64 output or input channels a 128 x 128 block tile leaves two or three
// of the four waves without a sub-tile.  Here the block tile is TM x TN (64 or 128 each, not both 128)
// and the waves that have no sub-tile of their own share the depth instead: the 4 / (TM/64 * TN/64) = KG
// waves on one 64 x 64 sub-tile each take every KG-th 16-wide k-step of a 16*KG-wide chunk, and their
// accumulators are added through LDS at the end, in a fixed order.  A chunk row is 64*KG bytes, so a
// row's loads cover whole 128-byte lines, and the LDS rows (16*KG + 4 floats) are free of bank conflicts
// for both the 16-byte stores and the 16-byte fragment reads.  One LDS stage; the next chunk waits in
// registers while the current one is multiplied.
struct GradProblem {
  const float *Y;   // [36][rows][ld]
  const float *V;   // [36][cols][ld]
  float *out;       // [ranges * 36][rows][cols]
  int rows, cols, ld;
  int kchunk;       // depth per range, a multiple of 64
  int tm, tn;
};

template <int TM, int TN>
static __global__ __launch_bounds__(kThreads, 3) void wino_grad_gemm_narrow_kernel(GradProblem p, TileGrid tg) {
  constexpr int SUB = (TM / 64) * (TN / 64);   // 64 x 64 sub-tiles of the block tile
  constexpr int KG = 4 / SUB;                  // waves per sub-tile
  static_assert(SUB == 1 || SUB == 2, "narrow tiles only: 64x64, 128x64, 64x128");
  constexpr int CH = BK * KG;                  // chunk depth
  constexpr int STRIDE = CH + 4;               // LDS row pitch in floats
  constexpr int LPR = CH / 4;                  // lanes (16-byte words) per row
  constexpr int RPP = kThreads / LPR;          // rows per pass
  constexpr int PA = TM / RPP, PB = TN / RPP;  // passes per operand
  constexpr int kOperands = (TM + TN) * STRIDE;
  constexpr int kReduce = (KG / 2) * SUB * 64 * 64;   // accumulators parked in one round of the final sum
  constexpr int kLds = kOperands > kReduce ? kOperands : kReduce;
  __shared__ __attribute__((aligned(16))) float lds[kLds];

  int z, tile_m, tile_n;
  if (!block_tile(tg, z, tile_m, tile_n)) return;
  const int range = z / kXi, xi = z - range * kXi;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = wave % SUB, g = wave / SUB;            // sub-tile and k-group of this wave
  const int wm0 = TM == 128 ? 64 * sub : 0, wn0 = TN == 128 ? 64 * sub : 0;
  const int m0 = tile_m * TM, n0 = tile_n * TN;
  const int kbegin = range * p.kchunk, kend = min(p.ld, kbegin + p.kchunk);

  // loaders: thread -> (row tid / LPR + RPP * pass, word tid % LPR); rows beyond the matrix and words
  // beyond the range read as zeros through an out-of-range offset
  const int quad = tid % LPR, prow = tid / LPR;
  const float *abase = p.Y + static_cast<int64_t>(xi) * p.rows * p.ld + static_cast<int64_t>(m0) * p.ld;
  const float *bbase = p.V + static_cast<int64_t>(xi) * p.cols * p.ld + static_cast<int64_t>(n0) * p.ld;
  const int arows = min(TM, p.rows - m0), brows = min(TN, p.cols - n0);
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(abase), 0, static_cast<int>(static_cast<int64_t>(arows) * p.ld * 4), kBufFlags);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(bbase), 0, static_cast<int>(static_cast<int64_t>(brows) * p.ld * 4), kBufFlags);
  unsigned a_voff[PA], b_voff[PB];
#pragma unroll
  for (int s = 0; s < PA; ++s) {
    const int row = prow + RPP * s;
    a_voff[s] = row < arows ? (static_cast<unsigned>(row) * static_cast<unsigned>(p.ld) + 4u * quad) * 4u : kOobOffset;
  }
#pragma unroll
  for (int s = 0; s < PB; ++s) {
    const int row = prow + RPP * s;
    b_voff[s] = row < brows ? (static_cast<unsigned>(row) * static_cast<unsigned>(p.ld) + 4u * quad) * 4u : kOobOffset;
  }
  u32x4 areg[PA], breg[PB];
  auto load = [&](int k0) {
    // ld is a multiple of 4 and so is every word's position: a word lies wholly inside the range or outside
    const bool in = k0 + 4 * quad < kend;
#pragma unroll
    for (int s = 0; s < PA; ++s) areg[s] = __builtin_amdgcn_raw_buffer_load_b128(ra, in ? a_voff[s] : kOobOffset, k0 * 4, 0);
#pragma unroll
    for (int s = 0; s < PB; ++s) breg[s] = __builtin_amdgcn_raw_buffer_load_b128(rb, in ? b_voff[s] : kOobOffset, k0 * 4, 0);
  };
  float *lds_a = lds, *lds_b = lds + TM * STRIDE;
  auto store = [&]() {
#pragma unroll
    for (int s = 0; s < PA; ++s) *reinterpret_cast<u32x4 *>(lds_a + (prow + RPP * s) * STRIDE + 4 * quad) = areg[s];
#pragma unroll
    for (int s = 0; s < PB; ++s) *reinterpret_cast<u32x4 *>(lds_b + (prow + RPP * s) * STRIDE + 4 * quad) = breg[s];
  };

  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  if (kbegin < kend) {
    load(kbegin);
    store();
  }
  __syncthreads();
  const bool live = m0 + wm0 < p.rows && n0 + wn0 < p.cols;
  for (int k0 = kbegin; k0 < kend; k0 += CH) {
    const bool more = k0 + CH < kend;
    if (more) load(k0 + CH);
    if (live) {
      // this wave's 16 of the chunk's k values: lanes 0-31 supply k = 8j + i, lanes 32-63 k = 8j + 4 + i
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        float fa[2][4], fb[2][4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const float4 qa = *reinterpret_cast<const float4 *>(lds_a + (wm0 + 32 * i + (lane & 31)) * STRIDE + BK * g + 8 * j +
                                                              4 * (lane >> 5));
          const float4 qb = *reinterpret_cast<const float4 *>(lds_b + (wn0 + 32 * i + (lane & 31)) * STRIDE + BK * g + 8 * j +
                                                              4 * (lane >> 5));
          fa[i][0] = qa.x, fa[i][1] = qa.y, fa[i][2] = qa.z, fa[i][3] = qa.w;
          fb[i][0] = qb.x, fb[i][1] = qb.y, fb[i][2] = qb.z, fb[i][3] = qb.w;
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
    __syncthreads();   // every wave has read the chunk
    if (more) {
      store();
      __syncthreads();
    }
  }

  // sum over the k-groups: the upper half parks its accumulators ([register][lane] per wave), the lower
  // half adds them; then once more until group 0 holds the sum.  The loop above ended with a barrier.
#pragma unroll
  for (int half = KG / 2; half >= 1; half /= 2) {
    float *park = lds + ((g - half) * SUB + sub) * (64 * 64) + lane;
    if (g >= half && g < 2 * half) {
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
          for (int e = 0; e < 16; ++e) park[((mi * 2 + ni) * 16 + e) * 64] = acc[mi][ni][e];
    }
    __syncthreads();
    if (g < half) {
      const float *from = lds + (g * SUB + sub) * (64 * 64) + lane;
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[mi][ni][e] += from[((mi * 2 + ni) * 16 + e) * 64];
    }
    __syncthreads();
  }
  if (g != 0 || !live) return;
  float *__restrict__ o = p.out + static_cast<int64_t>(z) * p.rows * p.cols;
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int n = n0 + wn0 + 32 * ni + (lane & 31);
    if (n >= p.cols) continue;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
      const int mb = m0 + wm0 + 32 * mi + 4 * (lane >> 5);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = mb + 8 * (e >> 2) + (e & 3);
        if (m < p.rows) o[static_cast<int64_t>(m) * p.cols + n] = acc[mi][ni][e];
      }
    }
  }
}

// ---------------------------------------------------------------- filter-gradient GEMMs, 128 x 128 tiles
// Same product and output layout as above.  The unit of work is one tile of one (range, xi) pair; the
// grid is NB resident blocks on every compute unit and block L (in the XCD-aware order) takes units
// L, L + G, L + 2G, ...: every block gets the same number of equal units when the host chooses the number
// of ranges so that the units fill a whole number of rounds, and the blocks of one XCD work at any time
// on the tiles of the same few (range, xi) pairs, which read the same rows of Y and V through that XCD's
// L2.  (With one tile per block, a launch of 576 or 864 blocks left a quarter of the matrix pipes idle
// in its last round, and a launch cut finer paid a prologue and a drained pipeline per block.)  As in the
// forward kernel, the next unit's first loads are issued before the finished unit's stores.  The LDS
// request is padded so that exactly NB blocks fit a compute unit: the dispatcher then cannot stack the
// grid unevenly.
template <int NB>
static __global__ __launch_bounds__(kThreads, NB) void wino_grad_gemm_kernel(GradProblem p, int units) {
  using Loader = KContigBufLoader<128>;
  using Lds = typename Loader::Lds;
  constexpr int kStage = 2 * Lds::kFloats;
  constexpr int kFit = (160 * 1024 / (NB + 1)) / 4 + 64;   // more than an (NB+1)-th of the LDS
  constexpr int kLds = 2 * kStage > kFit ? 2 * kStage : kFit;
  __shared__ __attribute__((aligned(16))) float lds[kLds];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
  const int per_group = p.tm * p.tn;
  const int G = gridDim.x;
  int u = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
  if (u >= units) return;

  int z, m0, n0, kbegin, kend;
  Loader la, lb;
  auto start = [&](int unit) {
    z = unit / per_group;
    const int tile = unit - z * per_group;
    const int tile_n = tile / p.tm;
    m0 = (tile - tile_n * p.tm) * 128;
    n0 = tile_n * 128;
    const int range = z / kXi, xi = z - range * kXi;
    kbegin = range * p.kchunk;
    kend = min(p.ld, kbegin + p.kchunk);
    typename Loader::Params ap{p.Y + static_cast<int64_t>(xi) * p.rows * p.ld, p.ld, p.rows, p.ld};
    typename Loader::Params bp{p.V + static_cast<int64_t>(xi) * p.cols * p.ld, p.ld, p.cols, p.ld};
    la.init(ap, m0, tid);
    lb.init(bp, n0, tid);
    la.load(kbegin, kend);
    lb.load(kbegin, kend);
  };
  start(u);

  for (;;) {
    acc16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    // the last k-step of the previous unit ended with a barrier: stage 0 is free
    la.store(lds, tid);
    lb.store(lds + Lds::kFloats, tid);
    __syncthreads();

    const bool live = m0 + wm0 < p.rows && n0 + wn0 < p.cols;
    int stage = 0;
    for (int k0 = kbegin; k0 < kend; k0 += BK) {
      const bool more = k0 + BK < kend;
      if (more) {
        la.load(k0 + BK, kend);
        lb.load(k0 + BK, kend);
      }
      if (live) {
        const float *sa = lds + stage * kStage, *sb = sa + Lds::kFloats;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float fa[2][4], fb[2][4];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            Lds::frag(sa, wm0 + 32 * i, j, lane, fa[i]);
            Lds::frag(sb, wn0 + 32 * i, j, lane, fb[i]);
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
        lb.store(sa + Lds::kFloats, tid);
      }
      __syncthreads();
      stage ^= 1;
    }

    float *__restrict__ o = p.out + static_cast<int64_t>(z) * p.rows * p.cols;
    const int om0 = m0 + wm0, on0 = n0 + wn0;
    u += G;
    const bool again = u < units;
    if (again) start(u);
    if (live) {
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const int n = on0 + 32 * ni + (lane & 31);
        if (n >= p.cols) continue;
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) {
          const int mb = om0 + 32 * mi + 4 * (lane >> 5);
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int m = mb + 8 * (e >> 2) + (e & 3);
            if (m < p.rows) o[static_cast<int64_t>(m) * p.cols + n] = acc[mi][ni][e];
          }
        }
      }
    }
    if (!again) break;
  }
}

// One resident round of blocks on `cus` compute units (with four per unit the 128 x 128 kernel ran 3 %
// faster over the launches of a VGG-16 step than with three), never more blocks than tiles.
template <int BM, int BN>
inline void launch_tiles(Problem p, hipStream_t st, int cus) {
  p.tm = (p.rows + BM - 1) / BM;
  p.tn = (p.ld + BN - 1) / BN;
  const int total = p.tm * p.tn * kXi;
  int grid = cus * gemm_blocks_per_cu<BM, BN>() / 8 * 8;
  if (grid > (total + 7) / 8 * 8) grid = (total + 7) / 8 * 8;
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL((wino_gemm_kernel<BM, BN>), dim3(grid), dim3(kThreads), 0, st, p, total);
}
inline void launch(const Problem &p, hipStream_t st, int cus) {
  if (p.rows <= 64)
    launch_tiles<64, 256>(p, st, cus);
  else
    launch_tiles<128, 128>(p, st, cus);
}

}  // namespace wg
}  // namespace tsplit
