// fp32 MFMA tile engine shared by MatMul and the three convolutions.
//
// D[M,N] = A[M,K] * B[K,N] with v_mfma_f32_32x32x2_f32.  A block of 256 threads (4 waves)
// owns a BM x BN tile; each wave owns a 64x64 sub-tile = 2x2 MFMA blocks (64 accumulator
// VGPRs), so one k-pair costs 2+2 operand registers for 4 MFMAs.  K advances in steps of
// BK = 16 through double-buffered LDS: the loads of step t+1 are issued before the MFMAs of
// step t and parked in registers, then written to the other LDS stage; one barrier per step.
//
// Each operand is staged in LDS in the orientation it has in memory, never transposed:
//   * "k-major"  [BK][MN+8]  for operands whose M/N index is contiguous in memory
//   * "mn-major" [MN][BK+4]  for operands whose K index is contiguous in memory
// This works because an MFMA only needs both operands to agree on WHICH k each lane
// supplies, not on the order: within a 16-wide step, lanes 0-31 supply k = 8j+i and lanes
// 32-63 supply k = 8j+4+i (j = 0,1; i = 0..3).  An mn-major operand then reads its four
// values with one 16-byte LDS read per lane; a k-major one with four 4-byte reads that are
// conflict-free because consecutive lanes touch consecutive addresses.
//
// Operand loaders (global -> registers -> LDS) are policy classes; the convolutions plug in
// gather loaders that compute im2col addresses on the fly.  The epilogue writes
// out[row_stride * m + colmap(n)], which covers row-major matrices, NCHW activations and the
// split-K partial buffers alike.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace tsplit {
namespace mg {

constexpr int BK = 16;
constexpr int kThreads = 256;
constexpr int kMnPad = 8;   // k-major rows: MN + 8 floats
constexpr int kKPad = 4;    // mn-major rows: BK + 4 floats

typedef float acc16 __attribute__((ext_vector_type(16)));

template <int MN>
struct KMajorLds {   // [BK][MN + 8]
  static constexpr int kStride = MN + kMnPad;
  static constexpr int kFloats = BK * kStride;
  // the 4 k-values (group j) this lane supplies for the 32-wide block starting at mn0
  static __device__ __forceinline__ void frag(const float *lds, int mn0, int j, int lane, float (&v)[4]) {
    const float *p = lds + (8 * j + 4 * (lane >> 5)) * kStride + mn0 + (lane & 31);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = p[i * kStride];
  }
};

template <int MN>
struct MnMajorLds {  // [MN][BK + 4]
  static constexpr int kStride = BK + kKPad;
  static constexpr int kFloats = MN * kStride;
  static __device__ __forceinline__ void frag(const float *lds, int mn0, int j, int lane, float (&v)[4]) {
    const float4 q = *reinterpret_cast<const float4 *>(lds + (mn0 + (lane & 31)) * kStride + 8 * j + 4 * (lane >> 5));
    v[0] = q.x;
    v[1] = q.y;
    v[2] = q.z;
    v[3] = q.w;
  }
};

// ------------------------------------------------------------------ dense-matrix loaders
// Operand whose K index is contiguous: element (mn, k) at p[mn * ld + k].
template <int MN>
struct KContigLoader {
  using Lds = MnMajorLds<MN>;
  struct Params {
    const float *p;
    int64_t ld;
    int mn_total;
    bool vec;   // ld % 4 == 0 and p 16-byte aligned
  };
  static constexpr int kPasses = MN / 64;   // 64 rows x 4 quads per pass
  float4 r[kPasses];
  const float *base[kPasses];
  bool row_ok[kPasses];
  int kq;
  bool vec;

  __device__ __forceinline__ void init(const Params &P, int mn0, int tid) {
    kq = tid & 3;
    vec = P.vec;
#pragma unroll
    for (int s = 0; s < kPasses; ++s) {
      const int row = mn0 + (tid >> 2) + 64 * s;
      row_ok[s] = row < P.mn_total;
      base[s] = P.p + static_cast<int64_t>(row_ok[s] ? row : 0) * P.ld;
    }
  }
  __device__ __forceinline__ void load(int k0, int kend) {
    const int k = k0 + 4 * kq;
#pragma unroll
    for (int s = 0; s < kPasses; ++s) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (row_ok[s]) {
        if (vec && k + 3 < kend) {
          v = *reinterpret_cast<const float4 *>(base[s] + k);
        } else {
          if (k < kend) v.x = base[s][k];
          if (k + 1 < kend) v.y = base[s][k + 1];
          if (k + 2 < kend) v.z = base[s][k + 2];
          if (k + 3 < kend) v.w = base[s][k + 3];
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

// Operand whose M/N index is contiguous: element (k, mn) at p[k * ld + mn].
template <int MN>
struct MnContigLoader {
  using Lds = KMajorLds<MN>;
  struct Params {
    const float *p;
    int64_t ld;
    int mn_total;
    bool vec;
  };
  static constexpr int kQuads = MN / 4;                 // 16-byte words per row
  static constexpr int kRowsPerPass = kThreads / kQuads;
  static constexpr int kPasses = BK / kRowsPerPass;
  float4 r[kPasses];
  const float *p;
  int64_t ld;
  int col, krow, ncols;   // first column of this thread's word, row within a pass, valid columns
  bool vec;

  __device__ __forceinline__ void init(const Params &P, int mn0, int tid) {
    p = P.p;
    ld = P.ld;
    vec = P.vec;
    col = mn0 + 4 * (tid % kQuads);
    krow = tid / kQuads;
    ncols = P.mn_total - col;   // <= 0: nothing valid
  }
  __device__ __forceinline__ void load(int k0, int kend) {
#pragma unroll
    for (int s = 0; s < kPasses; ++s) {
      const int k = k0 + krow + s * kRowsPerPass;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (k < kend && ncols > 0) {
        const float *q = p + static_cast<int64_t>(k) * ld + col;
        if (vec && ncols >= 4) {
          v = *reinterpret_cast<const float4 *>(q);
        } else {
          v.x = q[0];
          if (ncols > 1) v.y = q[1];
          if (ncols > 2) v.z = q[2];
          if (ncols > 3) v.w = q[3];
        }
      }
      r[s] = v;
    }
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int s = 0; s < kPasses; ++s)
      *reinterpret_cast<float4 *>(lds + (krow + s * kRowsPerPass) * Lds::kStride + 4 * (tid % kQuads)) = r[s];
  }
};

// ------------------------------------------------------------------ dense-matrix loaders on buffer loads
// The same two layouts read with raw buffer loads: a thread's byte offset is fixed when the tile
// starts and the k position of a step travels in the scalar offset, so a step costs no vector-ALU
// address arithmetic and no branch (vector-ALU instructions issued while the matrix pipe is
// saturated cost MFMA issue time).  Rows or columns outside the matrix get an offset beyond the
// buffer, for which the load returns 0; the buffer ends with the matrix, so the rows of a ragged
// last k-step read as zeros by themselves.  For matrices below 2 GiB (32-bit offsets); 16-byte
// loads need only 4-byte alignment here, so any leading dimension takes the wide path.
constexpr int kBufFlags = 0x00020000;           // raw buffer, 32-bit untyped data (gfx9 family)
constexpr unsigned kOobOffset = 0x80000000u;    // beyond any buffer these paths accept (< 2 GiB)
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct DenseParams {
  const float *p;
  int64_t ld;
  int mn_total;
  int k_total;
};

inline bool dense_fits_buffer(int64_t rows, int64_t ld, int tile_rows) {
  return rows * ld * 4 < (1ll << 31) && tile_rows * ld * 4 < (1ll << 31);
}

template <int MN>
struct KContigBufLoader {   // element (mn, k) at p[mn * ld + k]
  using Lds = MnMajorLds<MN>;
  using Params = DenseParams;
  static constexpr int kPasses = MN / 64;   // 64 rows x 4 quads per pass
  u32x4 r[kPasses];
  unsigned voff[kPasses];
  __amdgpu_buffer_rsrc_t rsrc;
  int kq;

  __device__ __forceinline__ void init(const Params &P, int mn0, int tid) {
    kq = tid & 3;
    const int rows_left = P.mn_total - mn0;
    const int64_t bytes = static_cast<int64_t>(rows_left) * P.ld * 4;
    // offsets count from the tile's first row
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.p) + static_cast<int64_t>(mn0) * P.ld, 0,
                                             static_cast<int>(bytes < 0x7fffffffll ? bytes : 0x7fffffffll), kBufFlags);
#pragma unroll
    for (int s = 0; s < kPasses; ++s) {
      const int row = (tid >> 2) + 64 * s;
      voff[s] = row < rows_left ? (static_cast<unsigned>(row) * static_cast<unsigned>(P.ld) + 4u * kq) * 4u : kOobOffset;
    }
  }
  __device__ __forceinline__ void load(int k0, int kend) {
    if (k0 + BK <= kend) {
#pragma unroll
      for (int s = 0; s < kPasses; ++s) r[s] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff[s], k0 * 4, 0);
    } else {
      // ragged last step: a word may run past the end of its row into the next one
      const int cnt = kend - (k0 + 4 * kq);
#pragma unroll
      for (int s = 0; s < kPasses; ++s) {
        u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, cnt > 0 ? voff[s] : kOobOffset, k0 * 4, 0);
        v.y = cnt >= 2 ? v.y : 0u;
        v.z = cnt >= 3 ? v.z : 0u;
        v.w = cnt >= 4 ? v.w : 0u;
        r[s] = v;
      }
    }
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int s = 0; s < kPasses; ++s)
      *reinterpret_cast<u32x4 *>(lds + ((tid >> 2) + 64 * s) * Lds::kStride + 4 * kq) = r[s];
  }
};

template <int MN>
struct MnContigBufLoader {   // element (k, mn) at p[k * ld + mn]
  using Lds = KMajorLds<MN>;
  using Params = DenseParams;
  static constexpr int kQuads = MN / 4;                 // 16-byte words per row
  static constexpr int kRowsPerPass = kThreads / kQuads;
  static constexpr int kPasses = BK / kRowsPerPass;
  u32x4 r[kPasses];
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned voff;
  int ncols, krow, row_bytes;   // valid columns of this thread's word (>= 4: all), row within a pass

  __device__ __forceinline__ void init(const Params &P, int mn0, int tid) {
    const int col = mn0 + 4 * (tid % kQuads);
    krow = tid / kQuads;
    ncols = P.mn_total - col;
    row_bytes = static_cast<int>(P.ld) * 4;
    const int64_t bytes = static_cast<int64_t>(P.k_total) * P.ld * 4;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.p), 0, static_cast<int>(bytes), kBufFlags);
    voff = ncols > 0 ? (static_cast<unsigned>(krow) * static_cast<unsigned>(P.ld) + static_cast<unsigned>(col)) * 4u
                     : kOobOffset;
  }
  __device__ __forceinline__ void load(int k0, int /*kend*/) {
#pragma unroll
    for (int s = 0; s < kPasses; ++s) {
      const int soff = (k0 + s * kRowsPerPass) * row_bytes;     // rows past the matrix end are out of range
      if (ncols >= 4 || ncols <= 0) {
        r[s] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0);
      } else {                                                   // the word holding the last 1-3 columns
        u32x4 v;
        v.x = __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, soff, 0);
        v.y = __builtin_amdgcn_raw_buffer_load_b32(rsrc, ncols > 1 ? voff + 4u : kOobOffset, soff, 0);
        v.z = __builtin_amdgcn_raw_buffer_load_b32(rsrc, ncols > 2 ? voff + 8u : kOobOffset, soff, 0);
        v.w = 0u;
        r[s] = v;
      }
    }
  }
  __device__ __forceinline__ void store(float *lds, int tid) const {
#pragma unroll
    for (int s = 0; s < kPasses; ++s)
      *reinterpret_cast<u32x4 *>(lds + (krow + s * kRowsPerPass) * Lds::kStride + 4 * (tid % kQuads)) = r[s];
  }
};

// ------------------------------------------------------------------ column maps
struct RowMajorCols {   // out[m * row_stride + n]
  __device__ __forceinline__ int64_t operator()(int n) const { return n; }
};

// ------------------------------------------------------------------ the kernel
// 1-D grid of grid_blocks(tm, tn, S) blocks; split z writes to out + z * z_stride.
//
// Block -> (tile, split) mapping.  The 8 XCDs of the chip each have their own L2 and the
// dispatcher deals consecutive workgroup ids to them round-robin, so blocks that read the same
// data should sit 8 ids apart.  The ids are therefore transposed (id % 8 selects a contiguous
// eighth of the logical order) and the logical order puts the sharers next to each other: the
// M tiles of one N tile (same gathered activations), then the N tiles, then the K splits (all
// tiles of one split read the same k-range of both operands).
struct TileGrid {
  int tm, tn, total;   // M tiles, N tiles, tm * tn * S
};
inline unsigned grid_blocks(int tm, int tn, int S) { return static_cast<unsigned>((tm * tn * S + 7) / 8 * 8); }

// One block's tile: out[m0.., n0..] (+)= A[m0.., kbegin..kend) B[kbegin..kend), n0..].
template <int BM, int BN, int WM, int WN, class ALoader, class BLoader, class ColMap>
__device__ __forceinline__ void mfma_gemm_tile(const typename ALoader::Params &ap, const typename BLoader::Params &bp,
                                               float *__restrict__ o, int64_t row_stride, const ColMap &colmap, int M,
                                               int N, int m0, int n0, int kbegin, int kend) {
  static_assert(WM * WN == 4 && BM / WM == 64 && BN / WN == 64, "each of the 4 waves owns a 64x64 sub-tile");
  using ALds = typename ALoader::Lds;
  using BLds = typename BLoader::Lds;
  __shared__ __attribute__((aligned(16))) float lds_a[2][ALds::kFloats];
  __shared__ __attribute__((aligned(16))) float lds_b[2][BLds::kFloats];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WN) * 64, wn0 = (wave % WN) * 64;

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
    la.store(lds_a[0], tid);
    lb.store(lds_b[0], tid);
  }
  __syncthreads();

  // A wave whose 64x64 sub-tile lies outside the matrix (ragged last tile) only helps with the
  // staging and leaves the matrix pipe to other blocks.  Two copies of the loop, chosen once: a
  // test inside the loop costs full tiles 20 %.
  auto k_loop = [&](auto with_mma) {
    int stage = 0;
    for (int k0 = kbegin; k0 < kend; k0 += BK) {
      const bool more = k0 + BK < kend;
      if (more) {
        la.load(k0 + BK, kend);
        lb.load(k0 + BK, kend);
      }
      if (decltype(with_mma)::value) {
        const float *sa = lds_a[stage], *sb = lds_b[stage];
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
        la.store(lds_a[stage ^ 1], tid);
        lb.store(lds_b[stage ^ 1], tid);
      }
      __syncthreads();
      stage ^= 1;
    }
  };
  if (m0 + wm0 < M && n0 + wn0 < N)
    k_loop(std::true_type{});
  else
    k_loop(std::false_type{});

  // epilogue: accumulator register e of a 32x32 block holds row 8*(e/4) + 4*(lane/32) + e%4,
  // column lane%32
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int n = n0 + wn0 + 32 * ni + (lane & 31);
    if (n >= N) continue;
    const int64_t coff = colmap(n);
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
      const int mb = m0 + wm0 + 32 * mi + 4 * (lane >> 5);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = mb + 8 * (e >> 2) + (e & 3);
        if (m < M) o[static_cast<int64_t>(m) * row_stride + coff] = acc[mi][ni][e];
      }
    }
  }
}

// block id -> (z, tile_m, tile_n) in the XCD-aware order described above; false for the blocks
// that only pad the grid to a multiple of 8
__device__ __forceinline__ bool block_tile(const TileGrid &tg, int &z, int &tile_m, int &tile_n) {
  const int logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (logical >= tg.total) return false;
  const int per_split = tg.tm * tg.tn;
  z = logical / per_split;
  const int rem = logical - z * per_split;
  tile_n = rem / tg.tm;
  tile_m = rem - tile_n * tg.tm;
  return true;
}

// split-K GEMM: split z covers k in [z*kchunk, (z+1)*kchunk) and writes to out + z * z_stride
template <int BM, int BN, int WM, int WN, class ALoader, class BLoader, class ColMap>
__global__ __launch_bounds__(kThreads) void mfma_gemm_kernel(typename ALoader::Params ap, typename BLoader::Params bp,
                                                             float *__restrict__ out, int64_t z_stride,
                                                             int64_t row_stride, ColMap colmap, int M, int N, int K,
                                                             int kchunk, TileGrid tg) {
  int z, tile_m, tile_n;
  if (!block_tile(tg, z, tile_m, tile_n)) return;
  const int kbegin = z * kchunk;
  mfma_gemm_tile<BM, BN, WM, WN, ALoader, BLoader, ColMap>(ap, bp, out + static_cast<int64_t>(z) * z_stride, row_stride,
                                                           colmap, M, N, tile_m * BM, tile_n * BN, kbegin,
                                                           min(K, kbegin + kchunk));
}

// batched GEMM: z is the batch index; operands and output advance by their batch strides
template <int BM, int BN, int WM, int WN, class ALoader, class BLoader>
__global__ __launch_bounds__(kThreads) void mfma_batched_gemm_kernel(typename ALoader::Params ap,
                                                                     typename BLoader::Params bp,
                                                                     float *__restrict__ out, int64_t a_zstride,
                                                                     int64_t b_zstride, int64_t c_zstride, int M, int N,
                                                                     int K, TileGrid tg) {
  int z, tile_m, tile_n;
  if (!block_tile(tg, z, tile_m, tile_n)) return;
  ap.p += static_cast<int64_t>(z) * a_zstride;
  bp.p += static_cast<int64_t>(z) * b_zstride;
  mfma_gemm_tile<BM, BN, WM, WN, ALoader, BLoader, RowMajorCols>(ap, bp, out + static_cast<int64_t>(z) * c_zstride,
                                                                 static_cast<int64_t>(N), RowMajorCols{}, M, N,
                                                                 tile_m * BM, tile_n * BN, 0, K);
}

// out[i] = sum_z part[z * stride + i], z ascending (deterministic split-K fold)
static __global__ __launch_bounds__(256) void splitk_fold_kernel(const float *__restrict__ part, float *__restrict__ out,
                                                          int64_t n, int64_t stride, int S) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  float s = part[i];
  for (int z = 1; z < S; ++z) s += part[z * stride + i];
  out[i] = s;
}

// How many K splits to use so that the launch fills the chip.  The aim is ONE full wave of
// resident blocks (blocks_per_cu on each of the 256 CUs): fewer leaves CUs idle, and a count
// such as 2.1 blocks per CU makes some CUs do 3 units of work while others do 2.
// kchunk is a multiple of BK.
inline void plan_splitk(int tiles, int K, int max_split, int blocks_per_cu, int &S, int &kchunk) {
  const int target = 256 * (blocks_per_cu > 0 ? blocks_per_cu : 2);
  int s = tiles >= target ? 1 : target / tiles;
  const int ksteps = (K + BK - 1) / BK;
  if (s > ksteps / 16) s = ksteps / 16;   // at least 16 k-steps per split: shorter ones are all prologue and epilogue
  if (s > max_split) s = max_split;
  if (s < 1) s = 1;
  int per = (ksteps + s - 1) / s;
  if (per < 1) per = 1;
  kchunk = per * BK;
  S = (K + kchunk - 1) / kchunk;
  if (S < 1) S = 1;
}

// resident blocks per CU of a kernel (register/LDS limited), asked once per kernel
template <class F>
inline int blocks_per_cu(F kernel) {
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, kThreads, 0) != hipSuccess || n < 1) {
    (void)hipGetLastError();
    n = 2;
  }
  return n;
}

}  // namespace mg
}  // namespace tsplit
