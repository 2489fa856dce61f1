// The 36 GEMMs of the Winograd routine with every fp32 operand split into three bf16 terms and the product
// taken as six bf16 matrix products accumulated in fp32 (opt-in; the default path multiplies in fp32).
//
// An fp32 number a is the exact sum a1 + a2 + a3 of three bf16 numbers: a1 = bf16(a) (round to nearest
// even), a2 = bf16(a - a1), a3 = a - a1 - a2 (each difference is exact in fp32, and the last one has at
// most 8 significant bits, so it is a bf16 number).  |a2| <= 2^-8 |a| and |a3| <= 2^-16 |a|.  A product
// a b is then the sum of nine exact bf16 x bf16 products; the six with i + j <= 4 are kept:
//     a1 b1 + (a1 b2 + a2 b1) + (a2 b2 + a1 b3 + a3 b1),
// and what is left out, a2 b3 + a3 b2 + a3 b3, is at most 2^-23 |a b|: the size of the rounding of one
// fp32 multiplication.  The bf16 matrix instruction (v_mfma_f32_32x32x16_bf16, fp32 accumulation) runs 16
// times the multiplications per cycle of the fp32 one, so six of them cost 3/8 of the fp32 instruction's
// time for the same product.  Not for operands above 2^127 (a1 would round to infinity).
//
// The operands stay fp32 in memory.  A block loads them as fp32, splits them in registers on their way to
// LDS, and keeps three bf16 planes per operand there, laid out so that a lane's 8 consecutive k values
// of one row (the instruction's operand) are one 16-byte word: plane[k / 8][row][k % 8].
#pragma once
#include "wino_gemm.h"

namespace tsplit {
namespace wg {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// (x, y) -> packed bf16 pair of the leading terms; x and y are left holding the remainders
__device__ __forceinline__ unsigned split_pair(float &x, float &y) {
  const f32x2 v = {x, y};
  const unsigned packed = __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
  x -= __uint_as_float(packed << 16);
  y -= __uint_as_float(packed & 0xffff0000u);
  return packed;
}

// eight fp32 values -> their three bf16 planes, 16 bytes each
__device__ __forceinline__ void split8(const float (&in)[8], u32x4 (&out)[3]) {
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = in[i];
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    out[s].x = split_pair(v[0], v[1]);
    out[s].y = split_pair(v[2], v[3]);
    out[s].z = split_pair(v[4], v[5]);
    out[s].w = split_pair(v[6], v[7]);
  }
}

// c + a b for one 32 x 32 x 16 step from the operands' three planes: the six products, smallest terms first
__device__ __forceinline__ acc16 split_products(const bf16x8 (&a)[3], const bf16x8 (&b)[3], acc16 c) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], b[0], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[2], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[1], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[0], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[1], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], c, 0, 0, 0);
  return c;
}

// M[xi] (rows x ld) = U[xi] (rows x depth, depth-contiguous) V[xi] (depth x ld, column-contiguous) on
// 128 x 128 tiles, 16 k values per step, the persistent XCD-aware walk and the epilogue of
// wino_gemm_kernel.  depth must be a multiple of 8.
constexpr int kSplitPlane = 2 * 128 * 8;             // bf16 elements of one plane of one operand (16 k x 128)
constexpr int kSplitStage = 2 * 3 * kSplitPlane;     // both operands, three planes each
static __global__ __launch_bounds__(kThreads, 3) void wino_gemm_split_kernel(Problem p, int total) {
  constexpr int BM = 128, BN = 128;
  __shared__ __attribute__((aligned(16))) __bf16 lds_h[2 * kSplitStage];   // 48 KB
  constexpr int kPitch = 64 + 4;
  static_assert(4 * 32 * kPitch * 4 <= 2 * kSplitStage * 2, "the epilogue's staging areas fit the operand stages");
  float *lds_f = reinterpret_cast<float *>(lds_h);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
  const int M = p.rows, N = p.ld, K = p.depth;
  const int per_xi = p.tm * p.tn;
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

  // loaders.  U: thread -> (row tid / 2, k half tid % 2): 8 consecutive k as two 16-byte loads.
  // V: thread -> (column tid % 128, k half tid / 128): 8 rows of one column as eight 4-byte loads, each of
  // which reads 256 contiguous bytes per wave.
  const int a_row = tid >> 1, a_half = tid & 1;
  const int b_col = tid & 127, b_half = __builtin_amdgcn_readfirstlane(tid >> 7);
  __amdgpu_buffer_rsrc_t ra, rb;
  unsigned a_voff, b_voff;
  int row_bytes = N * 4;
  float areg[8], breg[8];
  auto init = [&](int z, int m0, int n0) {
    const int rows_left = M - m0;
    const int64_t abytes = static_cast<int64_t>(rows_left) * K * 4;
    ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.U) + (static_cast<int64_t>(z) * M + m0) * K, 0,
                                           static_cast<int>(abytes < 0x7fffffffll ? abytes : 0x7fffffffll), kBufFlags);
    a_voff = a_row < rows_left ? (static_cast<unsigned>(a_row) * static_cast<unsigned>(K) + 8u * a_half) * 4u : kOobOffset;
    rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.V) + static_cast<int64_t>(z) * K * N, 0,
                                           static_cast<int>(static_cast<int64_t>(K) * N * 4), kBufFlags);
    b_voff = n0 + b_col < N ? static_cast<unsigned>(n0 + b_col) * 4u : kOobOffset;
  };
  auto load = [&](int k0) {
    // K is a multiple of 8: a thread's 8 values of U lie wholly inside the row or wholly beyond it
    const unsigned av = k0 + 8 * a_half < K ? a_voff : kOobOffset;
    const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(ra, av, k0 * 4, 0);
    const u32x4 hi = __builtin_amdgcn_raw_buffer_load_b128(ra, av, k0 * 4 + 16, 0);
    const unsigned w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) areg[j] = __uint_as_float(w[j]);
    // rows of V beyond the depth lie beyond the buffer and read as zeros
#pragma unroll
    for (int j = 0; j < 8; ++j)
      breg[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rb, b_voff, (k0 + 8 * b_half + j) * row_bytes, 0));
  };
  auto store = [&](__bf16 *stage) {
    u32x4 sa[3], sb[3];
    split8(areg, sa);
    split8(breg, sb);
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      *reinterpret_cast<u32x4 *>(stage + s * kSplitPlane + (a_half * 128 + a_row) * 8) = sa[s];
      *reinterpret_cast<u32x4 *>(stage + (3 + s) * kSplitPlane + (b_half * 128 + b_col) * 8) = sb[s];
    }
  };

  int z, m0, n0;
  locate(logical, z, m0, n0);
  init(z, m0, n0);
  load(0);
  float *mine = lds_f + wave * (32 * kPitch);
  const int r4 = lane >> 4, c4 = (lane & 15) * 4;
  const int frag = ((lane >> 5) * 128 + (lane & 31)) * 8;   // this lane's word within a plane, row 0 of a 32-row tile

  for (;;) {
    acc16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    __syncthreads();   // the staging areas of the previous tile's epilogue are the operand stages
    store(lds_h);
    __syncthreads();

    const bool live = m0 + wm0 < M && n0 + wn0 < N;
    int stage = 0;
    for (int k0 = 0; k0 < K; k0 += BK) {
      const bool more = k0 + BK < K;
      if (more) load(k0 + BK);
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
      if (more) store(lds_h + (stage ^ 1) * kSplitStage);
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
      init(z, m0, n0);
      load(0);
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

// ---------------------------------------------------------------- filter-gradient GEMMs, 128 x 128 tiles
// dU[xi] (rows x cols) = Y[xi] (rows x depth) V[xi]^T (cols x depth) over one range of the depth per unit, as
// wino_grad_gemm_kernel (same units, same walk, same output layout), the product taken in split bf16.  Both
// operands are depth-contiguous: a thread loads 8 consecutive k of one row as two 16-byte words, each of
// which lies wholly inside the range or outside it (ld and the range bounds are multiples of 4).
template <int NB>
static __global__ __launch_bounds__(kThreads, NB) void wino_grad_gemm_split_kernel(GradProblem p, int units) {
  constexpr int kFit = (160 * 1024 / (NB + 1)) / 2 + 128;   // bf16 elements: more than an (NB+1)-th of the LDS
  constexpr int kLds = 2 * kSplitStage > kFit ? 2 * kSplitStage : kFit;
  __shared__ __attribute__((aligned(16))) __bf16 lds_h[kLds];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
  const int per_group = p.tm * p.tn;
  const int G = gridDim.x;
  int u = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
  if (u >= units) return;

  const int row = tid >> 1, half = tid & 1;
  int z, m0, n0, kbegin, kend;
  __amdgpu_buffer_rsrc_t ra, rb;
  unsigned a_voff, b_voff;
  float areg[8], breg[8];
  auto load = [&](int k0) {
    const int k = k0 + 8 * half;
    const bool in0 = k < kend, in1 = k + 4 < kend;
    const u32x4 a0 = __builtin_amdgcn_raw_buffer_load_b128(ra, in0 ? a_voff : kOobOffset, k0 * 4, 0);
    const u32x4 a1 = __builtin_amdgcn_raw_buffer_load_b128(ra, in1 ? a_voff : kOobOffset, k0 * 4 + 16, 0);
    const u32x4 b0 = __builtin_amdgcn_raw_buffer_load_b128(rb, in0 ? b_voff : kOobOffset, k0 * 4, 0);
    const u32x4 b1 = __builtin_amdgcn_raw_buffer_load_b128(rb, in1 ? b_voff : kOobOffset, k0 * 4 + 16, 0);
    const unsigned wa[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const unsigned wb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      areg[j] = __uint_as_float(wa[j]);
      breg[j] = __uint_as_float(wb[j]);
    }
  };
  auto store = [&](__bf16 *stage) {
    u32x4 sa[3], sb[3];
    split8(areg, sa);
    split8(breg, sb);
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      *reinterpret_cast<u32x4 *>(stage + s * kSplitPlane + (half * 128 + row) * 8) = sa[s];
      *reinterpret_cast<u32x4 *>(stage + (3 + s) * kSplitPlane + (half * 128 + row) * 8) = sb[s];
    }
  };
  auto start = [&](int unit) {
    z = unit / per_group;
    const int tile = unit - z * per_group;
    const int tile_n = tile / p.tm;
    m0 = (tile - tile_n * p.tm) * 128;
    n0 = tile_n * 128;
    const int range = z / kXi, xi = z - range * kXi;
    kbegin = range * p.kchunk;
    kend = min(p.ld, kbegin + p.kchunk);
    const int arows = p.rows - m0, brows = p.cols - n0;
    const int64_t abytes = static_cast<int64_t>(arows) * p.ld * 4, bbytes = static_cast<int64_t>(brows) * p.ld * 4;
    ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.Y) + (static_cast<int64_t>(xi) * p.rows + m0) * p.ld, 0,
                                           static_cast<int>(abytes < 0x7fffffffll ? abytes : 0x7fffffffll), kBufFlags);
    rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.V) + (static_cast<int64_t>(xi) * p.cols + n0) * p.ld, 0,
                                           static_cast<int>(bbytes < 0x7fffffffll ? bbytes : 0x7fffffffll), kBufFlags);
    a_voff = row < arows ? (static_cast<unsigned>(row) * static_cast<unsigned>(p.ld) + 8u * half) * 4u : kOobOffset;
    b_voff = row < brows ? (static_cast<unsigned>(row) * static_cast<unsigned>(p.ld) + 8u * half) * 4u : kOobOffset;
    load(kbegin);
  };
  start(u);
  const int frag = ((lane >> 5) * 128 + (lane & 31)) * 8;

  for (;;) {
    acc16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    // the last k-step of the previous unit ended with a barrier: stage 0 is free
    store(lds_h);
    __syncthreads();

    const bool live = m0 + wm0 < p.rows && n0 + wn0 < p.cols;
    int stage = 0;
    for (int k0 = kbegin; k0 < kend; k0 += BK) {
      const bool more = k0 + BK < kend;
      if (more) load(k0 + BK);
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
      if (more) store(lds_h + (stage ^ 1) * kSplitStage);
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

inline void launch_split(Problem p, hipStream_t st, int cus) {
  p.tm = (p.rows + 127) / 128;
  p.tn = (p.ld + 127) / 128;
  const int total = p.tm * p.tn * kXi;
  const int grid = std::min(cus * 3 / 8 * 8, (total + 7) / 8 * 8);
  hipLaunchKernelGGL(wino_gemm_split_kernel, dim3(grid), dim3(kThreads), 0, st, p, total);
}

}  // namespace wg
}  // namespace tsplit
