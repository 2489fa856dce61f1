// CSR sparse x dense products behind the reference's cuSPARSE symbols
// (src/ops/CuSparseCsrmv.cu:3-64, src/ops/CuSparseCsrmm.cu:34-114).
//
// A is given as three 1-D arrays: values (fp32, nnz), row pointers (int32, nrow+1) and column
// indices (int32, nnz), zero based, as python/athena/ndarray.py:445-455 uploads them.  Dense
// operands and results are row-major.  All four transpose combinations of the matrix product
// are computed (the reference's GPU path asserts one of them away, CuSparseCsrmm.cu:48, its
// numpy path has all four, gpu_ops/CuSparse.py:150-163).
//
// All kernels are bound by HBM: per stored entry 8 bytes of A plus the gathered operand.
//   y = A x / C = A B     : a group of lanes per row, fixed summation order, no atomics
//   y = A^T x / C = A^T B : results are cleared, then every entry adds into its column's row
//                           with float atomics (the order of those additions is not fixed)
//   op(B) = B^T           : B is transposed into per-stream scratch first, then as above
// Entries whose column index or row range lies outside the matrix are skipped rather than
// dereferenced.
#include "common.h"

using namespace tsplit;

namespace {

constexpr int kThreads = 256;

struct Csr {
  const float *val;
  const int *ptr;
  const int *col;
  int nrow, ncol, nnz;
};

__device__ __forceinline__ void row_range(const Csr &A, int row, int &b, int &e) {
  b = max(0, min(A.ptr[row], A.nnz));
  e = max(b, min(A.ptr[row + 1], A.nnz));
}

// ---- matrix x vector ----------------------------------------------------------------
template <int LANES>
__global__ __launch_bounds__(kThreads) void csrmv_kernel(Csr A, const float *__restrict__ x, float *__restrict__ y) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int row = static_cast<int>(g / LANES), sub = static_cast<int>(g % LANES);
  float acc = 0.f;
  if (row < A.nrow) {
    int b, e;
    row_range(A, row, b, e);
    for (int j = b + sub; j < e; j += LANES) {
      const unsigned c = static_cast<unsigned>(A.col[j]);
      if (c < static_cast<unsigned>(A.ncol)) acc += A.val[j] * x[c];
    }
  }
#pragma unroll
  for (int d = LANES / 2; d > 0; d >>= 1) acc += __shfl_xor(acc, d, LANES);
  if (row < A.nrow && sub == 0) y[row] = acc;
}

template <int LANES>
__global__ __launch_bounds__(kThreads) void csrmv_trans_kernel(Csr A, const float *__restrict__ x,
                                                               float *__restrict__ y) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int row = static_cast<int>(g / LANES), sub = static_cast<int>(g % LANES);
  if (row >= A.nrow) return;
  int b, e;
  row_range(A, row, b, e);
  const float xv = x[row];
  for (int j = b + sub; j < e; j += LANES) {
    const unsigned c = static_cast<unsigned>(A.col[j]);
    if (c < static_cast<unsigned>(A.ncol)) atomicAdd(y + c, A.val[j] * xv);
  }
}

__global__ __launch_bounds__(kThreads) void zero_kernel(float *__restrict__ p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// ---- matrix x matrix: one thread per VEC consecutive outputs of a row ----------------
template <int VEC>
struct Pack;
template <>
struct Pack<1> {
  using T = float;
};
template <>
struct Pack<4> {
  using T = float4;
};

__device__ __forceinline__ void fma_into(float &a, float s, float b) { a += s * b; }
__device__ __forceinline__ void fma_into(float4 &a, float s, float4 b) {
  a.x += s * b.x;
  a.y += s * b.y;
  a.z += s * b.z;
  a.w += s * b.w;
}

// C[row, :] = sum_j val[j] * B[col[j], :]      (B: [ncol, n])
template <int VEC>
__global__ __launch_bounds__(kThreads) void csrmm_kernel(Csr A, const float *__restrict__ B, float *__restrict__ C,
                                                         int n) {
  using T = typename Pack<VEC>::T;
  const int nv = n / VEC;
  const int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (g >= static_cast<int64_t>(A.nrow) * nv) return;
  const int row = static_cast<int>(g / nv), t = static_cast<int>(g - static_cast<int64_t>(row) * nv);
  int b, e;
  row_range(A, row, b, e);
  T acc{};
  for (int j = b; j < e; ++j) {
    const unsigned c = static_cast<unsigned>(A.col[j]);
    if (c < static_cast<unsigned>(A.ncol))
      fma_into(acc, A.val[j], reinterpret_cast<const T *>(B + static_cast<int64_t>(c) * n)[t]);
  }
  reinterpret_cast<T *>(C + static_cast<int64_t>(row) * n)[t] = acc;
}

// C[col[j], :] += val[j] * B[row, :]           (B: [nrow, n], C: [ncol, n], cleared before)
__global__ __launch_bounds__(kThreads) void csrmm_trans_kernel(Csr A, const float *__restrict__ B,
                                                               float *__restrict__ C, int n) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (g >= static_cast<int64_t>(A.nrow) * n) return;
  const int row = static_cast<int>(g / n), t = static_cast<int>(g - static_cast<int64_t>(row) * n);
  int b, e;
  row_range(A, row, b, e);
  const float bv = B[g];
  for (int j = b; j < e; ++j) {
    const unsigned c = static_cast<unsigned>(A.col[j]);
    if (c < static_cast<unsigned>(A.ncol)) atomicAdd(C + static_cast<int64_t>(c) * n + t, A.val[j] * bv);
  }
}

unsigned blocks_for(int64_t threads) { return static_cast<unsigned>((threads + kThreads - 1) / kThreads); }

int lanes_for(const Csr &A) {
  const int mean = A.nrow > 0 ? (A.nnz + A.nrow - 1) / A.nrow : 1;
  int l = 1;
  while (l < 64 && l < mean) l <<= 1;
  return l;
}

#define LAUNCH_BY_LANES(kernel, lanes, ...)                                                                       \
  switch (lanes) {                                                                                                \
    case 1: hipLaunchKernelGGL((kernel<1>), dim3(blocks_for(int64_t(A.nrow) * 1)), dim3(kThreads), 0, st, __VA_ARGS__); break;   \
    case 2: hipLaunchKernelGGL((kernel<2>), dim3(blocks_for(int64_t(A.nrow) * 2)), dim3(kThreads), 0, st, __VA_ARGS__); break;   \
    case 4: hipLaunchKernelGGL((kernel<4>), dim3(blocks_for(int64_t(A.nrow) * 4)), dim3(kThreads), 0, st, __VA_ARGS__); break;   \
    case 8: hipLaunchKernelGGL((kernel<8>), dim3(blocks_for(int64_t(A.nrow) * 8)), dim3(kThreads), 0, st, __VA_ARGS__); break;   \
    case 16: hipLaunchKernelGGL((kernel<16>), dim3(blocks_for(int64_t(A.nrow) * 16)), dim3(kThreads), 0, st, __VA_ARGS__); break; \
    case 32: hipLaunchKernelGGL((kernel<32>), dim3(blocks_for(int64_t(A.nrow) * 32)), dim3(kThreads), 0, st, __VA_ARGS__); break; \
    default: hipLaunchKernelGGL((kernel<64>), dim3(blocks_for(int64_t(A.nrow) * 64)), dim3(kThreads), 0, st, __VA_ARGS__); break; \
  }

int csr_of(const char *who, const DLArray *data, const DLArray *row, const DLArray *col, int nrow, int ncol, Csr &A) {
  TS_REQUIRE(data && row && col, "%s: null CSR array", who);
  TS_REQUIRE(data->ndim == 1 && row->ndim == 1 && col->ndim == 1, "%s: the CSR arrays must be 1-D", who);
  TS_REQUIRE(nrow >= 0 && ncol >= 0, "%s: negative matrix extent", who);
  TS_REQUIRE(row->shape[0] == static_cast<int64_t>(nrow) + 1, "%s: %lld row pointers for %d rows (nrow + 1 expected)",
             who, static_cast<long long>(row->shape[0]), nrow);
  TS_REQUIRE(col->shape[0] == data->shape[0], "%s: %lld column indices for %lld values", who,
             static_cast<long long>(col->shape[0]), static_cast<long long>(data->shape[0]));
  TS_REQUIRE(data->shape[0] <= 0x7fffffff, "%s: more than 2^31-1 stored entries", who);
  TS_REQUIRE((data->shape[0] == 0 || (data->data && col->data)) && row->data, "%s: CSR array without data", who);
  A = Csr{static_cast<const float *>(data->data), static_cast<const int *>(row->data),
          static_cast<const int *>(col->data), nrow, ncol, static_cast<int>(data->shape[0])};
  return 0;
}

}  // namespace

extern "C" {

int CuSparse_DLGpuCsrmv(const DLArrayHandle data_handle, const DLArrayHandle row_handle,
                        const DLArrayHandle col_handle, int nrow, int ncol, bool transpose,
                        const DLArrayHandle input_handle, DLArrayHandle output_handle, DLStreamHandle stream_handle,
                        ProfilerHandle p) {
  const char *who = "CuSparse_DLGpuCsrmv";
  Csr A;
  if (csr_of(who, data_handle, row_handle, col_handle, nrow, ncol, A)) return -1;
  TS_REQUIRE(input_handle && output_handle && input_handle->ndim == 1 && output_handle->ndim == 1,
             "%s: the vectors must be 1-D", who);
  const int in_len = transpose ? nrow : ncol, out_len = transpose ? ncol : nrow;
  TS_REQUIRE(input_handle->shape[0] == in_len && output_handle->shape[0] == out_len,
             "%s: vector lengths %lld -> %lld, expected %d -> %d", who, static_cast<long long>(input_handle->shape[0]),
             static_cast<long long>(output_handle->shape[0]), in_len, out_len);
  hipStream_t st = stream_of(stream_handle);
  ProfileScope ps(p, st, 2ll * A.nnz + nrow + 1 + in_len, out_len, 0);
  const float *x = static_cast<const float *>(input_handle->data);
  float *y = static_cast<float *>(output_handle->data);
  const int lanes = lanes_for(A);
  if (!transpose) {
    if (nrow > 0) LAUNCH_BY_LANES(csrmv_kernel, lanes, A, x, y)
  } else {
    if (ncol > 0) hipLaunchKernelGGL(zero_kernel, dim3(blocks_for(ncol)), dim3(kThreads), 0, st, y, int64_t(ncol));
    if (nrow > 0 && A.nnz > 0) LAUNCH_BY_LANES(csrmv_trans_kernel, lanes, A, x, y)
  }
  return ps.finish();
}

int CuSparse_DLGpuCsrmm(const DLArrayHandle data_handle, const DLArrayHandle row_handle,
                        const DLArrayHandle col_handle, int nrow, int ncol, bool transposeA, const DLArrayHandle matB,
                        bool transposeB, DLArrayHandle matC, DLStreamHandle stream_handle, ProfilerHandle p) {
  const char *who = "CuSparse_DLGpuCsrmm";
  Csr A;
  if (csr_of(who, data_handle, row_handle, col_handle, nrow, ncol, A)) return -1;
  TS_REQUIRE(matB && matC && matB->ndim == 2 && matC->ndim == 2 && matB->data && matC->data,
             "%s: B and C must be 2-D arrays", who);
  const int64_t inner = transposeA ? nrow : ncol, outer = transposeA ? ncol : nrow;
  const int64_t b_rows = transposeB ? matB->shape[1] : matB->shape[0];
  const int64_t n = transposeB ? matB->shape[0] : matB->shape[1];
  TS_REQUIRE(b_rows == inner, "%s: op(A) has %lld columns, op(B) %lld rows", who, static_cast<long long>(inner),
             static_cast<long long>(b_rows));
  TS_REQUIRE(matC->shape[0] == outer && matC->shape[1] == n, "%s: C is [%lld,%lld], expected [%lld,%lld]", who,
             static_cast<long long>(matC->shape[0]), static_cast<long long>(matC->shape[1]),
             static_cast<long long>(outer), static_cast<long long>(n));
  TS_REQUIRE(n <= 0x7fffffff && outer * n < (1ll << 40), "%s: result too large", who);
  hipStream_t st = stream_of(stream_handle);
  const float *B = static_cast<const float *>(matB->data);
  float *C = static_cast<float *>(matC->data);
  int64_t ws_elems = 0;
  if (transposeB && inner > 0 && n > 0) {
    // op(B) = B^T: lay it out row-major [inner, n] in scratch
    float *Bt = static_cast<float *>(scratch_get(st, 6, static_cast<size_t>(inner) * n * 4));
    TS_REQUIRE(Bt, "%s: no scratch memory for the transposed operand", who);
    int64_t src_shape[2] = {n, inner}, dst_shape[2] = {inner, n};
    DLArray src{matB->data, matB->ctx, 2, src_shape}, dst{Bt, matB->ctx, 2, dst_shape};
    int perm[2] = {1, 0};
    if (DLGpuTranspose(&src, &dst, perm, stream_handle, nullptr)) return -1;
    B = Bt;
    ws_elems = inner * n;
  }
  ProfileScope ps(p, st, 2ll * A.nnz + nrow + 1 + inner * n, outer * n, ws_elems);
  const int ni = static_cast<int>(n);
  if (outer > 0 && n > 0) {
    if (!transposeA) {
      if (ni % 4 == 0 && aligned16(B) && aligned16(C))
        hipLaunchKernelGGL(csrmm_kernel<4>, dim3(blocks_for(outer * (n / 4))), dim3(kThreads), 0, st, A, B, C, ni);
      else
        hipLaunchKernelGGL(csrmm_kernel<1>, dim3(blocks_for(outer * n)), dim3(kThreads), 0, st, A, B, C, ni);
    } else {
      hipLaunchKernelGGL(zero_kernel, dim3(blocks_for(outer * n)), dim3(kThreads), 0, st, C, outer * n);
      if (nrow > 0 && A.nnz > 0)
        hipLaunchKernelGGL(csrmm_trans_kernel, dim3(blocks_for(int64_t(nrow) * n)), dim3(kThreads), 0, st, A, B, C, ni);
    }
  }
  return ps.finish();
}

}  // extern "C"
