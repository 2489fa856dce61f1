// DLGpuMatrixMultiply and DLGpuBatchMatrixMultiply: row-major C = op(A) op(B) on the fp32 MFMA
// tile engine.
//
// The four transpose combinations only change which loader stages each operand (a
// transposed operand is simply one whose other index is contiguous); nothing is ever
// transposed in memory.  Skinny problems (M <= 64, the fully-connected layers at batch 64)
// use 64x256 tiles; when the tile count cannot fill 256 CUs the K range is split across
// blocks and folded by a second deterministic kernel (the 64x25088x4096 layer streams a
// 392 MiB weight matrix and needs every CU pulling on HBM).  The batched form runs every
// leading index as one more grid dimension of the same kernel (no split-K: attention-sized
// batches already give thousands of tiles); narrow outputs (N <= 64) use 256x64 tiles.
#include "common.h"
#include "mfma_gemm.h"
#include "gemm_split.h"

namespace tsplit {
namespace {

using namespace mg;

// stored rows of an operand: (M or N, K) by (transposed or not)
inline int64_t stored_rows(bool k_rows, int mn, int K) { return k_rows ? K : mn; }

// BUF: both operands lie within 2 GiB and are read with buffer loads (the usual case)
template <int BM, int BN, int WM, int WN, bool TA, bool TB, bool BUF>
int launch_gemm(const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int M, int N, int K,
                hipStream_t s, int64_t *ws_elems) {
  using AL = typename std::conditional<
      BUF, typename std::conditional<TA, MnContigBufLoader<BM>, KContigBufLoader<BM>>::type,
      typename std::conditional<TA, MnContigLoader<BM>, KContigLoader<BM>>::type>::type;
  using BL = typename std::conditional<
      BUF, typename std::conditional<TB, KContigBufLoader<BN>, MnContigBufLoader<BN>>::type,
      typename std::conditional<TB, KContigLoader<BN>, MnContigLoader<BN>>::type>::type;
  typename AL::Params ap;
  typename BL::Params bp;
  if constexpr (BUF) {
    ap = {A, lda, M, K};
    bp = {B, ldb, N, K};
  } else {
    ap = {A, lda, M, lda % 4 == 0 && aligned16(A)};
    bp = {B, ldb, N, ldb % 4 == 0 && aligned16(B)};
  }
  const int tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
  int S, kchunk;
  static const int occ = blocks_per_cu(mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, RowMajorCols>);
  plan_splitk(tm * tn, K, 64, occ, S, kchunk);
  float *out = C;
  const int64_t mn = static_cast<int64_t>(M) * N;
  if (S > 1) {
    out = static_cast<float *>(scratch_get(s, 2, static_cast<size_t>(S) * mn * 4));
    TS_REQUIRE(out, "DLGpuMatrixMultiply: no scratch memory for split-K");
    *ws_elems = S * mn;
  }
  hipLaunchKernelGGL((mfma_gemm_kernel<BM, BN, WM, WN, AL, BL, RowMajorCols>), dim3(grid_blocks(tm, tn, S)),
                     dim3(kThreads), 0, s, ap, bp, out, mn, static_cast<int64_t>(N), RowMajorCols{}, M, N, K, kchunk,
                     TileGrid{tm, tn, tm * tn * S});
  if (S > 1)
    hipLaunchKernelGGL(splitk_fold_kernel, dim3(static_cast<unsigned>((mn + 255) / 256)), dim3(256), 0, s, out, C, mn,
                       mn, S);
  return 0;
}

// the same product with split-bf16 terms (opt-in): 128 x 128 tiles whatever M, the split-K plan and fold of above
template <bool TA, bool TB>
int launch_gemm_split(const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int M, int N, int K,
                      hipStream_t s, int64_t *ws_elems) {
  using AL = typename std::conditional<TA, SplitMnContigLoader, SplitKContigLoader>::type;
  using BL = typename std::conditional<TB, SplitKContigLoader, SplitMnContigLoader>::type;
  const typename AL::Params ap{A, lda, M, K};
  const typename BL::Params bp{B, ldb, N, K};
  const int tm = (M + 127) / 128, tn = (N + 127) / 128;
  int S, kchunk;
  plan_splitk(tm * tn, K, 64, 3, S, kchunk);
  float *out = C;
  const int64_t mn = static_cast<int64_t>(M) * N;
  if (S > 1) {
    out = static_cast<float *>(scratch_get(s, 2, static_cast<size_t>(S) * mn * 4));
    TS_REQUIRE(out, "DLGpuMatrixMultiply: no scratch memory for split-K");
    *ws_elems = S * mn;
  }
  hipLaunchKernelGGL((mfma_gemm_split_kernel<AL, BL>), dim3(grid_blocks(tm, tn, S)), dim3(kThreads), 0, s, ap, bp, out, mn,
                     M, N, K, kchunk, TileGrid{tm, tn, tm * tn * S});
  if (S > 1)
    hipLaunchKernelGGL(splitk_fold_kernel, dim3(static_cast<unsigned>((mn + 255) / 256)), dim3(256), 0, s, out, C, mn,
                       mn, S);
  return 0;
}

template <int BM, int BN, int WM, int WN, bool TA, bool TB>
int launch_gemm_any(const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int M, int N, int K,
                    hipStream_t s, int64_t *ws) {
  const bool buf = K < (1 << 29) && dense_fits_buffer(stored_rows(TA, M, K), lda, TA ? BK : BM) &&
                   dense_fits_buffer(stored_rows(!TB, N, K), ldb, TB ? BN : BK);
  if (buf) return launch_gemm<BM, BN, WM, WN, TA, TB, true>(A, lda, B, ldb, C, M, N, K, s, ws);
  return launch_gemm<BM, BN, WM, WN, TA, TB, false>(A, lda, B, ldb, C, M, N, K, s, ws);
}

template <bool TA, bool TB>
int dispatch_tile(const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int M, int N, int K,
                  hipStream_t s, int64_t *ws) {
  // split-bf16 products where asked for: K a multiple of 4 (a loaded word lies inside a row or outside it) and
  // both operands within reach of 32-bit byte offsets
  if (split_bf16_enabled() && K % 4 == 0 && K >= BK && K < (1 << 29) &&
      dense_fits_buffer(stored_rows(TA, M, K), lda, TA ? BK : 128) && dense_fits_buffer(stored_rows(!TB, N, K), ldb, TB ? 128 : BK))
    return launch_gemm_split<TA, TB>(A, lda, B, ldb, C, M, N, K, s, ws);
  if (M <= 64) return launch_gemm_any<64, 256, 1, 4, TA, TB>(A, lda, B, ldb, C, M, N, K, s, ws);
  return launch_gemm_any<128, 128, 2, 2, TA, TB>(A, lda, B, ldb, C, M, N, K, s, ws);
}

template <int BM, int BN, int WM, int WN, bool TA, bool TB, bool BUF>
int launch_batched(const float *A, int64_t lda, int64_t sa, const float *B, int64_t ldb, int64_t sb, float *C, int batch,
                   int M, int N, int K, hipStream_t s) {
  using AL = typename std::conditional<
      BUF, typename std::conditional<TA, MnContigBufLoader<BM>, KContigBufLoader<BM>>::type,
      typename std::conditional<TA, MnContigLoader<BM>, KContigLoader<BM>>::type>::type;
  using BL = typename std::conditional<
      BUF, typename std::conditional<TB, KContigBufLoader<BN>, MnContigBufLoader<BN>>::type,
      typename std::conditional<TB, KContigLoader<BN>, MnContigLoader<BN>>::type>::type;
  typename AL::Params ap;
  typename BL::Params bp;
  if constexpr (BUF) {
    ap = {A, lda, M, K};
    bp = {B, ldb, N, K};
  } else {
    ap = {A, lda, M, lda % 4 == 0 && sa % 4 == 0 && aligned16(A)};
    bp = {B, ldb, N, ldb % 4 == 0 && sb % 4 == 0 && aligned16(B)};
  }
  const int tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
  const int64_t blocks = static_cast<int64_t>(tm) * tn * batch;
  TS_REQUIRE(blocks < (1ll << 31) - 8, "DLGpuBatchMatrixMultiply: too many tiles");
  hipLaunchKernelGGL((mfma_batched_gemm_kernel<BM, BN, WM, WN, AL, BL>), dim3(grid_blocks(tm, tn, batch)),
                     dim3(kThreads), 0, s, ap, bp, C, sa, sb, static_cast<int64_t>(M) * N, M, N, K,
                     TileGrid{tm, tn, tm * tn * batch});
  return 0;
}

template <int BM, int BN, int WM, int WN, bool TA, bool TB>
int launch_batched_any(const float *A, int64_t lda, int64_t sa, const float *B, int64_t ldb, int64_t sb, float *C,
                       int batch, int M, int N, int K, hipStream_t s) {
  const bool buf = K < (1 << 29) && dense_fits_buffer(stored_rows(TA, M, K), lda, TA ? BK : BM) &&
                   dense_fits_buffer(stored_rows(!TB, N, K), ldb, TB ? BN : BK);
  if (buf) return launch_batched<BM, BN, WM, WN, TA, TB, true>(A, lda, sa, B, ldb, sb, C, batch, M, N, K, s);
  return launch_batched<BM, BN, WM, WN, TA, TB, false>(A, lda, sa, B, ldb, sb, C, batch, M, N, K, s);
}

template <bool TA, bool TB>
int dispatch_batched(const float *A, int64_t lda, int64_t sa, const float *B, int64_t ldb, int64_t sb, float *C,
                     int batch, int M, int N, int K, hipStream_t s) {
  if (M <= 64) return launch_batched_any<64, 256, 1, 4, TA, TB>(A, lda, sa, B, ldb, sb, C, batch, M, N, K, s);
  if (N <= 64) return launch_batched_any<256, 64, 4, 1, TA, TB>(A, lda, sa, B, ldb, sb, C, batch, M, N, K, s);
  return launch_batched_any<128, 128, 2, 2, TA, TB>(A, lda, sa, B, ldb, sb, C, batch, M, N, K, s);
}

}  // namespace
}  // namespace tsplit

using namespace tsplit;

extern "C" int DLGpuMatrixMultiply(const DLArrayHandle matA, bool transposeA, const DLArrayHandle matB,
                                   bool transposeB, DLArrayHandle matC, DLStreamHandle stream_handle,
                                   ProfilerHandle p) {
  TS_REQUIRE(matA && matB && matC, "DLGpuMatrixMultiply: NULL array");
  TS_REQUIRE(matA->ndim == 2 && matB->ndim == 2 && matC->ndim == 2, "DLGpuMatrixMultiply: 2-D arrays only");
  const int64_t M = matC->shape[0], N = matC->shape[1];
  const int64_t K = transposeA ? matA->shape[0] : matA->shape[1];
  const int64_t Am = transposeA ? matA->shape[1] : matA->shape[0];
  const int64_t Bk = transposeB ? matB->shape[1] : matB->shape[0];
  const int64_t Bn = transposeB ? matB->shape[0] : matB->shape[1];
  TS_REQUIRE(Am == M && Bn == N && Bk == K, "DLGpuMatrixMultiply: shapes do not conform: op(A) %lldx%lld, op(B) %lldx%lld, C %lldx%lld",
             (long long)Am, (long long)K, (long long)Bk, (long long)Bn, (long long)M, (long long)N);
  TS_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) - 64, "DLGpuMatrixMultiply: dimension too large");
  hipStream_t s = stream_of(stream_handle);
  int64_t ws = 0;
  ProfileScope ps(p, s, numel(matA) + numel(matB), M * N, 0);
  int rc = 0;
  if (M > 0 && N > 0) {
    const float *A = static_cast<const float *>(matA->data), *B = static_cast<const float *>(matB->data);
    float *C = static_cast<float *>(matC->data);
    const int64_t lda = matA->shape[1], ldb = matB->shape[1];
    const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K);
    if (!transposeA && !transposeB) rc = dispatch_tile<false, false>(A, lda, B, ldb, C, m, n, k, s, &ws);
    if (!transposeA && transposeB) rc = dispatch_tile<false, true>(A, lda, B, ldb, C, m, n, k, s, &ws);
    if (transposeA && !transposeB) rc = dispatch_tile<true, false>(A, lda, B, ldb, C, m, n, k, s, &ws);
    if (transposeA && transposeB) rc = dispatch_tile<true, true>(A, lda, B, ldb, C, m, n, k, s, &ws);
  }
  if (p) p->workspace_memory = mib(ws);
  if (rc) return rc;
  return ps.finish();
}

extern "C" int DLGpuBatchMatrixMultiply(const DLArrayHandle matA, bool transposeA, const DLArrayHandle matB,
                                        bool transposeB, DLArrayHandle matC, DLStreamHandle stream_handle) {
  TS_REQUIRE(matA && matB && matC, "DLGpuBatchMatrixMultiply: NULL array");
  const int nd = matC->ndim;
  TS_REQUIRE(nd >= 2 && matA->ndim == nd && matB->ndim == nd, "DLGpuBatchMatrixMultiply: ranks must agree and be >= 2");
  int64_t batch = 1;
  for (int d = 0; d < nd - 2; ++d) {
    TS_REQUIRE(matA->shape[d] == matC->shape[d] && matB->shape[d] == matC->shape[d],
               "DLGpuBatchMatrixMultiply: leading axis %d differs between the operands", d);
    batch *= matC->shape[d];
  }
  const int64_t a0 = matA->shape[nd - 2], a1 = matA->shape[nd - 1], b0 = matB->shape[nd - 2], b1 = matB->shape[nd - 1];
  const int64_t M = matC->shape[nd - 2], N = matC->shape[nd - 1];
  const int64_t K = transposeA ? a0 : a1, Am = transposeA ? a1 : a0;
  const int64_t Bk = transposeB ? b1 : b0, Bn = transposeB ? b0 : b1;
  TS_REQUIRE(Am == M && Bn == N && Bk == K,
             "DLGpuBatchMatrixMultiply: shapes do not conform: op(A) %lldx%lld, op(B) %lldx%lld, C %lldx%lld", (long long)Am,
             (long long)K, (long long)Bk, (long long)Bn, (long long)M, (long long)N);
  TS_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) - 64 && batch < (1ll << 31),
             "DLGpuBatchMatrixMultiply: dimension too large");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  int rc = 0;
  if (M > 0 && N > 0 && batch > 0) {
    const float *A = static_cast<const float *>(matA->data), *B = static_cast<const float *>(matB->data);
    float *C = static_cast<float *>(matC->data);
    const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K), b = static_cast<int>(batch);
    const int64_t sa = a0 * a1, sb = b0 * b1;
    if (!transposeA && !transposeB) rc = dispatch_batched<false, false>(A, a1, sa, B, b1, sb, C, b, m, n, k, s);
    if (!transposeA && transposeB) rc = dispatch_batched<false, true>(A, a1, sa, B, b1, sb, C, b, m, n, k, s);
    if (transposeA && !transposeB) rc = dispatch_batched<true, false>(A, a1, sa, B, b1, sb, C, b, m, n, k, s);
    if (transposeA && transposeB) rc = dispatch_batched<true, true>(A, a1, sa, B, b1, sb, C, b, m, n, k, s);
  }
  if (rc) return rc;
  return ps.finish();
}
