// Dropout forward / gradient behind the reference's cuDNN symbols
// (src/ops/CudnnDropout.cu:4-77, :79-151).
//
// Contract kept from the reference:
//   * `dropout` is the probability of zeroing an element; survivors are multiplied by
//     1/(1-dropout) (cudnnSetDropoutDescriptor / cudnnDropoutForward, CudnnDropout.cu:41,58).
//   * the generator is seeded with the same constant before every call (CudnnDropout.cu:33,41),
//     so a call with the same element count drops the same elements every time;
//   * the forward call with first_time == 1 sizes and allocates the reserve space from the
//     device pool and hands both back through the two pointers (CudnnDropout.cu:50-56); later
//     calls and the gradient reuse it; nobody frees it (as in the reference).
// The reserve space holds one bit per element (bit i%8 of byte i/8 = element i was kept).
//
// Which elements are dropped is this library's own choice (cuDNN's generator is closed):
// element i takes word i%4 of Philox-4x32-10(counter = (i/4, 0, 0, 0), key = seed) and is kept
// iff that word >= floor(dropout * 2^32).  One thread handles 8 consecutive elements: two
// generator calls, two 16-byte loads and stores, one mask byte.  HBM-bound: 8.125 B/element
// forward, 8.125 B/element gradient.
#include "common.h"

namespace tsplit {
void *device_pool_alloc(int device_id, size_t bytes);
}

using namespace tsplit;

namespace {

constexpr unsigned long long kSeed = 19260817ull;   // src/ops/CudnnDropout.cu:33
constexpr int kThreads = 256;

struct U4 {
  unsigned x, y, z, w;
};

__device__ __forceinline__ U4 philox4x32_10(unsigned c0, unsigned c1, unsigned k0, unsigned k1) {
  unsigned c2 = 0, c3 = 0;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const unsigned hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const unsigned hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    c0 = hi1 ^ c1 ^ k0;
    c1 = lo1;
    c2 = hi0 ^ c3 ^ k1;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return U4{c0, c1, c2, c3};
}

// keep bits of elements 8*t .. 8*t+7; `thr` = floor(dropout * 2^32) in 33 bits
__device__ __forceinline__ unsigned keep_byte(int64_t t, unsigned long long thr) {
  const unsigned long long g = static_cast<unsigned long long>(t) * 2;
  const U4 a = philox4x32_10(static_cast<unsigned>(g), static_cast<unsigned>(g >> 32),
                             static_cast<unsigned>(kSeed), static_cast<unsigned>(kSeed >> 32));
  const U4 b = philox4x32_10(static_cast<unsigned>(g + 1), static_cast<unsigned>((g + 1) >> 32),
                             static_cast<unsigned>(kSeed), static_cast<unsigned>(kSeed >> 32));
  unsigned m = 0;
  m |= (a.x >= thr) << 0;
  m |= (a.y >= thr) << 1;
  m |= (a.z >= thr) << 2;
  m |= (a.w >= thr) << 3;
  m |= (b.x >= thr) << 4;
  m |= (b.y >= thr) << 5;
  m |= (b.z >= thr) << 6;
  m |= (b.w >= thr) << 7;
  return m;
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 gate4(f32x4 v, unsigned m, float scale) {
  return f32x4{(m & 1) ? v.x * scale : 0.f, (m & 2) ? v.y * scale : 0.f, (m & 4) ? v.z * scale : 0.f,
               (m & 8) ? v.w * scale : 0.f};
}

// FROM_MASK = false: forward (generate the bits, write them); true: gradient (read them)
template <bool FROM_MASK, bool VEC>
__global__ __launch_bounds__(kThreads) void dropout_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                           unsigned char *__restrict__ mask, int64_t n,
                                                           unsigned long long thr, float scale) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t base = t * 8;
  if (base >= n) return;
  const unsigned m = FROM_MASK ? mask[t] : keep_byte(t, thr);
  if (!FROM_MASK) mask[t] = static_cast<unsigned char>(m);
  if (VEC && base + 8 <= n) {
    const f32x4 v0 = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(in + base));
    const f32x4 v1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(in + base) + 1);
    __builtin_nontemporal_store(gate4(v0, m, scale), reinterpret_cast<f32x4 *>(out + base));
    __builtin_nontemporal_store(gate4(v1, m >> 4, scale), reinterpret_cast<f32x4 *>(out + base) + 1);
  } else {
    const int cnt = static_cast<int>(min(static_cast<int64_t>(8), n - base));
    for (int i = 0; i < cnt; ++i) out[base + i] = ((m >> i) & 1) ? in[base + i] * scale : 0.f;
  }
}

int check_pair(const char *who, const DLArray *a, const DLArray *b) {
  TS_REQUIRE(a && b && a->data && b->data, "%s: null operand", who);
  TS_REQUIRE(a->ndim == b->ndim, "%s: operand ranks differ (%d vs %d)", who, a->ndim, b->ndim);
  for (int i = 0; i < a->ndim; ++i)
    TS_REQUIRE(a->shape[i] == b->shape[i], "%s: operand shapes differ on axis %d", who, i);
  return 0;
}

unsigned long long threshold_of(float dropout) {
  const double t = static_cast<double>(dropout) * 4294967296.0;
  return t >= 4294967296.0 ? (1ull << 32) : static_cast<unsigned long long>(t);
}

template <bool FROM_MASK>
void launch(const float *in, float *out, unsigned char *mask, int64_t n, float dropout, hipStream_t st) {
  const float scale = 1.0f / (1.0f - dropout);
  const int64_t threads = (n + 7) / 8;
  const unsigned blocks = static_cast<unsigned>((threads + kThreads - 1) / kThreads);
  if (aligned16(in) && aligned16(out))
    hipLaunchKernelGGL((dropout_kernel<FROM_MASK, true>), dim3(blocks), dim3(kThreads), 0, st, in, out, mask, n,
                       threshold_of(dropout), scale);
  else
    hipLaunchKernelGGL((dropout_kernel<FROM_MASK, false>), dim3(blocks), dim3(kThreads), 0, st, in, out, mask, n,
                       threshold_of(dropout), scale);
}

}  // namespace

extern "C" {

int CuDNN_DLGpuDropout(const DLArrayHandle input_X, const float dropout, DLArrayHandle output_Y, int *reserve_size,
                       void **reserve_space, int first_time, DLStreamHandle stream_handle, ProfilerHandle p) {
  const char *who = "CuDNN_DLGpuDropout";
  if (check_pair(who, input_X, output_Y)) return -1;
  TS_REQUIRE(reserve_size && reserve_space, "%s: null reserve pointers", who);
  TS_REQUIRE(dropout >= 0.f && dropout <= 1.f, "%s: dropout %g outside [0, 1]", who, dropout);
  const int64_t n = numel(input_X);
  const int64_t need = (n + 7) / 8;
  TS_REQUIRE(need <= 0x7fffffff, "%s: %lld elements exceed the int reserve size", who, static_cast<long long>(n));
  if (first_time == 1) {
    void *space = device_pool_alloc(input_X->ctx.device_id, static_cast<size_t>(need ? need : 1));
    TS_REQUIRE(space, "%s: no device memory for %lld reserve bytes", who, static_cast<long long>(need));
    *reserve_size = static_cast<int>(need);
    *reserve_space = space;
  }
  TS_REQUIRE(*reserve_space && *reserve_size >= need, "%s: reserve space of %d bytes, %lld needed (first_time not 1?)",
             who, *reserve_size, static_cast<long long>(need));
  hipStream_t st = stream_of(stream_handle);
  ProfileScope ps(p, st, n, n, 0);
  if (n > 0)
    launch<false>(static_cast<const float *>(input_X->data), static_cast<float *>(output_Y->data),
                  static_cast<unsigned char *>(*reserve_space), n, dropout, st);
  return ps.finish();
}

// output_Y carries the incoming gradient, input_X receives the result (the reference's naming).
int CuDNN_DLGpuDropout_gradient(const DLArrayHandle output_Y, const float dropout, DLArrayHandle input_X,
                                int *reserve_size, void **reserve_space, DLStreamHandle stream_handle,
                                ProfilerHandle p) {
  const char *who = "CuDNN_DLGpuDropout_gradient";
  if (check_pair(who, output_Y, input_X)) return -1;
  TS_REQUIRE(reserve_size && reserve_space && *reserve_space, "%s: no reserve space (forward not run?)", who);
  const int64_t n = numel(input_X);
  TS_REQUIRE(*reserve_size >= (n + 7) / 8, "%s: reserve space of %d bytes is too small for %lld elements", who,
             *reserve_size, static_cast<long long>(n));
  hipStream_t st = stream_of(stream_handle);
  ProfileScope ps(p, st, n, n, 0);
  if (n > 0)
    launch<true>(static_cast<const float *>(output_Y->data), static_cast<float *>(input_X->data),
                 static_cast<unsigned char *>(*reserve_space), n, dropout, st);
  return ps.finish();
}

}  // extern "C"
