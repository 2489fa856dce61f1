// Stand-alone measurement: can a SIMD of gfx950 issue vector instructions while its matrix pipe works?
//
// Every compute unit gets one block; waves w and w + 4 of a block share SIMD w % 4.  Each case runs the same
// number of loop iterations; an iteration is 8 independent fp32 MFMAs (16x16x4: 32 clocks each = 256 clocks of the
// matrix pipe) and / or 64 (56) independent fp32 FMAs (4 clocks of the issue port each = 256 (224) clocks).  If vector
// and matrix instructions overlapped, "MFMA waves + FMA waves" would take as long as either alone and the
// interleaved wave as long as its MFMAs alone; if they exclude each other, the sum.  The same with bf16 MFMAs
// (16x16x16: 8 per iteration) beside the FMAs.
//
//   hipcc --offload-arch=gfx950 -O3 -o issue_probe issue_probe.hip && ./issue_probe
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short bf16x4 __attribute__((ext_vector_type(4)));

enum Case { kAllMfma, kMfmaBesideFma, kMfmaAlone, kFmaAlone, kInterleaved, kFma56Alone, kBf16Alone, kBf16BesideFma };

template <int CASE>
__global__ __launch_bounds__(512) void probe_kernel(float *out, int iters) {
  const int wave = threadIdx.x >> 6;
  f32x4 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float a = threadIdx.x * 1e-3f, b = 1.0f + threadIdx.x * 1e-6f;
  const bf16x4 ha = {static_cast<short>(threadIdx.x), 1, 2, 3}, hb = {4, 5, 6, static_cast<short>(threadIdx.x)};
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = a + i;
  const bool first_half = wave < 4;
  const bool mfma = CASE == kAllMfma || ((CASE == kMfmaBesideFma || CASE == kMfmaAlone) && first_half);
  const bool bf16 = (CASE == kBf16Alone || CASE == kBf16BesideFma) && first_half;
  const bool fma = ((CASE == kMfmaBesideFma || CASE == kFmaAlone || CASE == kBf16BesideFma) && !first_half) || CASE == kFma56Alone;
  if (CASE == kInterleaved) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 7; ++j) v[(i + j) & 7] = __builtin_fmaf(v[(i + j) & 7], b, a);
      }
    }
  } else if (mfma) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
    }
  } else if (bf16) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ha, hb, acc[i], 0, 0, 0);
    }
  } else if (fma) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int r = 0; r < (CASE == kFma56Alone ? 7 : 8); ++r)
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_fmaf(v[i], b, a);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3] + v[i];
  if (s == 12345.678f) out[threadIdx.x] = s;     // keeps the work alive; never true
}

#define CHECK(call)                                                                         \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));                       \
      std::exit(1);                                                                         \
    }                                                                                       \
  } while (0)

template <int CASE>
float microseconds(float *out, int blocks, int threads, int iters) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  hipLaunchKernelGGL(probe_kernel<CASE>, dim3(blocks), dim3(threads), 0, 0, out, iters);
  CHECK(hipDeviceSynchronize());
  float best = 1e30f;
  for (int rep = 0; rep < 3; ++rep) {
    CHECK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(probe_kernel<CASE>, dim3(blocks), dim3(threads), 0, 0, out, iters);
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    best = ms < best ? ms : best;
  }
  CHECK(hipEventDestroy(e0));
  CHECK(hipEventDestroy(e1));
  return best * 1e3f;
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount, iters = 20000;
  float *out = nullptr;
  CHECK(hipMalloc(&out, 4096));
  std::printf("%s, %d compute units, one block per unit, %d iterations; best of 3 launches\n", prop.gcnArchName, cus, iters);
  std::printf("%-72s %9s\n", "case (per SIMD)", "us");
  std::printf("%-72s %9.1f\n", "2 waves, each 8 fp32 MFMA an iteration", microseconds<kAllMfma>(out, cus, 512, iters));
  std::printf("%-72s %9.1f\n", "1 wave 8 fp32 MFMA, the other idle", microseconds<kMfmaAlone>(out, cus, 512, iters));
  std::printf("%-72s %9.1f\n", "1 wave idle, the other 64 FMA", microseconds<kFmaAlone>(out, cus, 512, iters));
  std::printf("%-72s %9.1f\n", "1 wave 8 fp32 MFMA beside 1 wave 64 FMA", microseconds<kMfmaBesideFma>(out, cus, 512, iters));
  std::printf("%-72s %9.1f\n", "1 wave, 56 FMA an iteration", microseconds<kFma56Alone>(out, cus, 256, iters));
  std::printf("%-72s %9.1f\n", "1 wave, 8 fp32 MFMA with 7 independent FMA behind each", microseconds<kInterleaved>(out, cus, 256, iters));
  std::printf("%-72s %9.1f\n", "1 wave 8 bf16 MFMA (16x16x16), the other idle", microseconds<kBf16Alone>(out, cus, 512, iters));
  std::printf("%-72s %9.1f\n", "1 wave 8 bf16 MFMA (16x16x16) beside 1 wave 64 FMA", microseconds<kBf16BesideFma>(out, cus, 512, iters));
  CHECK(hipFree(out));
  return 0;
}
