// Wavefront-64 and block reductions used by the softmax, BatchNorm and split-K kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace tsplit {

constexpr int kWave = 64;

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of NW waves; every thread gets the result.  `smem` holds NW values.
template <typename T, int NW>
__device__ __forceinline__ T block_sum(T v, T *smem) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  __syncthreads();   // protects smem against a previous use
  if (lane == 0) smem[w] = v;
  __syncthreads();
  T r = smem[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r += smem[i];
  return r;
}

}  // namespace tsplit
