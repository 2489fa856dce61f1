// Sum reductions: ReduceSumAxisZero, Conv2d_reduce_sum and the general ReduceSum.
//
// The axes of the input are split into kept and reduced ones (each list collapsed,
// nd_index.h).  Two kernels cover every pattern:
//   - columns: the innermost input axis is kept.  A block owns 64 output elements (or 64
//     16-byte words of them) and four row-lanes share the walk over the reduced index space;
//     neighbouring lanes read neighbouring addresses on every step.
//   - rows: the innermost input axis is reduced.  A group of 64 or 256 threads owns one
//     output element, strides over the reduced index space (16-byte words along the
//     innermost axis where possible) and finishes with a shuffle / LDS reduction.
// When there are too few outputs to fill the chip, the reduced index space is cut into S
// slices (blockIdx.y); slice sums go to per-stream scratch and a second kernel adds them in
// a fixed order, so results do not depend on scheduling.  Accumulation is float32; a thread
// adds at most a few thousand terms before the tree takes over.
#include "common.h"
#include "nd_index.h"
#include "reduce.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct ReduceGeo {
  int nk, nr;
  FastDiv kext[kMaxDim];
  int64_t kstride[kMaxDim];
  FastDiv rext[kMaxDim];     // innermost counts words in the vector row kernel
  int64_t rstride[kMaxDim];
  uint32_t outputs;          // number of output elements (words in the vector column kernel)
  uint32_t rtotal;           // reduced index space (words in the vector row kernel)
  uint32_t chunk;            // reduced indices per slice
};

__device__ __forceinline__ int64_t kept_offset(const ReduceGeo &g, uint32_t o, int scale_inner) {
  int64_t off = 0;
  uint32_t rem = o;
  for (int d = g.nk - 1; d >= 0; --d) {
    const uint32_t q = g.kext[d].div(rem);
    uint32_t c = rem - q * g.kext[d].d;
    rem = q;
    if (d == g.nk - 1) c *= scale_inner;
    off += static_cast<int64_t>(c) * g.kstride[d];
  }
  return off;
}

__device__ __forceinline__ int64_t reduced_offset(const ReduceGeo &g, uint32_t r, int scale_inner) {
  int64_t off = 0;
  uint32_t rem = r;
  for (int d = g.nr - 1; d >= 0; --d) {
    const uint32_t q = g.rext[d].div(rem);
    uint32_t c = rem - q * g.rext[d].d;
    rem = q;
    if (d == g.nr - 1) c *= scale_inner;
    off += static_cast<int64_t>(c) * g.rstride[d];
  }
  return off;
}

// A block is 64 output units (VEC outputs each) wide and 4 row-lanes deep: row-lane ry adds
// the reduced indices r0 + ry, r0 + ry + 4, ... of the block's slice; the four partial sums
// are combined through LDS in a fixed order.  dst[slice][output].
constexpr int kColsWide = 64, kRowLanes = kThreads / kColsWide;
template <int VEC>
__global__ __launch_bounds__(kThreads) void reduce_cols_kernel(const float *__restrict__ in, float *__restrict__ dst,
                                                               ReduceGeo g) {
  __shared__ float sm[kRowLanes - 1][kColsWide][VEC];
  const int cx = threadIdx.x % kColsWide, ry = threadIdx.x / kColsWide;
  const uint32_t o = blockIdx.x * kColsWide + cx;
  const bool live = o < g.outputs;
  float acc[VEC] = {};
  if (live) {
    const float *p = in + kept_offset(g, o, VEC);
    const uint32_t r0 = blockIdx.y * g.chunk, r1 = min(r0 + g.chunk, g.rtotal);
    if (g.nr == 1) {
      const int64_t st = g.rstride[0] * kRowLanes;
      const float *q = p + static_cast<int64_t>(r0 + ry) * g.rstride[0];
#pragma unroll 8
      for (uint32_t r = r0 + ry; r < r1; r += kRowLanes, q += st) {
        if (VEC == 4) {
          const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(q));
          acc[0] += v.x;
          acc[1 % VEC] += v.y;
          acc[2 % VEC] += v.z;
          acc[3 % VEC] += v.w;
        } else {
          acc[0] += __builtin_nontemporal_load(q);
        }
      }
    } else {
#pragma unroll 4
      for (uint32_t r = r0 + ry; r < r1; r += kRowLanes) {
        const float *q = p + reduced_offset(g, r, 1);
        if (VEC == 4) {
          const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(q));
          acc[0] += v.x;
          acc[1 % VEC] += v.y;
          acc[2 % VEC] += v.z;
          acc[3 % VEC] += v.w;
        } else {
          acc[0] += __builtin_nontemporal_load(q);
        }
      }
    }
  }
  if (ry > 0) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) sm[ry - 1][cx][j] = acc[j];
  }
  __syncthreads();
  if (ry == 0 && live) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float t = acc[j];
#pragma unroll
      for (int l = 0; l < kRowLanes - 1; ++l) t += sm[l][cx][j];
      acc[j] = t;
    }
    float *d = dst + (static_cast<int64_t>(blockIdx.y) * g.outputs + o) * VEC;
    if (VEC == 4) {
      const f32x4 r = {acc[0], acc[1 % VEC], acc[2 % VEC], acc[3 % VEC]};
      *reinterpret_cast<f32x4 *>(d) = r;
    } else {
      d[0] = acc[0];
    }
  }
}

// G threads per output element; VEC elements per load along the innermost reduced axis
template <int G, int VEC>
__global__ __launch_bounds__(kThreads) void reduce_rows_kernel(const float *__restrict__ in, float *__restrict__ dst,
                                                               ReduceGeo g) {
  __shared__ float smem[kThreads / kWave];
  constexpr int per_block = kThreads / G;
  const uint32_t o = blockIdx.x * per_block + threadIdx.x / G;
  const int lane = threadIdx.x % G;
  const bool live = o < g.outputs;     // uniform per group; whole groups idle together
  float acc = 0.f;
  if (live) {
    const float *p = in + kept_offset(g, o, 1);
    const uint32_t r0 = blockIdx.y * g.chunk, r1 = min(r0 + g.chunk, g.rtotal);
    for (uint32_t r = r0 + lane; r < r1; r += G) {
      const float *q = p + reduced_offset(g, r, VEC);
      if (VEC == 4) {
        const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(q));
        acc += (v.x + v.y) + (v.z + v.w);
      } else {
        acc += *q;
      }
    }
  }
  if (G == kWave) {
    acc = wave_sum(acc);
  } else {
    acc = block_sum<float, kThreads / kWave>(acc, smem);
  }
  if (live && lane == 0) dst[static_cast<int64_t>(blockIdx.y) * g.outputs + o] = acc;
}

// out[o] = sum over slices of part[slice][o]: 64 outputs x 4 slice-lanes per block, slice-lane l
// adds slices l, l + 4, ...; the four sums are combined through LDS in a fixed order.
__global__ __launch_bounds__(kThreads) void fold_slices_kernel(const float *__restrict__ part, float *__restrict__ out,
                                                               uint32_t outputs, int slices) {
  __shared__ float sm[kRowLanes - 1][kColsWide];
  const int cx = threadIdx.x % kColsWide, ry = threadIdx.x / kColsWide;
  const uint32_t o = blockIdx.x * kColsWide + cx;
  float acc = 0.f;
  if (o < outputs) {
#pragma unroll 8
    for (int s = ry; s < slices; s += kRowLanes) acc += part[static_cast<int64_t>(s) * outputs + o];
  }
  if (ry > 0) sm[ry - 1][cx] = acc;
  __syncthreads();
  if (ry == 0 && o < outputs) {
#pragma unroll
    for (int l = 0; l < kRowLanes - 1; ++l) acc += sm[l][cx];
    out[o] = acc;
  }
}

__global__ __launch_bounds__(kThreads) void copy_kernel(const float *__restrict__ in, float *__restrict__ out, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) out[i] = in[i];
}

// Work a launch should offer before the reduced space is left unsliced.
constexpr int64_t kTargetThreads = 256 * 2048;

// out (dense over the kept axes, in order) = sum of `in` over the reduced axes.
// kept / reduced: axes outermost first with input strides.
int reduce_sum(const char *who, const float *in, float *out, Axis *kept, int nk, Axis *red, int nr, hipStream_t s) {
  nk = collapse_axes(kept, nk);
  nr = collapse_axes(red, nr);
  int64_t outputs = 1, rtotal = 1;
  for (int d = 0; d < nk; ++d) outputs *= kept[d].ext;
  for (int d = 0; d < nr; ++d) rtotal *= red[d].ext;
  if (outputs == 0) return 0;
  TS_REQUIRE(outputs < (1ll << 31) && rtotal < (1ll << 31), "%s: more than 2^31 kept or reduced elements", who);
  if (rtotal == 0) {   // empty sums
    hipLaunchKernelGGL(fold_slices_kernel, dim3(static_cast<unsigned>((outputs + kColsWide - 1) / kColsWide)),
                       dim3(kThreads), 0, s, in, out, static_cast<uint32_t>(outputs), 0);
    return 0;
  }
  if (rtotal == 1) {   // nothing to add: a (possibly strided) copy
    // reduced axes all have extent 1, so the kept axes are the whole dense input
    hipLaunchKernelGGL(copy_kernel, dim3(static_cast<unsigned>((outputs + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       s, in, out, outputs);
    return 0;
  }
  ReduceGeo g{};
  g.nk = nk;
  g.nr = nr;
  // which list holds the input's innermost (stride 1) axis?
  const bool rows = red[nr - 1].stride == 1 && red[nr - 1].ext > 1;
  bool vec;
  if (rows) {
    vec = red[nr - 1].ext % 4 == 0 && aligned16(in);
    for (int d = 0; d < nk && vec; ++d) vec = kept[d].stride % 4 == 0;
    for (int d = 0; d < nr - 1 && vec; ++d) vec = red[d].stride % 4 == 0;
  } else {
    vec = kept[nk - 1].stride == 1 && kept[nk - 1].ext % 4 == 0 && aligned16(in) && aligned16(out);
    for (int d = 0; d < nk - 1 && vec; ++d) vec = kept[d].stride % 4 == 0;
    for (int d = 0; d < nr && vec; ++d) vec = red[d].stride % 4 == 0;
  }
  for (int d = 0; d < nk; ++d) {
    g.kext[d] = FastDiv(static_cast<uint32_t>(!rows && vec && d == nk - 1 ? kept[d].ext / 4 : kept[d].ext));
    g.kstride[d] = kept[d].stride;
  }
  for (int d = 0; d < nr; ++d) {
    g.rext[d] = FastDiv(static_cast<uint32_t>(rows && vec && d == nr - 1 ? red[d].ext / 4 : red[d].ext));
    g.rstride[d] = red[d].stride;
  }
  const int64_t out_units = !rows && vec ? outputs / 4 : outputs;   // threads (columns) or groups (rows)
  const int64_t r_units = rows && vec ? rtotal / 4 : rtotal;
  g.outputs = static_cast<uint32_t>(out_units);
  g.rtotal = static_cast<uint32_t>(r_units);
  int group = 1;
  if (rows) group = r_units >= 2048 ? kThreads : kWave;
  // slices: enough blocks for the chip while every thread still has a few loads to overlap
  int64_t slices, chunk;
  if (rows) {
    const int64_t min_chunk = static_cast<int64_t>(group) * 8;
    slices = (kTargetThreads + out_units * group - 1) / (out_units * group);
    slices = std::min<int64_t>(slices, (r_units + min_chunk - 1) / min_chunk);
    slices = std::max<int64_t>(1, std::min<int64_t>(slices, 1024));
    chunk = (r_units + slices - 1) / slices;
    chunk = (chunk + group - 1) / group * group;
  } else {
    const int64_t out_blocks = (out_units + kColsWide - 1) / kColsWide, min_chunk = 8 * kRowLanes;
    slices = (kTargetThreads / kThreads + out_blocks - 1) / out_blocks;
    slices = std::min<int64_t>(slices, (r_units + min_chunk - 1) / min_chunk);
    slices = std::max<int64_t>(1, std::min<int64_t>(slices, 1024));
    chunk = (r_units + slices - 1) / slices;
  }
  slices = (r_units + chunk - 1) / chunk;
  g.chunk = static_cast<uint32_t>(chunk);
  float *dst = out;
  if (slices > 1) {
    dst = static_cast<float *>(scratch_get(s, 4, static_cast<size_t>(slices) * outputs * sizeof(float)));
    TS_REQUIRE(dst, "%s: out of device memory for %lld slice sums", who, (long long)(slices * outputs));
  }
  if (rows) {
    const int per_block = kThreads / group;
    const dim3 grid(static_cast<unsigned>((out_units + per_block - 1) / per_block), static_cast<unsigned>(slices));
    if (group == kWave) {
      if (vec)
        hipLaunchKernelGGL((reduce_rows_kernel<kWave, 4>), grid, dim3(kThreads), 0, s, in, dst, g);
      else
        hipLaunchKernelGGL((reduce_rows_kernel<kWave, 1>), grid, dim3(kThreads), 0, s, in, dst, g);
    } else {
      if (vec)
        hipLaunchKernelGGL((reduce_rows_kernel<kThreads, 4>), grid, dim3(kThreads), 0, s, in, dst, g);
      else
        hipLaunchKernelGGL((reduce_rows_kernel<kThreads, 1>), grid, dim3(kThreads), 0, s, in, dst, g);
    }
  } else {
    const dim3 grid(static_cast<unsigned>((out_units + kColsWide - 1) / kColsWide), static_cast<unsigned>(slices));
    if (vec)
      hipLaunchKernelGGL(reduce_cols_kernel<4>, grid, dim3(kThreads), 0, s, in, dst, g);
    else
      hipLaunchKernelGGL(reduce_cols_kernel<1>, grid, dim3(kThreads), 0, s, in, dst, g);
  }
  if (slices > 1)
    hipLaunchKernelGGL(fold_slices_kernel, dim3(static_cast<unsigned>((outputs + kColsWide - 1) / kColsWide)),
                       dim3(kThreads), 0, s, dst, out, static_cast<uint32_t>(outputs), static_cast<int>(slices));
  return 0;
}

inline const float *cf(const DLArray *a) { return static_cast<const float *>(a->data); }
inline float *mf(DLArray *a) { return static_cast<float *>(a->data); }

int axis_zero(const char *who, const DLArray *input, DLArray *output, DLStreamHandle sh, ProfilerHandle p,
              int64_t ws_elems) {
  TS_REQUIRE(input && output && input->data && output->data, "%s: NULL array", who);
  TS_REQUIRE(input->ndim >= 1, "%s: input must have an axis to reduce", who);
  const int64_t cols = numel(output);
  TS_REQUIRE(input->shape[0] * cols == numel(input), "%s: output must hold the input's trailing axes", who);
  hipStream_t s = stream_of(sh);
  ProfileScope ps(p, s, numel(input), cols, ws_elems);
  Axis kept[1], red[1];
  kept[0].ext = cols;
  kept[0].stride = 1;
  red[0].ext = input->shape[0];
  red[0].stride = cols;
  if (reduce_sum(who, cf(input), mf(output), kept, 1, red, 1, s)) return -1;
  return ps.finish();
}

}  // namespace
}  // namespace tsplit

using namespace tsplit;

extern "C" {

int DLGpuReduceSumAxisZero(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
                           ProfilerHandle p) {
  return axis_zero("DLGpuReduceSumAxisZero", input, output, stream_handle, p, 0);
}

int _DLGpuReduceSumAxisZero(const DLArrayHandle input, DLArrayHandle output, DLArrayHandle arr_workspace,
                            DLStreamHandle stream_handle, ProfilerHandle p) {
  // the caller's workspace is not needed; its size is still reported to the profiler
  return axis_zero("_DLGpuReduceSumAxisZero", input, output, stream_handle, p, arr_workspace ? numel(arr_workspace) : 0);
}

int DLGpuConv2d_reduce_sum(const DLArrayHandle input_x, DLArrayHandle output_y, DLStreamHandle stream_handle,
                           ProfilerHandle p) {
  TS_REQUIRE(input_x && output_y && input_x->data && output_y->data, "DLGpuConv2d_reduce_sum: NULL array");
  TS_REQUIRE(input_x->ndim == 4, "DLGpuConv2d_reduce_sum: input must be 4-D NCHW");
  const int64_t N = input_x->shape[0], C = input_x->shape[1], HW = input_x->shape[2] * input_x->shape[3];
  TS_REQUIRE(numel(output_y) == C, "DLGpuConv2d_reduce_sum: output must hold one value per channel");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input_x), C, 0);
  Axis kept[1], red[2];
  kept[0].ext = C;
  kept[0].stride = HW;
  red[0].ext = N;
  red[0].stride = C * HW;
  red[1].ext = HW;
  red[1].stride = 1;
  if (reduce_sum("DLGpuConv2d_reduce_sum", cf(input_x), mf(output_y), kept, 1, red, 2, s)) return -1;
  return ps.finish();
}

int DLGpuReduceSum(const DLArrayHandle in_arr, DLArrayHandle out_arr, int *axes, int num_ax,
                   DLStreamHandle stream_handle) {
  TS_REQUIRE(in_arr && out_arr && in_arr->data && out_arr->data, "DLGpuReduceSum: NULL array");
  const int nd = in_arr->ndim;
  TS_REQUIRE(nd >= 1 && nd <= kMaxDim, "DLGpuReduceSum: rank %d not supported", nd);
  TS_REQUIRE(num_ax >= 0 && (num_ax == 0 || axes), "DLGpuReduceSum: bad axes");
  bool reduced[kMaxDim] = {};
  for (int i = 0; i < num_ax; ++i) {
    TS_REQUIRE(axes[i] >= 0 && axes[i] < nd, "DLGpuReduceSum: axis %d out of range", axes[i]);
    reduced[axes[i]] = true;
  }
  Axis kept[kMaxDim], red[kMaxDim];
  int nk = 0, nr = 0;
  int64_t stride = 1, n_kept = 1;
  int64_t st[kMaxDim];
  for (int d = nd - 1; d >= 0; --d) {
    st[d] = stride;
    stride *= in_arr->shape[d];
  }
  for (int d = 0; d < nd; ++d) {
    Axis &a = reduced[d] ? red[nr++] : kept[nk++];
    a.ext = in_arr->shape[d];
    a.stride = st[d];
    if (!reduced[d]) n_kept *= in_arr->shape[d];
  }
  TS_REQUIRE(numel(out_arr) == n_kept, "DLGpuReduceSum: output holds %lld elements, the kept axes hold %lld",
             (long long)numel(out_arr), (long long)n_kept);
  if (nk == 0) kept[nk++] = Axis{};
  if (nr == 0) red[nr++] = Axis{};
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  if (reduce_sum("DLGpuReduceSum", cf(in_arr), mf(out_arr), kept, nk, red, nr, s)) return -1;
  return ps.finish();
}

}  // extern "C"
