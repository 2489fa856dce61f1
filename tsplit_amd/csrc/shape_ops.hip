// Data-movement operators: BroadcastTo, Conv2d_broadcast_to, BroadcastShape, Pad,
// Pad_gradient, Transpose, OneHot and the embedding lookup pair.
//
// The first six are one operation: out[o] = in[ sum_d (coord_d(o) - lo_d) * stride_d ], or a
// fill value where a coordinate leaves the input (Pad).  Broadcast axes have stride 0, a
// transpose permutes the strides, Pad_gradient is a window with lo < 0.  The host collapses
// the axes (nd_index.h) and picks
//   - the vector kernel when the innermost output extent is a multiple of 4: a thread
//     produces one 16-byte word with a non-temporal store; it reads one 16-byte word when the
//     input run is contiguous and aligned, one scalar when the axis is broadcast, else four
//     scalars;
//   - the tiled kernel for a transpose whose innermost output axis is not the innermost
//     input axis: 64x64 tiles go through LDS so that both the reads and the writes are
//     coalesced along their own contiguous axis;
//   - the scalar kernel otherwise (and for tensors of 2^32 elements or more).
#include <vector>

#include "common.h"
#include "nd_index.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct GatherGeo {
  FastDiv ext[kMaxDim];      // walk extents, outermost first (innermost counts words in the vector kernel)
  int64_t stride[kMaxDim];
  int32_t lo[kMaxDim];
  uint32_t in_ext[kMaxDim];  // coordinate c is read iff (uint32)(c - lo) < in_ext
  float fill;
  int vec_load;              // innermost input run is contiguous and 16-byte aligned
};

// NDIM axes, VEC elements per thread along the innermost one
template <int NDIM, int VEC>
__global__ __launch_bounds__(kThreads) void gather_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                          GatherGeo g, uint32_t total) {
  const uint32_t t = blockIdx.x * kThreads + threadIdx.x;
  if (t >= total) return;
  uint32_t rem = t;
  int64_t src = 0;
  bool inside = true;
  int32_t ci_inner = 0;
#pragma unroll
  for (int d = NDIM - 1; d >= 0; --d) {
    uint32_t c;
    if (d == 0) {
      c = rem;
    } else {
      const uint32_t q = g.ext[d].div(rem);
      c = rem - q * g.ext[d].d;
      rem = q;
    }
    if (d == NDIM - 1) {
      ci_inner = static_cast<int32_t>(c * VEC) - g.lo[d];
      src += static_cast<int64_t>(ci_inner) * g.stride[d];
    } else {
      const int32_t ci = static_cast<int32_t>(c) - g.lo[d];
      inside = inside && static_cast<uint32_t>(ci) < g.in_ext[d];
      src += static_cast<int64_t>(ci) * g.stride[d];
    }
  }
  constexpr int D = NDIM - 1;
  if (VEC == 1) {
    const bool ok = inside && static_cast<uint32_t>(ci_inner) < g.in_ext[D];
    out[t] = ok ? in[src] : g.fill;
  } else {
    f32x4 r;
    const bool all_in = inside && ci_inner >= 0 && static_cast<uint32_t>(ci_inner + 3) < g.in_ext[D];
    if (all_in && g.stride[D] == 0) {
      const float v = in[src];
      r = {v, v, v, v};
    } else if (all_in && g.vec_load && (src & 3) == 0) {
      r = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(in + src));
    } else {
      float e[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool ok = inside && static_cast<uint32_t>(ci_inner + j) < g.in_ext[D];
        e[j] = ok ? in[src + j * g.stride[D]] : g.fill;
      }
      r = {e[0], e[1], e[2], e[3]};
    }
    __builtin_nontemporal_store(r, reinterpret_cast<f32x4 *>(out) + t);
  }
}

// any rank, any size: 64-bit index arithmetic, one element per thread
struct GatherGeoBig {
  int ndim;
  int64_t ext[kMaxDim], stride[kMaxDim], lo[kMaxDim], in_ext[kMaxDim];
  float fill;
};
__global__ __launch_bounds__(kThreads) void gather_big_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                              GatherGeoBig g, int64_t total) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (t >= total) return;
  int64_t rem = t, src = 0;
  bool inside = true;
  for (int d = g.ndim - 1; d >= 0; --d) {
    const int64_t q = rem / g.ext[d];
    const int64_t ci = rem - q * g.ext[d] - g.lo[d];
    rem = q;
    inside = inside && ci >= 0 && ci < g.in_ext[d];
    src += ci * g.stride[d];
  }
  out[t] = inside ? in[src] : g.fill;
}

// ---- tiled transpose ----
// Output axes: [rest..., B-side..., A] where A is the innermost output axis (input stride sA != 1)
// and B is the output axis whose input stride is 1.  A block moves one 64(A) x 64(B) tile.
constexpr int kTile = 64;
struct TileGeo {
  int nrest;                 // other axes, enumerated by the block index after the two tile indices
  FastDiv tiles_a, tiles_b;
  FastDiv rest_ext[kMaxDim];
  int64_t rest_in[kMaxDim], rest_out[kMaxDim];
  int64_t ext_a, ext_b;
  int64_t in_stride_a;       // input stride of A (B's is 1)
  int64_t out_stride_b;      // output stride of B (A's is 1)
};

__global__ __launch_bounds__(kThreads) void transpose_tiled_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                                   TileGeo g) {
  __shared__ float tile[kTile][kTile + 1];
  uint32_t rem = blockIdx.x;
  uint32_t q = g.tiles_a.div(rem);
  const int64_t a0 = static_cast<int64_t>(rem - q * g.tiles_a.d) * kTile;
  rem = q;
  q = g.tiles_b.div(rem);
  const int64_t b0 = static_cast<int64_t>(rem - q * g.tiles_b.d) * kTile;
  rem = q;
  int64_t in_base = 0, out_base = 0;
  for (int d = g.nrest - 1; d >= 0; --d) {
    q = g.rest_ext[d].div(rem);
    const uint32_t c = rem - q * g.rest_ext[d].d;
    rem = q;
    in_base += static_cast<int64_t>(c) * g.rest_in[d];
    out_base += static_cast<int64_t>(c) * g.rest_out[d];
  }
  const int tx = threadIdx.x & (kTile - 1), ty = threadIdx.x / kTile;   // 64 x 4
  // read: lanes along B (contiguous in the input), rows along A
#pragma unroll 4
  for (int i = ty; i < kTile; i += kThreads / kTile) {
    const int64_t a = a0 + i, b = b0 + tx;
    if (a < g.ext_a && b < g.ext_b) tile[i][tx] = in[in_base + a * g.in_stride_a + b];
  }
  __syncthreads();
  // write: lanes along A (contiguous in the output), rows along B
#pragma unroll 4
  for (int i = ty; i < kTile; i += kThreads / kTile) {
    const int64_t a = a0 + tx, b = b0 + i;
    if (a < g.ext_a && b < g.ext_b) out[out_base + b * g.out_stride_b + a] = tile[tx][i];
  }
}

template <int VEC>
void launch_gather_ndim(int ndim, const float *in, float *out, const GatherGeo &g, uint32_t total, hipStream_t s) {
  const dim3 grid((total + kThreads - 1) / kThreads), block(kThreads);
  switch (ndim) {
    case 1: hipLaunchKernelGGL((gather_kernel<1, VEC>), grid, block, 0, s, in, out, g, total); break;
    case 2: hipLaunchKernelGGL((gather_kernel<2, VEC>), grid, block, 0, s, in, out, g, total); break;
    case 3: hipLaunchKernelGGL((gather_kernel<3, VEC>), grid, block, 0, s, in, out, g, total); break;
    case 4: hipLaunchKernelGGL((gather_kernel<4, VEC>), grid, block, 0, s, in, out, g, total); break;
    case 5: hipLaunchKernelGGL((gather_kernel<5, VEC>), grid, block, 0, s, in, out, g, total); break;
    case 6: hipLaunchKernelGGL((gather_kernel<6, VEC>), grid, block, 0, s, in, out, g, total); break;
    case 7: hipLaunchKernelGGL((gather_kernel<7, VEC>), grid, block, 0, s, in, out, g, total); break;
    default: hipLaunchKernelGGL((gather_kernel<8, VEC>), grid, block, 0, s, in, out, g, total); break;
  }
}

// out (dense, walked in order) = gather of `in` described by n axes (outermost first).
// Axis.stride is the input stride; Axis.stride2 is ignored.
void gather(const float *in, float *out, Axis *axes, int n, float fill, hipStream_t s) {
  n = collapse_axes(axes, n);
  int64_t total = 1;
  bool fits32 = true;
  for (int d = 0; d < n; ++d) {
    total *= axes[d].ext;
    fits32 = fits32 && axes[d].ext < (1ll << 31) && axes[d].lo > -(1ll << 31) && axes[d].lo < (1ll << 31);
  }
  if (total <= 0) return;
  if (total >= (1ll << 32) || !fits32) {
    GatherGeoBig g{};
    g.ndim = n;
    g.fill = fill;
    for (int d = 0; d < n; ++d) {
      g.ext[d] = axes[d].ext;
      g.stride[d] = axes[d].stride;
      g.lo[d] = axes[d].lo;
      g.in_ext[d] = axes[d].in_ext < 0 ? INT64_MAX : axes[d].in_ext;
    }
    hipLaunchKernelGGL(gather_big_kernel, dim3(static_cast<unsigned>((total + kThreads - 1) / kThreads)),
                       dim3(kThreads), 0, s, in, out, g, total);
    return;
  }
  const Axis &inner = axes[n - 1];
  const bool vec = inner.ext % 4 == 0 && aligned16(out);
  GatherGeo g{};
  g.fill = fill;
  for (int d = 0; d < n; ++d) {
    g.ext[d] = FastDiv(static_cast<uint32_t>(d == n - 1 && vec ? axes[d].ext / 4 : axes[d].ext));
    g.stride[d] = axes[d].stride;
    g.lo[d] = static_cast<int32_t>(axes[d].lo);
    g.in_ext[d] = axes[d].in_ext < 0 || axes[d].in_ext > INT32_MAX ? static_cast<uint32_t>(INT32_MAX)
                                                                   : static_cast<uint32_t>(axes[d].in_ext);
  }
  g.vec_load = inner.stride == 1 && aligned16(in);
  if (vec)
    launch_gather_ndim<4>(n, in, out, g, static_cast<uint32_t>(total / 4), s);
  else
    launch_gather_ndim<1>(n, in, out, g, static_cast<uint32_t>(total), s);
}

inline const float *cf(const DLArray *a) { return static_cast<const float *>(a->data); }
inline float *mf(DLArray *a) { return static_cast<float *>(a->data); }

// dense row-major strides of a DLArray
void dense_strides(const DLArray *a, int64_t *st) {
  int64_t m = 1;
  for (int d = a->ndim - 1; d >= 0; --d) {
    st[d] = m;
    m *= a->shape[d];
  }
}

// ---- OneHot: out[row, j] = (float(j) == ids[row]) ----
template <int VEC>
__global__ __launch_bounds__(kThreads) void one_hot_kernel(const float *__restrict__ ids, float *__restrict__ out,
                                                           FastDiv per_row, int64_t total) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (t >= total) return;
  int64_t row;
  uint32_t j;
  if (total < (1ll << 32)) {
    const uint32_t q = per_row.div(static_cast<uint32_t>(t));
    row = q;
    j = static_cast<uint32_t>(t) - q * per_row.d;
  } else {
    row = t / per_row.d;
    j = static_cast<uint32_t>(t - row * per_row.d);
  }
  const float id = ids[row];
  if (VEC == 1) {
    out[t] = static_cast<float>(j) == id ? 1.f : 0.f;
  } else {
    const float j0 = static_cast<float>(j * 4);
    const f32x4 r = {j0 == id ? 1.f : 0.f, j0 + 1.f == id ? 1.f : 0.f, j0 + 2.f == id ? 1.f : 0.f,
                     j0 + 3.f == id ? 1.f : 0.f};
    __builtin_nontemporal_store(r, reinterpret_cast<f32x4 *>(out) + t);
  }
}

// ---- Embedding: out[row, :] = table[int(ids[row]), :]; rows whose id is outside the table read as 0 ----
template <typename W>
__global__ __launch_bounds__(kThreads) void embedding_kernel(const W *__restrict__ table, const float *__restrict__ ids,
                                                             W *__restrict__ out, FastDiv per_row, int64_t vocab,
                                                             int64_t total) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (t >= total) return;
  int64_t row;
  uint32_t j;
  if (total < (1ll << 32)) {
    const uint32_t q = per_row.div(static_cast<uint32_t>(t));
    row = q;
    j = static_cast<uint32_t>(t) - q * per_row.d;
  } else {
    row = t / per_row.d;
    j = static_cast<uint32_t>(t - row * per_row.d);
  }
  const float idf = ids[row];
  const int64_t id = static_cast<int64_t>(idf);
  W v{};
  if (idf > -1.f && id < vocab) v = table[id * per_row.d + j];
  out[t] = v;
}

// table_grad[int(ids[row]), :] += dy[row, :]   (table_grad zeroed beforehand)
__global__ __launch_bounds__(kThreads) void embedding_grad_kernel(const float *__restrict__ dy,
                                                                  const float *__restrict__ ids,
                                                                  float *__restrict__ table_grad, FastDiv per_row,
                                                                  int64_t vocab, int64_t total) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (t >= total) return;
  int64_t row;
  uint32_t j;
  if (total < (1ll << 32)) {
    const uint32_t q = per_row.div(static_cast<uint32_t>(t));
    row = q;
    j = static_cast<uint32_t>(t) - q * per_row.d;
  } else {
    row = t / per_row.d;
    j = static_cast<uint32_t>(t - row * per_row.d);
  }
  const float idf = ids[row];
  const int64_t id = static_cast<int64_t>(idf);
  if (idf > -1.f && id < vocab) unsafeAtomicAdd(table_grad + id * per_row.d + j, dy[t]);
}

__global__ __launch_bounds__(kThreads) void zero_kernel(float *__restrict__ p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

unsigned blocks_for(int64_t n) { return static_cast<unsigned>((n + kThreads - 1) / kThreads); }

int pad_axes(const char *who, const DLArray *small, const DLArray *big, const int *paddings, int pad_len, size_t mode,
             int64_t *lo) {
  TS_REQUIRE(small && big && small->data && big->data, "%s: NULL array", who);
  TS_REQUIRE(mode == 0, "%s: only mode 0 (CONSTANT) is implemented", who);
  TS_REQUIRE(small->ndim == 4 && big->ndim == 4, "%s: arrays must be 4-D", who);
  TS_REQUIRE(pad_len >= 0 && pad_len <= 8 && pad_len % 2 == 0, "%s: pad_len must be an even number <= 8", who);
  TS_REQUIRE(pad_len == 0 || paddings, "%s: NULL paddings", who);
  const int first = 4 - pad_len / 2;
  for (int d = 0; d < 4; ++d) {
    const int64_t before = d < first ? 0 : paddings[(d - first) * 2], after = d < first ? 0 : paddings[(d - first) * 2 + 1];
    TS_REQUIRE(before >= 0 && after >= 0, "%s: negative padding", who);
    TS_REQUIRE(small->shape[d] + before + after == big->shape[d], "%s: axis %d: %lld + %lld + %lld != %lld", who, d,
               (long long)small->shape[d], (long long)before, (long long)after, (long long)big->shape[d]);
    lo[d] = before;
  }
  return 0;
}

}  // namespace
}  // namespace tsplit

using namespace tsplit;

extern "C" {

int DLGpuBroadcastTo(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input && output && input->data && output->data, "DLGpuBroadcastTo: NULL array");
  const int64_t n_in = numel(input), n_out = numel(output);
  TS_REQUIRE(n_in > 0 && n_out % n_in == 0, "DLGpuBroadcastTo: output size %lld is not a multiple of the input size %lld",
             (long long)n_out, (long long)n_in);
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, n_in, n_out, 0);
  Axis ax[2];
  ax[0].ext = n_out / n_in;
  ax[0].stride = 0;
  ax[1].ext = n_in;
  ax[1].stride = 1;
  gather(cf(input), mf(output), ax, 2, 0.f, s);
  return ps.finish();
}

int DLGpuConv2d_broadcast_to(const DLArrayHandle input_x, DLArrayHandle output_y, DLStreamHandle stream_handle,
                             ProfilerHandle p) {
  TS_REQUIRE(input_x && output_y && input_x->data && output_y->data, "DLGpuConv2d_broadcast_to: NULL array");
  TS_REQUIRE(output_y->ndim == 4, "DLGpuConv2d_broadcast_to: output must be 4-D NCHW");
  TS_REQUIRE(numel(input_x) == output_y->shape[1], "DLGpuConv2d_broadcast_to: input must hold one value per channel");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input_x), numel(output_y), 0);
  Axis ax[3];
  ax[0].ext = output_y->shape[0];
  ax[0].stride = 0;
  ax[1].ext = output_y->shape[1];
  ax[1].stride = 1;
  ax[2].ext = output_y->shape[2] * output_y->shape[3];
  ax[2].stride = 0;
  gather(cf(input_x), mf(output_y), ax, 3, 0.f, s);
  return ps.finish();
}

int DLGpuBroadcastShape(const DLArrayHandle in_arr, DLArrayHandle out_arr, int *add_axes, DLStreamHandle stream_handle) {
  TS_REQUIRE(in_arr && out_arr && in_arr->data && out_arr->data, "DLGpuBroadcastShape: NULL array");
  const int nd = out_arr->ndim, diff = nd - in_arr->ndim;
  TS_REQUIRE(nd >= 1 && nd <= kMaxDim && diff >= 0, "DLGpuBroadcastShape: bad ranks (%d -> %d)", in_arr->ndim, nd);
  // input axis feeding each output axis, or -1 for a new axis
  int from[kMaxDim];
  if (!add_axes) {
    for (int d = 0; d < nd; ++d) from[d] = d < diff ? -1 : d - diff;
  } else {
    bool is_new[kMaxDim] = {};
    for (int i = 0; i < diff; ++i) {
      TS_REQUIRE(add_axes[i] >= 0 && add_axes[i] < nd && !is_new[add_axes[i]], "DLGpuBroadcastShape: bad add_axes[%d]", i);
      is_new[add_axes[i]] = true;
    }
    int k = 0;
    for (int d = 0; d < nd; ++d) from[d] = is_new[d] ? -1 : k++;
  }
  int64_t st[kMaxDim];
  dense_strides(in_arr, st);
  Axis ax[kMaxDim];
  for (int d = 0; d < nd; ++d) {
    ax[d].ext = out_arr->shape[d];
    if (from[d] < 0 || in_arr->shape[from[d]] == 1) {
      ax[d].stride = 0;
    } else {
      TS_REQUIRE(in_arr->shape[from[d]] == out_arr->shape[d], "DLGpuBroadcastShape: axis %d: %lld cannot broadcast to %lld",
                 d, (long long)in_arr->shape[from[d]], (long long)out_arr->shape[d]);
      ax[d].stride = st[from[d]];
    }
  }
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  gather(cf(in_arr), mf(out_arr), ax, nd, 0.f, s);
  return ps.finish();
}

int DLGpuPad(const DLArrayHandle input_X, DLArrayHandle output_Y, int *paddings, int pad_len, size_t mode,
             float constant_values, DLStreamHandle stream_handle, ProfilerHandle p) {
  int64_t lo[4];
  if (pad_axes("DLGpuPad", input_X, output_Y, paddings, pad_len, mode, lo)) return -1;
  int64_t st[kMaxDim];
  dense_strides(input_X, st);
  Axis ax[4];
  for (int d = 0; d < 4; ++d) {
    ax[d].ext = output_Y->shape[d];
    ax[d].stride = st[d];
    ax[d].lo = lo[d];
    ax[d].in_ext = input_X->shape[d];
  }
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input_X), numel(output_Y), 0);
  if (numel(input_X) == 0) {   // nothing to read: the output is all fill
    for (int d = 0; d < 4; ++d) ax[d].stride = 0;
  }
  gather(cf(input_X), mf(output_Y), ax, 4, constant_values, s);
  return ps.finish();
}

int DLGpuPad_gradient(const DLArrayHandle output_gradient_Y, DLArrayHandle input_gradient_X, int *paddings, int pad_len,
                      size_t mode, DLStreamHandle stream_handle, ProfilerHandle p) {
  int64_t lo[4];
  if (pad_axes("DLGpuPad_gradient", input_gradient_X, output_gradient_Y, paddings, pad_len, mode, lo)) return -1;
  int64_t st[kMaxDim];
  dense_strides(output_gradient_Y, st);
  Axis ax[4];
  int64_t offset = 0;
  for (int d = 0; d < 4; ++d) {
    ax[d].ext = input_gradient_X->shape[d];
    ax[d].stride = st[d];
    offset += lo[d] * st[d];
  }
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(output_gradient_Y), numel(input_gradient_X), 0);
  gather(cf(output_gradient_Y) + offset, mf(input_gradient_X), ax, 4, 0.f, s);
  return ps.finish();
}

int DLGpuTranspose(const DLArrayHandle input, DLArrayHandle output, int *perm, DLStreamHandle stream_handle,
                   ProfilerHandle p) {
  TS_REQUIRE(input && output && perm && input->data && output->data, "DLGpuTranspose: NULL argument");
  const int nd = input->ndim;
  TS_REQUIRE(nd >= 1 && nd <= kMaxDim && output->ndim == nd, "DLGpuTranspose: bad ranks");
  bool seen[kMaxDim] = {};
  int64_t st[kMaxDim], ost[kMaxDim];
  dense_strides(input, st);
  dense_strides(output, ost);
  Axis ax[kMaxDim];
  for (int d = 0; d < nd; ++d) {
    TS_REQUIRE(perm[d] >= 0 && perm[d] < nd && !seen[perm[d]], "DLGpuTranspose: perm is not a permutation");
    seen[perm[d]] = true;
    TS_REQUIRE(output->shape[d] == input->shape[perm[d]], "DLGpuTranspose: output axis %d has extent %lld, expected %lld", d,
               (long long)output->shape[d], (long long)input->shape[perm[d]]);
    ax[d].ext = output->shape[d];
    ax[d].stride = st[perm[d]];
    ax[d].stride2 = ost[d];
  }
  hipStream_t s = stream_of(stream_handle);
  const int64_t total = numel(output);
  ProfileScope ps(p, s, total, total, 0);
  if (total == 0) return ps.finish();
  int n = collapse_axes(ax, nd);
  // tiled path: the innermost output axis is strided in the input and another axis is the input's contiguous one
  int b = -1;
  for (int d = 0; d < n - 1; ++d)
    if (ax[d].stride == 1) b = d;
  bool fits = total < (1ll << 31);
  if (n >= 2 && ax[n - 1].stride != 1 && b >= 0 && ax[b].ext >= 8 && ax[n - 1].ext >= 8 && fits) {
    TileGeo g{};
    g.ext_a = ax[n - 1].ext;
    g.ext_b = ax[b].ext;
    g.in_stride_a = ax[n - 1].stride;
    g.out_stride_b = ax[b].stride2;
    const int64_t ta = (g.ext_a + kTile - 1) / kTile, tb = (g.ext_b + kTile - 1) / kTile;
    g.tiles_a = FastDiv(static_cast<uint32_t>(ta));
    g.tiles_b = FastDiv(static_cast<uint32_t>(tb));
    int64_t blocks = ta * tb;
    for (int d = 0; d < n - 1; ++d) {
      if (d == b) continue;
      g.rest_ext[g.nrest] = FastDiv(static_cast<uint32_t>(ax[d].ext));
      g.rest_in[g.nrest] = ax[d].stride;
      g.rest_out[g.nrest] = ax[d].stride2;
      ++g.nrest;
      blocks *= ax[d].ext;
    }
    if (blocks < (1ll << 31)) {
      hipLaunchKernelGGL(transpose_tiled_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s, cf(input),
                         mf(output), g);
      return ps.finish();
    }
  }
  gather(cf(input), mf(output), ax, n, 0.f, s);
  return ps.finish();
}

int DLGpuOneHot(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle) {
  TS_REQUIRE(input && output && input->data && output->data, "DLGpuOneHot: NULL array");
  TS_REQUIRE(output->ndim == input->ndim + 1, "DLGpuOneHot: output rank must be input rank + 1");
  for (int d = 0; d < input->ndim; ++d)
    TS_REQUIRE(input->shape[d] == output->shape[d], "DLGpuOneHot: leading output axes must equal the input shape");
  const int64_t classes = output->shape[output->ndim - 1], total = numel(output);
  TS_REQUIRE(classes < (1ll << 24), "DLGpuOneHot: class count must stay exactly representable in float32");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  if (total > 0) {
    if (classes % 4 == 0 && aligned16(output->data))
      hipLaunchKernelGGL(one_hot_kernel<4>, dim3(blocks_for(total / 4)), dim3(kThreads), 0, s, cf(input), mf(output),
                         FastDiv(static_cast<uint32_t>(classes / 4)), total / 4);
    else
      hipLaunchKernelGGL(one_hot_kernel<1>, dim3(blocks_for(total)), dim3(kThreads), 0, s, cf(input), mf(output),
                         FastDiv(static_cast<uint32_t>(classes)), total);
  }
  return ps.finish();
}

int DLGpuEmbeddingLookUp(const DLArrayHandle input, const DLArrayHandle ids, DLArrayHandle output,
                         DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input && ids && output && input->data && ids->data && output->data, "DLGpuEmbeddingLookUp: NULL array");
  TS_REQUIRE(input->ndim == 2, "DLGpuEmbeddingLookUp: the table must be 2-D");
  TS_REQUIRE(output->ndim == ids->ndim + 1, "DLGpuEmbeddingLookUp: output rank must be ids rank + 1");
  for (int d = 0; d < ids->ndim; ++d)
    TS_REQUIRE(ids->shape[d] == output->shape[d], "DLGpuEmbeddingLookUp: leading output axes must equal the ids shape");
  const int64_t width = input->shape[1], vocab = input->shape[0], rows = numel(ids);
  TS_REQUIRE(output->shape[output->ndim - 1] == width, "DLGpuEmbeddingLookUp: last output axis must be the table width");
  TS_REQUIRE(width < (1ll << 31), "DLGpuEmbeddingLookUp: table too wide");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(input) + rows, numel(output), 0);
  const int64_t total = rows * width;
  if (total > 0) {
    if (width % 4 == 0 && aligned16(input->data) && aligned16(output->data))
      hipLaunchKernelGGL(embedding_kernel<float4>, dim3(blocks_for(total / 4)), dim3(kThreads), 0, s,
                         static_cast<const float4 *>(input->data), cf(ids), static_cast<float4 *>(output->data),
                         FastDiv(static_cast<uint32_t>(width / 4)), vocab, total / 4);
    else
      hipLaunchKernelGGL(embedding_kernel<float>, dim3(blocks_for(total)), dim3(kThreads), 0, s, cf(input), cf(ids),
                         mf(output), FastDiv(static_cast<uint32_t>(width)), vocab, total);
  }
  return ps.finish();
}

int DLGpuEmbeddingLookUp_Gradient(const DLArrayHandle output_grad, const DLArrayHandle ids, DLArrayHandle input_grad,
                                  DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(output_grad && ids && input_grad && output_grad->data && ids->data && input_grad->data,
             "DLGpuEmbeddingLookUp_Gradient: NULL array");
  TS_REQUIRE(input_grad->ndim == 2, "DLGpuEmbeddingLookUp_Gradient: the table gradient must be 2-D");
  TS_REQUIRE(output_grad->ndim == ids->ndim + 1, "DLGpuEmbeddingLookUp_Gradient: gradient rank must be ids rank + 1");
  for (int d = 0; d < ids->ndim; ++d)
    TS_REQUIRE(ids->shape[d] == output_grad->shape[d],
               "DLGpuEmbeddingLookUp_Gradient: leading gradient axes must equal the ids shape");
  const int64_t width = input_grad->shape[1], vocab = input_grad->shape[0], rows = numel(ids);
  TS_REQUIRE(output_grad->shape[output_grad->ndim - 1] == width,
             "DLGpuEmbeddingLookUp_Gradient: last gradient axis must be the table width");
  TS_REQUIRE(width < (1ll << 31), "DLGpuEmbeddingLookUp_Gradient: table too wide");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(p, s, numel(output_grad) + rows, numel(input_grad), 0);
  const int64_t n_table = numel(input_grad), total = rows * width;
  if (n_table > 0) hipLaunchKernelGGL(zero_kernel, dim3(blocks_for(n_table)), dim3(kThreads), 0, s, mf(input_grad), n_table);
  if (total > 0)
    hipLaunchKernelGGL(embedding_grad_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, s, cf(output_grad), cf(ids),
                       mf(input_grad), FastDiv(static_cast<uint32_t>(width)), vocab, total);
  return ps.finish();
}

}  // extern "C"
