// Filter gradient of the Winograd F(4x4, 3x3) convolution in ONE kernel (plus the small final transform):
//   dU[xi][o][c] = sum over tiles (A dy A^T)[xi][o][tile] * (B^T d B)[xi][c][tile],   dw = G^T dU G.
// The three-kernel routine writes both transformed tensors (2.25 times the activations each) to memory and
// reads them back; with few channels that traffic is what it spends its time on.  Here a block transforms
// the patches of 8 tiles on the way into LDS and multiplies them there.
//
// The result of one (64 produced) x (64 gathered) band, 36 x 64 x 64 sums, is more than a block's registers
// hold, so the 36 points are dealt to six blocks: block group R owns row R of the 6 x 6 grid of points (6
// points: 24 accumulator tiles of 16 x 16 per wave, 96 registers a lane, so that two blocks share a compute
// unit and one multiplies while the other loads, transforms or waits).  Of B^T d B it needs row R only: one of
// the six first-pass combinations of each patch column (from three or four of the patch's six rows), then the
// full second pass on that row; the same for A dy A^T.  So the six groups together do the arithmetic of one
// full transform; only the loads of the patches are repeated (from the L2: the groups of a tile range run
// side by side).
//
// A block walks a contiguous range of tiles (numbered image-major, so 8 consecutive tiles are neighbours in a
// row of tiles) in steps of 8:
//   * thread (slot = t % 8, cg = t / 8) transforms, for tile slot `slot`, the patches of gathered channels
//     cg and cg + 32 and the tiles of produced channels cg and cg + 32 of its band, from registers that were
//     loaded during the previous step's products (aligned quads through buffer loads; rows and tiles outside the
//     tensor get an offset beyond the buffer and read as zeros; the two patch columns beside a quad are columns
//     of the neighbouring tiles' quads, so their first-pass values come from the neighbouring lanes - for the
//     slots at the ends from the step before and the step after, which is why the second pass runs one step
//     behind the first), and stores the 6 points of each into LDS;
//   * wave w owns produced channels 16 w .. 16 w + 15 of the band: per point one 8-byte LDS read of Y (a lane's
//     two values are tiles 2 j, 2 j + 1, j = lane / 16: the depth index of two successive matrix instructions)
//     and four of X (the four blocks of 16 gathered channels), then 8 v_mfma_f32_16x16x4_f32.
// At the end the block stores its 6 x 64 x 64 partial sums; wino_filter_grad_kernel adds the ranges' partial
// sums in a fixed order and applies G^T . G, as for the three-kernel routine.
//
// Included by winograd.hip behind wino_fused.h (buffer loads, lane shifts) and the filter gradient's
// transforms (a_rows).
#pragma once

namespace fgrad {

using fused::buf_load4;
using fused::f32x4;
using fused::from_lane_above;
using fused::from_lane_below;
using fused::kBufFlagsF;
using fused::kOobF;

typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kStep = 8;      // tiles per step
constexpr int kPts = 6;       // points per block: one row of the 6 x 6 grid
constexpr int kBandF = 64;    // channels per band, produced and gathered
// LDS layout of one operand: [point][block of 16 channels][j = slot / 2][channel % 16][slot % 2], so that the 8 bytes a
// lane reads (its channel, slots 2 j and 2 j + 1) lie lane after lane; a j-group starts 16 words further on than it
// would, so that the transforms' stores (8 slots x 8 channels per wave) spread over all banks
constexpr int kJPitch = 16 * 2 + 16;              // words per j-group
constexpr int kBlockWords = 4 * kJPitch;          // words per (point, block of 16 channels)
constexpr int kOperandWords = kPts * 4 * kBlockWords;

struct FGradGeo {
  int C, O;                   // channels of x / of dy (multiples of 64)
  int H, W;                   // plane (multiples of 4)
  int tw, th;                 // tiles per plane
  int tiles;                  // images * th * tw
  int steps_per_range, ranges;
  int cbands, obands;
  int items;                  // ranges * obands * cbands * 6: one per block
};

// row R of B^T applied to (d0 .. d5), with bt_rows' expressions (entries the row does not read are never touched)
template <int R>
__device__ __forceinline__ float bt_row(const float d[6]) {
  if constexpr (R == 0) return 4.0f * d[0] - 5.0f * d[2] + d[4];
  if constexpr (R == 1) return d[3] + d[4] - 4.0f * (d[1] + d[2]);
  if constexpr (R == 2) return 4.0f * (d[1] - d[2]) - d[3] + d[4];
  if constexpr (R == 3) return 2.0f * (d[3] - d[1]) - d[2] + d[4];
  if constexpr (R == 4) return 2.0f * (d[1] - d[3]) - d[2] + d[4];
  return 4.0f * d[1] - 5.0f * d[3] + d[5];
}
// which of the patch's six rows row R of B^T reads
template <int R>
constexpr bool x_row_used(int a) {
  return R == 0 ? (a == 0 || a == 2 || a == 4) : R == 5 ? (a == 1 || a == 3 || a == 5) : (a >= 1 && a <= 4);
}
// row R of A applied to (d0 .. d3), with a_rows' expressions
template <int R>
__device__ __forceinline__ float a_row(const float d[4]) {
  if constexpr (R == 0) return d[0];
  if constexpr (R == 5) return d[3];
  const float e = d[0] + d[2], f = d[1] + d[3], p = d[0] + 4.0f * d[2], q = 2.0f * d[1] + 8.0f * d[3];
  if constexpr (R == 1) return e + f;
  if constexpr (R == 2) return e - f;
  if constexpr (R == 3) return p + q;
  return p - q;
}
template <int R>
constexpr bool y_row_used(int a) {
  return R == 0 ? a == 0 : R == 5 ? a == 3 : true;
}

// what a thread holds of a step between its loads and its first pass: per channel k the quads of the patch rows
// its group reads and the quads of the gradient tile's rows
struct Raw {
  f32x4 xq[2][6];
  f32x4 yq[2][4];
};

// where a thread's tile lies
struct TileAt {
  int n, ty, tx;
  bool live;
};

template <int R>
__device__ __forceinline__ void load_raw(__amdgpu_buffer_rsrc_t rx, __amdgpu_buffer_rsrc_t ry, const FGradGeo &g, const TileAt &at,
                                         const unsigned xc[2], const unsigned yc[2], Raw &raw) {
  const unsigned row_bytes = static_cast<unsigned>(g.W) * 4u, plane_bytes = row_bytes * static_cast<unsigned>(g.H);
  // byte offset of the quad in patch row 1 (image row 4 ty) of channel 0 of the image
  const unsigned x0 = static_cast<unsigned>(at.n) * static_cast<unsigned>(g.C) * plane_bytes +
                      static_cast<unsigned>(4 * at.ty) * row_bytes + static_cast<unsigned>(16 * at.tx);
  const unsigned y0 = static_cast<unsigned>(at.n) * static_cast<unsigned>(g.O) * plane_bytes +
                      static_cast<unsigned>(4 * at.ty) * row_bytes + static_cast<unsigned>(16 * at.tx);
  const bool top = at.ty > 0, bottom = at.ty < g.th - 1;       // patch rows 0 / 5 lie inside the plane
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const unsigned base = at.live ? x0 + xc[k] : kOobF;
#pragma unroll
    for (int a = 0; a < 6; ++a) {
      if (!x_row_used<R>(a)) continue;
      if (a == 0)
        raw.xq[k][0] = buf_load4(rx, at.live && top ? base - row_bytes : kOobF, 0u);
      else if (a == 5)
        raw.xq[k][5] = buf_load4(rx, at.live && bottom ? base : kOobF, 4u * row_bytes);
      else
        raw.xq[k][a] = buf_load4(rx, base, static_cast<unsigned>(a - 1) * row_bytes);
    }
    const unsigned ybase = at.live ? y0 + yc[k] : kOobF;
#pragma unroll
    for (int a = 0; a < 4; ++a)
      if (y_row_used<R>(a)) raw.yq[k][a] = buf_load4(ry, ybase, static_cast<unsigned>(a) * row_bytes);
  }
}

// The first pass of a step: row R of B^T (of A) applied down the four columns of every quad.  A patch's two
// outer columns are columns of the neighbouring tiles' quads (patch column 0 is the left neighbour's quad
// column 3, patch column 5 the right neighbour's quad column 0), so their first-pass values are the
// neighbours' and are fetched from them in the second pass: nothing beside the quads is ever loaded.
struct Half {
  float x[2][4];     // per channel k: first pass of quad columns 0 .. 3 = patch columns 1 .. 4
  float y[2][4];
  bool has_left, has_right;     // the tile has a neighbour in its row of tiles
};

template <int R>
__device__ __forceinline__ void first_pass(const Raw &raw, Half &h) {
#pragma unroll
  for (int k = 0; k < 2; ++k) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float col[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int a = 0; a < 6; ++a)
        if (x_row_used<R>(a)) col[a] = raw.xq[k][a][q];
      h.x[k][q] = bt_row<R>(col);
      float row[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int a = 0; a < 4; ++a)
        if (y_row_used<R>(a)) row[a] = raw.yq[k][a][q];
      h.y[k][q] = a_row<R>(row);
    }
  }
}

// the value of the lane 7 above / below within a row of 16 lanes: for slot 0 the same channel's slot 7 and
// the other way round (a row of 16 lanes is two channels' 8 slots)
__device__ __forceinline__ float from_lane_7_above(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x107, 0xf, 0xf, false));
}
__device__ __forceinline__ float from_lane_7_below(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x117, 0xf, 0xf, false));
}

// The second pass of step s, one step late: `cur` is the first pass of step s, `before_x3` quad column 3 of
// step s - 1 and `after` the first pass of step s + 1 (slot 0's left neighbour is slot 7 of the step before, slot
// 7's right neighbour slot 0 of the step after).  The 6 points of every patch and gradient tile go into LDS
// (layout above); channel cg + 32 k is channel cg % 16 of block cg / 16 + 2 k.
__device__ __forceinline__ void second_pass(const Half &cur, const float before_x3[2], const Half &after, int slot, int cg,
                                            float *__restrict__ Xl, float *__restrict__ Yl) {
  const int word = (cg >> 4) * kBlockWords + (slot >> 1) * kJPitch + (cg & 15) * 2 + (slot & 1);
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const float left_in = from_lane_below(cur.x[k][3]), left_out = from_lane_7_above(before_x3[k]);
    const float right_in = from_lane_above(cur.x[k][0]), right_out = from_lane_7_below(after.x[k][0]);
    const float t[6] = {!cur.has_left ? 0.0f : slot > 0 ? left_in : left_out, cur.x[k][0], cur.x[k][1], cur.x[k][2], cur.x[k][3],
                        !cur.has_right ? 0.0f : slot < kStep - 1 ? right_in : right_out};
    float v[6];
    bt_rows(t, v);
    float *dst = Xl + word + 2 * k * kBlockWords;
#pragma unroll
    for (int q = 0; q < 6; ++q) dst[q * (4 * kBlockWords)] = v[q];
  }
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    float v[6];
    a_rows(cur.y[k], v);
    float *dst = Yl + word + 2 * k * kBlockWords;
#pragma unroll
    for (int q = 0; q < 6; ++q) dst[q * (4 * kBlockWords)] = v[q];
  }
}

template <int R>
__device__ __forceinline__ void fgrad_block(const float *__restrict__ x, const float *__restrict__ dy, float *__restrict__ part,
                                            const FGradGeo &g, int range, int ob, int cb, float *__restrict__ lds) {
  float *Xl = lds, *Yl = lds + kOperandWords;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int slot = t & (kStep - 1), cg = t >> 3;
  const unsigned plane_bytes = static_cast<unsigned>(g.H) * static_cast<unsigned>(g.W) * 4u;
  const int per_img = g.th * g.tw, imgs = g.tiles / per_img;
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(x), 0, static_cast<int>(static_cast<unsigned>(imgs) * static_cast<unsigned>(g.C) * plane_bytes), kBufFlagsF);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(dy), 0, static_cast<int>(static_cast<unsigned>(imgs) * static_cast<unsigned>(g.O) * plane_bytes), kBufFlagsF);
  unsigned xc[2], yc[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    xc[k] = static_cast<unsigned>(cb * kBandF + cg + 32 * k) * plane_bytes;
    yc[k] = static_cast<unsigned>(ob * kBandF + cg + 32 * k) * plane_bytes;
  }
  const int steps = (g.tiles + kStep - 1) / kStep;
  const int step0 = range * g.steps_per_range, step1 = min(steps, step0 + g.steps_per_range);

  f32x4 acc[kPts][4];
#pragma unroll
  for (int e = 0; e < kPts; ++e)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[e][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  // Iteration s of the loop does the first pass of step s and the second pass and the products of step s - 1;
  // in front of it, the first passes of steps step0 - 1 and step0 (the tiles that border the range belong to other
  // blocks, but their quads hold the outer columns of the range's first and last tile).
  TileAt at;          // this thread's tile in the step being loaded
  {
    const int ti = (step0 - 1) * kStep + slot;
    at.live = ti >= 0 && ti < g.tiles;
    const int tl = at.live ? ti : 0;
    at.n = tl / per_img;
    const int rem = tl - at.n * per_img;
    at.ty = rem / g.tw;
    at.tx = at.live ? rem - at.ty * g.tw : slot - kStep;       // (before the first tile: 8 further on is tile `slot`)
  }
  auto advance = [&](int next_step) {
    at.tx += kStep;
    while (at.tx >= g.tw) {
      at.tx -= g.tw;
      ++at.ty;
    }
    while (at.ty >= g.th) {
      at.ty -= g.th;
      ++at.n;
    }
    at.live = next_step <= step1 && next_step * kStep + slot < g.tiles;
  };
  Raw raw;
  Half cur;                     // first pass of step s - 1
  float before_x3[2];           // quad column 3 of step s - 2
  load_raw<R>(rx, ry, g, at, xc, yc, raw);
  first_pass<R>(raw, cur);
#pragma unroll
  for (int k = 0; k < 2; ++k) before_x3[k] = cur.x[k][3];
  advance(step0);
  load_raw<R>(rx, ry, g, at, xc, yc, raw);
  first_pass<R>(raw, cur);
  cur.has_left = at.tx > 0;
  cur.has_right = at.tx < g.tw - 1;
  advance(step0 + 1);
  load_raw<R>(rx, ry, g, at, xc, yc, raw);
  // a lane's 8-byte word of (point e, block b of 16 channels): word index e * kPointVecs + b * kBlockVecs + this
  constexpr int kBlockVecs = kBlockWords / 2, kPointVecs = 4 * kBlockVecs;
  const int lane_vec = (lane >> 4) * (kJPitch / 2) + (lane & 15);
  const f32x2 *Xv = reinterpret_cast<const f32x2 *>(Xl) + lane_vec;
  const f32x2 *Yv = reinterpret_cast<const f32x2 *>(Yl) + wave * kBlockVecs + lane_vec;

  for (int step = step0 + 1; step <= step1; ++step) {
    // two LDS buffers take turns, so that one barrier a step is enough: a wave writes the points of the next step
    // while slower waves still read the other buffer, and by the time it writes this buffer again every wave
    // has passed the barrier behind the step in between, that is, has finished reading it
    const int buf = (step & 1) * (2 * kOperandWords);
    {
      Half after;
      first_pass<R>(raw, after);
      after.has_left = at.tx > 0;
      after.has_right = at.tx < g.tw - 1;
      second_pass(cur, before_x3, after, slot, cg, Xl + buf, Yl + buf);
#pragma unroll
      for (int k = 0; k < 2; ++k) before_x3[k] = cur.x[k][3];
      cur = after;
    }
    __syncthreads();
    advance(step + 1);         // the next step's tile of this thread: 8 further on in the image-major numbering
    load_raw<R>(rx, ry, g, at, xc, yc, raw);
    // (the scheduling barriers keep those loads in front of the products, which cover their way from memory, and
    // every point's LDS reads one point ahead of its products: left alone the compiler sinks the loads behind
    // the products and the reads next to their uses)
    __builtin_amdgcn_sched_barrier(0);
    const f32x2 *Xb = Xv + buf / 2, *Yb = Yv + buf / 2;
    f32x2 a = Yb[0], b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = Xb[j * kBlockVecs];
#pragma unroll
    for (int e = 0; e < kPts; ++e) {
      f32x2 an = a, bn[4] = {b[0], b[1], b[2], b[3]};
      if (e + 1 < kPts) {
        an = Yb[(e + 1) * kPointVecs];
#pragma unroll
        for (int j = 0; j < 4; ++j) bn[j] = Xb[(e + 1) * kPointVecs + j * kBlockVecs];
      }
      __builtin_amdgcn_sched_barrier(0);
      // (a matrix instruction that accumulates into the result of the one before it waits for it: the four
      // accumulators of a point take turns)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[e][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b[j].x, acc[e][j], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[e][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b[j].y, acc[e][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      a = an;
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = bn[j];
    }
  }

  // partial sums of this range: part[((range * 36) + point) * O * C + o * C + c]
  const int64_t oc = static_cast<int64_t>(g.O) * g.C;
  float *out = part + (static_cast<int64_t>(range) * 36 + kPts * R) * oc +
               static_cast<int64_t>(ob * kBandF + 16 * wave + 4 * (lane >> 4)) * g.C + cb * kBandF + (lane & 15);
#pragma unroll
  for (int e = 0; e < kPts; ++e)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) out[e * oc + static_cast<int64_t>(v) * g.C + 16 * j] = acc[e][j][v];
}

// grid: items rounded up to a multiple of 8 blocks; item = ((range * obands + ob) * cbands + cb) * 6 + group, dealt to
// the 8 XCDs in contiguous stretches so that the blocks of one range (which read the same activations) share an L2
__global__ __launch_bounds__(256, 2) void wino_fgrad_fused_kernel(const float *__restrict__ x, const float *__restrict__ dy,
                                                                  float *__restrict__ part, FGradGeo g) {
  __shared__ __attribute__((aligned(16))) float lds[2 * 2 * kOperandWords];      // two buffers of 36 864 bytes
  const int per_xcd = gridDim.x >> 3;
  const int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (item >= g.items) return;
  const int group = item % 6, rest = item / 6;
  const int cb = rest % g.cbands, ob = (rest / g.cbands) % g.obands, range = rest / (g.cbands * g.obands);
  switch (group) {
    case 0: fgrad_block<0>(x, dy, part, g, range, ob, cb, lds); break;
    case 1: fgrad_block<1>(x, dy, part, g, range, ob, cb, lds); break;
    case 2: fgrad_block<2>(x, dy, part, g, range, ob, cb, lds); break;
    case 3: fgrad_block<3>(x, dy, part, g, range, ob, cb, lds); break;
    case 4: fgrad_block<4>(x, dy, part, g, range, ob, cb, lds); break;
    default: fgrad_block<5>(x, dy, part, g, range, ob, cb, lds); break;
  }
}

// ranges of tiles: as many as fill one to three rounds of two blocks per compute unit best, each at least 16 steps long
inline void fgrad_plan(FGradGeo &g, int cus) {
  const int steps = (g.tiles + kStep - 1) / kStep;
  const int per_range = 6 * g.obands * g.cbands, slots = 2 * cus;
  const int max_ranges = std::max(1, steps / 16);
  int best = 1;
  double best_fill = 0.0;
  for (int rounds = 1; rounds <= 3; ++rounds) {
    const int ranges = std::min(max_ranges, std::max(1, rounds * slots / per_range));
    const int blocks = ranges * per_range;
    const double fill = static_cast<double>(blocks) / (static_cast<double>((blocks + slots - 1) / slots) * slots);
    if (fill > best_fill + 0.02) {
      best_fill = fill;
      best = ranges;
    }
  }
  g.steps_per_range = (steps + best - 1) / best;
  g.ranges = (steps + g.steps_per_range - 1) / g.steps_per_range;      // no empty range
  g.items = g.ranges * per_range;
}

}  // namespace fgrad
