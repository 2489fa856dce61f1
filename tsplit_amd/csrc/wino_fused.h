// Winograd F(4x4, 3x3) in ONE kernel for layers that produce their output in bands of 64 channels from
// a multiple of 16 gathered channels (the caller takes it up to 256 on either side): the input transform happens on the way into LDS and the output transform
// comes straight from the accumulators, so neither V nor M (2.25 times the activations each) touches
// memory.  With so few channels the three-kernel routine is bound by exactly that traffic (a 64 -> 64
// layer at 224 x 224 moves 2.3 GB for 0.4 GB of activations); here the activations are read once per
// band and written once, and the transformed filter comes from the L2 cache.
//
// Included by winograd.hip behind its transforms (g_rows, bt_rows, at_rows).
//
// One block of 256 threads (4 waves) owns a group of at most 16 tiles of one image (a rectangle of gw x gh tiles:
// 8 x 2 at 224 x 224, 4 x 4 at 112 x 112; or, where no rectangle fills the 16 slots as well, 16 consecutive tiles
// row after row: 56 x 56; either way neighbouring lanes hold neighbouring tiles) and one band of 64 produced
// channels, for all 36 points xi.  Two blocks share a compute unit (a wave
// needs 256 registers: 144 of them accumulators) and run out of step, so that one multiplies while the other
// transforms or waits for its activations:
//   * the gathered channels go by in chunks of 16.  A thread loads the 6 x 6 patch of one tile slot in one
//     channel of the chunk (six aligned quads, the two columns beside them from the neighbouring lanes or,
//     where the neighbouring tile is not in a neighbouring lane, from memory; zeros outside the plane),
//     transforms it (B^T d B) and stores the 36 values into LDS in the order the matrix instruction reads
//     them.  A wave's 64 threads are the 16 slots x the 4 channels that share c % 4, so that one store
//     instruction touches all 32 LDS banks (16 consecutive 16-byte words, element c / 4 of each);
//   * wave w owns produced channels 16 * w .. + 15 (and all 16 tile slots) and multiplies,
//     for every xi, U[xi] (16 channels x 16 gathered, from memory: 16 bytes per lane, laid out for this by
//     wino_filter_fused_kernel) with V[xi] (16 gathered x 16 slots, from LDS: 16 bytes per lane) in four
//     v_mfma_f32_16x16x4_f32 into its own accumulator of that xi: 36 accumulators of 4 registers;
//   * at the end every lane holds, for 4 channels and one tile, all 36 points: the output transform
//     (A^T M A) is lane-local, and the tile's four rows leave as 16-byte stores.
// Optionally each block leaves one partial (sum, sum of squares) per channel of what it stored, for a
// BatchNorm that follows.
#pragma once

namespace fused {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// the value of the lane below / above within a row of 16 lanes (a data-parallel move, no trip through LDS);
// the row's first / last lane gets its own value back and does not use it
__device__ __forceinline__ float from_lane_below(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, false));
}
__device__ __forceinline__ float from_lane_above(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x101, 0xf, 0xf, false));
}

constexpr int kThreadsF = 256;
constexpr int kSlots = 16;      // tile slots per block
constexpr int kChunk = 16;      // gathered channels per step
constexpr int kAhead = 6;       // filter words a wave keeps in flight (divides 36; 4 ran the same, 9 and 12 spill and ran 25 - 40 % slower)
constexpr int kBand = 64;       // produced channels per block

// Filter transform into the layout the kernel reads: word (chunk, xi, ob, lane) holds, for produced channel
// o = 16 * ob + lane % 16 and gathered channels c = 16 * chunk + 4 * kk + lane / 16 (kk = 0 .. 3), the four
// U[xi][o][c].  `bands` bands of 64 produced channels lie one behind the other; `slack_words` words behind
// each band's last word are read ahead by the kernel and never used.
inline size_t fused_filter_floats(int produced, int gathered) {
  const size_t band = static_cast<size_t>(gathered / kChunk) * kXi * 4 * 64 * 4;
  return static_cast<size_t>(produced / kBand) * (band + static_cast<size_t>(kAhead) * 4 * 64 * 4);
}

__global__ __launch_bounds__(256) void wino_filter_fused_kernel(const float *__restrict__ w, float *__restrict__ Uf, int produced,
                                                                int gathered, bool rotated, int slack_words) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= produced * gathered) return;
  const int o = i / gathered, c = i - o * gathered;
  const float *g = w + (rotated ? static_cast<int64_t>(c) * produced + o : static_cast<int64_t>(o) * gathered + c) * 9;
  float k[9];
#pragma unroll
  for (int j = 0; j < 9; ++j) k[j] = rotated ? g[8 - j] : g[j];
  float t[3][6];
#pragma unroll
  for (int col = 0; col < 3; ++col) g_rows(k[col], k[3 + col], k[6 + col], t[col]);
  const int band = o / kBand, ob = (o % kBand) / 16, chunk = c / kChunk, kk = (c % kChunk) / 4;
  const int lane = (c % 4) * 16 + o % 16;
  const size_t band_floats = static_cast<size_t>(gathered / kChunk) * kXi * 4 * 64 * 4 + static_cast<size_t>(slack_words) * 4 * 64 * 4;
  float *dst = Uf + band * band_floats + ((static_cast<size_t>(chunk) * kXi * 4 + ob) * 64 + lane) * 4 + kk;
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    float u[6];
    g_rows(t[0][r], t[1][r], t[2][r], u);
#pragma unroll
    for (int q = 0; q < 6; ++q) dst[static_cast<size_t>(r * 6 + q) * 4 * 64 * 4] = u[q];
  }
}

struct FusedGeo {
  int gathered, produced;   // channels
  int H, W;                 // plane (multiples of 4)
  int tw, th;               // tiles per plane
  int gw, gh;               // tiles per group, gw * gh <= 16; tw % gw == 0, th % gh == 0; gw = 0: runs of 16 tiles
  int groups_w, groups;     // groups per row of groups (rectangles only), per image
  int items;                // images * groups * bands: one per block
};

// the six quads of one thread's patch: the middle four columns of its six rows
struct Patch {
  f32x4 mid[6];
};

typedef unsigned int u32x4f __attribute__((ext_vector_type(4)));
constexpr int kBufFlagsF = 0x00020000;           // raw buffer, 32-bit untyped data
constexpr unsigned kOobF = 0x80000000u;          // an offset beyond any buffer used here: such a load returns 0

__device__ __forceinline__ f32x4 buf_load4(__amdgpu_buffer_rsrc_t rsrc, unsigned voff, unsigned soff) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0));
}

// What a thread reads of its image: byte offsets (within the image's gathered planes) of the aligned quads of
// its six patch rows in the chunk's first channel set, kOobF for rows outside the plane and for threads without
// a tile; they do not change from chunk to chunk, which advances through the scalar offset.  `edge` is the
// distance in bytes from a quad to the one value a thread at the group's edge fetches beside it (0: none).
struct PatchAddr {
  unsigned row[6];
  int edge;
};

__device__ __forceinline__ void load_patch(__amdgpu_buffer_rsrc_t rx, const PatchAddr &pa, unsigned chunk_off, Patch &p) {
#pragma unroll
  for (int r = 0; r < 6; ++r) p.mid[r] = buf_load4(rx, pa.row[r], chunk_off);
}

// B^T d B of the patch into LDS: value xi of (channel c of the chunk, slot) goes where lane
// (c % 4) * 16 + slot of every wave reads it as element c / 4 of its 16-byte word.
// The columns beside the quads come from the neighbouring lanes, which hold the neighbouring tiles of the
// same row of the group; at the group's edges they are fetched here (lines the neighbouring block's quads
// brought into the cache; zero beyond the plane) rather than held in registers through the products
// (fetching them with the quads, a step ahead, measured 8 % slower: six more loads in front of the
// filter words, which return in order).
template <bool RUNS>
__device__ __forceinline__ void transform_patch(const Patch &p, __amdgpu_buffer_rsrc_t rx, const PatchAddr &pa, unsigned chunk_off,
                                                bool at_left, bool at_right, int c, int slot, float *__restrict__ Vl) {
  float edge[6];
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    const unsigned off = (pa.edge != 0 && pa.row[r] != kOobF) ? pa.row[r] + static_cast<unsigned>(pa.edge) : kOobF;
    edge[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, off, chunk_off, 0));
  }
  float d[6][6];
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    const float from_left = from_lane_below(p.mid[r].w), from_right = from_lane_above(p.mid[r].x);
    // (zero beyond the plane: no edge value is fetched there.  In a run of consecutive tiles a thread can be at the
    // run's end on one side and at the plane's edge on the other: the one value it fetched belongs to one side only)
    d[r][0] = !at_left ? from_left : (!RUNS || pa.edge < 0) ? edge[r] : 0.0f;
    d[r][1] = p.mid[r].x;
    d[r][2] = p.mid[r].y;
    d[r][3] = p.mid[r].z;
    d[r][4] = p.mid[r].w;
    d[r][5] = !at_right ? from_right : (!RUNS || pa.edge > 0) ? edge[r] : 0.0f;
  }
  float tmp[6][6];
#pragma unroll
  for (int q = 0; q < 6; ++q) {
    const float col[6] = {d[0][q], d[1][q], d[2][q], d[3][q], d[4][q], d[5][q]};
    bt_rows(col, tmp[q]);
  }
  float *dst = Vl + ((c & 3) * 16 + slot) * 4 + (c >> 2);
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    const float row[6] = {tmp[0][r], tmp[1][r], tmp[2][r], tmp[3][r], tmp[4][r], tmp[5][r]};
    float v[6];
    bt_rows(row, v);
#pragma unroll
    for (int q = 0; q < 6; ++q) dst[(r * 6 + q) * (64 * 4)] = v[q];
  }
}

// grid: images * groups * bands work items rounded up to a multiple of 8 blocks; item i: band = i % bands (the
// items of one group of tiles, which read the same activations, follow each other), then the group, then the image.
template <bool STATS, bool RUNS>
__global__ __launch_bounds__(kThreadsF, 2) void wino_fused_kernel(const float *__restrict__ x, const float *__restrict__ Uf,
                                                               float *__restrict__ y, FusedGeo g, float *__restrict__ stats) {
  __shared__ __attribute__((aligned(16))) float Vl[kXi * 64 * 4];      // 36 864 bytes
  const int bands = g.produced / kBand;
  // Workgroup ids go round the 8 XCDs, each with its own L2: block b takes work item (b % 8) * per_xcd + b / 8,
  // so that an XCD owns a contiguous stretch of groups and the rows and columns neighbouring groups share
  // (a patch overlaps its neighbours by two rows and two columns) come from that L2 and not from memory again.
  const int per_xcd = gridDim.x >> 3;
  const int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (item >= g.items) return;
  const int band = item % bands;
  const int grp = (item / bands) % g.groups, n = item / bands / g.groups;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // ---- the loader's tile and channel: lanes 16 apart hold the channels that share c % 4
  const int slot = t & 15, cl = (((t >> 4) & 3) << 2) | wave;
  // a slot's tile, whether it exists, and whether the tile to its left / right sits in the neighbouring lane
  const auto tile_of = [&](int s, int &ty_, int &tx_, bool &left_, bool &right_) {
    if (RUNS) {      // a run of 16 consecutive tiles of the image, row after row
      const int idx = grp * kSlots + s;
      ty_ = idx / g.tw;
      tx_ = idx - ty_ * g.tw;
      left_ = s == 0 || tx_ == 0;
      right_ = s == kSlots - 1 || tx_ == g.tw - 1;
      return idx < g.tw * g.th;
    }
    const int GY = grp / g.groups_w, GX = grp - GY * g.groups_w;
    const int gy = s / g.gw, gx = s - gy * g.gw;
    ty_ = GY * g.gh + gy;
    tx_ = GX * g.gw + gx;
    left_ = gx == 0;
    right_ = gx == g.gw - 1;
    return s < g.gw * g.gh;
  };
  int ty, tx;
  bool at_left, at_right;      // the column beside the quad does not come from the neighbouring lane
  const bool live = tile_of(slot, ty, tx, at_left, at_right);
  const int64_t plane_elems = static_cast<int64_t>(g.H) * g.W;
  const unsigned plane_bytes = static_cast<unsigned>(plane_elems) * 4u;
  // the image's gathered planes as one buffer: rows outside the plane get an offset beyond it and read as zeros
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(x) + static_cast<int64_t>(n) * g.gathered * plane_elems, 0, static_cast<int>(g.gathered * plane_bytes), kBufFlagsF);
  PatchAddr pa;
  pa.edge = !live ? 0 : (at_left && tx > 0) ? -4 : (at_right && tx < g.tw - 1) ? 16 : 0;
#pragma unroll
  for (int r = 0; r < 6; ++r) {
    const int h = 4 * ty - 1 + r;
    pa.row[r] = (live && h >= 0 && h < g.H) ? static_cast<unsigned>(cl) * plane_bytes + static_cast<unsigned>(h * g.W + 4 * tx) * 4u : kOobF;
  }
  const unsigned chunk_bytes = kChunk * plane_bytes;
  // ---- the multiplier's share
  const int ob = wave;
  const int chunks = g.gathered / kChunk;
  const size_t band_floats = static_cast<size_t>(chunks) * kXi * 4 * 64 * 4 + static_cast<size_t>(kAhead) * 4 * 64 * 4;
  // the band's filter words as one buffer: word e of this lane at byte (e * 256 + ob * 64 + lane) * 16
  const __amdgpu_buffer_rsrc_t ru = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(Uf) + band * band_floats, 0,
                                                                     static_cast<int>(band_floats * 4), kBufFlagsF);
  const unsigned uoff = static_cast<unsigned>(ob * 64 + lane) * 16u;
  const f32x4 *vw = reinterpret_cast<const f32x4 *>(Vl) + lane;                                  // point xi: vw[xi * 64]

  f32x4 acc[kXi];
#pragma unroll
  for (int xi = 0; xi < kXi; ++xi) acc[xi] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  Patch patch;
  load_patch(rx, pa, 0u, patch);
  f32x4 ua[kAhead];
#pragma unroll
  for (int j = 0; j < kAhead; ++j) ua[j] = buf_load4(ru, uoff, static_cast<unsigned>(j) * 4096u);

  for (int ch = 0; ch < chunks; ++ch) {
    transform_patch<RUNS>(patch, rx, pa, static_cast<unsigned>(ch) * chunk_bytes, at_left, at_right, cl, slot, Vl);
    __syncthreads();
    if (ch + 1 < chunks) load_patch(rx, pa, static_cast<unsigned>(ch + 1) * chunk_bytes, patch);
    const unsigned ubase = static_cast<unsigned>(ch * kXi + kAhead) * 4096u;     // the word kAhead points on
    // (the scheduling barriers keep every filter word's load kAhead points ahead of its use and the LDS
    // reads a pair of points ahead: left alone the compiler sinks them next to their uses to save
    // registers and every point then waits out the cache's latency; a single point ahead was slower)
    f32x4 vb0 = vw[0], vb1 = vw[64];
#pragma unroll
    for (int xi = 0; xi < kXi; xi += 2) {
      const f32x4 b0 = vb0, b1 = vb1;
      if (xi + 2 < kXi) {
        vb0 = vw[(xi + 2) * 64];
        vb1 = vw[(xi + 3) * 64];
      }
      const f32x4 a0 = ua[xi % kAhead], a1 = ua[(xi + 1) % kAhead];
      ua[xi % kAhead] = buf_load4(ru, uoff, ubase + static_cast<unsigned>(xi) * 4096u);       // (behind the last chunk: the slack words)
      ua[(xi + 1) % kAhead] = buf_load4(ru, uoff, ubase + static_cast<unsigned>(xi + 1) * 4096u);
      __builtin_amdgcn_sched_barrier(0);
      acc[xi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.x, b0.x, acc[xi], 0, 0, 0);
      acc[xi + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.x, b1.x, acc[xi + 1], 0, 0, 0);
      acc[xi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.y, b0.y, acc[xi], 0, 0, 0);
      acc[xi + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.y, b1.y, acc[xi + 1], 0, 0, 0);
      acc[xi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.z, b0.z, acc[xi], 0, 0, 0);
      acc[xi + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.z, b1.z, acc[xi + 1], 0, 0, 0);
      acc[xi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.w, b0.w, acc[xi], 0, 0, 0);
      acc[xi + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.w, b1.w, acc[xi + 1], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  }

  // ---- output transform from the accumulators: lane holds channels o0 .. o0 + 3 of tile slot `os`
  const int os = lane & 15;
  int oty, otx;
  bool unused_left, unused_right;
  const bool olive = tile_of(os, oty, otx, unused_left, unused_right);
  const int o0 = band * kBand + ob * 16 + (lane >> 4) * 4;
  float s[4] = {0.0f, 0.0f, 0.0f, 0.0f}, sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int r4 = 0; r4 < 4; ++r4) {
    float tmp[6][4];
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      const float col[6] = {acc[q][r4], acc[6 + q][r4], acc[12 + q][r4], acc[18 + q][r4], acc[24 + q][r4], acc[30 + q][r4]};
      at_rows(col, tmp[q]);
    }
    float *plane = y + (static_cast<int64_t>(n) * g.produced + o0 + r4) * plane_elems + static_cast<int64_t>(4 * oty) * g.W + 4 * otx;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float row[6] = {tmp[0][r], tmp[1][r], tmp[2][r], tmp[3][r], tmp[4][r], tmp[5][r]};
      float v[4];
      at_rows(row, v);
      if (olive) {
        *reinterpret_cast<f32x4 *>(plane + static_cast<int64_t>(r) * g.W) = f32x4{v[0], v[1], v[2], v[3]};
        if (STATS) {
          s[r4] += (v[0] + v[1]) + (v[2] + v[3]);
          sq[r4] += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        }
      }
    }
  }
  if (STATS) {
    // the 16 lanes that share lane / 16 hold the same four channels: one partial per block and channel
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
#pragma unroll
      for (int m = 1; m < 16; m <<= 1) {
        s[r4] += __shfl_xor(s[r4], m);
        sq[r4] += __shfl_xor(sq[r4], m);
      }
    }
    if ((lane & 15) == 0) {
      const int64_t k = item / bands;     // partial index: (image, group)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        float *dst = stats + (k * g.produced + o0 + r4) * 2;
        dst[0] = s[r4];
        dst[1] = sq[r4];
      }
    }
  }
}

// How a plane's tw x th tiles are dealt to groups of at most 16: the largest rectangle (wider first, at least two wide)
// that tiles the plane exactly, or - where that leaves more slots empty - runs of 16 consecutive tiles, row after
// row (gw = 0; 14 x 14 tiles: 13 runs with 196 of 208 slots filled, where rows of 14 fill 14 of 16).  False if
// less than three quarters of the slots would carry a tile.
inline bool fused_group(int tw, int th, int &gw, int &gh, int &groups) {
  int best = 0;
  for (int w = 2; w <= tw && w <= kSlots; ++w) {
    if (tw % w) continue;
    for (int h = 1; h <= th && w * h <= kSlots; ++h) {
      if (th % h) continue;
      if (w * h > best || (w * h == best && w > gw)) {
        best = w * h;
        gw = w;
        gh = h;
      }
    }
  }
  const int tiles = tw * th, runs = (tiles + kSlots - 1) / kSlots;
  if (best > 0 && best * runs >= tiles) {        // the rectangles fill their slots at least as well
    groups = (tw / gw) * (th / gh);
    return best >= 12;
  }
  gw = gh = 0;
  groups = runs;
  return 4 * tiles >= 3 * runs * kSlots;
}

}  // namespace fused
