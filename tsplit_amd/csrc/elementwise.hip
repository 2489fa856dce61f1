// HBM-streaming elementwise kernels: graph-closure ops, Relu, elementwise math, Where and
// the optimizer updates.
//
// One template serves all of them.  Every thread moves one 16-byte word per array,
// consecutive lanes touch consecutive words, and loads and stores are non-temporal: these
// tensors are far larger than the caches and are touched once per kernel, and on MI355X a
// read+write stream measured 6.5 TB/s this way against 5.7 TB/s with 4 words per thread and
// cached accesses.  Arrays that are not 16-byte aligned (micro-tensor views can start
// anywhere on a 4-byte boundary) take the scalar variant.
#include <array>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "common.h"

namespace tsplit {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 1;
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int N>
struct Ptrs {
  float *p[N];
};

// Op contract: static constexpr int N (arrays), LOAD / STORE bit masks over the arrays,
// and  __device__ void apply(float (&v)[N]) const  transforming one element of each.
template <class Op>
__global__ __launch_bounds__(kThreads) void ew_vec_kernel(Op op, Ptrs<Op::N> a, int64_t n) {
  constexpr int N = Op::N;
  const int64_t n4 = n >> 2;
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * kUnroll) * kThreads + threadIdx.x;
  f32x4 v[kUnroll][N];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t i = first + static_cast<int64_t>(u) * kThreads;
    if (i < n4) {
#pragma unroll
      for (int k = 0; k < N; ++k)
        if (Op::LOAD & (1 << k)) v[u][k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(a.p[k]) + i);
    }
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t i = first + static_cast<int64_t>(u) * kThreads;
    if (i < n4) {
      float e[4][N];
#pragma unroll
      for (int k = 0; k < N; ++k) {
        e[0][k] = v[u][k].x;
        e[1][k] = v[u][k].y;
        e[2][k] = v[u][k].z;
        e[3][k] = v[u][k].w;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) op.apply(e[j]);
#pragma unroll
      for (int k = 0; k < N; ++k)
        if (Op::STORE & (1 << k)) {
          const f32x4 r = {e[0][k], e[1][k], e[2][k], e[3][k]};
          __builtin_nontemporal_store(r, reinterpret_cast<f32x4 *>(a.p[k]) + i);
        }
    }
  }
  // the last (n % 4) elements
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
    const int64_t i = (n4 << 2) + threadIdx.x;
    float e[N];
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (Op::LOAD & (1 << k)) e[k] = a.p[k][i];
    op.apply(e);
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (Op::STORE & (1 << k)) a.p[k][i] = e[k];
  }
}

template <class Op>
__global__ __launch_bounds__(kThreads) void ew_scalar_kernel(Op op, Ptrs<Op::N> a, int64_t n) {
  constexpr int N = Op::N;
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * kUnroll) * kThreads + threadIdx.x;
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t i = first + static_cast<int64_t>(u) * kThreads;
    if (i < n) {
      float e[N];
#pragma unroll
      for (int k = 0; k < N; ++k)
        if (Op::LOAD & (1 << k)) e[k] = a.p[k][i];
      op.apply(e);
#pragma unroll
      for (int k = 0; k < N; ++k)
        if (Op::STORE & (1 << k)) a.p[k][i] = e[k];
    }
  }
}

template <class Op>
void launch(Op op, Ptrs<Op::N> a, int64_t n, hipStream_t s) {
  if (n <= 0) return;
  bool vec = true;
  for (int k = 0; k < Op::N; ++k) vec = vec && aligned16(a.p[k]);
  const int64_t per_block = static_cast<int64_t>(kThreads) * kUnroll;
  if (vec) {
    const int64_t n4 = n >> 2;
    int64_t blocks = (n4 + per_block - 1) / per_block;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(ew_vec_kernel<Op>, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s, op, a, n);
  } else {
    const int64_t blocks = (n + per_block - 1) / per_block;
    hipLaunchKernelGGL(ew_scalar_kernel<Op>, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0, s, op, a, n);
  }
}

// ---- ops.  Array 0 is the output unless noted. ----
struct SetOp {   // out = c
  static constexpr int N = 1, LOAD = 0, STORE = 1;
  float c;
  __device__ void apply(float (&v)[1]) const { v[0] = c; }
};
struct CopyOp {  // out = a
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  __device__ void apply(float (&v)[2]) const { v[0] = v[1]; }
};
struct AddOp {   // out = a + b
  static constexpr int N = 3, LOAD = 6, STORE = 1;
  __device__ void apply(float (&v)[3]) const { v[0] = v[1] + v[2]; }
};
struct MulOp {
  static constexpr int N = 3, LOAD = 6, STORE = 1;
  __device__ void apply(float (&v)[3]) const { v[0] = v[1] * v[2]; }
};
struct AddConstOp {
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  float c;
  __device__ void apply(float (&v)[2]) const { v[0] = v[1] + c; }
};
struct MulConstOp {
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  float c;
  __device__ void apply(float (&v)[2]) const { v[0] = v[1] * c; }
};
struct ReluOp {
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  __device__ void apply(float (&v)[2]) const { v[0] = fmaxf(v[1], 0.f); }
};
struct ReluGradOp {   // out = (sign(x)+1)*0.5*dy ; arrays: out, x, dy
  static constexpr int N = 3, LOAD = 6, STORE = 1;
  __device__ void apply(float (&v)[3]) const {
    const float x = v[1];
    const float sgn = x > 0.f ? 1.f : (x < 0.f ? -1.f : x);   // keeps +-0 and NaN like np.sign
    v[0] = (sgn + 1.f) * 0.5f * v[2];
  }
};
struct DivOp {    // out = a / b
  static constexpr int N = 3, LOAD = 6, STORE = 1;
  __device__ void apply(float (&v)[3]) const { v[0] = v[1] / v[2]; }
};
struct DivConstOp {   // out = c / a  (src/ops/DivideConst.cu:6)
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  float c;
  __device__ void apply(float (&v)[2]) const { v[0] = c / v[1]; }
};
struct NegOp {
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  __device__ void apply(float (&v)[2]) const { v[0] = -v[1]; }
};
struct SqrtOp {
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  __device__ void apply(float (&v)[2]) const { v[0] = sqrtf(v[1]); }
};
struct RsqrtOp {  // correctly rounded quotient rather than the approximate rsqrt instruction
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  __device__ void apply(float (&v)[2]) const { v[0] = 1.f / sqrtf(v[1]); }
};
struct TanhOp {
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  __device__ void apply(float (&v)[2]) const { v[0] = tanhf(v[1]); }
};
struct SigmoidOp {   // 1/(1+1/exp(x)) (src/ops/Sigmoid.cu:6); saturates to 0 and 1 without NaN
  static constexpr int N = 2, LOAD = 2, STORE = 1;
  __device__ void apply(float (&v)[2]) const { v[0] = 1.f / (1.f + expf(-v[1])); }
};
struct WhereOp {     // out = cond != 0 ? a : b ; arrays: out, cond, a, b
  static constexpr int N = 4, LOAD = 14, STORE = 1;
  __device__ void apply(float (&v)[4]) const { v[0] = v[1] != 0.f ? v[2] : v[3]; }
};
// optimizers: arrays param, grad, state...; evaluation order of src/ops/Optimizers.cu
struct SgdOp {
  static constexpr int N = 2, LOAD = 3, STORE = 1;
  float lr;
  __device__ void apply(float (&v)[2]) const { v[0] = v[0] - lr * v[1]; }
};
struct MomentumOp {   // param, grad, velocity
  static constexpr int N = 3, LOAD = 7, STORE = 5;
  float lr, mom;
  __device__ void apply(float (&v)[3]) const {
    v[2] = mom * v[2] - lr * v[1];
    v[0] = v[0] + v[2];
  }
};
struct NesterovOp {
  static constexpr int N = 3, LOAD = 7, STORE = 5;
  float lr, mom;
  __device__ void apply(float (&v)[3]) const {
    const float t = lr * v[1];
    v[2] = mom * (v[2] - t);
    v[0] = v[0] + v[2] - t;
  }
};
struct AdaGradOp {    // param, grad, acc
  static constexpr int N = 3, LOAD = 7, STORE = 5;
  float lr, eps;
  __device__ void apply(float (&v)[3]) const {
    v[2] = v[2] + v[1] * v[1];
    v[0] = v[0] - lr * v[1] / (sqrtf(v[2]) + eps);
  }
};
struct AdamOp {       // param, grad, m, v
  static constexpr int N = 4, LOAD = 15, STORE = 13;
  float lr, b1, b2, b1t, b2t, eps;
  __device__ void apply(float (&v)[4]) const {
    v[2] = b1 * v[2] + (1.f - b1) * v[1];
    v[3] = b2 * v[3] + (1.f - b2) * v[1] * v[1];
    const float mc = v[2] / (1.f - b1t);
    const float vc = v[3] / (1.f - b2t);
    v[0] = v[0] - lr * mc / (sqrtf(vc) + eps);
  }
};

inline float *fp(const DLArray *a) { return static_cast<float *>(a->data); }

}  // namespace
}  // namespace tsplit

using namespace tsplit;

// ---- one launch over many arrays (optimizer updates of a whole model) ----
// A model's update is dozens of launches, most of them on vectors of a few hundred values that cost
// a launch each (4 us) for nanoseconds of work.  Here the arrays are listed in a table in device
// memory and one grid walks all of them: block b takes kMultiWords 16-byte words of the array
// blocks[b] names.  Arithmetic per element is the single-array kernel's, so results are the same bits.
constexpr int kMultiPerThread = 4;
constexpr int kMultiWords = kThreads * kMultiPerThread;

template <int N>
struct MultiTensor {
  float *p[N];
  int64_t n;
};
struct MultiBlock {
  int tensor;
  unsigned first_word;
};

template <class Op>
__global__ __launch_bounds__(kThreads) void ew_multi_kernel(Op op, const MultiTensor<Op::N> *__restrict__ tensors,
                                                            const MultiBlock *__restrict__ blocks) {
  constexpr int N = Op::N;
  const MultiBlock b = blocks[blockIdx.x];
  const MultiTensor<N> t = tensors[b.tensor];
  const int64_t n4 = t.n >> 2;
  f32x4 v[kMultiPerThread][N];
#pragma unroll
  for (int u = 0; u < kMultiPerThread; ++u) {
    const int64_t i = static_cast<int64_t>(b.first_word) + u * kThreads + threadIdx.x;
    if (i < n4) {
#pragma unroll
      for (int k = 0; k < N; ++k)
        if (Op::LOAD & (1 << k)) v[u][k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(t.p[k]) + i);
    }
  }
#pragma unroll
  for (int u = 0; u < kMultiPerThread; ++u) {
    const int64_t i = static_cast<int64_t>(b.first_word) + u * kThreads + threadIdx.x;
    if (i < n4) {
      float e[4][N];
#pragma unroll
      for (int k = 0; k < N; ++k) {
        e[0][k] = v[u][k].x;
        e[1][k] = v[u][k].y;
        e[2][k] = v[u][k].z;
        e[3][k] = v[u][k].w;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) op.apply(e[j]);
#pragma unroll
      for (int k = 0; k < N; ++k)
        if (Op::STORE & (1 << k)) {
          const f32x4 r = {e[0][k], e[1][k], e[2][k], e[3][k]};
          __builtin_nontemporal_store(r, reinterpret_cast<f32x4 *>(t.p[k]) + i);
        }
    }
  }
  // the array's last (n % 4) elements, by its first block
  if (b.first_word == 0 && threadIdx.x < (t.n & 3)) {
    const int64_t i = (n4 << 2) + threadIdx.x;
    float e[N];
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (Op::LOAD & (1 << k)) e[k] = t.p[k][i];
    op.apply(e);
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (Op::STORE & (1 << k)) t.p[k][i] = e[k];
  }
}

// The table of one stream's last multi-array call: uploaded again only when the arrays or the device
// buffer under it changed (a trainer passes the same parameters every step, and a recorded step must
// not copy from the host).  The copy reads a pinned staging buffer of its own, rewritten only after
// the previous upload has finished.
struct MultiTable {
  std::vector<char> host;          // the table as last uploaded
  char *dev = nullptr;             // the device buffer it was uploaded into
  // two staging buffers the asynchronous copies read in turn, each with an event recorded behind its last upload:
  // the host waits only for the upload before the last one (lists that change from call to call would
  // otherwise tie the host to the stream)
  char *pinned[2] = {nullptr, nullptr};
  size_t pinned_bytes[2] = {0, 0};
  hipEvent_t uploaded[2] = {nullptr, nullptr};
  int turn = 0;
  bool in_graph = false;           // a recorded step launches with this table at `dev`
};
std::mutex g_multi_mu;
std::map<hipStream_t, MultiTable> g_multi;

void multi_table_release(MultiTable &mt) {
  for (int i = 0; i < 2; ++i) {
    if (mt.uploaded[i]) {
      (void)hipEventSynchronize(mt.uploaded[i]);
      (void)hipEventDestroy(mt.uploaded[i]);
    }
    if (mt.pinned[i]) (void)hipHostFree(mt.pinned[i]);
  }
  mt = MultiTable{};
}

bool stream_is_recording(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  return s && hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}

std::atomic<int> tsplit::g_updates_pending{0};
int pending_run_locked();
extern std::mutex g_pending_mu;
void tsplit::updates_flush_all() {
  std::lock_guard<std::mutex> lk(g_pending_mu);
  if (pending_run_locked()) std::fprintf(stderr, "tsplit: a deferred optimizer update could not be launched\n");
}

// The stream is about to be destroyed (it has drained): its table's device buffer goes with the
// stream's scratch, and a later stream may get the same handle value.
void tsplit::multi_update_drop_stream(hipStream_t stream) {
  std::lock_guard<std::mutex> lk(g_multi_mu);
  auto it = g_multi.find(stream);
  if (it == g_multi.end()) return;
  multi_table_release(it->second);
  g_multi.erase(it);
}

// arrays[k][i]: array k of tensor i.  Tensors whose arrays are not all 16-byte aligned go through the
// single-array launch.
template <class Op>
int launch_multi(Op op, const std::vector<std::array<float *, Op::N>> &arrays, const std::vector<int64_t> &sizes,
                 hipStream_t s, const char *who) {
  constexpr int N = Op::N;
  std::vector<MultiTensor<N>> tensors;
  std::vector<MultiBlock> blocks;
  for (size_t i = 0; i < arrays.size(); ++i) {
    if (sizes[i] <= 0) continue;
    bool vec = true;
    Ptrs<N> a;
    for (int k = 0; k < N; ++k) {
      a.p[k] = arrays[i][k];
      vec = vec && aligned16(a.p[k]);
    }
    TS_REQUIRE(sizes[i] < (1ll << 33), "%s: array too large", who);
    if (!vec) {
      launch(op, a, sizes[i], s);
      continue;
    }
    MultiTensor<N> t;
    for (int k = 0; k < N; ++k) t.p[k] = a.p[k];
    t.n = sizes[i];
    const int64_t words = std::max<int64_t>(1, sizes[i] >> 2);      // at least the block that does the tail
    for (int64_t w = 0; w < words; w += kMultiWords)
      blocks.push_back(MultiBlock{static_cast<int>(tensors.size()), static_cast<unsigned>(w)});
    tensors.push_back(t);
  }
  if (blocks.empty()) return 0;
  const size_t tbytes = (tensors.size() * sizeof(MultiTensor<N>) + 15) / 16 * 16, bbytes = blocks.size() * sizeof(MultiBlock);
  std::vector<char> table(tbytes + bbytes);
  std::memcpy(table.data(), tensors.data(), tensors.size() * sizeof(MultiTensor<N>));
  std::memcpy(table.data() + tbytes, blocks.data(), bbytes);
  const bool recording = stream_is_recording(s);
  {
    std::lock_guard<std::mutex> lk(g_multi_mu);
    MultiTable &mt = g_multi[s];
    if (mt.in_graph && mt.host != table && !recording) {
      // a recorded step replays with the table that lies in the device buffer: other arrays on this
      // stream go through one launch each and leave that table alone
      for (const MultiTensor<N> &t : tensors) {
        Ptrs<N> a;
        for (int k = 0; k < N; ++k) a.p[k] = t.p[k];
        launch(op, a, t.n, s);
      }
      return 0;
    }
  }
  char *dev = static_cast<char *>(scratch_get(s, 8, table.size()));
  TS_REQUIRE(dev, "%s: no scratch memory", who);
  {
    std::lock_guard<std::mutex> lk(g_multi_mu);
    MultiTable &mt = g_multi[s];
    if (mt.dev != dev || mt.host != table) {
      TS_REQUIRE(!recording, "%s: the list of arrays changed while a step is being recorded; run the step once before recording it", who);
      const int b = mt.turn;
      mt.turn ^= 1;
      if (mt.uploaded[b]) TS_HIP(hipEventSynchronize(mt.uploaded[b]));   // this staging buffer is free again
      if (mt.pinned_bytes[b] < table.size()) {
        if (mt.pinned[b]) (void)hipHostFree(mt.pinned[b]);
        mt.pinned[b] = nullptr;
        mt.pinned_bytes[b] = 0;
        const size_t want = (table.size() + 4095) / 4096 * 4096;
        TS_HIP(hipHostMalloc(reinterpret_cast<void **>(&mt.pinned[b]), want, hipHostMallocDefault));
        mt.pinned_bytes[b] = want;
      }
      if (!mt.uploaded[b]) TS_HIP(hipEventCreateWithFlags(&mt.uploaded[b], hipEventDisableTiming));
      std::memcpy(mt.pinned[b], table.data(), table.size());
      mt.dev = nullptr;   // until the copy below is queued nothing valid lies there
      TS_HIP(hipMemcpyAsync(dev, mt.pinned[b], table.size(), hipMemcpyHostToDevice, s));
      TS_HIP(hipEventRecord(mt.uploaded[b], s));
      mt.host = table;
      mt.dev = dev;
      mt.in_graph = false;
    }
    mt.in_graph |= recording;
  }
  hipLaunchKernelGGL(ew_multi_kernel<Op>, dim3(static_cast<unsigned>(blocks.size())), dim3(kThreads), 0, s, op,
                     reinterpret_cast<const MultiTensor<N> *>(dev), reinterpret_cast<const MultiBlock *>(dev + tbytes));
  return 0;
}

// ---- the list of optimizer updates that wait for their neighbours (common.h)
struct PendingUpdates {
  hipStream_t stream = nullptr;
  int device = 0;
  int rule = 0;                     // 0: SGD, 1: momentum, 2: Nesterov momentum
  float lr = 0.0f, momentum = 0.0f;
  std::vector<std::array<float *, 3>> arrays;      // param, grad, velocity (SGD: velocity unused)
  std::vector<int64_t> sizes;
};
std::mutex g_pending_mu;
PendingUpdates g_pending;

bool lazy_updates_enabled() {
  static const bool on = [] {
    const char *e = std::getenv("TSPLIT_LAZY_UPDATES");
    return !e || std::atoi(e) != 0;
  }();
  return on;
}

// one array of the list as a launch of its own
void pending_run_one(const PendingUpdates &job, size_t i) {
  Ptrs<3> a{{job.arrays[i][0], job.arrays[i][1], job.arrays[i][2]}};
  if (job.rule == 0)
    launch(SgdOp{job.lr}, Ptrs<2>{{a.p[0], a.p[1]}}, job.sizes[i], job.stream);
  else if (job.rule == 1)
    launch(MomentumOp{job.lr, job.momentum}, a, job.sizes[i], job.stream);
  else
    launch(NesterovOp{job.lr, job.momentum}, a, job.sizes[i], job.stream);
}

// runs the list (the caller holds g_pending_mu)
int pending_run_locked() {
  if (g_pending.arrays.empty()) return 0;
  PendingUpdates job;
  std::swap(job, g_pending);
  tsplit::g_updates_pending.store(0, std::memory_order_relaxed);
  int now = job.device;
  (void)hipGetDevice(&now);
  if (now != job.device) (void)hipSetDevice(job.device);      // the list runs on the device its stream lives on
  // Arrays the one launch can take (16-byte aligned, below its size limit) go into it; the others, and all of
  // them if the launch cannot be set up, run one by one: no update is ever dropped or done twice.
  PendingUpdates many;
  many.stream = job.stream, many.rule = job.rule, many.lr = job.lr, many.momentum = job.momentum;
  std::vector<size_t> listed;
  for (size_t i = 0; i < job.arrays.size(); ++i) {
    const bool takes = job.arrays.size() > 1 && job.sizes[i] < (1ll << 33) && aligned16(job.arrays[i][0]) &&
                       aligned16(job.arrays[i][1]) && (job.rule == 0 || aligned16(job.arrays[i][2]));
    if (!takes) {
      pending_run_one(job, i);
      continue;
    }
    many.arrays.push_back(job.arrays[i]);
    many.sizes.push_back(job.sizes[i]);
    listed.push_back(i);
  }
  int rc = 0;
  if (listed.size() == 1) {
    pending_run_one(job, listed[0]);
  } else if (!listed.empty()) {
    const char *who = "optimizer update";
    if (job.rule == 0) {
      std::vector<std::array<float *, 2>> two(many.arrays.size());
      for (size_t i = 0; i < two.size(); ++i) two[i] = {many.arrays[i][0], many.arrays[i][1]};
      rc = launch_multi(SgdOp{job.lr}, two, many.sizes, job.stream, who);
    } else {
      rc = job.rule == 1 ? launch_multi(MomentumOp{job.lr, job.momentum}, many.arrays, many.sizes, job.stream, who)
                         : launch_multi(NesterovOp{job.lr, job.momentum}, many.arrays, many.sizes, job.stream, who);
    }
    if (rc)       // set-up failed before the launch: nothing of the list has run
      for (size_t i : listed) pending_run_one(job, i);
  }
  if (now != job.device) (void)hipSetDevice(now);
  return 0;
}

// Puts one update on the list (running the list first if this one does not fit it).  False: the caller runs
// the update itself, now (recording streams, or the list switched off).
bool pending_add(hipStream_t s, int rule, float lr, float momentum, float *param, float *grad, float *velocity, int64_t n) {
  if (!lazy_updates_enabled() || stream_is_recording(s)) {
    tsplit::updates_flush_if_any();
    return false;
  }
  int device = 0;
  (void)hipGetDevice(&device);
  std::lock_guard<std::mutex> lk(g_pending_mu);
  bool fits = g_pending.arrays.empty() || (g_pending.stream == s && g_pending.device == device && g_pending.rule == rule &&
                                           g_pending.lr == lr && g_pending.momentum == momentum);
  if (fits) {
    // one launch updates all listed arrays at once: an array this update writes must not be read or written by a
    // listed one, nor may it read what a listed one writes (the same parameter updated twice in a row)
    const auto overlap = [](const float *a, int64_t na, const float *b, int64_t nb) {
      return a && b && a < b + nb && b < a + na;
    };
    for (size_t i = 0; fits && i < g_pending.arrays.size(); ++i) {
      const std::array<float *, 3> &o = g_pending.arrays[i];
      const int64_t m = g_pending.sizes[i];
      for (int k = 0; k < 3 && fits; ++k) {
        if (overlap(param, n, o[k], m) || overlap(velocity, n, o[k], m)) fits = false;      // writes against anything listed
        if (k != 1 && overlap(grad, n, o[k], m)) fits = false;                              // reads against listed writes
      }
    }
  }
  if (!fits) (void)pending_run_locked();
  g_pending.stream = s;
  g_pending.device = device;
  g_pending.rule = rule;
  g_pending.lr = lr;
  g_pending.momentum = momentum;
  g_pending.arrays.push_back({param, grad, velocity});
  g_pending.sizes.push_back(n);
  tsplit::g_updates_pending.store(1, std::memory_order_relaxed);
  return true;
}

#define SAME_SIZE(a, b, name) \
  TS_REQUIRE(numel(a) == numel(b), name ": operand sizes differ (%lld vs %lld)", (long long)numel(a), (long long)numel(b))

extern "C" {

int DLGpuArraySet(DLArrayHandle arr, float value, DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(arr && arr->data, "DLGpuArraySet: NULL array");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(arr);
  ProfileScope ps(p, s, 0, n, 0);
  launch(SetOp{value}, Ptrs<1>{{fp(arr)}}, n, s);
  return ps.finish();
}

int DLGpuMatrixElementwiseAdd(const DLArrayHandle matA, const DLArrayHandle matB, DLArrayHandle output,
                              DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(matA && matB && output, "DLGpuMatrixElementwiseAdd: NULL array");
  SAME_SIZE(matA, output, "DLGpuMatrixElementwiseAdd");
  SAME_SIZE(matB, output, "DLGpuMatrixElementwiseAdd");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, 2 * n, n, 0);
  launch(AddOp{}, Ptrs<3>{{fp(output), fp(matA), fp(matB)}}, n, s);
  return ps.finish();
}

int DLGpuMatrixElementwiseMultiply(const DLArrayHandle matA, const DLArrayHandle matB, DLArrayHandle output,
                                   DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(matA && matB && output, "DLGpuMatrixElementwiseMultiply: NULL array");
  SAME_SIZE(matA, output, "DLGpuMatrixElementwiseMultiply");
  SAME_SIZE(matB, output, "DLGpuMatrixElementwiseMultiply");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, 2 * n, n, 0);
  launch(MulOp{}, Ptrs<3>{{fp(output), fp(matA), fp(matB)}}, n, s);
  return ps.finish();
}

int DLGpuMatrixElementwiseAddByConst(const DLArrayHandle input, float val, DLArrayHandle output,
                                     DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input && output, "DLGpuMatrixElementwiseAddByConst: NULL array");
  SAME_SIZE(input, output, "DLGpuMatrixElementwiseAddByConst");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, n, n, 0);
  launch(AddConstOp{val}, Ptrs<2>{{fp(output), fp(input)}}, n, s);
  return ps.finish();
}

int DLGpuMatrixMultiplyByConst(const DLArrayHandle input, float val, DLArrayHandle output,
                               DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input && output, "DLGpuMatrixMultiplyByConst: NULL array");
  SAME_SIZE(input, output, "DLGpuMatrixMultiplyByConst");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, n, n, 0);
  launch(MulConstOp{val}, Ptrs<2>{{fp(output), fp(input)}}, n, s);
  return ps.finish();
}

int DLGpuReshape(const DLArrayHandle in_arr, DLArrayHandle out_arr, DLStreamHandle stream_handle,
                 ProfilerHandle p) {
  TS_REQUIRE(in_arr && out_arr, "DLGpuReshape: NULL array");
  SAME_SIZE(in_arr, out_arr, "DLGpuReshape");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(out_arr);
  ProfileScope ps(p, s, n, n, 0);
  if (in_arr->data != out_arr->data) launch(CopyOp{}, Ptrs<2>{{fp(out_arr), fp(in_arr)}}, n, s);
  return ps.finish();
}

int DLGpuRelu(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input && output, "DLGpuRelu: NULL array");
  SAME_SIZE(input, output, "DLGpuRelu");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, n, n, 0);
  launch(ReluOp{}, Ptrs<2>{{fp(output), fp(input)}}, n, s);
  return ps.finish();
}

int DLGpuReluGradient(const DLArrayHandle input, const DLArrayHandle in_grad, DLArrayHandle output,
                      DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(input && in_grad && output, "DLGpuReluGradient: NULL array");
  SAME_SIZE(input, output, "DLGpuReluGradient");
  SAME_SIZE(in_grad, output, "DLGpuReluGradient");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, 2 * n, n, 0);
  launch(ReluGradOp{}, Ptrs<3>{{fp(output), fp(input), fp(in_grad)}}, n, s);
  return ps.finish();
}

#define UNARY_ENTRY(symbol, OP)                                                                                      \
  int symbol(const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle, ProfilerHandle p) {     \
    TS_REQUIRE(input && output, #symbol ": NULL array");                                                             \
    SAME_SIZE(input, output, #symbol);                                                                               \
    hipStream_t s = stream_of(stream_handle);                                                                        \
    const int64_t n = numel(output);                                                                                 \
    ProfileScope ps(p, s, n, n, 0);                                                                                  \
    launch(OP{}, Ptrs<2>{{fp(output), fp(input)}}, n, s);                                                            \
    return ps.finish();                                                                                              \
  }

UNARY_ENTRY(DLGpuOpposite, NegOp)
UNARY_ENTRY(DLGpuSqrt, SqrtOp)
UNARY_ENTRY(DLGpuReciprocalSqrt, RsqrtOp)
UNARY_ENTRY(DLGpuTanh, TanhOp)
UNARY_ENTRY(DLGpuSigmoid, SigmoidOp)
#undef UNARY_ENTRY

int DLGpuMatrixElementwiseDivide(const DLArrayHandle matA, const DLArrayHandle matB, DLArrayHandle output,
                                 DLStreamHandle stream_handle, ProfilerHandle p) {
  TS_REQUIRE(matA && matB && output, "DLGpuMatrixElementwiseDivide: NULL array");
  SAME_SIZE(matA, output, "DLGpuMatrixElementwiseDivide");
  SAME_SIZE(matB, output, "DLGpuMatrixElementwiseDivide");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, 2 * n, n, 0);
  launch(DivOp{}, Ptrs<3>{{fp(output), fp(matA), fp(matB)}}, n, s);
  return ps.finish();
}

int DLGpuMatrixDivConst(float val, const DLArrayHandle input, DLArrayHandle output, DLStreamHandle stream_handle,
                        ProfilerHandle p) {
  TS_REQUIRE(input && output, "DLGpuMatrixDivConst: NULL array");
  SAME_SIZE(input, output, "DLGpuMatrixDivConst");
  hipStream_t s = stream_of(stream_handle);
  const int64_t n = numel(output);
  ProfileScope ps(p, s, n, n, 0);
  launch(DivConstOp{val}, Ptrs<2>{{fp(output), fp(input)}}, n, s);
  return ps.finish();
}

int DLGpuWhere(const DLArrayHandle cond, const DLArrayHandle arr1, const DLArrayHandle arr2, DLArrayHandle output,
               DLStreamHandle stream_handle) {
  TS_REQUIRE(cond && arr1 && arr2 && output, "DLGpuWhere: NULL array");
  SAME_SIZE(cond, output, "DLGpuWhere");
  SAME_SIZE(arr1, output, "DLGpuWhere");
  SAME_SIZE(arr2, output, "DLGpuWhere");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  launch(WhereOp{}, Ptrs<4>{{fp(output), fp(cond), fp(arr1), fp(arr2)}}, numel(output), s);
  return ps.finish();
}

int SGDOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, float lr, DLStreamHandle stream_handle) {
  TS_REQUIRE(param && grad, "SGDOptimizerUpdate: NULL array");
  SAME_SIZE(param, grad, "SGDOptimizerUpdate");
  hipStream_t s = stream_of_update(stream_handle);
  if (numel(param) > 0 && pending_add(s, 0, lr, 0.0f, fp(param), fp(grad), nullptr, numel(param))) return 0;
  ProfileScope ps(nullptr, s, 0, 0, 0);
  launch(SgdOp{lr}, Ptrs<2>{{fp(param), fp(grad)}}, numel(param), s);
  return ps.finish();
}

int MomentumOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, DLArrayHandle velocity, float lr,
                            float momentum, bool nesterov, DLStreamHandle stream_handle) {
  TS_REQUIRE(param && grad && velocity, "MomentumOptimizerUpdate: NULL array");
  SAME_SIZE(param, grad, "MomentumOptimizerUpdate");
  SAME_SIZE(param, velocity, "MomentumOptimizerUpdate");
  hipStream_t s = stream_of_update(stream_handle);
  if (numel(param) > 0 && pending_add(s, nesterov ? 2 : 1, lr, momentum, fp(param), fp(grad), fp(velocity), numel(param))) return 0;
  ProfileScope ps(nullptr, s, 0, 0, 0);
  Ptrs<3> a{{fp(param), fp(grad), fp(velocity)}};
  if (nesterov)
    launch(NesterovOp{lr, momentum}, a, numel(param), s);
  else
    launch(MomentumOp{lr, momentum}, a, numel(param), s);
  return ps.finish();
}

// SGD / momentum update of `count` parameters in one launch: the arithmetic of SGDOptimizerUpdate /
// MomentumOptimizerUpdate per element (velocities == NULL: plain SGD).
int TSplit_OptimizerUpdateMulti(DLArrayHandle *params, const DLArrayHandle *grads, DLArrayHandle *velocities, int count,
                                float lr, float momentum, int nesterov, DLStreamHandle stream_handle) {
  const char *who = "TSplit_OptimizerUpdateMulti";
  TS_REQUIRE(count >= 0 && (count == 0 || (params && grads)), "%s: NULL table", who);
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  std::vector<int64_t> sizes(count);
  for (int i = 0; i < count; ++i) {
    TS_REQUIRE(params[i] && grads[i] && (!velocities || velocities[i]), "%s: NULL array", who);
    TS_REQUIRE(numel(params[i]) == numel(grads[i]) && (!velocities || numel(params[i]) == numel(velocities[i])),
               "%s: operand sizes of parameter %d differ", who, i);
    sizes[i] = numel(params[i]);
  }
  int rc;
  if (!velocities) {
    std::vector<std::array<float *, 2>> a(count);
    for (int i = 0; i < count; ++i) a[i] = {fp(params[i]), fp(grads[i])};
    rc = launch_multi(SgdOp{lr}, a, sizes, s, who);
  } else {
    std::vector<std::array<float *, 3>> a(count);
    for (int i = 0; i < count; ++i) a[i] = {fp(params[i]), fp(grads[i]), fp(velocities[i])};
    rc = nesterov ? launch_multi(NesterovOp{lr, momentum}, a, sizes, s, who) : launch_multi(MomentumOp{lr, momentum}, a, sizes, s, who);
  }
  if (rc) return rc;
  return ps.finish();
}

int AdaGradOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, DLArrayHandle acc, float lr, float eps,
                           DLStreamHandle stream_handle) {
  TS_REQUIRE(param && grad && acc, "AdaGradOptimizerUpdate: NULL array");
  SAME_SIZE(param, grad, "AdaGradOptimizerUpdate");
  SAME_SIZE(param, acc, "AdaGradOptimizerUpdate");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  launch(AdaGradOp{lr, eps}, Ptrs<3>{{fp(param), fp(grad), fp(acc)}}, numel(param), s);
  return ps.finish();
}

int AdamOptimizerUpdate(DLArrayHandle param, const DLArrayHandle grad, DLArrayHandle expavg, DLArrayHandle expavgsq,
                        float lr, float beta1, float beta2, float beta1t, float beta2t, float eps,
                        DLStreamHandle stream_handle) {
  TS_REQUIRE(param && grad && expavg && expavgsq, "AdamOptimizerUpdate: NULL array");
  SAME_SIZE(param, grad, "AdamOptimizerUpdate");
  SAME_SIZE(param, expavg, "AdamOptimizerUpdate");
  SAME_SIZE(param, expavgsq, "AdamOptimizerUpdate");
  hipStream_t s = stream_of(stream_handle);
  ProfileScope ps(nullptr, s, 0, 0, 0);
  launch(AdamOp{lr, beta1, beta2, beta1t, beta2t, eps}, Ptrs<4>{{fp(param), fp(grad), fp(expavg), fp(expavgsq)}},
         numel(param), s);
  return ps.finish();
}

}  // extern "C"
