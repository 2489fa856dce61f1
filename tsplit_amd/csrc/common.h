// Shared host-side helpers of the operator library: argument checks, stream lookup,
// the ProfilerHandle contract, and per-stream scratch memory for kernels that need it.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>

#include "../../include/c_runtime_api.h"

namespace tsplit {

inline int64_t numel(const DLArray *a) {
  int64_t n = 1;
  for (int i = 0; i < a->ndim; ++i) n *= a->shape[i];
  return n;
}

// ---- what a convolution leaves behind for the BatchNorm that follows it (runtime.cpp) ----
// A forward convolution whose epilogue can sum its output per channel at no extra pass notes, for the
// range of memory it wrote, where those sums lie.  CuDNN_DLGpuBatch_Normalization on exactly that range
// (one note, or the notes of consecutive batch micro-tensors that tile it in ascending order), on the same
// stream, takes its batch statistics from them instead of reading the tensor twice.  A note may only be
// used while nothing has written the range since: EVERY operator of the library obtains its stream through
// stream_of(), which drops all notes (a convolution drops the notes its own output overlaps and keeps the
// others, so that micro-tensors accumulate); so do copies without a stream, graph launches and stream
// destruction.  Only calls made through this library are seen: memory written behind its back (another
// library in the process) is not, as with any of its scratch buffers.  TSPLIT_BN_LOOKBEHIND=0 switches
// the notes off.
struct ConvNote {
  hipStream_t stream;
  const char *begin;     // the convolution's output
  size_t bytes;
  int images, channels, plane;
  const double *sums;    // [channels][2]: sum and sum of squares over this output
};
extern std::atomic<int> g_conv_notes_live;
void conv_notes_drop_all();
// drops the notes that overlap [begin, begin + bytes)
void conv_notes_drop_overlapping(const void *begin, size_t bytes);
// room for one more note's sums on `stream` (nullptr: none; the caller then makes no note)
double *conv_note_sums(hipStream_t stream, int channels);
void conv_note_add(const ConvNote &note);
// the notes that tile [begin, begin + bytes) of a [*, channels, plane] tensor on `stream`: returns their
// number (0: none) and the first one's sums, behind which the others' lie at channels * 2 doubles each
int conv_notes_take(hipStream_t stream, const void *begin, size_t bytes, int channels, int plane, const double **sums);
bool conv_notes_enabled();

// ---- Optimizer updates wait for their neighbours.  SGDOptimizerUpdate / MomentumOptimizerUpdate are called once
// per parameter (42 times a VGG-16 step, 449 times an Inception-v4 step), most of them on vectors of a few hundred
// values for which a launch costs more than the work.  Such a call only puts its arrays on a list; the list is
// run as ONE launch (the kernel behind TSplit_OptimizerUpdateMulti: the same arithmetic per element) as soon as
// anything else is asked of the library - every entry point that takes a stream comes through the functions
// below, which run the list first, and so do copies without a stream, freeing an array, destroying a stream and
// starting a recording.  So no call into the library can see a parameter before its update, and the updates stay
// in their order on their stream.  A call with another stream, rule or rate than the list's runs the list first.
// TSPLIT_LAZY_UPDATES=0 makes every update run at once.
extern std::atomic<int> g_updates_pending;
void updates_flush_all();
inline void updates_flush_if_any() {
  if (g_updates_pending.load(std::memory_order_relaxed)) updates_flush_all();
}

inline hipStream_t raw_stream(DLStreamHandle h) {
  return h ? *static_cast<hipStream_t *>(h->handle) : static_cast<hipStream_t>(nullptr);
}

// the stream of a call that cannot change a tensor (the notes above stay)
inline hipStream_t stream_keep_notes(DLStreamHandle h) {
  updates_flush_if_any();
  return raw_stream(h);
}

// The stream an operator runs on.  Every operator writes somewhere: the notes above end here.
inline hipStream_t stream_of(DLStreamHandle h) {
  if (g_conv_notes_live.load(std::memory_order_relaxed)) conv_notes_drop_all();
  return stream_keep_notes(h);
}

// the stream of an optimizer update that may join the list: the list is not run
inline hipStream_t stream_of_update(DLStreamHandle h) {
  if (g_conv_notes_live.load(std::memory_order_relaxed)) conv_notes_drop_all();
  return raw_stream(h);
}

inline float mib(int64_t elems) { return static_cast<float>(elems) * 4.0f / (1024.0f * 1024.0f); }

// Grow-only device scratch, one buffer per (stream, slot), kept until the process ends.
// Kernels launched on one stream are ordered, so a buffer may be reused by the next op on
// that stream without waiting; ops on different streams never share one.
void *scratch_get(hipStream_t stream, int slot, size_t bytes);

// Forgets the table of arrays TSplit_OptimizerUpdateMulti keeps for a stream (elementwise.hip);
// called by DLStreamDestroy once the stream has drained, before its scratch is dropped.
void multi_update_drop_stream(hipStream_t stream);

// whether contractions take their products in split bf16 (TSplit_SplitBf16; winograd.hip)
bool split_bf16_enabled();

// Where a convolution leaves per-channel partial sums of its output for a BatchNorm that follows:
// partial k of channel c is the pair (sum, sum of squares) at part[(k * channels + c) * 2]; `used`
// counts the partials written so far (a call may run as several launches).
struct StatsSink {
  float *part;
  int channels;
  int capacity;   // partials the buffer holds per channel
  int used;
};

// Per-channel (sum, sum of squares) of a 4-D NCHW array by a pass of its own, as doubles: dst[c * 2],
// dst[c * 2 + 1] (batchnorm.hip).
int bn_channel_sums(const DLArray *y, double *dst, hipStream_t st);

// Looks up, once per device, the address of the fixed scratch array behind
// TSplit_SoftmaxCrossEntropyNoAlloc (called from the per-device init call).
void softmax_noalloc_setup(int device_id);


#define TS_FAIL(...)                                  \
  do {                                                \
    std::fprintf(stderr, "[libc_runtime_api] ");      \
    std::fprintf(stderr, __VA_ARGS__);                \
    std::fprintf(stderr, "\n");                       \
    return -1;                                        \
  } while (0)

#define TS_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) TS_FAIL(__VA_ARGS__); \
  } while (0)

#define TS_HIP(call)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) TS_FAIL("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
  } while (0)

// ProfilerHandle contract of the reference (e.g. src/ops/Relu.cu:15-51): with a non-NULL
// profiler the call records operand sizes in MiB, times the launch with events and blocks
// until it has finished.  Usage:
//   ProfileScope ps(p, stream, in_elems, out_elems, ws_elems);  ... launches ...  return ps.finish();
class ProfileScope {
 public:
  ProfileScope(ProfilerHandle p, hipStream_t s, int64_t in_elems, int64_t out_elems, int64_t ws_elems)
      : p_(p), s_(s) {
    if (!p_) return;
    p_->input_memory = mib(in_elems);
    p_->output_memory = mib(out_elems);
    p_->workspace_memory = mib(ws_elems);
    ok_ = hipEventCreate(&a_) == hipSuccess && hipEventCreate(&b_) == hipSuccess &&
          hipEventRecord(a_, s_) == hipSuccess;
  }
  int finish() {
    hipError_t le = hipGetLastError();
    if (le != hipSuccess) {
      std::fprintf(stderr, "[libc_runtime_api] kernel launch failed: %s\n", hipGetErrorString(le));
      return -1;
    }
    if (!p_) return 0;
    if (!ok_) return -1;
    float ms = -1.f;
    bool good = hipEventRecord(b_, s_) == hipSuccess && hipEventSynchronize(b_) == hipSuccess &&
                hipEventElapsedTime(&ms, a_, b_) == hipSuccess;
    p_->time = ms;
    return good ? 0 : -1;
  }
  ~ProfileScope() {   // also on the early-return paths of an operator call
    if (a_) (void)hipEventDestroy(a_);
    if (b_) (void)hipEventDestroy(b_);
  }
  ProfileScope(const ProfileScope &) = delete;
  ProfileScope &operator=(const ProfileScope &) = delete;

 private:
  ProfilerHandle p_;
  hipStream_t s_;
  hipEvent_t a_{}, b_{};
  bool ok_ = false;
};

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace tsplit
