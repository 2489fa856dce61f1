// Runtime half of the C ABI: array lifecycle, copies, streams, events, the pooled
// allocator's public face, micro-tensor views.  No kernels here.
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <set>
#include <stdexcept>
#include <vector>

#include "common.h"
#include "pool.h"

namespace tsplit {
namespace {

std::mutex g_mu;

// ---------------------------------------------------------------- device pool
size_t env_bytes(const char *name, size_t dflt) {
  const char *v = std::getenv(name);
  if (!v || !*v) return dflt;
  return static_cast<size_t>(std::strtoull(v, nullptr, 10));
}

void *dev_alloc(size_t bytes, void *) {
  void *p = nullptr;
  if (hipMalloc(&p, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return p;
}
void dev_release(void *p, void *) { (void)hipFree(p); }
size_t dev_available(void *) {
  size_t free_b = 0, total_b = 0;
  if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return 0;
  // head-room for kernels' code objects, scratch and the runtime itself
  // (the reference keeps 500 MB back: gpu_memory_manager.cc:246)
  const size_t keep = 512ull << 20;
  return free_b > keep ? free_b - keep : 0;
}

std::map<int, BinnedPool *> g_pools;

BinnedPool *pool_for(int dev) {
  auto it = g_pools.find(dev);
  if (it != g_pools.end()) return it->second;
  PoolBacking b{dev_alloc, dev_release, dev_available, nullptr};
  size_t slab = env_bytes("TSPLIT_POOL_SLAB_BYTES", 1ull << 30);
  size_t limit = env_bytes("TSPLIT_POOL_LIMIT_BYTES", ~size_t(0));
  BinnedPool *p = new BinnedPool(b, slab, limit, env_bytes("TSPLIT_POOL_SPLIT_SLACK_BYTES", BinnedPool::kSplitSlack));
  g_pools[dev] = p;
  return p;
}

int current_or(int dev) {
  (void)hipSetDevice(dev);
  return dev;
}

// ---------------------------------------------------------------- host memory
// Host tensors are pinned when a device is present (the reference's GPU build does the
// same: src/common/cpu_device_api.cc:30-36) so that stream copies really are asynchronous;
// on a machine without a device they are plain aligned memory.  With MEMORY_MANAGE_RULE != 0
// they come from a pool of pinned slabs (same best-fit core as the device pool): pinning costs
// hundreds of microseconds per call, and an executor that swaps tensors out and in allocates a
// host buffer per tensor and step.  Rule 0 pins and unpins per tensor.
std::set<void *> g_pinned;

bool have_device() {
  static const bool yes = [] {
    int n = 0;
    const bool ok = hipGetDeviceCount(&n) == hipSuccess && n > 0;
    if (!ok) (void)hipGetLastError();
    return ok;
  }();
  return yes;
}

void *host_raw_alloc(size_t bytes) {
  if (bytes == 0) bytes = 4;
  void *p = nullptr;
  if (have_device()) {
    if (hipHostMalloc(&p, bytes, hipHostMallocDefault) == hipSuccess) {
      g_pinned.insert(p);
      return p;
    }
    (void)hipGetLastError();
  }
  if (posix_memalign(&p, 256, bytes) != 0) return nullptr;
  return p;
}

void host_raw_free(void *p) {
  auto it = g_pinned.find(p);
  if (it != g_pinned.end()) {
    g_pinned.erase(it);
    (void)hipHostFree(p);
  } else {
    std::free(p);
  }
}

void *host_slab_alloc(size_t bytes, void *) { return host_raw_alloc(bytes); }
void host_slab_release(void *p, void *) { host_raw_free(p); }
size_t host_slab_available(void *) { return ~size_t(0) >> 1; }

BinnedPool *host_pool() {
  static BinnedPool *pool = new BinnedPool(PoolBacking{host_slab_alloc, host_slab_release, host_slab_available, nullptr},
                                           env_bytes("TSPLIT_HOST_POOL_SLAB_BYTES", 256ull << 20),
                                           env_bytes("TSPLIT_HOST_POOL_LIMIT_BYTES", ~size_t(0)));
  return pool;
}

void *host_alloc(size_t bytes, int rule) { return rule != 0 ? host_pool()->Malloc(bytes) : host_raw_alloc(bytes); }

void host_free(void *p, int rule) {
  if (rule != 0 && host_pool()->Free(p)) return;
  host_raw_free(p);
}

size_t byte_size(const DLArray *a) { return static_cast<size_t>(numel(a)) * 4; }

void *data_alloc(DLContext ctx, size_t bytes, int rule) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (ctx.device_type == kCPU) {
    void *hp = host_alloc(bytes, rule);
    if (!hp) throw std::runtime_error("out of host memory");
    return hp;
  }
  if (ctx.device_type != kGPU) throw std::runtime_error("unknown device type");
  current_or(ctx.device_id);
  void *p = nullptr;
  if (rule == 0) {
    if (hipMalloc(&p, bytes ? bytes : 4) != hipSuccess) {
      (void)hipGetLastError();
      p = nullptr;
    }
  } else {
    p = pool_for(ctx.device_id)->Malloc(bytes);
  }
  if (!p) throw std::runtime_error("out of device memory");
  return p;
}

void data_free(DLContext ctx, void *p, int rule) {
  if (!p) return;
  std::lock_guard<std::mutex> lk(g_mu);
  if (ctx.device_type == kCPU) {
    host_free(p, rule);
    return;
  }
  current_or(ctx.device_id);
  if (rule != 0) {
    if (pool_for(ctx.device_id)->Free(p)) return;
    throw std::runtime_error("pointer was not allocated from the pool");
  }
  (void)hipFree(p);
}

DLArray *new_array(const index_t *shape, index_t ndim, DLContext ctx) {
  DLArray *a = new DLArray();
  a->data = nullptr;
  a->ctx = ctx;
  a->ndim = static_cast<int>(ndim);
  a->shape = new int64_t[ndim > 0 ? ndim : 1];
  for (index_t i = 0; i < ndim; ++i) a->shape[i] = shape[i];
  return a;
}

// ---------------------------------------------------------------- scratch
struct ScratchKey {
  hipStream_t s;
  int slot;
  bool operator<(const ScratchKey &o) const { return s != o.s ? s < o.s : slot < o.slot; }
};
struct ScratchBuf {
  void *p;
  size_t bytes;
  bool recorded;   // handed out while a step was being recorded: a graph holds this address
};
std::map<ScratchKey, ScratchBuf> g_scratch;
// Buffers a recorded step still refers to after their (stream, slot) moved on to a larger one or
// the stream was destroyed; owned here until the last graph is gone.
std::vector<void *> g_scratch_parked;
int g_live_graphs = 0;
int g_open_recordings = 0;

// g_mu held.  A buffer no recording refers to is freed, one a recording got is parked.
void scratch_retire(ScratchBuf &b) {
  if (!b.p) return;
  if (b.recorded)
    g_scratch_parked.push_back(b.p);
  else
    (void)hipFree(b.p);
  b.p = nullptr;
  b.bytes = 0;
  b.recorded = false;
}

// g_mu held.  With no graph alive and none being recorded nothing refers to a parked buffer.
void scratch_release_parked() {
  if (g_live_graphs > 0 || g_open_recordings > 0) return;
  for (void *p : g_scratch_parked) (void)hipFree(p);
  g_scratch_parked.clear();
  for (auto &kv : g_scratch) kv.second.recorded = false;
}

}  // namespace

// Pool memory for an operator that must hand a buffer to its caller (dropout's reserve space);
// nullptr when the device has none left.
void *device_pool_alloc(int device_id, size_t bytes) {
  try {
    return data_alloc(DLContext{device_id, kGPU}, bytes, 1);
  } catch (const std::exception &) {
    return nullptr;
  }
}

void *scratch_get(hipStream_t stream, int slot, size_t bytes) {
  std::lock_guard<std::mutex> lk(g_mu);
  ScratchBuf &b = g_scratch[ScratchKey{stream, slot}];
  hipStreamCaptureStatus recording = hipStreamCaptureStatusNone;
  const bool in_recording =
      stream && hipStreamIsCapturing(stream, &recording) == hipSuccess && recording != hipStreamCaptureStatusNone;
  if (b.bytes >= bytes && b.p) {
    b.recorded |= in_recording;
    return b.p;
  }
  if (b.p) {
    // growing is set-up, not part of a step: a recording cannot allocate on the way
    if (in_recording) {
      std::fprintf(stderr, "[libc_runtime_api] scratch memory would have to grow while a step is being recorded; "
                           "run the step once before recording it\n");
      return nullptr;
    }
    // the old buffer may still be read by a kernel in flight on this stream; a recorded step that
    // got it keeps its address, so such a buffer is parked instead of freed
    (void)hipStreamSynchronize(stream);
    scratch_retire(b);
  }
  size_t want = (bytes + (1 << 20) - 1) >> 20 << 20;
  if (hipMalloc(&b.p, want) != hipSuccess) {
    (void)hipGetLastError();
    b.p = nullptr;
    return nullptr;
  }
  b.bytes = want;
  b.recorded = in_recording;
  return b.p;
}

// Bytes of scratch a destroyed stream leaves behind would stay allocated for good, keyed by a
// handle value a later stream may get again: called by DLStreamDestroy after the stream has drained.
void scratch_drop_stream(hipStream_t stream) {
  std::lock_guard<std::mutex> lk(g_mu);
  for (auto it = g_scratch.begin(); it != g_scratch.end();) {
    if (it->first.s == stream) {
      scratch_retire(it->second);
      it = g_scratch.erase(it);
    } else {
      ++it;
    }
  }
}

// ---------------------------------------------------------------- notes of convolutions for BatchNorm
namespace {
std::mutex g_notes_mu;
std::vector<ConvNote> g_notes;
// the sums of the notes of a stream lie one behind the other in that stream's scratch slot 9
constexpr size_t kNoteBytes = 1 << 20;
std::map<hipStream_t, size_t> g_note_used;
}  // namespace
std::atomic<int> g_conv_notes_live{0};

bool conv_notes_enabled() {
  static const bool on = [] {
    const char *e = std::getenv("TSPLIT_BN_LOOKBEHIND");
    return !(e && e[0] == '0');
  }();
  return on;
}

void conv_notes_drop_all() {
  std::lock_guard<std::mutex> lk(g_notes_mu);
  g_notes.clear();
  g_note_used.clear();
  g_conv_notes_live.store(0, std::memory_order_relaxed);
}

void conv_notes_drop_overlapping(const void *begin, size_t bytes) {
  if (!g_conv_notes_live.load(std::memory_order_relaxed)) return;
  std::lock_guard<std::mutex> lk(g_notes_mu);
  const char *b = static_cast<const char *>(begin), *e = b + bytes;
  bool dropped = false;
  for (auto it = g_notes.begin(); it != g_notes.end();) {
    if (it->begin < e && b < it->begin + it->bytes) {
      it = g_notes.erase(it);
      dropped = true;
    } else {
      ++it;
    }
  }
  if (g_notes.empty()) {
    g_note_used.clear();
    g_conv_notes_live.store(0, std::memory_order_relaxed);
  } else if (dropped) {
    // the remaining notes keep their sums; nothing is handed out twice because offsets only grow until
    // the list is empty
  }
}

double *conv_note_sums(hipStream_t stream, int channels) {
  const size_t want = static_cast<size_t>(channels) * 2 * sizeof(double);
  size_t used;
  {
    std::lock_guard<std::mutex> lk(g_notes_mu);
    used = g_note_used[stream];
    if (used + want > kNoteBytes) return nullptr;
    g_note_used[stream] = used + want;
  }
  char *base = static_cast<char *>(scratch_get(stream, 9, kNoteBytes));
  return base ? reinterpret_cast<double *>(base + used) : nullptr;
}

void conv_note_add(const ConvNote &note) {
  std::lock_guard<std::mutex> lk(g_notes_mu);
  g_notes.push_back(note);
  g_conv_notes_live.store(1, std::memory_order_relaxed);
}

int conv_notes_take(hipStream_t stream, const void *begin, size_t bytes, int channels, int plane, const double **sums) {
  if (!g_conv_notes_live.load(std::memory_order_relaxed)) return 0;
  std::lock_guard<std::mutex> lk(g_notes_mu);
  const char *at = static_cast<const char *>(begin), *end = at + bytes;
  const double *first = nullptr, *expect = nullptr;
  int n = 0;
  // the notes are in the order their convolutions were issued: the pieces must come in ascending order,
  // one behind the other in memory and in the sums' buffer
  for (const ConvNote &c : g_notes) {
    if (c.begin != at) continue;
    if (c.stream != stream || c.channels != channels || c.plane != plane || at + c.bytes > end) return 0;
    if (c.bytes != static_cast<size_t>(c.images) * channels * plane * sizeof(float)) return 0;
    if (n == 0) {
      first = c.sums;
    } else if (c.sums != expect) {
      return 0;
    }
    expect = c.sums + static_cast<size_t>(channels) * 2;
    at += c.bytes;
    ++n;
    if (at == end) break;
  }
  if (n == 0 || at != end) return 0;
  *sums = first;
  return n;
}

void scratch_recording_opened() {
  std::lock_guard<std::mutex> lk(g_mu);
  ++g_open_recordings;
}
void scratch_recording_closed(bool graph_made) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_open_recordings > 0) --g_open_recordings;
  if (graph_made) ++g_live_graphs;
  scratch_release_parked();
}
void scratch_graph_destroyed() {
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_live_graphs > 0) --g_live_graphs;
  scratch_release_parked();
}

}  // namespace tsplit

using namespace tsplit;

#define API_BEGIN() try {
#define API_END()                                                        \
  }                                                                      \
  catch (const std::exception &e) {                                      \
    std::fprintf(stderr, "[libc_runtime_api] %s\n", e.what());           \
    return -1;                                                           \
  }                                                                      \
  return 0;

extern "C" {

int ProfilerAlloc(ProfilerHandle *handle) {
  Profiler *p = new Profiler();
  p->time = p->input_memory = p->output_memory = p->workspace_memory = -1.f;
  *handle = p;
  return 0;
}

// ------------------------------------------------------------ streams / events
int DLStreamCreate(size_t dev_id, DLStreamHandle *handle) {
  TS_HIP(hipSetDevice(static_cast<int>(dev_id)));
  hipStream_t *s = new hipStream_t();
  hipError_t e = hipStreamCreate(s);   // default priority, blocking w.r.t. the NULL stream
  if (e != hipSuccess) {
    delete s;
    TS_FAIL("hipStreamCreate failed: %s", hipGetErrorString(e));
  }
  DLStream *h = new DLStream();
  h->device_id = static_cast<int>(dev_id);
  h->handle = s;
  *handle = h;
  return 0;
}

int DLStreamDestroy(DLStreamHandle handle) {
  if (!handle) return 0;
  hipStream_t *s = static_cast<hipStream_t *>(handle->handle);
  if (s) {
    updates_flush_if_any();           // optimizer updates that waited on this stream run before it drains
    (void)hipStreamSynchronize(*s);
    conv_notes_drop_all();            // their sums lie in this stream's scratch
    multi_update_drop_stream(*s);
    scratch_drop_stream(*s);
    TS_HIP(hipStreamDestroy(*s));
    delete s;
  }
  delete handle;
  return 0;
}

int DLStreamSync(DLStreamHandle handle) {
  TS_HIP(hipStreamSynchronize(stream_keep_notes(handle)));   // waiting writes nothing
  return 0;
}

int DLEventCreate(size_t dev_id, DLEventHandle *handle) {
  TS_HIP(hipSetDevice(static_cast<int>(dev_id)));
  hipEvent_t *ev = new hipEvent_t();
  hipError_t e = hipEventCreate(ev);
  if (e != hipSuccess) {
    delete ev;
    TS_FAIL("hipEventCreate failed: %s", hipGetErrorString(e));
  }
  DLEvent *h = new DLEvent();
  h->device_id = static_cast<int>(dev_id);
  h->handle = ev;
  *handle = h;
  return 0;
}

int DLEventDestroy(DLEventHandle handle) {
  if (!handle) return 0;
  hipEvent_t *ev = static_cast<hipEvent_t *>(handle->handle);
  if (ev) {
    TS_HIP(hipEventDestroy(*ev));
    delete ev;
  }
  delete handle;
  return 0;
}

int DLEventRecord(DLStreamHandle stream_handle, DLEventHandle event_handle) {
  TS_REQUIRE(event_handle != nullptr, "DLEventRecord: NULL event");
  // (marking a point on a stream writes nothing: the convolutions' notes stay)
  TS_HIP(hipEventRecord(*static_cast<hipEvent_t *>(event_handle->handle), stream_keep_notes(stream_handle)));
  return 0;
}

int DLEventSync(DLEventHandle handle) {
  TS_REQUIRE(handle != nullptr, "DLEventSync: NULL event");
  TS_HIP(hipEventSynchronize(*static_cast<hipEvent_t *>(handle->handle)));
  return 0;
}

int DLEventQuery(DLEventHandle handle) {
  if (!handle) return 0;
  hipError_t e = hipEventQuery(*static_cast<hipEvent_t *>(handle->handle));
  if (e == hipSuccess) return 1;
  (void)hipGetLastError();   // hipErrorNotReady is sticky in the last-error slot otherwise
  return 0;
}

// ------------------------------------------------------------ recorded steps (HIP graphs)
int TSplit_StreamBeginRecord(DLStreamHandle stream) {
  TS_REQUIRE(stream != nullptr && stream->handle != nullptr, "TSplit_StreamBeginRecord: a created stream is required");
  // relaxed mode: device allocations made by this thread while recording (a new pool slab) are allowed
  TS_HIP(hipStreamBeginCapture(stream_of(stream), hipStreamCaptureModeRelaxed));
  scratch_recording_opened();
  return 0;
}

int TSplit_StreamEndRecord(DLStreamHandle stream, DLGraphHandle *out) {
  TS_REQUIRE(stream != nullptr && stream->handle != nullptr && out != nullptr, "TSplit_StreamEndRecord: NULL argument");
  *out = nullptr;
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(stream_of(stream), &graph);
  if (e != hipSuccess || graph == nullptr) {
    (void)hipGetLastError();
    if (graph) (void)hipGraphDestroy(graph);
    scratch_recording_closed(false);
    TS_FAIL("TSplit_StreamEndRecord: the recording was invalidated (%s)", hipGetErrorString(e));
  }
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    scratch_recording_closed(false);
    TS_FAIL("TSplit_StreamEndRecord: hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  scratch_recording_closed(true);
  DLGraph *g = new DLGraph();
  g->device_id = stream->device_id;
  g->handle = exec;
  *out = g;
  return 0;
}

int TSplit_GraphLaunch(DLGraphHandle graph, DLStreamHandle stream) {
  TS_REQUIRE(graph != nullptr && graph->handle != nullptr, "TSplit_GraphLaunch: NULL graph");
  TS_REQUIRE(stream != nullptr && stream->handle != nullptr, "TSplit_GraphLaunch: a created stream is required");
  TS_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph->handle), stream_of(stream)));
  return 0;
}

int TSplit_GraphDestroy(DLGraphHandle graph) {
  if (!graph) return 0;
  if (graph->handle) TS_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph->handle)));
  delete graph;
  scratch_graph_destroyed();
  return 0;
}

void cuda_init(void) {
  int d = 0;
  if (hipGetDevice(&d) == hipSuccess) (void)hipSetDevice(d);
}
void cudnn_init(size_t dev_id, DLStreamHandle) {
  (void)hipSetDevice(static_cast<int>(dev_id));
  softmax_noalloc_setup(static_cast<int>(dev_id));
}
void cublas_init(size_t dev_id, DLStreamHandle) { (void)hipSetDevice(static_cast<int>(dev_id)); }
void cusp_init(size_t dev_id, DLStreamHandle) { (void)hipSetDevice(static_cast<int>(dev_id)); }

// ------------------------------------------------------------ pool introspection
static int current_device() {
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess) {
    (void)hipGetLastError();
    d = 0;
  }
  return d;
}

void DLMemoryManager_PrintState(void *t, int type) {
  std::lock_guard<std::mutex> lk(g_mu);
  *static_cast<int *>(t) = pool_for(current_device())->FreeChunkCount(type != 0);
}

void DLMemoryManager_Try_to_Malloc(size_t memory_size, void *p) {
  std::lock_guard<std::mutex> lk(g_mu);
  *static_cast<int *>(p) = pool_for(current_device())->Try(memory_size) ? 1 : 0;
}

void DLMemoryManager_GPU_Usage(size_t *used_size, size_t *unused_unavailable_size,
                               size_t *unused_available_size) {
  std::lock_guard<std::mutex> lk(g_mu);
  pool_for(current_device())->Usage(used_size, unused_unavailable_size, unused_available_size);
}

// ------------------------------------------------------------ arrays
int DLArrayAlloc(const index_t *shape, index_t ndim, DLContext ctx, DLArrayHandle *out,
                 int MEMORY_MANAGE_RULE) {
  DLArray *a = nullptr;
  try {
    a = new_array(shape, ndim, ctx);
    a->data = data_alloc(ctx, byte_size(a), MEMORY_MANAGE_RULE);
    *out = a;
  } catch (const std::exception &e) {
    std::fprintf(stderr, "[libc_runtime_api] DLArrayAlloc: %s\n", e.what());
    if (a) {
      delete[] a->shape;
      delete a;
    }
    return -1;
  }
  return 0;
}

int DLArrayAllocSelf(DLArrayHandle handle, int MEMORY_MANAGE_RULE) {
  API_BEGIN();
  handle->data = data_alloc(handle->ctx, byte_size(handle), MEMORY_MANAGE_RULE);
  API_END();
}

int DLArrayFree(DLArrayHandle handle, int MEMORY_MANAGE_RULE) {
  API_BEGIN();
  // An optimizer update that waits may name this array.  Memory of the pool stays mapped and is next written by a
  // call that runs the waiting updates first; memory that goes back to the driver must be done with now.
  if (MEMORY_MANAGE_RULE == 0) updates_flush_if_any();
  if (handle) {
    void *d = handle->data;
    DLContext ctx = handle->ctx;
    delete[] handle->shape;
    delete handle;
    data_free(ctx, d, MEMORY_MANAGE_RULE);
  }
  API_END();
}

int DLArrayFreeSelf(DLArrayHandle handle, int MEMORY_MANAGE_RULE) {
  API_BEGIN();
  if (MEMORY_MANAGE_RULE == 0) updates_flush_if_any();
  void *d = handle->data;
  handle->data = nullptr;
  data_free(handle->ctx, d, MEMORY_MANAGE_RULE);
  API_END();
}

int DLArrayCopyFromTo(DLArrayHandle from, DLArrayHandle to, DLStreamHandle stream) {
  TS_REQUIRE(from && to, "DLArrayCopyFromTo: NULL array");
  size_t bytes = byte_size(from);
  TS_REQUIRE(bytes == byte_size(to), "DLArrayCopyFromTo: sizes differ (%zu vs %zu bytes)", bytes,
             byte_size(to));
  if (bytes == 0) return 0;
  const bool fg = from->ctx.device_type == kGPU, tg = to->ctx.device_type == kGPU;
  if (!fg && !tg) {
    std::memcpy(to->data, from->data, bytes);
    return 0;
  }
  hipMemcpyKind kind = fg && tg ? hipMemcpyDeviceToDevice : (fg ? hipMemcpyDeviceToHost : hipMemcpyHostToDevice);
  TS_HIP(hipSetDevice(fg ? from->ctx.device_id : to->ctx.device_id));
  if (stream) {
    TS_HIP(hipMemcpyAsync(to->data, from->data, bytes, kind, stream_of(stream)));
  } else {
    conv_notes_drop_all();            // (the branch above went through stream_of)
    updates_flush_if_any();
    TS_HIP(hipMemcpy(to->data, from->data, bytes, kind));
  }
  return 0;
}

int DLArrayReuseAlloc(DLContext ctx, int MEMORY_MANAGE_RULE, const index_t *input_shape,
                      index_t input_ndim, DLArrayHandle *input, const index_t *output_shape,
                      index_t output_ndim, DLArrayHandle *output, int pieces, int overlap_pieces) {
  TS_REQUIRE(pieces > 0 && overlap_pieces >= 0 && overlap_pieces <= pieces,
             "DLArrayReuseAlloc: bad pieces/overlap (%d/%d)", pieces, overlap_pieces);
  DLArray *in = nullptr, *out = nullptr;
  try {
    in = new_array(input_shape, input_ndim, ctx);
    out = new_array(output_shape, output_ndim, ctx);
    const size_t in_b = byte_size(in), out_b = byte_size(out);
    const size_t total = out_b + in_b / pieces * (pieces - overlap_pieces);
    if (total < in_b) throw std::runtime_error("DLArrayReuseAlloc: output smaller than the overlapped part of the input");
    char *base = static_cast<char *>(data_alloc(ctx, total, MEMORY_MANAGE_RULE));
    out->data = base;                      // output at the base
    in->data = base + (total - in_b);      // input flush with the end
    *input = in;
    *output = out;
  } catch (const std::exception &e) {
    std::fprintf(stderr, "[libc_runtime_api] %s\n", e.what());
    for (DLArray *a : {in, out})
      if (a) {
        delete[] a->shape;
        delete a;
      }
    return -1;
  }
  return 0;
}

int DLArraySliceForMicroTensor(DLArrayHandle input, DLArrayHandle *output, int total_number,
                               int index, int dimension) {
  TS_REQUIRE(input && input->ndim >= 1, "DLArraySliceForMicroTensor: bad input");
  TS_REQUIRE(total_number > 0 && index >= 0 && index < total_number,
             "DLArraySliceForMicroTensor: index %d of %d", index, total_number);
  const int d = dimension == 0 ? 0 : 1;
  TS_REQUIRE(d < input->ndim, "DLArraySliceForMicroTensor: dimension %d of a %d-d array", d, input->ndim);
  DLArray *v = new_array(input->shape, input->ndim, input->ctx);
  const int64_t D = input->shape[d];
  const int64_t len = D ? numel(input) / D : 0;   // elements per index of the split dimension
  const int64_t base = D / total_number, extra = D % total_number;
  // pieces [0, extra) hold base+1 indices, the rest hold base
  const int64_t before = static_cast<int64_t>(index) * base + (index < extra ? index : extra);
  v->shape[d] = base + (index < extra ? 1 : 0);
  // For d == 1 this is, like the reference, a contiguous chunk re-labelled [N, C/k, ...]:
  // a true channel slice only when N == 1.
  v->data = static_cast<float *>(input->data) + before * len;
  *output = v;
  return 0;
}

}  // extern "C"
