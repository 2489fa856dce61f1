// Host-only C face of the pool core over a fake address range, for the CPU unit tests.
// Nothing is ever dereferenced: "allocating" backing memory just advances a counter.
#include "pool.h"

namespace {
struct FakeDevice {
  size_t capacity;
  size_t handed_out;
  uintptr_t next;
  int alloc_calls;
};
void *fake_alloc(size_t bytes, void *u) {
  FakeDevice *d = static_cast<FakeDevice *>(u);
  if (d->handed_out + bytes > d->capacity) return nullptr;
  d->handed_out += bytes;
  void *p = reinterpret_cast<void *>(d->next);
  d->next += (bytes + 4095) / 4096 * 4096 + 4096;   // slabs are never adjacent
  d->alloc_calls++;
  return p;
}
void fake_release(void *, void *) {}
size_t fake_available(void *u) {
  FakeDevice *d = static_cast<FakeDevice *>(u);
  return d->capacity - d->handed_out;
}
struct Handle {
  FakeDevice dev;
  tsplit::BinnedPool *pool;
};
}  // namespace

extern "C" {
void *pool_test_create(size_t device_capacity, size_t slab_bytes, size_t limit_bytes) {
  Handle *h = new Handle{{device_capacity, 0, 0x10000000u, 0}, nullptr};
  tsplit::PoolBacking b{fake_alloc, fake_release, fake_available, &h->dev};
  h->pool = new tsplit::BinnedPool(b, slab_bytes, limit_bytes);
  return h;
}
void pool_test_destroy(void *hh) {
  Handle *h = static_cast<Handle *>(hh);
  delete h->pool;
  delete h;
}
uintptr_t pool_test_malloc(void *hh, size_t bytes) {
  return reinterpret_cast<uintptr_t>(static_cast<Handle *>(hh)->pool->Malloc(bytes));
}
int pool_test_free(void *hh, uintptr_t p) {
  return static_cast<Handle *>(hh)->pool->Free(reinterpret_cast<void *>(p)) ? 1 : 0;
}
int pool_test_try(void *hh, size_t bytes) { return static_cast<Handle *>(hh)->pool->Try(bytes) ? 1 : 0; }
void pool_test_usage(void *hh, size_t *used, size_t *uu, size_t *ua) {
  static_cast<Handle *>(hh)->pool->Usage(used, uu, ua);
}
int pool_test_free_chunks(void *hh) { return static_cast<Handle *>(hh)->pool->FreeChunkCount(false); }
size_t pool_test_reserved(void *hh) { return static_cast<Handle *>(hh)->pool->Reserved(); }
int pool_test_backing_calls(void *hh) { return static_cast<Handle *>(hh)->dev.alloc_calls; }
}
