// Device-agnostic core of the pooled tensor allocator behind DLArrayAlloc(rule != 0).
//
// Role of the reference's DLMemoryManager (src/cuda_common/gpu_memory_manager.cc:97-318):
// best-fit search over free chunks, split on allocation, coalesce with free neighbours
// on release, plus the used / unused-unavailable / unused-available accounting that the
// memory-policy executors poll.  Differences, chosen for a 288 GB device:
//   * the reference grabs (free - 500 MB) in one cudaMalloc at start-up; here the pool grows
//     by slabs on demand, so a process only holds what its tensors ever needed;
//   * free chunks live in one size-ordered set (the same answer as the reference's 30
//     power-of-two bins searched upward, in O(log n));
//   * a capacity limit can emulate a smaller device.
// The core never dereferences the memory it manages and gets its backing store through
// function pointers, so the host tests drive it over a fake address range.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <map>
#include <set>
#include <utility>
#include <vector>

namespace tsplit {

struct PoolBacking {
  void *(*alloc)(size_t bytes, void *user);   // returns nullptr on failure
  void (*release)(void *ptr, void *user);
  size_t (*available)(void *user);            // bytes the backing store could still hand out
  void *user;
};

class BinnedPool {
 public:
  static constexpr size_t kAlign = 256;                 // ref: chunk granularity 256 B
  static constexpr size_t kSplitSlack = 128ull << 20;   // ref: gpu_memory_manager.cc:222-223

  // split_slack: a free block at most twice the request is handed out whole unless the part left over
  // would reach this many bytes (the reference's 128 MiB by default; 0 splits always, which wastes
  // nothing and is what a capacity limit close to the tensors' own total needs)
  BinnedPool(PoolBacking backing, size_t slab_bytes, size_t limit_bytes, size_t split_slack = kSplitSlack)
      : backing_(backing), slab_bytes_(slab_bytes), limit_(limit_bytes), split_slack_(split_slack) {}

  ~BinnedPool() {
    for (Chunk *c : all_) delete c;
    for (void *s : slabs_) backing_.release(s, backing_.user);
  }

  static size_t RoundUp(size_t n) { return n == 0 ? kAlign : (n + kAlign - 1) / kAlign * kAlign; }

  void *Malloc(size_t bytes) {
    const size_t need = RoundUp(bytes);
    Chunk *c = Search(need);
    if (c == nullptr && !Grow(need)) return nullptr;
    if (c == nullptr) c = Search(need);
    if (c == nullptr) return nullptr;
    free_.erase({c->size, c});
    c->in_use = true;
    c->used = bytes;
    // split rule of the reference: only when the block is more than twice the request or
    // the slack reaches 128 MiB; smaller slack stays attached ("unused unavailable").
    if (c->size > need && (c->size > 2 * need || c->size - need >= split_slack_)) Split(c, need);
    live_[c->ptr] = c;
    return c->ptr;
  }

  bool Free(void *ptr) {
    auto it = live_.find(static_cast<char *>(ptr));
    if (it == live_.end()) return false;
    Chunk *c = it->second;
    live_.erase(it);
    c->in_use = false;
    c->used = 0;
    if (c->prev && !c->prev->in_use) c = Merge(c->prev, c);
    if (c->next && !c->next->in_use) c = Merge(c, c->next);
    free_.insert({c->size, c});
    return true;
  }

  bool Owns(void *ptr) const { return live_.count(static_cast<char *>(ptr)) != 0; }

  // Would Malloc(bytes) succeed right now (from a free chunk or by growing)?
  bool Try(size_t bytes) {
    const size_t need = RoundUp(bytes);
    if (Search(need)) return true;
    return need <= Growable();
  }

  // used: bytes requested by live tensors; unused_unavailable: slack inside live chunks;
  // unused_available: free chunks plus what the pool may still take from the device.
  void Usage(size_t *used, size_t *unused_unavailable, size_t *unused_available) {
    size_t u = 0, uu = 0, ua = 0;
    for (Chunk *c : all_) {
      if (c->in_use) {
        u += c->used;
        uu += c->size - c->used;
      } else {
        ua += c->size;
      }
    }
    *used = u;
    *unused_unavailable = uu;
    *unused_available = ua + Growable();
  }

  int FreeChunkCount(bool print) {
    int n = 0;
    if (print) std::printf("------------ pool state: %zu slabs, %zu bytes reserved ------------\n", slabs_.size(), reserved_);
    for (Chunk *c : all_) {
      if (!c->in_use) ++n;
      if (print) std::printf("  chunk %p size %zu %s used %zu\n", (void *)c->ptr, c->size, c->in_use ? "LIVE" : "free", c->used);
    }
    if (print) std::printf("------------ pool state end ------------\n");
    return n;
  }

  size_t Reserved() const { return reserved_; }
  size_t SlabCount() const { return slabs_.size(); }

 private:
  struct Chunk {
    char *ptr;
    size_t size;
    size_t used;
    bool in_use;
    Chunk *prev;   // address-order neighbours inside the same slab
    Chunk *next;
  };
  struct BySizeThenAddr {
    bool operator()(const std::pair<size_t, Chunk *> &a, const std::pair<size_t, Chunk *> &b) const {
      if (a.first != b.first) return a.first < b.first;
      return a.second->ptr < b.second->ptr;
    }
  };

  Chunk *Search(size_t need) {
    // lower_bound needs a key object; a stack chunk with a null address sorts first
    Chunk probe{nullptr, need, 0, false, nullptr, nullptr};
    auto it = free_.lower_bound({need, &probe});
    return it == free_.end() ? nullptr : it->second;
  }

  size_t Growable() {
    size_t dev = backing_.available(backing_.user);
    size_t cap = limit_ > reserved_ ? limit_ - reserved_ : 0;
    return dev < cap ? dev : cap;
  }

  bool Grow(size_t need) {
    size_t room = Growable();
    if (need > room) return false;
    size_t want = need > slab_bytes_ ? need : slab_bytes_;
    if (want > room) want = room / kAlign * kAlign;
    if (want < need) return false;
    void *p = backing_.alloc(want, backing_.user);
    if (p == nullptr && want > need) {
      want = need;
      p = backing_.alloc(want, backing_.user);
    }
    if (p == nullptr) return false;
    slabs_.push_back(p);
    reserved_ += want;
    Chunk *c = new Chunk{static_cast<char *>(p), want, 0, false, nullptr, nullptr};
    all_.insert(c);
    free_.insert({c->size, c});
    return true;
  }

  void Split(Chunk *c, size_t need) {
    Chunk *rest = new Chunk{c->ptr + need, c->size - need, 0, false, c, c->next};
    if (c->next) c->next->prev = rest;
    c->next = rest;
    c->size = need;
    all_.insert(rest);
    free_.insert({rest->size, rest});
  }

  Chunk *Merge(Chunk *a, Chunk *b) {   // a directly precedes b, both free; b is absorbed
    if (free_.count({a->size, a})) free_.erase({a->size, a});
    if (free_.count({b->size, b})) free_.erase({b->size, b});
    a->size += b->size;
    a->next = b->next;
    if (b->next) b->next->prev = a;
    all_.erase(b);
    delete b;
    return a;
  }

  struct ByAddr {
    bool operator()(const Chunk *a, const Chunk *b) const { return a->ptr < b->ptr; }
  };

  PoolBacking backing_;
  size_t slab_bytes_;
  size_t limit_;
  size_t split_slack_;
  size_t reserved_ = 0;
  std::vector<void *> slabs_;
  std::set<Chunk *, ByAddr> all_;
  std::set<std::pair<size_t, Chunk *>, BySizeThenAddr> free_;
  std::map<char *, Chunk *> live_;
};

}  // namespace tsplit
