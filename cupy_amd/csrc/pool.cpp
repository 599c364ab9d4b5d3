// mi355rt: device memory pool (native core of the MemoryPool API).
//
// Layout of the cache: one arena per stream identity; inside an arena free
// blocks hang in size bins (size -> LIFO list), looked up with lower_bound so a
// request takes the smallest cached block that fits ("best fit") and the most
// recently freed block of that size (still warm in the TLB).  A block that is
// larger than the request is split; the tail goes back into its bin.  Blocks
// carved from one underlying allocation form a doubly linked list in address
// order, so freeing merges with free neighbours in O(1).
//
// Stream order is what makes reuse safe without synchronisation: a block freed
// while kernels of stream S still use it is handed out again only on S, whose
// later work runs after those kernels.
//
// Locking: one mutex per pool guards the bookkeeping and nothing else.  The
// allocator callbacks (hipMalloc / hipFree, or a host-language allocator that
// may run arbitrary code, a garbage collector included) are only ever called
// with the mutex RELEASED: a request that misses the cache reserves its bytes
// against the limit, unlocks, allocates, and locks again to register the block;
// blocks to be given back are unlinked under the lock and released after it.
// rt_pool_free never blocks: when the mutex is busy the address goes onto a
// lock-free list that the next holder of the mutex works off
// (cupy/cuda/memory.pyx:1364-1398 takes the same two precautions).
#include "mi355rt.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <map>
#include <mutex>
#include <new>
#include <unordered_map>
#include <vector>

void rt_set_last_error_(const char* text);

namespace {

struct Chunk {
  uint64_t base;      // address of the underlying allocation
  size_t base_size;   // size of the underlying allocation
  size_t offset;      // offset of this block inside it
  size_t size;
  uint64_t stream;    // arena this block belongs to
  bool in_use;
  Chunk* prev;        // address-order neighbours inside the same allocation
  Chunk* next;
  Chunk* bin_prev;    // neighbours inside the size bin (free blocks only)
  Chunk* bin_next;
  uint64_t address() const { return base + offset; }
};

struct Bin {
  Chunk* head = nullptr;
  size_t count = 0;
};

struct Arena {
  std::map<size_t, Bin> bins;

  void insert(Chunk* c) {
    Bin& b = bins[c->size];
    c->bin_prev = nullptr;
    c->bin_next = b.head;
    if (b.head) b.head->bin_prev = c;
    b.head = c;
    ++b.count;
  }

  void remove(Chunk* c) {
    auto it = bins.find(c->size);
    Bin& b = it->second;
    if (c->bin_prev) c->bin_prev->bin_next = c->bin_next;
    else b.head = c->bin_next;
    if (c->bin_next) c->bin_next->bin_prev = c->bin_prev;
    c->bin_prev = c->bin_next = nullptr;
    if (--b.count == 0) bins.erase(it);
  }

  Chunk* take_best_fit(size_t size) {
    auto it = bins.lower_bound(size);
    if (it == bins.end()) return nullptr;
    Chunk* c = it->second.head;
    remove(c);
    return c;
  }
};

int default_alloc(void*, size_t size, uint64_t* address) {
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, size);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return static_cast<int>(e);
  }
  *address = reinterpret_cast<uint64_t>(p);
  return 0;
}

void default_free(void*, uint64_t address, size_t) {
  if (hipFree(reinterpret_cast<void*>(address)) != hipSuccess) (void)hipGetLastError();
}

struct PendingFree {
  uint64_t address;
  PendingFree* next;
};

struct Released {
  uint64_t base;
  size_t size;
};

struct Pool {
  std::mutex mutex;
  rt_pool_alloc_fn alloc_fn = default_alloc;
  rt_pool_free_fn free_fn = default_free;
  void* ctx = nullptr;
  size_t limit = 0;
  size_t total_bytes = 0;  // bytes obtained from the allocator (in use + cached)
  size_t used_bytes = 0;
  size_t reserved_bytes = 0;  // requests that are at the allocator right now
  std::unordered_map<uint64_t, Arena> arenas;
  std::unordered_map<uint64_t, Chunk*> in_use;
  std::atomic<PendingFree*> pending{nullptr};

  // ---- everything below expects the mutex to be held ----

  // Returns one block to its arena, merging it with free neighbours.
  int put_back(uint64_t address) {
    auto it = in_use.find(address);
    if (it == in_use.end()) return RT_ERR_INVALID;
    Chunk* c = it->second;
    in_use.erase(it);
    c->in_use = false;
    used_bytes -= c->size;
    Arena& arena = arenas[c->stream];
    if (c->next && !c->next->in_use) {
      Chunk* n = c->next;
      arena.remove(n);
      c->size += n->size;
      c->next = n->next;
      if (n->next) n->next->prev = c;
      delete n;
    }
    if (c->prev && !c->prev->in_use) {
      Chunk* q = c->prev;
      arena.remove(q);
      q->size += c->size;
      q->next = c->next;
      if (c->next) c->next->prev = q;
      delete c;
      c = q;
    }
    arena.insert(c);
    return 0;
  }

  // Works off the frees that found the mutex busy.
  void drain_pending() {
    PendingFree* node = pending.exchange(nullptr, std::memory_order_acquire);
    while (node) {
      PendingFree* next = node->next;
      (void)put_back(node->address);
      delete node;
      node = next;
    }
  }

  // Unlinks cached blocks that are whole allocations (never split, or fully
  // re-merged) and lists them in `out`; the caller hands them to free_fn once
  // the mutex is released.  Split blocks stay: part of their allocation is
  // still in use.
  void unlink_arena(Arena& arena, std::vector<Released>* out) {
    std::vector<Chunk*> victims;
    for (auto& kv : arena.bins)
      for (Chunk* c = kv.second.head; c; c = c->bin_next)
        if (!c->prev && !c->next) victims.push_back(c);
    for (Chunk* c : victims) {
      arena.remove(c);
      out->push_back(Released{c->base, c->base_size});
      total_bytes -= c->base_size;
      delete c;
    }
  }

  void unlink_all(std::vector<Released>* out) {
    for (auto& kv : arenas) unlink_arena(kv.second, out);
  }

  // ---- and this one expects it to be released ----
  void give_back(const std::vector<Released>& blocks) {
    for (const Released& r : blocks) free_fn(ctx, r.base, r.size);
  }
};

// Holds the pool's mutex; frees that piled up meanwhile are worked off on
// entry and again after leaving, so none waits for the next unrelated call.
class Locked {
 public:
  explicit Locked(Pool* p) : p_(p) { lock(); }
  ~Locked() {
    if (held_) unlock();
  }
  void lock() {
    p_->mutex.lock();
    held_ = true;
    p_->drain_pending();
  }
  void unlock() {
    p_->mutex.unlock();
    held_ = false;
    while (p_->pending.load(std::memory_order_acquire) && p_->mutex.try_lock()) {
      p_->drain_pending();
      p_->mutex.unlock();
    }
  }

 private:
  Pool* p_;
  bool held_ = false;
};

}  // namespace

extern "C" {

size_t rt_pool_round_size(size_t size) {
  return (size + RT_POOL_UNIT - 1) / RT_POOL_UNIT * RT_POOL_UNIT;
}

int rt_pool_create(void** pool) {
  return rt_pool_create_with_allocator(pool, nullptr, nullptr, nullptr);
}

int rt_pool_create_with_allocator(void** pool, rt_pool_alloc_fn alloc_fn, rt_pool_free_fn free_fn,
                                  void* ctx) {
  if (!pool) {
    rt_set_last_error_("rt_pool_create: null output");
    return RT_ERR_INVALID;
  }
  if ((alloc_fn == nullptr) != (free_fn == nullptr)) {
    rt_set_last_error_("rt_pool_create: alloc and free callbacks must be given together");
    return RT_ERR_INVALID;
  }
  Pool* p = new (std::nothrow) Pool();
  if (!p) {
    rt_set_last_error_("rt_pool_create: out of host memory");
    return RT_ERR_INVALID;
  }
  if (alloc_fn) {
    p->alloc_fn = alloc_fn;
    p->free_fn = free_fn;
    p->ctx = ctx;
  }
  *pool = p;
  return 0;
}

int rt_pool_destroy(void* pool) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p) return 0;
  std::vector<Released> blocks;
  {
    Locked lock(p);
    p->unlink_all(&blocks);
    // Free blocks that are still split cannot be returned piecewise; drop the
    // bookkeeping and hand whole allocations back once per base address.
    std::unordered_map<uint64_t, size_t> bases;
    for (auto& kv : p->arenas)
      for (auto& bin : kv.second.bins)
        for (Chunk* c = bin.second.head; c;) {
          Chunk* next = c->bin_next;
          bases[c->base] = c->base_size;
          delete c;
          c = next;
        }
    for (auto& kv : p->in_use) {
      bases.erase(kv.second->base);  // still referenced by the caller: leak it
      delete kv.second;
    }
    for (auto& kv : bases) blocks.push_back(Released{kv.first, kv.second});
    p->arenas.clear();
    p->in_use.clear();
  }
  p->give_back(blocks);
  delete p;
  return 0;
}

int rt_pool_malloc(void* pool, size_t size, uint64_t stream_ident, uint64_t* address) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p || !address || size == 0) {
    rt_set_last_error_("rt_pool_malloc: null pool/output or zero size");
    return RT_ERR_INVALID;
  }
  size = rt_pool_round_size(size);
  Locked lock(p);
  Chunk* c = p->arenas[stream_ident].take_best_fit(size);
  if (c) {
    if (c->size > size) {
      Chunk* tail = new (std::nothrow) Chunk{c->base, c->base_size, c->offset + size,
                                             c->size - size, c->stream, false,
                                             c, c->next, nullptr, nullptr};
      if (tail) {
        if (c->next) c->next->prev = tail;
        c->next = tail;
        c->size = size;
        p->arenas[stream_ident].insert(tail);
      }
    }
  } else {
    // Cache miss.  The request is booked against the limit first, so that
    // requests running side by side cannot exceed it together; cached blocks
    // are given back to the allocator before the request is refused
    // (cupy/cuda/memory.pyx:1518-1563).
    std::vector<Released> blocks;
    auto over_limit = [&] {
      return p->limit != 0 && p->total_bytes + p->reserved_bytes + size > p->limit;
    };
    if (over_limit()) {
      p->unlink_all(&blocks);
      if (over_limit()) {
        lock.unlock();
        p->give_back(blocks);
        rt_set_last_error_("rt_pool_malloc: out of memory");
        return RT_ERR_POOL_OOM;
      }
    }
    p->reserved_bytes += size;
    lock.unlock();
    p->give_back(blocks);
    uint64_t base = 0;
    bool ok = p->alloc_fn(p->ctx, size, &base) == 0;
    if (!ok) {
      blocks.clear();
      lock.lock();
      p->unlink_all(&blocks);
      lock.unlock();
      p->give_back(blocks);
      ok = p->alloc_fn(p->ctx, size, &base) == 0;
    }
    if (ok) {
      c = new (std::nothrow) Chunk{base, size, 0, size, stream_ident, false,
                                   nullptr, nullptr, nullptr, nullptr};
      if (!c) p->free_fn(p->ctx, base, size);
    }
    lock.lock();
    p->reserved_bytes -= size;
    if (!c) {
      rt_set_last_error_(ok ? "rt_pool_malloc: out of host memory"
                            : "rt_pool_malloc: out of memory");
      return RT_ERR_POOL_OOM;
    }
    p->total_bytes += size;
  }
  c->in_use = true;
  p->used_bytes += c->size;
  p->in_use[c->address()] = c;
  *address = c->address();
  return 0;
}

int rt_pool_free(void* pool, uint64_t address) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p) {
    rt_set_last_error_("rt_pool_free: null pool");
    return RT_ERR_INVALID;
  }
  if (!p->mutex.try_lock()) {
    // Somebody else is inside the pool (possibly further up this very thread's
    // stack, e.g. a finaliser run by a signal or collector): leave the address
    // for the next holder of the mutex.  An address the pool does not know is
    // then dropped silently when the list is worked off.
    PendingFree* node = new (std::nothrow) PendingFree{address, nullptr};
    if (!node) {
      rt_set_last_error_("rt_pool_free: out of host memory");
      return RT_ERR_INVALID;
    }
    node->next = p->pending.load(std::memory_order_relaxed);
    while (!p->pending.compare_exchange_weak(node->next, node, std::memory_order_release,
                                             std::memory_order_relaxed)) {
    }
    // The holder may have left between the failed try and the push.
    if (p->mutex.try_lock()) {
      p->drain_pending();
      p->mutex.unlock();
    }
    return 0;
  }
  p->drain_pending();
  int status = p->put_back(address);
  p->mutex.unlock();
  if (status != 0)
    rt_set_last_error_("rt_pool_free: address is not an in-use block of this pool");
  return status;
}

int rt_pool_free_all_blocks(void* pool, int all_streams, uint64_t stream_ident) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p) {
    rt_set_last_error_("rt_pool_free_all_blocks: null pool");
    return RT_ERR_INVALID;
  }
  std::vector<Released> blocks;
  {
    Locked lock(p);
    if (all_streams) {
      p->unlink_all(&blocks);
    } else {
      auto it = p->arenas.find(stream_ident);
      if (it != p->arenas.end()) p->unlink_arena(it->second, &blocks);
    }
  }
  p->give_back(blocks);
  return 0;
}

int rt_pool_stats(void* pool, size_t* used_bytes, size_t* free_bytes, size_t* total_bytes,
                  size_t* n_free_blocks) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p) {
    rt_set_last_error_("rt_pool_stats: null pool");
    return RT_ERR_INVALID;
  }
  Locked lock(p);
  size_t blocks = 0;
  for (auto& kv : p->arenas)
    for (auto& bin : kv.second.bins) blocks += bin.second.count;
  if (used_bytes) *used_bytes = p->used_bytes;
  if (free_bytes) *free_bytes = p->total_bytes - p->used_bytes;
  if (total_bytes) *total_bytes = p->total_bytes;
  if (n_free_blocks) *n_free_blocks = blocks;
  return 0;
}

int rt_pool_set_limit(void* pool, size_t limit_bytes) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p) {
    rt_set_last_error_("rt_pool_set_limit: null pool");
    return RT_ERR_INVALID;
  }
  Locked lock(p);
  p->limit = limit_bytes;
  return 0;
}

int rt_pool_get_limit(void* pool, size_t* limit_bytes) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p || !limit_bytes) {
    rt_set_last_error_("rt_pool_get_limit: null argument");
    return RT_ERR_INVALID;
  }
  Locked lock(p);
  *limit_bytes = p->limit;
  return 0;
}

}  // extern "C"
