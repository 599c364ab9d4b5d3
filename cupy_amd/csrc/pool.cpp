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
#include "mi355rt.h"

#include <hip/hip_runtime.h>

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

struct Pool {
  std::mutex mutex;
  rt_pool_alloc_fn alloc_fn = default_alloc;
  rt_pool_free_fn free_fn = default_free;
  void* ctx = nullptr;
  size_t limit = 0;
  size_t total_bytes = 0;  // bytes obtained from the allocator (in use + cached)
  size_t used_bytes = 0;
  std::unordered_map<uint64_t, Arena> arenas;
  std::unordered_map<uint64_t, Chunk*> in_use;

  // Releases cached blocks that are whole allocations (never split, or fully
  // re-merged).  Split blocks stay: part of their allocation is still in use.
  void release_arena(Arena& arena) {
    std::vector<Chunk*> victims;
    for (auto& kv : arena.bins)
      for (Chunk* c = kv.second.head; c; c = c->bin_next)
        if (!c->prev && !c->next) victims.push_back(c);
    for (Chunk* c : victims) {
      arena.remove(c);
      free_fn(ctx, c->base, c->base_size);
      total_bytes -= c->base_size;
      delete c;
    }
  }

  void release_all() {
    for (auto& kv : arenas) release_arena(kv.second);
  }

  // Obtain a fresh allocation, honouring the limit; cached blocks are given
  // back to the driver before the request is refused.
  int allocate_fresh(size_t size, uint64_t* address) {
    if (limit != 0 && total_bytes + size > limit) {
      release_all();
      if (total_bytes + size > limit) return RT_ERR_POOL_OOM;
    }
    if (alloc_fn(ctx, size, address) == 0) return 0;
    release_all();
    if (alloc_fn(ctx, size, address) == 0) return 0;
    return RT_ERR_POOL_OOM;
  }
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
  {
    std::lock_guard<std::mutex> lock(p->mutex);
    p->release_all();
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
    for (auto& kv : bases) p->free_fn(p->ctx, kv.first, kv.second);
  }
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
  std::lock_guard<std::mutex> lock(p->mutex);
  Arena& arena = p->arenas[stream_ident];
  Chunk* c = arena.take_best_fit(size);
  if (!c) {
    uint64_t base = 0;
    int status = p->allocate_fresh(size, &base);
    if (status != 0) {
      rt_set_last_error_("rt_pool_malloc: out of memory");
      return status;
    }
    c = new (std::nothrow) Chunk{base, size, 0, size, stream_ident, false,
                                 nullptr, nullptr, nullptr, nullptr};
    if (!c) {
      p->free_fn(p->ctx, base, size);
      rt_set_last_error_("rt_pool_malloc: out of host memory");
      return RT_ERR_POOL_OOM;
    }
    p->total_bytes += size;
  } else if (c->size > size) {
    Chunk* tail = new (std::nothrow) Chunk{c->base, c->base_size, c->offset + size,
                                           c->size - size, c->stream, false,
                                           c, c->next, nullptr, nullptr};
    if (tail) {
      if (c->next) c->next->prev = tail;
      c->next = tail;
      c->size = size;
      arena.insert(tail);
    }
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
  std::lock_guard<std::mutex> lock(p->mutex);
  auto it = p->in_use.find(address);
  if (it == p->in_use.end()) {
    rt_set_last_error_("rt_pool_free: address is not an in-use block of this pool");
    return RT_ERR_INVALID;
  }
  Chunk* c = it->second;
  p->in_use.erase(it);
  c->in_use = false;
  p->used_bytes -= c->size;
  Arena& arena = p->arenas[c->stream];
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

int rt_pool_free_all_blocks(void* pool, int all_streams, uint64_t stream_ident) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p) {
    rt_set_last_error_("rt_pool_free_all_blocks: null pool");
    return RT_ERR_INVALID;
  }
  std::lock_guard<std::mutex> lock(p->mutex);
  if (all_streams) {
    p->release_all();
  } else {
    auto it = p->arenas.find(stream_ident);
    if (it != p->arenas.end()) p->release_arena(it->second);
  }
  return 0;
}

int rt_pool_stats(void* pool, size_t* used_bytes, size_t* free_bytes, size_t* total_bytes,
                  size_t* n_free_blocks) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p) {
    rt_set_last_error_("rt_pool_stats: null pool");
    return RT_ERR_INVALID;
  }
  std::lock_guard<std::mutex> lock(p->mutex);
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
  std::lock_guard<std::mutex> lock(p->mutex);
  p->limit = limit_bytes;
  return 0;
}

int rt_pool_get_limit(void* pool, size_t* limit_bytes) {
  Pool* p = static_cast<Pool*>(pool);
  if (!p || !limit_bytes) {
    rt_set_last_error_("rt_pool_get_limit: null argument");
    return RT_ERR_INVALID;
  }
  std::lock_guard<std::mutex> lock(p->mutex);
  *limit_bytes = p->limit;
  return 0;
}

}  // extern "C"
