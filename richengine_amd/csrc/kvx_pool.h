// The page pool: sole owner of page references and of which extents hold
// memory.  Written against an abstract extent storage so the same code runs
// over device extents (through the C ABI) and over an accounting-only storage
// in host tests.  Behaviour follows the reference's engine::KvPool
// (runtime/engine/cache/KvPool.hpp:64-115, KvPool.cpp).
#pragma once

#include <cstdint>
#include <vector>

#include "kvx.h"

namespace kvx {

// What the pool needs of its memory (reference: kv::ExtentStorage,
// runtime/ops/PagedKv.hpp:56-76).  Status codes are the KVX_* values.
class ExtentStorage {
public:
  virtual ~ExtentStorage() = default;
  virtual uint32_t page_count() const = 0;
  virtual uint64_t bytes_per_page() const = 0;
  virtual uint32_t extent_pages() const = 0;
  virtual int allocate_extent(uint32_t extent) = 0;
  virtual int release_extent(uint32_t extent) = 0;
  virtual int copy_pages(const kvx_page_copy *copies, uint32_t n) = 0;
};

struct PageMoves {
  uint32_t first_page = 0;
  std::vector<uint32_t> destinations;  // by offset in the emptied extent
  uint32_t moved = 0;
  bool empty() const { return destinations.empty(); }
  uint32_t follow(uint32_t page) const {
    return page >= first_page && page - first_page < destinations.size()
               ? destinations[page - first_page]
               : page;
  }
};

class KvPool {
public:
  // status() != KVX_OK after construction when the runway was refused
  // (KVX_ENOMEM) or the geometry is invalid (KVX_EINVAL).
  KvPool(ExtentStorage &storage, uint32_t runway_pages);
  int status() const { return status_; }

  int acquire(uint32_t count, uint32_t *pages);
  int retain(uint32_t page, bool prefix_owner);
  int release(uint32_t page, bool prefix_owner);
  bool page_active(uint32_t page) const { return pages_[page].active != 0; }
  uint32_t page_count() const { return uint32_t(pages_.size()); }
  uint32_t extent_pages() const { return extent_pages_; }
  uint32_t free_pages() const { return free_pages_; }
  uint64_t allocated_bytes() const;
  uint32_t reusable_pages() const { return allocated_extents_ * extent_pages_ - active_pages_; }
  int reclaim_empty(bool keep_runway, uint32_t limit, uint64_t *released);
  int compact_extent(const uint32_t *fixed, uint32_t n_fixed, PageMoves *moves);
  void snapshot(kvx_pool_snapshot *out) const;

private:
  static constexpr uint32_t kNone = 0xffffffffu;
  struct Page {
    uint32_t active = 0;
    uint32_t prev = kNone, next = kNone;
    bool prefix = false, listed = false;
  };
  struct Extent {
    uint32_t used = 0;
    uint32_t free_head = kNone, free_count = 0;
    uint32_t prev_reclaimable = kNone, next_reclaimable = kNone;
    bool allocated = false, reclaimable = false;
  };
  bool is_free(uint32_t page) const { return !pages_[page].active && !pages_[page].prefix; }
  uint32_t extent_of(uint32_t page) const { return page / extent_pages_; }
  void list_insert(uint32_t page);
  void list_remove(uint32_t page);
  uint32_t packing_extent();
  void mark_used(uint32_t page);
  void mark_free(uint32_t page);
  void set_allocated(uint32_t extent, bool allocated);
  void set_reclaimable(uint32_t extent, bool reclaimable);
  int allocate_extent(uint32_t extent);
  int release_extent(uint32_t extent);

  ExtentStorage &storage_;
  int status_ = KVX_OK;
  uint32_t extent_pages_ = 0;
  std::vector<Page> pages_;
  std::vector<Extent> extents_;
  uint32_t free_pages_ = 0, active_pages_ = 0, prefix_pages_ = 0, allocated_extents_ = 0;
  uint32_t packing_ = kNone;
  uint32_t reclaimable_head_ = kNone, reclaimable_count_ = 0;
  uint64_t allocations_ = 0, releases_ = 0, compactions_ = 0, moved_ = 0;
  double allocate_max_ms_ = 0, release_max_ms_ = 0;
};

}  // namespace kvx
