// The page pool: sole owner of page references and of which extents hold
// memory.  Written against an abstract extent storage so the same code runs
// over device extents (through the C ABI) and over an accounting-only storage
// in host tests.
//
// What is fixed from outside is behaviour, held by the reference's pool cases
// (dev/tests/engine/elastic_kv_pool_test.cpp:40-383; interface
// runtime/engine/cache/KvPool.hpp:64-115): which page ids an acquisition hands
// out, which extents a reclaim gives back, which pages a compaction moves and
// where.  The bookkeeping behind it is this file's own:
//  - every extent keeps its free pages on a stack (last freed, first reused;
//    a fresh extent is stacked lowest page on top).  A page that is taken out
//    of the middle of a stack (a reference to a page that was free) leaves a
//    stale entry behind, told from a live one by the page's ticket; stale
//    entries are dropped when they reach the top or when a stack has grown to
//    twice its extent;
//  - the extents that can serve an acquisition sit in an ordered set keyed by
//    (unheld pages, extent index), so the fullest extent with a free page, the
//    lowest index among equals, is its first element;
//  - an extent without held pages remembers when it became idle; a reclaim
//    visits idle extents latest first.
#pragma once

#include <cstdint>
#include <set>
#include <utility>
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

// Where the pages of an emptied extent went (reference: KvPageMoves,
// runtime/engine/cache/KvPool.hpp:39-52).
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
  bool page_active(uint32_t page) const { return page_[page].holders != 0; }
  // More than one holder, or the prefix cache among them: a holder that wants
  // to write the page needs a copy of its own first.
  bool page_shared(uint32_t page) const {
    return page_[page].holders + (page_[page].cached ? 1u : 0u) > 1;
  }
  // Whole-page copies through the pool's storage (kv_page_copy on device storage).
  int copy_pages(const kvx_page_copy *copies, uint32_t n) { return storage_.copy_pages(copies, n); }
  uint32_t page_count() const { return uint32_t(page_.size()); }
  uint32_t extent_pages() const { return span_; }
  uint32_t free_pages() const { return free_total_; }
  uint64_t allocated_bytes() const;
  uint32_t reusable_pages() const { return resident_ * span_ - active_total_; }
  int reclaim_empty(bool keep_runway, uint32_t limit, uint64_t *released);
  // Pages that a compaction frees are reusable at once in the pool's books, while
  // the copy that empties them is only enqueued (device storage copies on the
  // stream the caller names): whoever writes such a page next must do so on that
  // stream, or after it.
  int compact_extent(const uint32_t *fixed, uint32_t n_fixed, PageMoves *moves);
  void snapshot(kvx_pool_snapshot *out) const;

private:
  struct PageBook {
    uint32_t holders = 0;  // counted references of sequences
    uint64_t ticket = 0;   // of the page's live stack entry; 0 = not on a stack
    bool cached = false;   // the prefix cache's one reference
    bool held() const { return holders || cached; }
  };
  struct FreeEntry {
    uint64_t ticket;
    uint32_t page;
  };
  struct ExtentBook {
    std::vector<FreeEntry> stack;  // top = back
    uint32_t free = 0;             // live entries of the stack
    uint32_t held = 0;             // pages with a reference
    uint64_t idle_since = 0;       // 0 = holds pages, or has no memory
    bool resident = false;
  };
  using FillKey = std::pair<uint32_t, uint32_t>;  // (unheld pages, extent)

  uint32_t extent_of(uint32_t page) const { return page / span_; }
  bool live(const FreeEntry &e) const { return page_[e.page].ticket == e.ticket; }
  void stack_push(uint32_t page);
  uint32_t stack_pop(uint32_t extent);
  void stack_forget(uint32_t page);
  // The first `count` free pages of an extent in the order pops would yield them.
  void stack_peek(uint32_t extent, uint32_t count, std::vector<uint32_t> *out) const;
  void refile(uint32_t extent, uint32_t held_before, uint32_t free_before);
  void hold(uint32_t page);    // a page that had no reference gets its first
  void unhold(uint32_t page);  // a page lost its last reference
  int bring_in(uint32_t extent);
  int give_up(uint32_t extent);

  ExtentStorage &storage_;
  int status_ = KVX_OK;
  uint32_t span_ = 0;  // pages per extent
  std::vector<PageBook> page_;
  std::vector<ExtentBook> extent_;
  std::set<FillKey> fill_order_;  // resident extents with a free page, fullest first
  uint64_t next_ticket_ = 0;
  uint64_t idle_clock_ = 0;
  uint32_t free_total_ = 0, active_total_ = 0, cached_total_ = 0, resident_ = 0, idle_ = 0;
  uint64_t allocations_ = 0, releases_ = 0, compactions_ = 0, moved_ = 0;
  double allocate_max_ms_ = 0, release_max_ms_ = 0;
};

}  // namespace kvx
