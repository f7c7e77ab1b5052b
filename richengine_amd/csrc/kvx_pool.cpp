#include "kvx_pool.h"

#include <algorithm>
#include <chrono>
#include <numeric>

namespace kvx {

namespace {
using Clock = std::chrono::steady_clock;
double ms_since(Clock::time_point start) {
  return std::chrono::duration<double, std::milli>(Clock::now() - start).count();
}
}  // namespace

KvPool::KvPool(ExtentStorage &storage, uint32_t runway_pages)
    : storage_(storage), extent_pages_(storage.extent_pages()), pages_(storage.page_count()) {
  if (pages_.empty() || !storage.bytes_per_page() || !extent_pages_ ||
      pages_.size() % extent_pages_ || runway_pages > pages_.size()) {
    status_ = KVX_EINVAL;
    return;
  }
  extents_.resize(pages_.size() / extent_pages_);
  for (uint32_t extent = 0; extent * extent_pages_ < runway_pages; ++extent) {
    if (int rc = allocate_extent(extent)) {
      status_ = rc;
      return;
    }
  }
}

uint64_t KvPool::allocated_bytes() const {
  return uint64_t(allocated_extents_) * extent_pages_ * storage_.bytes_per_page();
}

// A freed page goes to the head of its extent's list, so the page released
// last is handed out first.
void KvPool::list_insert(uint32_t page) {
  Page &p = pages_[page];
  Extent &e = extents_[extent_of(page)];
  p.prev = kNone;
  p.next = e.free_head;
  p.listed = true;
  if (e.free_head != kNone) pages_[e.free_head].prev = page;
  e.free_head = page;
  ++e.free_count;
  ++free_pages_;
  packing_ = kNone;
}

void KvPool::list_remove(uint32_t page) {
  Page &p = pages_[page];
  Extent &e = extents_[extent_of(page)];
  if (p.prev == kNone) e.free_head = p.next;
  else pages_[p.prev].next = p.next;
  if (p.next != kNone) pages_[p.next].prev = p.prev;
  p.prev = p.next = kNone;
  p.listed = false;
  --e.free_count;
  --free_pages_;
}

// The allocated extent with the most held pages that still has a free one;
// ties go to the lowest index and an empty extent loses to any used one.
uint32_t KvPool::packing_extent() {
  if (packing_ != kNone && extents_[packing_].free_count) return packing_;
  uint32_t best = kNone;
  for (uint32_t i = 0; i < extents_.size(); ++i)
    if (extents_[i].free_count && (best == kNone || extents_[i].used > extents_[best].used))
      best = i;
  packing_ = best;
  return best;
}

void KvPool::mark_used(uint32_t page) {
  const uint32_t x = extent_of(page);
  if (pages_[page].listed) {
    list_remove(page);
    if (x != packing_) packing_ = kNone;
  }
  if (!extents_[x].used) set_reclaimable(x, false);
  ++extents_[x].used;
}

void KvPool::mark_free(uint32_t page) {
  const uint32_t x = extent_of(page);
  --extents_[x].used;
  list_insert(page);
  if (!extents_[x].used) set_reclaimable(x, true);
}

void KvPool::set_reclaimable(uint32_t x, bool on) {
  Extent &e = extents_[x];
  if (e.reclaimable == on) return;
  if (on) {  // newest at the head
    e.prev_reclaimable = kNone;
    e.next_reclaimable = reclaimable_head_;
    if (reclaimable_head_ != kNone) extents_[reclaimable_head_].prev_reclaimable = x;
    reclaimable_head_ = x;
    ++reclaimable_count_;
  } else {
    if (e.prev_reclaimable == kNone) reclaimable_head_ = e.next_reclaimable;
    else extents_[e.prev_reclaimable].next_reclaimable = e.next_reclaimable;
    if (e.next_reclaimable != kNone)
      extents_[e.next_reclaimable].prev_reclaimable = e.prev_reclaimable;
    e.prev_reclaimable = e.next_reclaimable = kNone;
    --reclaimable_count_;
  }
  e.reclaimable = on;
}

void KvPool::set_allocated(uint32_t x, bool on) {
  Extent &e = extents_[x];
  const uint32_t first = x * extent_pages_;
  if (on) {
    e.allocated = true;
    ++allocated_extents_;
    // Inserted highest first so the lowest page ends at the head.
    for (uint32_t page = first + extent_pages_; page > first;) list_insert(--page);
    set_reclaimable(x, true);
    return;
  }
  set_reclaimable(x, false);
  for (uint32_t page = first; page < first + extent_pages_; ++page) list_remove(page);
  e.allocated = false;
  --allocated_extents_;
}

int KvPool::allocate_extent(uint32_t x) {
  const auto start = Clock::now();
  if (int rc = storage_.allocate_extent(x)) return rc;
  ++allocations_;
  allocate_max_ms_ = std::max(allocate_max_ms_, ms_since(start));
  set_allocated(x, true);
  return KVX_OK;
}

int KvPool::release_extent(uint32_t x) {
  const auto start = Clock::now();
  if (int rc = storage_.release_extent(x)) return rc;  // a refusal changes nothing
  ++releases_;
  release_max_ms_ = std::max(release_max_ms_, ms_since(start));
  set_allocated(x, false);
  return KVX_OK;
}

int KvPool::acquire(uint32_t count, uint32_t *out) {
  if (!count) return KVX_OK;
  std::vector<uint32_t> selected;
  selected.reserve(count);
  auto give_back = [&] {
    for (auto it = selected.rbegin(); it != selected.rend(); ++it) list_insert(*it);
  };
  while (selected.size() < count) {
    if (free_pages_) {
      const uint32_t page = extents_[packing_extent()].free_head;
      list_remove(page);
      selected.push_back(page);
      continue;
    }
    uint32_t x = kNone;
    for (uint32_t i = 0; i < extents_.size(); ++i)
      if (!extents_[i].allocated) {
        x = i;
        break;
      }
    if (x == kNone) {  // page ids ran out before the budget did
      give_back();
      return KVX_ESTATE;
    }
    if (int rc = allocate_extent(x)) {
      // Extents this call did allocate stay, reclaimable, for the retry.
      give_back();
      return rc;
    }
  }
  for (uint32_t page : selected) {
    mark_used(page);
    pages_[page].active = 1;
    ++active_pages_;
  }
  std::copy(selected.begin(), selected.end(), out);
  return KVX_OK;
}

int KvPool::retain(uint32_t page, bool prefix_owner) {
  if (page >= pages_.size()) return KVX_ERANGE;
  if (!extents_[extent_of(page)].allocated) return KVX_ESTATE;
  Page &p = pages_[page];
  if (prefix_owner && p.prefix) return KVX_ESTATE;
  if (!prefix_owner && p.active == 0xffffffffu) return KVX_ESTATE;
  if (is_free(page)) mark_used(page);
  if (prefix_owner) {
    p.prefix = true;
    ++prefix_pages_;
  } else if (!p.active++) {
    ++active_pages_;
  }
  return KVX_OK;
}

int KvPool::release(uint32_t page, bool prefix_owner) {
  if (page >= pages_.size()) return KVX_ERANGE;
  Page &p = pages_[page];
  if (prefix_owner ? !p.prefix : !p.active) return KVX_ESTATE;
  if (prefix_owner) {
    p.prefix = false;
    --prefix_pages_;
  } else if (!--p.active) {
    --active_pages_;
  }
  if (is_free(page)) mark_free(page);
  return KVX_OK;
}

int KvPool::reclaim_empty(bool keep_runway, uint32_t limit, uint64_t *released) {
  uint32_t reclaimed = 0;
  bool kept = false;
  int rc = KVX_OK;
  for (uint32_t x = reclaimable_head_; x != kNone && reclaimed < limit;) {
    const uint32_t next = extents_[x].next_reclaimable;
    if (keep_runway && !kept) {
      kept = true;
    } else {
      if ((rc = release_extent(x))) break;
      ++reclaimed;
    }
    x = next;
  }
  if (released) *released = uint64_t(reclaimed) * extent_pages_ * storage_.bytes_per_page();
  return rc;
}

int KvPool::compact_extent(const uint32_t *fixed, uint32_t n_fixed, PageMoves *moves) {
  *moves = {};
  // Pages move only into extents that already hold pages.
  uint32_t free_in_use = 0;
  for (const Extent &e : extents_)
    if (e.allocated && e.used) free_in_use += e.free_count;
  uint32_t emptied = kNone;
  for (uint32_t i = 0; i < extents_.size(); ++i) {
    const Extent &e = extents_[i];
    if (!e.allocated || !e.used || e.used > free_in_use - e.free_count) continue;
    if (emptied != kNone && e.used >= extents_[emptied].used) continue;
    bool pinned = false;
    for (uint32_t f = 0; f < n_fixed && !pinned; ++f) pinned = extent_of(fixed[f]) == i;
    if (!pinned) emptied = i;
  }
  if (emptied == kNone) return KVX_OK;

  std::vector<uint32_t> receivers;
  for (uint32_t i = 0; i < extents_.size(); ++i) {
    const Extent &e = extents_[i];
    if (i != emptied && e.allocated && e.used && e.free_count) receivers.push_back(i);
  }
  std::stable_sort(receivers.begin(), receivers.end(), [&](uint32_t a, uint32_t b) {
    return extents_[a].used > extents_[b].used;
  });
  const uint32_t first = emptied * extent_pages_;
  std::vector<kvx_page_copy> copies;
  size_t r = 0;
  uint32_t to = extents_[receivers[r]].free_head;
  for (uint32_t page = first; page < first + extent_pages_; ++page) {
    if (is_free(page)) continue;
    while (to == kNone) to = extents_[receivers[++r]].free_head;
    copies.push_back({page, to});
    to = pages_[to].next;
  }
  if (int rc = storage_.copy_pages(copies.data(), uint32_t(copies.size()))) return rc;

  moves->first_page = first;
  moves->destinations.resize(extent_pages_);
  std::iota(moves->destinations.begin(), moves->destinations.end(), first);
  for (const kvx_page_copy &c : copies) {
    mark_used(c.to);
    pages_[c.to].active = pages_[c.from].active;
    pages_[c.from].active = 0;
    pages_[c.to].prefix = pages_[c.from].prefix;
    pages_[c.from].prefix = false;
    mark_free(c.from);
    moves->destinations[c.from - first] = c.to;
  }
  moves->moved = uint32_t(copies.size());
  ++compactions_;
  moved_ += copies.size();
  return KVX_OK;
}

void KvPool::snapshot(kvx_pool_snapshot *out) const {
  out->pages_allocated = allocated_extents_ * extent_pages_;
  out->pages_free = free_pages_;
  out->pages_active = active_pages_;
  out->pages_prefix = prefix_pages_;
  out->allocated_bytes = allocated_bytes();
  out->reclaimable_bytes = uint64_t(reclaimable_count_) * extent_pages_ * storage_.bytes_per_page();
  out->extent_allocations = allocations_;
  out->extent_releases = releases_;
  out->extent_allocate_max_ms = allocate_max_ms_;
  out->extent_release_max_ms = release_max_ms_;
  out->extent_compactions = compactions_;
  out->pages_moved = moved_;
}

}  // namespace kvx
