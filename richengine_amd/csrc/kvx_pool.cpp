// The page pool; the header describes its bookkeeping.
#include "kvx_pool.h"

#include <algorithm>
#include <chrono>

namespace kvx {

namespace {
double elapsed_ms(std::chrono::steady_clock::time_point since) {
  return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - since).count();
}
}  // namespace

KvPool::KvPool(ExtentStorage &storage, uint32_t runway_pages)
    : storage_(storage), span_(storage.extent_pages()) {
  const uint32_t pages = storage.page_count();
  if (!pages || !span_ || pages % span_ || !storage.bytes_per_page() || runway_pages > pages) {
    status_ = KVX_EINVAL;
    return;
  }
  page_.resize(pages);
  extent_.resize(pages / span_);
  const uint32_t runway_extents = (runway_pages + span_ - 1) / span_;
  for (uint32_t x = 0; x < runway_extents && status_ == KVX_OK; ++x) status_ = bring_in(x);
}

uint64_t KvPool::allocated_bytes() const {
  return uint64_t(resident_) * span_ * storage_.bytes_per_page();
}

// ---- free stacks ---------------------------------------------------------------

void KvPool::stack_push(uint32_t page) {
  ExtentBook &x = extent_[extent_of(page)];
  page_[page].ticket = ++next_ticket_;  // never 0, which means "not on a stack"
  x.stack.push_back({next_ticket_, page});
  ++x.free;
  ++free_total_;
  if (x.stack.size() > 2u * span_) {  // squeeze the stale entries out, order kept
    size_t kept = 0;
    for (const FreeEntry &e : x.stack)
      if (live(e)) x.stack[kept++] = e;
    x.stack.resize(kept);
  }
}

uint32_t KvPool::stack_pop(uint32_t extent) {
  ExtentBook &x = extent_[extent];
  while (!live(x.stack.back())) x.stack.pop_back();
  const uint32_t page = x.stack.back().page;
  x.stack.pop_back();
  page_[page].ticket = 0;
  --x.free;
  --free_total_;
  return page;
}

void KvPool::stack_forget(uint32_t page) {
  page_[page].ticket = 0;
  --extent_[extent_of(page)].free;
  --free_total_;
}

void KvPool::stack_peek(uint32_t extent, uint32_t count, std::vector<uint32_t> *out) const {
  const ExtentBook &x = extent_[extent];
  for (size_t i = x.stack.size(); i > 0 && count; --i)
    if (live(x.stack[i - 1])) {
      out->push_back(x.stack[i - 1].page);
      --count;
    }
}

// ---- the fill order -------------------------------------------------------------

// Moves an extent to its place in the fill order after `held` or `free` changed;
// the arguments are what they were when it was last filed.
void KvPool::refile(uint32_t extent, uint32_t held_before, uint32_t free_before) {
  const ExtentBook &x = extent_[extent];
  if (free_before) fill_order_.erase(FillKey(span_ - held_before, extent));
  if (x.resident && x.free) fill_order_.insert(FillKey(span_ - x.held, extent));
}

void KvPool::hold(uint32_t page) {
  const uint32_t e = extent_of(page);
  ExtentBook &x = extent_[e];
  const uint32_t held = x.held, free = x.free;
  if (page_[page].ticket) stack_forget(page);
  if (!x.held++) {
    x.idle_since = 0;
    --idle_;
  }
  refile(e, held, free);
}

void KvPool::unhold(uint32_t page) {
  const uint32_t e = extent_of(page);
  ExtentBook &x = extent_[e];
  const uint32_t held = x.held, free = x.free;
  stack_push(page);
  if (!--x.held) {
    x.idle_since = ++idle_clock_;
    ++idle_;
  }
  refile(e, held, free);
}

// ---- extents --------------------------------------------------------------------

int KvPool::bring_in(uint32_t extent) {
  const auto start = std::chrono::steady_clock::now();
  if (const int rc = storage_.allocate_extent(extent)) return rc;
  allocate_max_ms_ = std::max(allocate_max_ms_, elapsed_ms(start));
  ++allocations_;
  ExtentBook &x = extent_[extent];
  x.resident = true;
  ++resident_;
  x.idle_since = ++idle_clock_;
  ++idle_;
  // Highest page first, so that the lowest ends on top.
  for (uint32_t i = span_; i > 0; --i) stack_push(extent * span_ + i - 1);
  refile(extent, 0, 0);
  return KVX_OK;
}

int KvPool::give_up(uint32_t extent) {
  const auto start = std::chrono::steady_clock::now();
  if (const int rc = storage_.release_extent(extent)) return rc;  // a refusal changes nothing
  release_max_ms_ = std::max(release_max_ms_, elapsed_ms(start));
  ++releases_;
  ExtentBook &x = extent_[extent];
  const uint32_t free = x.free;
  for (uint32_t i = 0; i < span_; ++i) page_[extent * span_ + i].ticket = 0;
  free_total_ -= x.free;
  x.free = 0;
  x.stack.clear();
  x.resident = false;
  --resident_;
  x.idle_since = 0;
  --idle_;
  refile(extent, 0, free);
  return KVX_OK;
}

// ---- references -------------------------------------------------------------------

int KvPool::acquire(uint32_t count, uint32_t *out) {
  // Pages are only taken off their stacks here and get their reference once all
  // of them are found: a refused growth puts them back in reverse, which leaves
  // every stack, the fill order and the idle order as they were.
  std::vector<uint32_t> taken;
  taken.reserve(count);
  int rc = KVX_OK;
  while (taken.size() < count) {
    if (!fill_order_.empty()) {
      const uint32_t e = fill_order_.begin()->second;
      const uint32_t held = extent_[e].held, free = extent_[e].free;
      taken.push_back(stack_pop(e));
      refile(e, held, free);
      continue;
    }
    uint32_t absent = 0;
    while (absent < extent_.size() && extent_[absent].resident) ++absent;
    rc = absent == extent_.size() ? KVX_ESTATE  // page ids ran out before the budget did
                                  : bring_in(absent);
    if (rc) break;
  }
  if (rc) {
    // Extents this call did bring in stay, idle, for the retry.
    for (size_t i = taken.size(); i > 0; --i) {
      const uint32_t e = extent_of(taken[i - 1]);
      const uint32_t held = extent_[e].held, free = extent_[e].free;
      stack_push(taken[i - 1]);
      refile(e, held, free);
    }
    return rc;
  }
  for (uint32_t i = 0; i < count; ++i) {
    hold(taken[i]);
    page_[taken[i]].holders = 1;
    out[i] = taken[i];
  }
  active_total_ += count;
  return KVX_OK;
}

int KvPool::retain(uint32_t page, bool prefix_owner) {
  if (page >= page_.size()) return KVX_ERANGE;
  if (!extent_[extent_of(page)].resident) return KVX_ESTATE;
  PageBook &p = page_[page];
  if (prefix_owner ? p.cached : p.holders == UINT32_MAX) return KVX_ESTATE;
  if (!p.held()) hold(page);
  if (prefix_owner) {
    p.cached = true;
    ++cached_total_;
  } else if (!p.holders++) {
    ++active_total_;
  }
  return KVX_OK;
}

int KvPool::release(uint32_t page, bool prefix_owner) {
  if (page >= page_.size()) return KVX_ERANGE;
  PageBook &p = page_[page];
  if (prefix_owner ? !p.cached : !p.holders) return KVX_ESTATE;
  if (prefix_owner) {
    p.cached = false;
    --cached_total_;
  } else if (!--p.holders) {
    --active_total_;
  }
  if (!p.held()) unhold(page);
  return KVX_OK;
}

// ---- giving memory back -----------------------------------------------------------

int KvPool::reclaim_empty(bool keep_runway, uint32_t limit, uint64_t *released) {
  std::vector<std::pair<uint64_t, uint32_t>> idle;  // (idle since, extent)
  for (uint32_t e = 0; e < extent_.size(); ++e)
    if (extent_[e].resident && !extent_[e].held) idle.emplace_back(extent_[e].idle_since, e);
  std::sort(idle.begin(), idle.end(), std::greater<>());  // latest first
  uint32_t given = 0;
  int rc = KVX_OK;
  // The extent that fell idle last stays as the runway when asked to.
  for (size_t i = keep_runway ? 1 : 0; i < idle.size() && given < limit; ++i) {
    if ((rc = give_up(idle[i].second))) break;
    ++given;
  }
  if (released) *released = uint64_t(given) * span_ * storage_.bytes_per_page();
  return rc;
}

int KvPool::compact_extent(const uint32_t *fixed, uint32_t n_fixed, PageMoves *moves) {
  *moves = {};
  // Pages only move into extents that hold pages already, so what counts is the
  // free room of those.
  uint32_t room = 0;
  for (const ExtentBook &x : extent_)
    if (x.resident && x.held) room += x.free;
  std::vector<bool> pinned(extent_.size(), false);
  for (uint32_t i = 0; i < n_fixed; ++i)
    if (fixed[i] < page_.size()) pinned[extent_of(fixed[i])] = true;
  // The extent to empty: the one with the fewest held pages that the others can
  // take in, the lowest index among equals.
  uint32_t victim = UINT32_MAX;
  for (uint32_t e = 0; e < extent_.size(); ++e) {
    const ExtentBook &x = extent_[e];
    if (!x.resident || !x.held || pinned[e] || x.held > room - x.free) continue;
    if (victim == UINT32_MAX || x.held < extent_[victim].held) victim = e;
  }
  if (victim == UINT32_MAX) return KVX_OK;

  // Receivers fullest first (lowest index among equals); each gives its free
  // pages in the order an acquisition would.
  std::vector<std::pair<uint32_t, uint32_t>> receivers;  // (unheld pages, extent)
  for (uint32_t e = 0; e < extent_.size(); ++e) {
    const ExtentBook &x = extent_[e];
    if (e != victim && x.resident && x.held && x.free) receivers.emplace_back(span_ - x.held, e);
  }
  std::sort(receivers.begin(), receivers.end());
  std::vector<uint32_t> landing;
  uint32_t wanted = extent_[victim].held;
  for (size_t r = 0; r < receivers.size() && wanted; ++r) {
    const uint32_t take = std::min(wanted, extent_[receivers[r].second].free);
    stack_peek(receivers[r].second, take, &landing);
    wanted -= take;
  }
  // One sweep over the victim, lowest page first, pairs every held page with the
  // next landing place.
  std::vector<kvx_page_copy> copies;
  copies.reserve(landing.size());
  const uint32_t first = victim * span_;
  for (uint32_t page = first; page < first + span_; ++page)
    if (page_[page].held()) copies.push_back({page, landing[copies.size()]});
  if (const int rc = storage_.copy_pages(copies.data(), uint32_t(copies.size()))) return rc;

  moves->first_page = first;
  moves->destinations.resize(span_);
  for (uint32_t i = 0; i < span_; ++i) moves->destinations[i] = first + i;
  for (const kvx_page_copy &c : copies) {
    hold(c.to);
    page_[c.to].holders = page_[c.from].holders;
    page_[c.to].cached = page_[c.from].cached;
    page_[c.from].holders = 0;
    page_[c.from].cached = false;
    unhold(c.from);
    moves->destinations[c.from - first] = c.to;
  }
  moves->moved = uint32_t(copies.size());
  moved_ += copies.size();
  ++compactions_;
  return KVX_OK;
}

void KvPool::snapshot(kvx_pool_snapshot *out) const {
  const uint64_t extent_bytes = uint64_t(span_) * storage_.bytes_per_page();
  out->pages_allocated = resident_ * span_;
  out->pages_free = free_total_;
  out->pages_active = active_total_;
  out->pages_prefix = cached_total_;
  out->allocated_bytes = resident_ * extent_bytes;
  out->reclaimable_bytes = idle_ * extent_bytes;
  out->extent_allocations = allocations_;
  out->extent_releases = releases_;
  out->extent_allocate_max_ms = allocate_max_ms_;
  out->extent_release_max_ms = release_max_ms_;
  out->extent_compactions = compactions_;
  out->pages_moved = moved_;
}

}  // namespace kvx
