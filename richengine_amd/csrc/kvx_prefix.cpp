// Prefix page cache and per-sequence page lists; see kvx_prefix.h.
#include "kvx_prefix.h"

#include <algorithm>

namespace kvx {

// A 64-bit FNV-1a over the key's words.  The hash only spreads keys over the
// map's buckets; equality is the map's comparison of whole keys.
size_t PrefixCache::ContentKeyHash::operator()(const ContentKey &key) const {
  uint64_t h = 0xcbf29ce484222325ull;
  auto fold = [&h](uint64_t word) {
    h ^= word;
    h *= 0x100000001b3ull;
  };
  fold(key.parent);
  for (uint32_t i = 0; i < KVX_PAGE_TOKENS; i += 2)
    fold(uint64_t(key.tokens[i]) | uint64_t(key.tokens[i + 1]) << 32);
  fold(key.image_lo);
  fold(key.image_hi);
  return size_t(h ^ (h >> 29));
}

PrefixCache::ContentKey PrefixCache::key_of(uint64_t parent, const uint32_t *tokens,
                                            uint64_t image_lo, uint64_t image_hi) {
  ContentKey key;
  key.parent = parent;
  key.image_lo = image_lo;
  key.image_hi = image_hi;
  std::copy(tokens, tokens + KVX_PAGE_TOKENS, key.tokens.begin());
  return key;
}

PrefixCache::~PrefixCache() {
  for (const auto &entry : blocks_)
    if (entry.second.page != kNoPage) pool_.release(entry.second.page, true);
}

const PrefixCache::Block *PrefixCache::get(uint64_t id) const {
  const auto found = blocks_.find(id);
  return found == blocks_.end() ? nullptr : &found->second;
}
PrefixCache::Block *PrefixCache::get(uint64_t id) {
  const auto found = blocks_.find(id);
  return found == blocks_.end() ? nullptr : &found->second;
}

// KvCache::reindex (KvCache.cpp:577-592), resident tier only: a block nobody
// uses and without children waits in the eviction order.
void PrefixCache::reindex(Block &b) {
  if (b.listed) {
    leaves_.erase(std::make_pair(b.listed_at, b.id));
    b.listed = false;
  }
  if (b.active_users || b.children) return;
  leaves_.emplace(std::make_pair(b.last_used, b.id), b.id);
  b.listed = true;
  b.listed_at = b.last_used;
}

// A block id is never reused, so a key under a parent that no longer exists
// cannot be in the map: an unknown parent simply finds nothing.
bool PrefixCache::find(uint64_t parent, const uint32_t *tokens, uint32_t n_tokens, uint64_t image_lo,
                       uint64_t image_hi, uint64_t *block, uint32_t *page) const {
  if (n_tokens != KVX_PAGE_TOKENS) return false;
  const auto hit = by_content_.find(key_of(parent, tokens, image_lo, image_hi));
  if (hit == by_content_.end()) return false;
  if (block) *block = hit->second;
  if (page) *page = get(hit->second)->page;
  return true;
}

int PrefixCache::insert(uint64_t parent, const uint32_t *tokens, uint32_t n_tokens, uint32_t page,
                        uint64_t image_lo, uint64_t image_hi, uint64_t *block,
                        uint32_t *canonical_page) {
  if (n_tokens != KVX_PAGE_TOKENS) return KVX_EINVAL;  // one full page
  if (page >= pool_.page_count()) return KVX_ERANGE;
  // One probe either finds the content or reserves its place.
  const auto placed = by_content_.try_emplace(key_of(parent, tokens, image_lo, image_hi), 0);
  if (!placed.second) {  // cached already: the caller gets the canonical block and page
    if (block) *block = placed.first->second;
    if (canonical_page) *canonical_page = get(placed.first->second)->page;
    return KVX_OK;
  }
  Block *above = parent ? get(parent) : nullptr;
  int rc = KVX_OK;
  if (parent && !above) rc = KVX_EINVAL;           // unknown parent
  else if (block_on_page_[page]) rc = KVX_ESTATE;  // the page already holds a block
  else rc = pool_.retain(page, true);
  if (rc) {
    by_content_.erase(placed.first);
    return rc;
  }
  const uint64_t id = next_id_++;
  placed.first->second = id;
  Block &fresh = blocks_[id];
  fresh.id = id;
  fresh.key = placed.first->first;
  fresh.page = page;
  fresh.depth = above ? above->depth + 1 : 1;
  fresh.last_used = ++clock_;
  block_on_page_[page] = id;
  if (above) {  // no longer a leaf
    ++above->children;
    reindex(*above);
  }
  reindex(fresh);
  ++generation_;
  if (block) *block = id;
  if (canonical_page) *canonical_page = page;
  return KVX_OK;
}

int PrefixCache::chain_length(uint64_t block, uint32_t *length) const {
  const Block *b = get(block);
  if (!b) return KVX_ERANGE;
  *length = b->depth;
  return KVX_OK;
}

int PrefixCache::chain(uint64_t block, std::vector<uint64_t> *blocks,
                       std::vector<uint32_t> *pages) const {
  const Block *b = get(block);
  if (!b) return KVX_ERANGE;
  blocks->assign(b->depth, 0);
  pages->assign(b->depth, kNoPage);
  for (uint32_t index = b->depth; index > 0; --index) {
    if (!b) return KVX_ESTATE;
    (*blocks)[index - 1] = b->id;
    (*pages)[index - 1] = b->page;
    b = b->key.parent ? get(b->key.parent) : nullptr;
  }
  return b ? KVX_ESTATE : KVX_OK;
}

int PrefixCache::page_of(uint64_t block, uint32_t *page) const {
  const Block *b = get(block);
  if (!b) return KVX_ERANGE;
  *page = b->page;
  return KVX_OK;
}

int PrefixCache::retain_active(uint64_t block) {
  Block *b = get(block);
  if (!b) return KVX_ERANGE;
  ++b->active_users;
  b->last_used = ++clock_;
  reindex(*b);
  return KVX_OK;
}

int PrefixCache::release_active(uint64_t block) {
  Block *b = get(block);
  if (!b) return KVX_ERANGE;
  if (!b->active_users) return KVX_ESTATE;
  --b->active_users;
  // A released leaf is the newest; a parent keeps the recency its children
  // pass on (KvCache.cpp:237-249).
  if (!b->active_users && !b->children) b->last_used = ++clock_;
  reindex(*b);
  return KVX_OK;
}

int PrefixCache::touch(uint64_t block) {
  Block *b = get(block);
  if (!b) return KVX_ERANGE;
  b->last_used = ++clock_;
  reindex(*b);
  return KVX_OK;
}

int PrefixCache::eviction_candidate(uint64_t after, uint64_t *block, bool *found) const {
  *found = false;
  auto position = leaves_.begin();
  if (after) {
    const Block *b = get(after);
    if (!b) return KVX_ERANGE;
    position = leaves_.upper_bound(std::make_pair(b->last_used, b->id));
  }
  if (position == leaves_.end()) return KVX_OK;
  *block = position->second;
  *found = true;
  return KVX_OK;
}

int PrefixCache::erase(uint64_t block) {
  Block *b = get(block);
  if (!b) return KVX_ERANGE;
  if (b->children || b->active_users) return KVX_ESTATE;  // a referenced block stays
  const uint64_t parent = b->key.parent, last_used = b->last_used;
  const uint32_t page = b->page;
  if (b->listed) leaves_.erase(std::make_pair(b->listed_at, b->id));
  by_content_.erase(b->key);
  blocks_.erase(block);
  ++generation_;
  block_on_page_[page] = 0;
  if (parent) {
    Block &p = *get(parent);
    --p.children;
    // KvCache::inherit (KvCache.cpp:441-446): an exposed parent is at least as
    // recent as the leaf it lost.
    if (!p.children && !p.active_users) p.last_used = std::max(p.last_used, last_used);
    reindex(p);
  }
  return pool_.release(page, true);
}

void PrefixCache::follow_pages(const PageMoves &moves) {
  for (uint32_t offset = 0; offset < moves.destinations.size(); ++offset) {
    const uint32_t from = moves.first_page + offset, to = moves.destinations[offset];
    if (to == from) continue;
    const uint64_t id = block_on_page_[from];
    block_on_page_[from] = 0;
    if (!id) continue;
    get(id)->page = to;
    block_on_page_[to] = id;
  }
}

// The identity is a value that travels with a block's key (and would be persisted
// with it), so its bits are the reference's: two chains with their own seeds fold,
// for every span that overlaps the block, the span's content digest, its grid, its
// place in the prompt and the block's start.  `a ^= v + golden + (a << 6) + (a >> 2)`
// is the fold of both chains; the second takes the complement of every value.
void block_image_identity(uint64_t block_begin, uint32_t block_tokens, const kvx_image_span *spans,
                          uint32_t n_spans, uint64_t *lo, uint64_t *hi) {
  const auto fold = [](uint64_t a, uint64_t v) {
    return a ^ (v + 0x9e3779b97f4a7c15ull + (a << 6) + (a >> 2));
  };
  uint64_t chain_lo = 0, chain_hi = 0;
  const uint64_t block_end = block_begin + block_tokens;
  for (uint32_t i = 0; i < n_spans; ++i) {
    const kvx_image_span &span = spans[i];
    if (span.offset >= block_end) break;  // spans are sorted by offset
    if (uint32_t(span.offset + span.tokens) <= block_begin) continue;  // 32-bit end, as ImageSpan::end()
    const uint64_t words[5] = {span.digest_lo, span.digest_hi,
                               uint64_t(span.grid_height) << 32 | span.grid_width,
                               uint64_t(span.offset) << 32 | span.tokens, block_begin};
    if (!chain_lo) chain_lo = 0x243f6a8885a308d3ull;
    if (!chain_hi) chain_hi = 0x13198a2e03707344ull;
    for (const uint64_t word : words) {
      chain_lo = fold(chain_lo, word);
      chain_hi = fold(chain_hi, ~word);
    }
  }
  *lo = chain_lo;
  *hi = chain_hi;
}

namespace {
// The spans that can still overlap the block at `block_begin` or a later one (Cache.cpp:16-22):
// sorted and disjoint, a span that ends before a block ends before every later block too.
void spans_from(const kvx_image_span *&spans, uint32_t &n_spans, uint64_t block_begin) {
  while (n_spans && uint32_t(spans->offset + spans->tokens) <= block_begin) {
    ++spans;
    --n_spans;
  }
}
}  // namespace

uint64_t PrefixCache::extend_match(std::vector<uint64_t> *blocks, const uint32_t *prompt, uint64_t n,
                                   const kvx_image_span *spans, uint32_t n_spans) const {
  if (!n) return 0;
  // Leave one real input token to compute the first logits from.
  const uint64_t maximum = (n - 1) / KVX_PAGE_TOKENS;
  uint64_t hashed = 0;
  for (uint64_t index = blocks->size(); index < maximum; ++index) {
    const uint64_t begin = index * KVX_PAGE_TOKENS;
    const uint64_t parent = blocks->empty() ? 0 : blocks->back();
    spans_from(spans, n_spans, begin);
    uint64_t image_lo = 0, image_hi = 0;
    block_image_identity(begin, KVX_PAGE_TOKENS, spans, n_spans, &image_lo, &image_hi);
    ++hashed;
    uint64_t id = 0;
    if (!find(parent, prompt + begin, KVX_PAGE_TOKENS, image_lo, image_hi, &id, nullptr)) break;
    blocks->push_back(id);
  }
  return hashed;
}

// ---- sequences ----------------------------------------------------------------

SequenceCache::~SequenceCache() {
  std::vector<uint64_t> ids;
  for (const auto &entry : sequences_) ids.push_back(entry.first);
  for (uint64_t id : ids) end(id);
}

int SequenceCache::begin(uint64_t id) {
  if (!id || sequences_.count(id)) return KVX_EINVAL;
  sequences_.emplace(id, Sequence{});
  return KVX_OK;
}

int SequenceCache::end(uint64_t id) {
  const auto found = sequences_.find(id);
  if (found == sequences_.end()) return KVX_OK;
  for (uint32_t page : found->second.pages) pool_.release(page, false);
  if (!found->second.blocks.empty()) prefix_.release_active(found->second.blocks.back());
  sequences_.erase(found);
  return KVX_OK;
}

int SequenceCache::restore(uint64_t id, uint64_t last_block) {
  const auto found = sequences_.find(id);
  if (found == sequences_.end()) return KVX_ERANGE;
  Sequence &s = found->second;
  if (!s.pages.empty() || !s.blocks.empty()) return KVX_ESTATE;  // already owns pages
  std::vector<uint64_t> blocks;
  std::vector<uint32_t> pages;
  if (const int rc = prefix_.chain(last_block, &blocks, &pages)) return rc;
  prefix_.retain_active(blocks.back());
  for (uint32_t page : pages) pool_.retain(page, false);
  s.pages = std::move(pages);
  s.blocks = std::move(blocks);
  changed(s, 0);
  return KVX_OK;
}

int SequenceCache::ensure_tokens(uint64_t id, uint64_t tokens) {
  const auto found = sequences_.find(id);
  if (found == sequences_.end()) return KVX_ERANGE;
  Sequence &s = found->second;
  const uint64_t needed = (tokens + KVX_PAGE_TOKENS - 1) / KVX_PAGE_TOKENS;
  if (needed > 0xffffffffull) return KVX_EINVAL;
  const uint32_t previous = uint32_t(s.pages.size());
  if (needed <= previous) return KVX_OK;
  std::vector<uint32_t> acquired(needed - previous);
  if (const int rc = pool_.acquire(uint32_t(acquired.size()), acquired.data())) return rc;
  s.pages.insert(s.pages.end(), acquired.begin(), acquired.end());
  changed(s, previous);
  return KVX_OK;
}

int SequenceCache::fork(uint64_t id, uint64_t source, uint64_t tokens) {
  const auto found = sequences_.find(id), origin = sequences_.find(source);
  if (found == sequences_.end() || origin == sequences_.end()) return KVX_ERANGE;
  Sequence &s = found->second;
  const Sequence &from = origin->second;
  if (id == source || !s.pages.empty() || !s.blocks.empty()) return KVX_ESTATE;
  const uint64_t pages = (tokens + KVX_PAGE_TOKENS - 1) / KVX_PAGE_TOKENS;
  if (pages > from.pages.size()) return KVX_EINVAL;  // more than the source holds
  if (!pages) return KVX_OK;
  for (uint64_t i = 0; i < pages; ++i)
    if (const int rc = pool_.retain(from.pages[i], false)) {
      while (i > 0) pool_.release(from.pages[--i], false);
      return rc;
    }
  s.pages.assign(from.pages.begin(), from.pages.begin() + pages);
  // Blocks exist for published whole pages only.
  const uint64_t blocks = std::min<uint64_t>(tokens / KVX_PAGE_TOKENS, from.blocks.size());
  s.blocks.assign(from.blocks.begin(), from.blocks.begin() + blocks);
  if (blocks) prefix_.retain_active(s.blocks.back());
  changed(s, 0);
  return KVX_OK;
}

// The counterpart of ensure_tokens after a speculative rollback: the reference keeps
// "the pages of tokens + scratch" by never asking for more (Engine.cpp:1190-1193) and lets
// rejected rows lie where they are (abi/PagedAttention.h:33-38); a tree of 16 draft rows can
// leave a whole page without a committed token, which goes back to the pool here.
int SequenceCache::truncate(uint64_t id, uint64_t tokens, uint32_t *released) {
  *released = 0;
  const auto found = sequences_.find(id);
  if (found == sequences_.end()) return KVX_ERANGE;
  Sequence &s = found->second;
  const uint64_t keep = (tokens + KVX_PAGE_TOKENS - 1) / KVX_PAGE_TOKENS;
  if (keep < s.blocks.size()) return KVX_ESTATE;  // a published page is history, not scratch
  if (keep >= s.pages.size()) return KVX_OK;
  for (size_t index = size_t(keep); index < s.pages.size(); ++index) pool_.release(s.pages[index], false);
  *released = uint32_t(s.pages.size() - keep);
  s.pages.resize(size_t(keep));
  changed(s, uint32_t(keep));
  return KVX_OK;
}

int SequenceCache::ensure_writable(uint64_t id, uint64_t token, bool *copied, uint32_t *from,
                                   uint32_t *to) {
  *copied = false;
  const auto found = sequences_.find(id);
  if (found == sequences_.end()) return KVX_ERANGE;
  Sequence &s = found->second;
  const uint64_t logical = token / KVX_PAGE_TOKENS;
  if (logical >= s.pages.size()) return KVX_EINVAL;  // ensure_tokens comes first
  // A published page never changes again: rows stored at or after `token` lie past it.
  if (logical < s.blocks.size()) return KVX_ESTATE;
  const uint32_t shared = s.pages[logical];
  if (!pool_.page_shared(shared)) return KVX_OK;
  uint32_t mine = 0;
  if (pool_.acquire(1, &mine)) return KVX_ENOMEM;  // refused growth, or no page id left
  const kvx_page_copy copy{shared, mine};
  if (const int rc = pool_.copy_pages(&copy, 1)) {
    pool_.release(mine, false);
    return rc;
  }
  s.pages[logical] = mine;
  changed(s, uint32_t(logical));
  pool_.release(shared, false);
  *copied = true;
  *from = shared;
  *to = mine;
  return KVX_OK;
}

// Cache::publishCommittedBlocks (Cache.cpp:294-333): every newly full page
// becomes a block; where the content is already cached the sequence moves to
// the canonical page and gives its own back.
int SequenceCache::publish(uint64_t id, const uint32_t *tokens, uint64_t n_tokens,
                           uint32_t committed, const kvx_image_span *spans, uint32_t n_spans) {
  const auto found = sequences_.find(id);
  if (found == sequences_.end()) return KVX_ERANGE;
  Sequence &s = found->second;
  if (committed > n_tokens) return KVX_EINVAL;
  const uint32_t full = committed / KVX_PAGE_TOKENS;
  const uint64_t required = (uint64_t(committed) + KVX_PAGE_TOKENS - 1) / KVX_PAGE_TOKENS;
  if (required > s.pages.size()) return KVX_ESTATE;  // committed KV without a page
  if (full < s.blocks.size()) return KVX_ESTATE;     // history moved backwards
  while (s.blocks.size() < full) {
    const uint32_t logical = uint32_t(s.blocks.size());
    const uint64_t parent = logical ? s.blocks.back() : 0;
    uint64_t block = 0;
    uint32_t canonical = 0;
    const uint32_t writer = s.pages[logical];
    const uint64_t begin = uint64_t(logical) * KVX_PAGE_TOKENS;
    spans_from(spans, n_spans, begin);
    uint64_t image_lo = 0, image_hi = 0;
    block_image_identity(begin, KVX_PAGE_TOKENS, spans, n_spans, &image_lo, &image_hi);
    if (const int rc = prefix_.insert(parent, tokens + begin, KVX_PAGE_TOKENS, writer, image_lo,
                                      image_hi, &block, &canonical))
      return rc;
    const bool replace = canonical != writer;
    if (replace) pool_.retain(canonical, false);
    prefix_.retain_active(block);
    s.blocks.push_back(block);
    if (replace) {
      s.pages[logical] = canonical;
      changed(s, logical);
      pool_.release(writer, false);
    }
    if (parent) prefix_.release_active(parent);
  }
  return KVX_OK;
}

int SequenceCache::view(uint64_t id, View *out) const {
  const auto found = sequences_.find(id);
  if (found == sequences_.end()) return KVX_ERANGE;
  const Sequence &s = found->second;
  *out = {s.pages.data(), uint32_t(s.pages.size()), s.revision, s.first_changed, s.blocks.data(),
          uint32_t(s.blocks.size())};
  return KVX_OK;
}

int SequenceCache::compact_extent(PageMoves *moves) {
  if (const int rc = pool_.compact_extent(nullptr, 0, moves)) return rc;
  if (moves->empty()) return KVX_OK;
  prefix_.follow_pages(*moves);
  for (auto &entry : sequences_) {
    Sequence &s = entry.second;
    size_t first = s.pages.size();
    for (size_t index = 0; index < s.pages.size(); ++index) {
      const uint32_t destination = moves->follow(s.pages[index]);
      if (destination == s.pages[index]) continue;
      s.pages[index] = destination;
      first = std::min(first, index);
    }
    if (first < s.pages.size()) changed(s, uint32_t(first));
  }
  return KVX_OK;
}

}  // namespace kvx
