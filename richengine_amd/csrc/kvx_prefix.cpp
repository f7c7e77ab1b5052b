// Prefix page cache and per-sequence page lists; see kvx_prefix.h.
#include "kvx_prefix.h"

#include <algorithm>

namespace kvx {
namespace {

// runtime/engine/cache/KvCache.cpp:12-25
uint64_t mix(uint64_t hash, uint64_t value) {
  hash ^= value + 0x9e3779b97f4a7c15ULL + (hash << 6) + (hash >> 2);
  return hash;
}
uint64_t index_hash(uint64_t parent_hash, const uint32_t *tokens, uint64_t lo, uint64_t hi) {
  uint64_t hash = mix(0x6a09e667f3bcc909ULL, parent_hash);
  for (uint32_t i = 0; i < KVX_PAGE_TOKENS; ++i) hash = mix(hash, tokens[i]);
  hash = mix(hash, lo);
  return mix(hash, hi);
}

}  // namespace

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

bool PrefixCache::find(uint64_t parent, const uint32_t *tokens, uint32_t n_tokens, uint64_t image_lo,
                       uint64_t image_hi, uint64_t *block, uint32_t *page) const {
  if (n_tokens != KVX_PAGE_TOKENS) return false;
  const Block *above = parent ? get(parent) : nullptr;
  if (parent && !above) return false;
  const uint64_t hash = index_hash(above ? above->index_hash : 0, tokens, image_lo, image_hi);
  const auto range = index_.equal_range(hash);
  for (auto candidate = range.first; candidate != range.second; ++candidate) {
    const Block &entry = *get(candidate->second);
    // Hashes filter candidates; equality needs the complete key.
    if (entry.parent == parent && entry.image_lo == image_lo && entry.image_hi == image_hi &&
        std::equal(entry.tokens.begin(), entry.tokens.end(), tokens)) {
      if (block) *block = entry.id;
      if (page) *page = entry.page;
      return true;
    }
  }
  return false;
}

int PrefixCache::insert(uint64_t parent, const uint32_t *tokens, uint32_t n_tokens, uint32_t page,
                        uint64_t image_lo, uint64_t image_hi, uint64_t *block,
                        uint32_t *canonical_page) {
  if (n_tokens != KVX_PAGE_TOKENS) return KVX_EINVAL;  // one full page
  if (page >= pool_.page_count()) return KVX_ERANGE;
  uint64_t existing = 0;
  uint32_t existing_page = kNoPage;
  if (find(parent, tokens, n_tokens, image_lo, image_hi, &existing, &existing_page)) {
    if (block) *block = existing;
    if (canonical_page) *canonical_page = existing_page;
    return KVX_OK;
  }
  Block *above = parent ? get(parent) : nullptr;
  if (parent && !above) return KVX_EINVAL;  // unknown parent
  if (block_on_page_[page]) return KVX_ESTATE;  // the page already holds a block
  if (const int rc = pool_.retain(page, true)) return rc;
  Block entry;
  entry.id = next_id_++;
  entry.parent = parent;
  entry.index_hash = index_hash(above ? above->index_hash : 0, tokens, image_lo, image_hi);
  std::copy(tokens, tokens + KVX_PAGE_TOKENS, entry.tokens.begin());
  entry.image_lo = image_lo;
  entry.image_hi = image_hi;
  entry.page = page;
  entry.depth = above ? above->depth + 1 : 1;
  const uint64_t id = entry.id;
  index_.emplace(entry.index_hash, id);
  blocks_.emplace(id, entry);
  block_on_page_[page] = id;
  if (parent) {
    Block &p = *get(parent);
    ++p.children;
    reindex(p);
  }
  Block &placed = *get(id);
  placed.last_used = ++clock_;
  reindex(placed);
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
    b = b->parent ? get(b->parent) : nullptr;
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
  const uint64_t parent = b->parent, hash = b->index_hash, last_used = b->last_used;
  const uint32_t page = b->page;
  if (b->listed) leaves_.erase(std::make_pair(b->listed_at, b->id));
  const auto range = index_.equal_range(hash);
  for (auto it = range.first; it != range.second; ++it)
    if (it->second == block) {
      index_.erase(it);
      break;
    }
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

uint64_t PrefixCache::extend_match(std::vector<uint64_t> *blocks, const uint32_t *prompt,
                                   uint64_t n) const {
  if (!n) return 0;
  // Leave one real input token to compute the first logits from.
  const uint64_t maximum = (n - 1) / KVX_PAGE_TOKENS;
  uint64_t hashed = 0;
  for (uint64_t index = blocks->size(); index < maximum; ++index) {
    const uint64_t parent = blocks->empty() ? 0 : blocks->back();
    ++hashed;
    uint64_t id = 0;
    if (!find(parent, prompt + index * KVX_PAGE_TOKENS, KVX_PAGE_TOKENS, 0, 0, &id, nullptr)) break;
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

// Cache::publishCommittedBlocks (Cache.cpp:294-333): every newly full page
// becomes a block; where the content is already cached the sequence moves to
// the canonical page and gives its own back.
int SequenceCache::publish(uint64_t id, const uint32_t *tokens, uint64_t n_tokens,
                           uint32_t committed) {
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
    if (const int rc = prefix_.insert(parent, tokens + uint64_t(logical) * KVX_PAGE_TOKENS,
                                      KVX_PAGE_TOKENS, writer, 0, 0, &block, &canonical))
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
