// Prefix reuse at whole-page granularity: the RAM tier of the reference's
// engine::KvCache (runtime/engine/cache/KvCache.hpp:40-241, KvCache.cpp) and
// the part of engine::Cache that keeps each sequence's page list
// (runtime/engine/cache/Cache.cpp:143-166, 179-199, 284-333, 381-413, 700-731,
// 748-785).  Blocks are keyed by (parent block, the page's 32 tokens, image
// identity); a block owns one prefix reference of its page in the pool.  The
// disk tier, recurrent states and poisoning of the reference are not part of
// the KV data path and have no counterpart here.
//
// Blocks are found through one hash map whose key is the whole content key
// (parent block id, the 32 tokens, both halves of the image identity), so a
// lookup is a single probe that compares complete keys, and a block's place in
// the tree is its parent's id, not a hash chained down from the root.
#pragma once

#include <array>
#include <cstdint>
#include <map>
#include <unordered_map>
#include <utility>
#include <vector>

#include "kvx_pool.h"

namespace kvx {

// engine::blockImageIdentity (runtime/engine/cache/KvCache.cpp:29-52).
void block_image_identity(uint64_t block_begin, uint32_t block_tokens, const kvx_image_span *spans,
                          uint32_t n_spans, uint64_t *lo, uint64_t *hi);

class PrefixCache {
public:
  static constexpr uint32_t kNoPage = 0xffffffffu;
  explicit PrefixCache(KvPool &pool) : pool_(pool), block_on_page_(pool.page_count(), 0) {}
  ~PrefixCache();
  PrefixCache(const PrefixCache &) = delete;
  PrefixCache &operator=(const PrefixCache &) = delete;

  // KvCache::find: true with the block and its page when the exact key exists.
  bool find(uint64_t parent, const uint32_t *tokens, uint32_t n_tokens, uint64_t image_lo,
            uint64_t image_hi, uint64_t *block, uint32_t *page) const;
  // KvCache::insert: existing content is returned as it is.
  int insert(uint64_t parent, const uint32_t *tokens, uint32_t n_tokens, uint32_t page,
             uint64_t image_lo, uint64_t image_hi, uint64_t *block, uint32_t *canonical_page);
  bool contains(uint64_t block) const { return blocks_.count(block) != 0; }
  int chain_length(uint64_t block, uint32_t *length) const;
  int chain(uint64_t block, std::vector<uint64_t> *blocks, std::vector<uint32_t> *pages) const;
  int page_of(uint64_t block, uint32_t *page) const;
  int retain_active(uint64_t block);
  int release_active(uint64_t block);
  int touch(uint64_t block);
  // KvCache::evictionCandidate: idle resident leaves, oldest first; `after` = 0
  // starts the scan.  False when there is none.
  int eviction_candidate(uint64_t after, uint64_t *block, bool *found) const;
  int erase(uint64_t block);
  // KvCache::followPages after an extent compaction.
  void follow_pages(const PageMoves &moves);
  // Cache::extendMatch: appends matched blocks, leaving at least one prompt token
  // unmatched; returns how many pages were looked up.  Every block is looked up
  // under the identity of the prompt's images that overlap it (`spans` sorted by
  // offset and disjoint; none for a text-only prompt).
  uint64_t extend_match(std::vector<uint64_t> *blocks, const uint32_t *prompt, uint64_t n,
                        const kvx_image_span *spans = nullptr, uint32_t n_spans = 0) const;
  uint64_t generation() const { return generation_; }
  uint64_t block_count() const { return blocks_.size(); }

private:
  struct ContentKey {
    uint64_t parent = 0, image_lo = 0, image_hi = 0;
    std::array<uint32_t, KVX_PAGE_TOKENS> tokens{};
    bool operator==(const ContentKey &o) const {
      return parent == o.parent && image_lo == o.image_lo && image_hi == o.image_hi &&
             tokens == o.tokens;
    }
  };
  struct ContentKeyHash {
    size_t operator()(const ContentKey &key) const;
  };
  static ContentKey key_of(uint64_t parent, const uint32_t *tokens, uint64_t image_lo,
                           uint64_t image_hi);
  struct Block {
    uint64_t id = 0;
    ContentKey key;
    uint32_t page = kNoPage, depth = 0, children = 0, active_users = 0;
    uint64_t last_used = 0, listed_at = 0;
    bool listed = false;
  };
  const Block *get(uint64_t id) const;
  Block *get(uint64_t id);
  void reindex(Block &b);

  KvPool &pool_;
  std::unordered_map<uint64_t, Block> blocks_;
  std::unordered_map<ContentKey, uint64_t, ContentKeyHash> by_content_;  // key -> block id
  std::map<std::pair<uint64_t, uint64_t>, uint64_t> leaves_;  // (last used, id) -> id
  std::vector<uint64_t> block_on_page_;
  uint64_t next_id_ = 1, clock_ = 0, generation_ = 0;
};

// One sequence's pages: engine::Cache's Request record.
class SequenceCache {
public:
  SequenceCache(KvPool &pool, PrefixCache &prefix) : pool_(pool), prefix_(prefix) {}
  ~SequenceCache();
  int begin(uint64_t id);                                   // Cache::beginRequest
  int end(uint64_t id);                                     // Cache::endRequest
  int restore(uint64_t id, uint64_t last_block);            // Cache::restoreRequest, resident chain
  int ensure_tokens(uint64_t id, uint64_t tokens);          // Cache::ensureTokens
  // Copy-on-write sharing, which the reference does not have (it shares whole
  // published pages only, Cache.cpp:183-184, :774).  fork: the empty sequence `id`
  // takes the pages that hold the first `tokens` tokens of `source` by reference,
  // the partly filled last one included, and the source's blocks over those pages.
  // ensure_writable: before rows are stored at `token` and after, the page that
  // holds it is replaced by a private copy (all layers, on the pool's copy stream)
  // when anyone else holds it too; *copied says whether, *from / *to which pages.
  int fork(uint64_t id, uint64_t source, uint64_t tokens);
  // Gives back the pages past those that hold the first `tokens` tokens (a rollback
  // that emptied them); *released says how many.  Published pages stay.
  int truncate(uint64_t id, uint64_t tokens, uint32_t *released);
  int ensure_writable(uint64_t id, uint64_t token, bool *copied, uint32_t *from, uint32_t *to);
  int publish(uint64_t id, const uint32_t *tokens, uint64_t n_tokens, uint32_t committed,
              const kvx_image_span *spans = nullptr, uint32_t n_spans = 0);
  struct View {                                             // Cache::pageTable
    const uint32_t *pages;
    uint32_t count;
    uint64_t revision;
    uint32_t first_changed;
    const uint64_t *blocks;
    uint32_t block_count;
  };
  int view(uint64_t id, View *out) const;
  // Cache::compactExtent: empties one extent, re-points blocks and sequences.
  int compact_extent(PageMoves *moves);

private:
  struct Sequence {
    std::vector<uint32_t> pages;
    std::vector<uint64_t> blocks;
    uint64_t revision = 0;
    uint32_t first_changed = 0;
  };
  static void changed(Sequence &s, uint32_t first) {
    ++s.revision;
    s.first_changed = first;
  }
  KvPool &pool_;
  PrefixCache &prefix_;
  std::unordered_map<uint64_t, Sequence> sequences_;
};

}  // namespace kvx
