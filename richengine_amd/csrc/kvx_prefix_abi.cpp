// C ABI of the prefix page cache and the per-sequence page lists.
#include "kvx_internal.h"
#include "kvx_pool.h"
#include "kvx_prefix.h"

// Defined with the pool's ABI: the pool object behind a kvx_pool handle and the
// stream its page copies go to.
kvx::KvPool &kvx_pool_object(kvx_pool *pool);
void kvx_pool_set_stream(kvx_pool *pool, void *stream);

struct kvx_prefix {
  kvx::PrefixCache cache;
  explicit kvx_prefix(kvx_pool *pool) : cache(kvx_pool_object(pool)) {}
};

struct kvx_sequences {
  kvx_pool *pool;
  kvx::SequenceCache sequences;
  kvx_sequences(kvx_pool *p, kvx_prefix *prefix)
      : pool(p), sequences(kvx_pool_object(p), prefix->cache) {}
};

namespace {
int report(int rc, const char *what) { return rc ? kvx::fail(rc, what) : rc; }
}  // namespace

extern "C" {

int kvx_prefix_create(kvx_pool *pool, kvx_prefix **out) {
  if (!pool || !out) return kvx::fail(KVX_EINVAL, "kvx_prefix_create: null argument");
  *out = new kvx_prefix(pool);
  return KVX_OK;
}
void kvx_prefix_destroy(kvx_prefix *prefix) { delete prefix; }

int kvx_prefix_find(const kvx_prefix *prefix, uint64_t parent, const uint32_t *tokens,
                    uint32_t n_tokens, uint64_t image_lo, uint64_t image_hi, uint64_t *block,
                    uint32_t *page) {
  return prefix->cache.find(parent, tokens, n_tokens, image_lo, image_hi, block, page) ? 1 : 0;
}
int kvx_prefix_insert(kvx_prefix *prefix, uint64_t parent, const uint32_t *tokens,
                      uint32_t n_tokens, uint32_t page, uint64_t image_lo, uint64_t image_hi,
                      uint64_t *block, uint32_t *canonical_page) {
  const int rc =
      prefix->cache.insert(parent, tokens, n_tokens, page, image_lo, image_hi, block, canonical_page);
  switch (rc) {
  case KVX_EINVAL:
    return kvx::fail(rc, "KV cache block needs one full page of tokens and a known parent");
  case KVX_ERANGE:
    return kvx::fail(rc, "KV cache physical page is out of range");
  case KVX_ESTATE:
    return kvx::fail(rc, "KV cache page already holds a block, or is not held");
  default:
    return rc;
  }
}
int kvx_prefix_contains(const kvx_prefix *prefix, uint64_t block) {
  return prefix->cache.contains(block) ? 1 : 0;
}
uint64_t kvx_prefix_generation(const kvx_prefix *prefix) { return prefix->cache.generation(); }
uint64_t kvx_prefix_block_count(const kvx_prefix *prefix) { return prefix->cache.block_count(); }
int kvx_prefix_chain(const kvx_prefix *prefix, uint64_t block, uint64_t *blocks, uint32_t *pages,
                     uint32_t capacity, uint32_t *length) {
  std::vector<uint64_t> ids;
  std::vector<uint32_t> held;
  if (const int rc = prefix->cache.chain(block, &ids, &held))
    return report(rc, "unknown KV cache block");
  if (length) *length = uint32_t(ids.size());
  for (uint32_t i = 0; i < ids.size() && i < capacity; ++i) {
    if (blocks) blocks[i] = ids[i];
    if (pages) pages[i] = held[i];
  }
  return KVX_OK;
}
int kvx_prefix_retain_active(kvx_prefix *prefix, uint64_t block) {
  return report(prefix->cache.retain_active(block), "unknown KV cache block");
}
int kvx_prefix_release_active(kvx_prefix *prefix, uint64_t block) {
  return report(prefix->cache.release_active(block), "KV cache block has no active user");
}
int kvx_prefix_touch(kvx_prefix *prefix, uint64_t block) {
  return report(prefix->cache.touch(block), "unknown KV cache block");
}
int kvx_prefix_eviction_candidate(const kvx_prefix *prefix, uint64_t after, uint64_t *block) {
  bool found = false;
  uint64_t id = 0;
  if (const int rc = prefix->cache.eviction_candidate(after, &id, &found))
    return report(rc, "unknown KV cache block");
  if (found && block) *block = id;
  return found ? 1 : 0;
}
int kvx_prefix_erase(kvx_prefix *prefix, uint64_t block) {
  const int rc = prefix->cache.erase(block);
  return rc == KVX_ESTATE ? kvx::fail(rc, "cannot evict a referenced KV cache block")
                          : report(rc, "unknown KV cache block");
}
void kvx_prefix_follow_pages(kvx_prefix *prefix, uint32_t first_page, const uint32_t *destinations,
                             uint32_t n) {
  kvx::PageMoves moves;
  moves.first_page = first_page;
  moves.destinations.assign(destinations, destinations + n);
  prefix->cache.follow_pages(moves);
}
uint64_t kvx_prefix_match(const kvx_prefix *prefix, const uint32_t *prompt, uint64_t n_tokens,
                          uint64_t *blocks, uint32_t capacity, uint32_t *matched) {
  return kvx_prefix_match_images(prefix, prompt, n_tokens, nullptr, 0, blocks, capacity, matched);
}
uint64_t kvx_prefix_match_images(const kvx_prefix *prefix, const uint32_t *prompt, uint64_t n_tokens,
                                 const kvx_image_span *spans, uint32_t n_spans, uint64_t *blocks,
                                 uint32_t capacity, uint32_t *matched) {
  std::vector<uint64_t> chain;
  const uint64_t hashed =
      prefix->cache.extend_match(&chain, prompt, n_tokens, spans, spans ? n_spans : 0);
  if (matched) *matched = uint32_t(chain.size());
  for (uint32_t i = 0; i < chain.size() && i < capacity; ++i) blocks[i] = chain[i];
  return hashed;
}

void kvx_block_image_identity(uint64_t block_begin, uint32_t block_tokens,
                              const kvx_image_span *spans, uint32_t n_spans, uint64_t *lo,
                              uint64_t *hi) {
  kvx::block_image_identity(block_begin, block_tokens, spans, n_spans, lo, hi);
}

int kvx_sequences_create(kvx_pool *pool, kvx_prefix *prefix, kvx_sequences **out) {
  if (!pool || !prefix || !out) return kvx::fail(KVX_EINVAL, "kvx_sequences_create: null argument");
  *out = new kvx_sequences(pool, prefix);
  return KVX_OK;
}
void kvx_sequences_destroy(kvx_sequences *sequences) { delete sequences; }
int kvx_sequence_begin(kvx_sequences *s, uint64_t id) {
  return report(s->sequences.begin(id), "invalid or duplicate sequence id");
}
int kvx_sequence_end(kvx_sequences *s, uint64_t id) { return s->sequences.end(id); }
int kvx_sequence_restore(kvx_sequences *s, uint64_t id, uint64_t last_block) {
  const int rc = s->sequences.restore(id, last_block);
  return rc == KVX_ESTATE ? kvx::fail(rc, "restore target already owns KV pages")
                          : report(rc, "unknown sequence or KV cache block");
}
int kvx_sequence_ensure_tokens(kvx_sequences *s, uint64_t id, uint64_t tokens) {
  const int rc = s->sequences.ensure_tokens(id, tokens);
  return rc == KVX_ENOMEM ? rc : report(rc, "unknown sequence, or KV target past the page id range");
}
int kvx_sequence_fork(kvx_sequences *s, uint64_t id, uint64_t source, uint64_t tokens) {
  const int rc = s->sequences.fork(id, source, tokens);
  switch (rc) {
  case KVX_ESTATE:
    return kvx::fail(rc, "fork target already owns KV pages, or is its own source");
  case KVX_EINVAL:
    return kvx::fail(rc, "fork point past the pages the source holds");
  default:
    return report(rc, "unknown sequence");
  }
}
int kvx_sequence_truncate(kvx_sequences *s, uint64_t id, uint64_t tokens, uint32_t *released_pages) {
  uint32_t released = 0;
  const int rc = s->sequences.truncate(id, tokens, &released);
  if (released_pages) *released_pages = released;
  if (rc == KVX_ESTATE) return kvx::fail(rc, "truncation would drop a published page");
  return report(rc, "unknown sequence");
}
int kvx_sequence_ensure_writable(kvx_sequences *s, uint64_t id, uint64_t token, uint32_t *copied,
                                 uint32_t *from_page, uint32_t *to_page, void *stream) {
  bool did = false;
  uint32_t from = KVX_NO_PAGE, to = KVX_NO_PAGE;
  kvx_pool_set_stream(s->pool, stream);
  const int rc = s->sequences.ensure_writable(id, token, &did, &from, &to);
  kvx_pool_set_stream(s->pool, nullptr);
  if (copied) *copied = did ? 1u : 0u;
  if (from_page) *from_page = from;
  if (to_page) *to_page = to;
  switch (rc) {
  case KVX_ESTATE:
    return kvx::fail(rc, "the page is published: rows before the token's page boundary are final");
  case KVX_EINVAL:
    return kvx::fail(rc, "the sequence holds no page for this token");
  case KVX_ENOMEM:
    return rc;
  default:
    return report(rc, "unknown sequence");
  }
}
int kvx_sequence_publish(kvx_sequences *s, uint64_t id, const uint32_t *tokens, uint64_t n_tokens,
                         uint32_t committed_tokens) {
  return kvx_sequence_publish_images(s, id, tokens, n_tokens, committed_tokens, nullptr, 0);
}
int kvx_sequence_publish_images(kvx_sequences *s, uint64_t id, const uint32_t *tokens,
                                uint64_t n_tokens, uint32_t committed_tokens,
                                const kvx_image_span *spans, uint32_t n_spans) {
  const int rc =
      s->sequences.publish(id, tokens, n_tokens, committed_tokens, spans, spans ? n_spans : 0);
  switch (rc) {
  case KVX_EINVAL:
    return kvx::fail(rc, "committed KV exceeds exact token history");
  case KVX_ESTATE:
    return kvx::fail(rc, "committed KV has no physical page, or history moved backwards");
  default:
    return report(rc, "unknown sequence");
  }
}
int kvx_sequence_view(const kvx_sequences *s, uint64_t id, kvx_sequence_pages *out) {
  kvx::SequenceCache::View view{};
  if (const int rc = s->sequences.view(id, &view)) return report(rc, "unknown sequence");
  out->pages = view.pages;
  out->page_count = view.count;
  out->revision = view.revision;
  out->first_changed = view.first_changed;
  out->blocks = view.blocks;
  out->block_count = view.block_count;
  return KVX_OK;
}
int kvx_sequences_compact_extent(kvx_sequences *s, uint32_t *first_page, uint32_t *destinations,
                                 uint32_t *moved_pages, void *stream) {
  kvx::PageMoves moves;
  kvx_pool_set_stream(s->pool, stream);
  const int rc = s->sequences.compact_extent(&moves);
  kvx_pool_set_stream(s->pool, nullptr);
  if (rc) return rc;
  if (moved_pages) *moved_pages = moves.moved;
  if (!moves.empty()) {
    if (first_page) *first_page = moves.first_page;
    if (destinations)
      for (size_t i = 0; i < moves.destinations.size(); ++i) destinations[i] = moves.destinations[i];
  }
  return KVX_OK;
}

}  // extern "C"
