// C ABI of the page pool over device extent storage.
#include "kvx_internal.h"
#include "kvx_pool.h"

namespace {

// The pool's view of a kvx_storage: extents through the storage calls, page
// moves through the copy kernel on the stream of the current compaction.
class DeviceExtents final : public kvx::ExtentStorage {
public:
  explicit DeviceExtents(kvx_storage *storage) : storage_(storage) {}
  uint32_t page_count() const override { return kvx_storage_page_count(storage_); }
  uint64_t bytes_per_page() const override { return kvx_storage_bytes_per_page(storage_); }
  uint32_t extent_pages() const override { return kvx_storage_extent_pages(storage_); }
  int allocate_extent(uint32_t extent) override {
    return kvx_storage_allocate_extent(storage_, extent);
  }
  int release_extent(uint32_t extent) override {
    return kvx_storage_release_extent(storage_, extent);
  }
  int copy_pages(const kvx_page_copy *copies, uint32_t n) override {
    return kv_page_copy(storage_, copies, n, stream);
  }
  void *stream = nullptr;

private:
  kvx_storage *storage_;
};

}  // namespace

struct kvx_pool {
  DeviceExtents extents;
  kvx::KvPool pool;
  kvx_pool(kvx_storage *storage, uint32_t runway) : extents(storage), pool(extents, runway) {}
};

kvx::KvPool &kvx_pool_object(kvx_pool *pool) { return pool->pool; }
void kvx_pool_set_stream(kvx_pool *pool, void *stream) { pool->extents.stream = stream; }

extern "C" {

int kvx_pool_create(kvx_storage *storage, uint32_t runway_pages, kvx_pool **out) {
  if (!storage || !out) return kvx::fail(KVX_EINVAL, "kvx_pool_create: null argument");
  *out = nullptr;
  auto *p = new kvx_pool(storage, runway_pages);
  if (const int rc = p->pool.status()) {
    delete p;
    return rc == KVX_EINVAL ? kvx::fail(rc, "invalid KV extent storage or runway") : rc;
  }
  *out = p;
  return KVX_OK;
}
void kvx_pool_destroy(kvx_pool *pool) { delete pool; }
int kvx_pool_acquire(kvx_pool *pool, uint32_t count, uint32_t *pages) {
  const int rc = pool->pool.acquire(count, pages);
  if (rc == KVX_ESTATE) return kvx::fail(rc, "KV page ids ran out before the memory budget did");
  return rc;
}
int kvx_pool_retain(kvx_pool *pool, uint32_t page, int prefix_owner) {
  const int rc = pool->pool.retain(page, prefix_owner != 0);
  return rc ? kvx::fail(rc, "invalid KV page retain") : rc;
}
int kvx_pool_release(kvx_pool *pool, uint32_t page, int prefix_owner) {
  const int rc = pool->pool.release(page, prefix_owner != 0);
  return rc ? kvx::fail(rc, "invalid KV page release") : rc;
}
int kvx_pool_page_active(const kvx_pool *pool, uint32_t page) {
  return page < pool->pool.page_count() && pool->pool.page_active(page);
}
uint32_t kvx_pool_free_pages(const kvx_pool *pool) { return pool->pool.free_pages(); }
int kvx_pool_reclaim_empty(kvx_pool *pool, int keep_runway, uint32_t limit, uint64_t *released) {
  return pool->pool.reclaim_empty(keep_runway != 0, limit, released);
}
int kvx_pool_compact_extent(kvx_pool *pool, const uint32_t *fixed, uint32_t n_fixed,
                            uint32_t *first_page, uint32_t *destinations, uint32_t *moved_pages,
                            void *stream) {
  kvx::PageMoves moves;
  pool->extents.stream = stream;
  const int rc = pool->pool.compact_extent(fixed, n_fixed, &moves);
  pool->extents.stream = nullptr;
  if (rc) return rc;
  if (moved_pages) *moved_pages = moves.moved;
  if (!moves.empty()) {
    if (first_page) *first_page = moves.first_page;
    if (destinations)
      for (size_t i = 0; i < moves.destinations.size(); ++i) destinations[i] = moves.destinations[i];
  }
  return KVX_OK;
}
int kvx_pool_snapshot_get(const kvx_pool *pool, kvx_pool_snapshot *out) {
  pool->pool.snapshot(out);
  return KVX_OK;
}

}  // extern "C"
