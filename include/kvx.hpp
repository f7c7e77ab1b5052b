// kvx.hpp -- header-only C++17 mirror of RichEngine's KV host interface over
// the C ABI of libkvx (kvx.h).
//
// Same names, argument meaning and error behaviour as the reference's
// runtime/ops (kv::Layout, kv::PageStorage, ops::PagedAttention) and
// runtime/engine/cache (KvPool), so code and tests written against those read
// the same here.  Differences forced by the device:
//   - a metal::MetalBuffer becomes a device pointer into HBM the caller owns;
//   - a metal::CommandGraph becomes the hipStream_t work is enqueued on (passed
//     as void*, nullptr = the default stream);
//   - partials and statistics live in one workspace buffer (partials first,
//     statistics at the next 256-byte boundary);
//   - status codes of the C ABI are raised as the reference's exceptions:
//     std::invalid_argument, std::logic_error, std::out_of_range;
//     a refused allocation is a value (AllocationFailure), as in the reference.
#pragma once

#include <algorithm>
#include <array>
#include <cstdint>
#include <new>
#include <stdexcept>
#include <string>
#include <vector>

#include "kvx.h"

namespace kvx {

class DeviceError : public std::runtime_error {
  using std::runtime_error::runtime_error;
};

// Raises what the reference would throw for a failed call.  KVX_ENOMEM is a
// value for callers that report refusals (allocateExtent, acquirePages).
inline void check(int status) {
  switch (status) {
  case KVX_OK:
    return;
  case KVX_EINVAL:
    throw std::invalid_argument(kvx_last_error());
  case KVX_ESTATE:
    throw std::logic_error(kvx_last_error());
  case KVX_ERANGE:
    throw std::out_of_range(kvx_last_error());
  case KVX_ENOMEM:
    throw std::bad_alloc();
  default:
    throw DeviceError(kvx_last_error());
  }
}

namespace kv {

// runtime/ops/PagedKv.hpp:16
enum class Format : uint32_t {
  Int8 = KVX_FMT_INT8,
  BFloat16 = KVX_FMT_BF16,
  Int4 = KVX_FMT_INT4,
  Float8E4M3 = KVX_FMT_FP8E4M3
};

inline constexpr uint32_t kPageTokens = KVX_PAGE_TOKENS;
inline constexpr uint32_t kVerifyRows = KVX_VERIFY_ROWS;
inline constexpr uint32_t kTreeVerifyNodes = KVX_TREE_NODES;
inline constexpr uint32_t kVerifyChunkStride = KVX_VERIFY_CHUNK_STRIDE;
inline constexpr uint32_t kVerifyMaximumSplits = KVX_VERIFY_MAX_SPLITS;
inline constexpr uint32_t kPrefillTokenBudget = KVX_PREFILL_TOKEN_BUDGET;

using ChunkedPrefillParams = kvx_chunk_params;    // abi/PagedAttention.h:39-45
using PrefillAttentionParams = kvx_prefill_params;  // abi/PagedAttention.h:52-61
using VerifyAttentionParams = kvx_verify_params;  // abi/PagedAttention.h:72-84
using PageCopy = kvx_page_copy;                   // PagedKv.hpp:48-51
using KvLayer = kvx_kv_layer;                     // abi/KvExtent.h:93-96 (RichKvLayer)

// runtime/ops/PagedKv.hpp:125-232
struct Layout final {
  uint32_t attentionLayers = 0;
  uint32_t kvHeads = 0;
  uint32_t headDimension = 0;
  Format format = Format::Int8;
  float scoreScale = 0.0F;

  kvx_layout c() const noexcept {
    return {attentionLayers, kvHeads, headDimension, static_cast<uint32_t>(format), scoreScale};
  }
  bool valid() const noexcept { const auto l = c(); return kvx_layout_valid(&l) != 0; }
  bool quantized() const noexcept { return format != Format::BFloat16; }
  uint64_t dataBytesPerLayerPage() const noexcept { const auto l = c(); return kvx_layout_data_bytes_per_layer_page(&l); }
  uint64_t scaleBytesPerLayerPage() const noexcept { const auto l = c(); return kvx_layout_scale_bytes_per_layer_page(&l); }
  uint64_t bytesPerLayerPage() const noexcept { const auto l = c(); return kvx_layout_bytes_per_layer_page(&l); }
  uint64_t bytesPerModelPage() const noexcept { const auto l = c(); return kvx_layout_bytes_per_model_page(&l); }
  uint32_t extentAlignmentPages() const noexcept { const auto l = c(); return kvx_layout_extent_alignment_pages(&l); }
  uint32_t minimumExtentPages() const noexcept { const auto l = c(); return kvx_layout_minimum_extent_pages(&l); }
  uint32_t maximumExtentPages() const noexcept { const auto l = c(); return kvx_layout_maximum_extent_pages(&l); }
  uint32_t extentPagesFor(uint64_t pages) const noexcept { const auto l = c(); return kvx_layout_extent_pages_for(&l, pages); }
  // No counterpart in the reference: the largest extent the page entry allows.
  uint32_t largestExtentPages() const noexcept { const auto l = c(); return kvx_layout_largest_extent_pages(&l); }
};

// runtime/ops/PagedAttention.hpp:54-95
inline uint32_t verifyAttentionSplits(uint32_t historyTokens, uint32_t rows = kVerifyRows) {
  return kvx_verify_splits(historyTokens, rows);
}
inline const char *chunkedPrefillValidationError(const ChunkedPrefillParams &params) {
  static const char *const names[] = {nullptr, "chunk_tokens_out_of_range", "context_out_of_range",
                                      "chunk_stride_invalid", "page_table_too_short"};
  return names[kvx_chunk_validation(&params)];
}

// runtime/metal/MetalBackend.hpp:18-45, reduced to what the path reports
enum class AllocationFailure { None, EngineBudget, DriverRejected };

// runtime/ops/PagedKv.hpp:56-76
class ExtentStorage {
public:
  virtual ~ExtentStorage() = default;
  virtual uint32_t pageCount() const noexcept = 0;
  virtual uint64_t bytesPerPage() const noexcept = 0;
  virtual uint32_t extentPages() const noexcept = 0;
  virtual AllocationFailure allocateExtent(uint32_t extent) = 0;
  virtual void releaseExtent(uint32_t extent) = 0;
  virtual void copyPages(const PageCopy *copies, size_t count) = 0;
};

// runtime/ops/PageStorage.hpp:27-102 over HBM extents.
class PageStorage final : public ExtentStorage {
public:
  // aligned = false takes any extent size the page index allows, as the
  // reference's test pools do (dev/tuning/HostKvExtents.hpp:158-169).
  PageStorage(Layout layout, uint32_t pageCount, uint32_t extentPages, bool aligned = true,
              void *stream = nullptr)
      : layout_(layout), stream_(stream) {
    const kvx_layout l = layout.c();
    check(kvx_storage_create(&l, pageCount, extentPages, aligned ? 1 : 0, &storage_));
  }
  ~PageStorage() override { kvx_storage_destroy(storage_); }
  PageStorage(const PageStorage &) = delete;
  PageStorage &operator=(const PageStorage &) = delete;

  uint32_t pageCount() const noexcept override { return kvx_storage_page_count(storage_); }
  uint64_t bytesPerPage() const noexcept override { return kvx_storage_bytes_per_page(storage_); }
  uint32_t extentPages() const noexcept override { return kvx_storage_extent_pages(storage_); }
  uint64_t extentBytes() const noexcept { return kvx_storage_extent_bytes(storage_); }
  uint64_t allocatedBytes() const noexcept { return kvx_storage_allocated_bytes(storage_); }
  bool allocated(uint32_t page) const noexcept { return kvx_storage_is_allocated(storage_, page) != 0; }
  // The admission budget of the reference's allocation callback; 0 = none.
  void setBudget(uint64_t bytes) { kvx_storage_set_budget(storage_, bytes); budget_ = bytes; }

  AllocationFailure allocateExtent(uint32_t extent) override {
    const int status = kvx_storage_allocate_extent(storage_, extent);
    if (status == KVX_ENOMEM)
      return budget_ ? AllocationFailure::EngineBudget : AllocationFailure::DriverRejected;
    check(status);
    return AllocationFailure::None;
  }
  void releaseExtent(uint32_t extent) override { check(kvx_storage_release_extent(storage_, extent)); }
  void copyPages(const PageCopy *copies, size_t count) override {
    check(kv_page_copy(storage_, copies, static_cast<uint32_t>(count), stream_));
  }
  void copyPages(const std::vector<PageCopy> &copies) { copyPages(copies.data(), copies.size()); }
  // The pages' spans (PageStorage::spans, PageStorage.mm:143-167) as one linear
  // buffer, page after page: what a host or disk tier demotes and restores
  // (engine::KvPageTier).  `buffer` is device memory or pinned host memory.
  void exportPages(const std::vector<uint32_t> &pages, void *buffer) const {
    check(kv_page_export(storage_, pages.data(), static_cast<uint32_t>(pages.size()), buffer, stream_));
  }
  void importPages(const std::vector<uint32_t> &pages, const void *buffer) {
    check(kv_page_import(storage_, pages.data(), static_cast<uint32_t>(pages.size()), buffer, stream_));
  }

  KvLayer layer(uint32_t index) const {
    KvLayer out{};
    check(kvx_storage_layer(storage_, index, &out));
    return out;
  }
  // writeEntries (PageStorage.mm:127-141) into a host array ...
  void entries(const std::vector<uint32_t> &pages, uint32_t first, uint64_t *tableHost) const {
    check(kvx_storage_entries(storage_, pages.data(), static_cast<uint32_t>(pages.size()), first, tableHost));
  }
  // ... and into a device table of `capacity` entries, on the storage's stream.
  void writeEntries(const std::vector<uint32_t> &pages, uint32_t first, uint64_t *tableDevice,
                    uint64_t capacity) const {
    check(kvx_storage_write_entries(storage_, pages.data(), static_cast<uint32_t>(pages.size()), first,
                                    tableDevice, capacity, stream_));
  }
  // spans(page) for memory the host cannot map: the page's bytes, staged.
  std::vector<uint8_t> readPage(uint32_t page) const {
    std::vector<uint8_t> bytes(bytesPerPage());
    check(kvx_storage_page_read(storage_, page, bytes.data()));
    return bytes;
  }
  void writePage(uint32_t page, const std::vector<uint8_t> &bytes) {
    if (bytes.size() != bytesPerPage()) throw std::invalid_argument("page bytes have the wrong size");
    check(kvx_storage_page_write(storage_, page, bytes.data()));
  }
  const Layout &layout() const noexcept { return layout_; }
  kvx_storage *handle() const noexcept { return storage_; }
  void *stream() const noexcept { return stream_; }

private:
  Layout layout_;
  kvx_storage *storage_ = nullptr;
  void *stream_ = nullptr;
  uint64_t budget_ = 0;
};

}  // namespace kv

namespace engine {

using KvPoolSnapshot = kvx_pool_snapshot;  // runtime/engine/cache/KvPool.hpp:12-35

// runtime/engine/cache/KvPool.hpp:39-52
struct KvPageMoves final {
  uint32_t firstPage = 0;
  std::vector<uint32_t> destinations;
  bool empty() const noexcept { return destinations.empty(); }
  uint32_t follow(uint32_t page) const noexcept {
    return page >= firstPage && page - firstPage < destinations.size() ? destinations[page - firstPage]
                                                                      : page;
  }
};

// runtime/engine/cache/KvPool.hpp:54-62
struct KvPageAcquisition {
  std::vector<uint32_t> pages;
  kv::AllocationFailure failure = kv::AllocationFailure::None;
  bool granted() const noexcept { return failure == kv::AllocationFailure::None; }
};

// runtime/engine/cache/KvPool.hpp:75-115 over a kv::PageStorage.
class KvPool final {
public:
  KvPool(kv::PageStorage &storage, uint32_t runwayPages) : storage_(storage) {
    check(kvx_pool_create(storage.handle(), runwayPages, &pool_));
  }
  ~KvPool() { kvx_pool_destroy(pool_); }
  KvPool(const KvPool &) = delete;
  KvPool &operator=(const KvPool &) = delete;

  KvPageAcquisition acquirePages(uint32_t count) {
    KvPageAcquisition result;
    result.pages.resize(count);
    const int status = kvx_pool_acquire(pool_, count, result.pages.data());
    if (status == KVX_ENOMEM) {
      result.pages.clear();
      result.failure = kv::AllocationFailure::DriverRejected;
      return result;
    }
    check(status);
    return result;
  }
  void retainPage(uint32_t page, bool prefixOwner) { check(kvx_pool_retain(pool_, page, prefixOwner)); }
  void releasePage(uint32_t page, bool prefixOwner) { check(kvx_pool_release(pool_, page, prefixOwner)); }
  uint32_t pageCount() const noexcept { return storage_.pageCount(); }
  uint64_t bytesPerPage() const noexcept { return storage_.bytesPerPage(); }
  uint32_t extentPages() const noexcept { return storage_.extentPages(); }
  uint32_t freePageCount() const noexcept { return kvx_pool_free_pages(pool_); }
  bool pageActive(uint32_t page) const {
    const int status = kvx_pool_page_active(pool_, page);
    if (status < 0) check(status);
    return status != 0;
  }
  uint64_t allocatedBytes() const noexcept { return snapshot().allocated_bytes; }
  uint64_t reclaimEmptyExtents(bool keepRunway, uint32_t limit) {
    uint64_t released = 0;
    check(kvx_pool_reclaim_empty(pool_, keepRunway, limit, &released));
    return released;
  }
  KvPageMoves compactExtent(const std::vector<uint32_t> &fixed = {}) {
    KvPageMoves moves;
    std::vector<uint32_t> destinations(storage_.extentPages());
    uint32_t moved = 0;
    check(kvx_pool_compact_extent(pool_, fixed.data(), static_cast<uint32_t>(fixed.size()),
                                  &moves.firstPage, destinations.data(), &moved, storage_.stream()));
    if (moved) moves.destinations = std::move(destinations);
    return moves;
  }
  KvPoolSnapshot snapshot() const noexcept {
    KvPoolSnapshot out{};
    kvx_pool_snapshot_get(pool_, &out);
    return out;
  }

private:
  kv::PageStorage &storage_;
  kvx_pool *pool_ = nullptr;
};

// runtime/engine/cache/KvCache.hpp:25-32, KvCache.cpp:29-52: what the images that overlap
// tokens [blockBegin, blockBegin + blockTokens) add to that block's cache key.
using ImageSpan = kvx_image_span;
struct ImageIdentity final {
  uint64_t lo = 0, hi = 0;
  bool operator==(const ImageIdentity &o) const noexcept { return lo == o.lo && hi == o.hi; }
};
inline ImageIdentity blockImageIdentity(uint64_t blockBegin, uint32_t blockTokens,
                                        const std::vector<ImageSpan> &spans) noexcept {
  ImageIdentity identity;
  kvx_block_image_identity(blockBegin, blockTokens, spans.data(), static_cast<uint32_t>(spans.size()),
                           &identity.lo, &identity.hi);
  return identity;
}

}  // namespace engine

namespace ops {

// runtime/ops/PagedAttention.hpp:101-104
struct AttentionWorkspace final {
  uint64_t partialsBytes = 0;
  uint64_t statisticsBytes = 0;
  // One buffer: partials, then statistics at the next 256-byte boundary.
  uint64_t bytes() const noexcept { return (partialsBytes + 255) / 256 * 256 + statisticsBytes; }
};

// runtime/ops/PagedAttention.hpp:109-136, without the Metal pipeline names
struct PrefillAttentionPlan final {
  kv::Format format;
  uint32_t rows;
  uint32_t splits;
  AttentionWorkspace workspace;
  uint32_t queryHeads;
  float scoreScale;
};

// runtime/ops/PagedAttention.hpp:138-183; any lane count
struct VerifyAttentionPlan final {
  kv::Format format;
  uint32_t lanes;
  std::vector<uint32_t> laneSplits;
  uint32_t splits;  // their maximum
  AttentionWorkspace workspace;
  uint32_t rowCapacity;
  uint32_t queryHeads;
  float scoreScale;
};

// runtime/ops/PagedAttention.hpp:185-197
struct PagedVerifyBuffers final {
  const void *chunkKeys = nullptr;
  const void *chunkValues = nullptr;
  const void *queries = nullptr;
  void *workspace = nullptr;
  uint64_t workspaceBytes = 0;
  void *output = nullptr;
  const uint64_t *const *pageTables = nullptr;  // host array of device table addresses
  const uint32_t *treeMasks = nullptr;
};

// runtime/ops/PagedAttention.hpp:199-324 (the KV part of it)
class PagedAttention final {
public:
  static PrefillAttentionPlan prefillPlan(uint32_t rows, uint32_t queryHeads, kv::Layout layout) {
    requireShape(queryHeads, layout);
    if (!rows || rows > kv::kPrefillTokenBudget)
      throw std::invalid_argument("paged prefill attention rows exceed the execution geometry");
    PrefillAttentionPlan plan{layout.format, rows, kvx_prefill_splits(rows), {}, queryHeads, layout.scoreScale};
    const kvx_layout l = layout.c();
    check(kvx_prefill_workspace(rows, queryHeads, &l, &plan.workspace.partialsBytes,
                                &plan.workspace.statisticsBytes));
    return plan;
  }
  // The same with the split count sized for the GPU (kvx_prefill_plan_for): the
  // reference rule gives chunks of 256 rows and more one split, which leaves
  // most of 1024 SIMDs idle until the chunk has about 2048 rows.
  // sequences: how many chunks of this shape one addPrefillBatch call holds (its launches
  // carry every sequence's waves, so a batch often fills the GPU with fewer splits).
  static PrefillAttentionPlan prefillPlan(uint32_t historyTokens, uint32_t rows, uint32_t queryHeads,
                                          kv::Layout layout, uint32_t sequences = 1) {
    PrefillAttentionPlan plan = prefillPlan(rows, queryHeads, layout);
    const kvx_layout l = layout.c();
    plan.splits = kvx_prefill_plan_for(&l, historyTokens, rows, queryHeads, sequences);
    if (!plan.splits) throw std::invalid_argument("paged prefill plan: no sequences");
    check(kvx_prefill_workspace_for(rows, plan.splits, queryHeads, &l, &plan.workspace.partialsBytes,
                                    &plan.workspace.statisticsBytes));
    return plan;
  }
  // decode = true selects the batched-decode split rule of this library
  // (rows = 1 per lane, one split per 32 visible pages).  sizedForGpu = true
  // takes the split counts from kvx_decode_plan_for / kvx_verify_plan, which look at
  // the whole batch and give the launch one round of waves, instead of the
  // reference's per-lane rules.
  static VerifyAttentionPlan verifyPlan(uint32_t lanes, uint32_t queryHeads, kv::Layout layout,
                                        const std::vector<uint32_t> &historyTokens, bool tree = false,
                                        bool decode = false, bool sizedForGpu = false) {
    requireShape(queryHeads, layout);
    if (!lanes || historyTokens.size() != lanes)
      throw std::invalid_argument("paged verify attention needs one history per lane");
    if (tree && layout.format == kv::Format::Float8E4M3)
      throw std::invalid_argument("fp8 KV has no tree verify");
    const uint32_t rows = decode ? 1 : tree ? kv::kTreeVerifyNodes : kv::kVerifyRows;
    VerifyAttentionPlan plan{layout.format, lanes, {}, 0, {}, rows, queryHeads, layout.scoreScale};
    if (sizedForGpu) {
      plan.laneSplits.resize(lanes);
      const kvx_layout l = layout.c();
      check(decode ? kvx_decode_plan_for(&l, historyTokens.data(), lanes, plan.laneSplits.data())
                   : kvx_verify_plan(historyTokens.data(), lanes, rows, layout.kvHeads, queryHeads,
                                     static_cast<uint32_t>(layout.format), plan.laneSplits.data()));
      for (uint32_t splits : plan.laneSplits) plan.splits = std::max(plan.splits, splits);
    } else {
      for (uint32_t history : historyTokens) {
        const uint32_t splits = decode ? kvx_decode_splits(history, 1) : kvx_verify_splits(history, rows);
        plan.laneSplits.push_back(splits);
        plan.splits = std::max(plan.splits, splits);
      }
    }
    const uint32_t group = queryHeads / layout.kvHeads;
    uint64_t fusedRows = 0;
    for (uint32_t splits : plan.laneSplits) fusedRows += uint64_t{splits} * layout.kvHeads * rows * group;
    plan.workspace.partialsBytes = fusedRows * layout.headDimension * sizeof(float);
    plan.workspace.statisticsBytes = fusedRows * 2 * sizeof(float);
    return plan;
  }
  static AttentionWorkspace prefillWorkspace(uint32_t maximumRows, uint32_t queryHeads, kv::Layout layout) {
    AttentionWorkspace w;
    const kvx_layout l = layout.c();
    check(kvx_prefill_workspace_bound(maximumRows, queryHeads, &l, &w.partialsBytes, &w.statisticsBytes));
    return w;
  }
  static AttentionWorkspace verifyWorkspace(uint32_t lanes, uint32_t queryHeads, kv::Layout layout,
                                            uint32_t rowCapacity = kv::kVerifyRows) {
    AttentionWorkspace w;
    const kvx_layout l = layout.c();
    check(kvx_verify_workspace(lanes, rowCapacity, queryHeads, &l, &w.partialsBytes, &w.statisticsBytes));
    return w;
  }

  static kv::ChunkedPrefillParams prefillParams(uint64_t logicalPosition, uint32_t chunkTokens,
                                                uint32_t chunkStride, uint32_t pageTableEntries) {
    const kv::ChunkedPrefillParams p{static_cast<uint32_t>(logicalPosition), chunkTokens, chunkStride,
                                     pageTableEntries, {}};
    if (logicalPosition > UINT32_MAX || kvx_chunk_validation(&p))
      throw std::invalid_argument(std::string("chunked prefill parameters: ") +
                                  (logicalPosition > UINT32_MAX ? "context_out_of_range"
                                                                : kv::chunkedPrefillValidationError(p)));
    return p;
  }
  static kv::ChunkedPrefillParams verifyParams(uint64_t logicalPosition, uint32_t pageTableEntries,
                                               uint32_t rows = kv::kVerifyRows) {
    return prefillParams(logicalPosition, rows, kv::kVerifyChunkStride, pageTableEntries);
  }
  // The reference stores 15 live tree rows (PagedAttention.cpp:418-422); up to
  // 16 are accepted here.
  static kv::ChunkedPrefillParams verifyTreeParams(uint64_t logicalPosition, uint32_t pageTableEntries,
                                                   uint32_t rows = kv::kTreeVerifyNodes - 1) {
    return prefillParams(logicalPosition, rows, kv::kVerifyChunkStride, pageTableEntries);
  }

  static void addPrefillStore(void *stream, const kv::PageStorage &storage, uint32_t layer,
                              const void *chunkKeys, const void *chunkValues, const uint64_t *pageTable,
                              const kv::ChunkedPrefillParams &params) {
    const uint64_t *tables[1] = {pageTable};
    check(kv_append(storage.handle(), layer, chunkKeys, chunkValues, tables, &params, 1, 0, 0, stream));
  }
  // addPrefillQkv / addVerifyQkv followed by the store (runtime/ops/PagedAttention.cpp:299-320,
  // 351-371, then 424-440 / 467-500) as one dispatch: norms, rotation and layout of the packed
  // projection rows, queries out, keys and values quantized straight into their page slots.
  // `rows` rows per lane lie in packed / ropeCos / ropeSin; each lane's chunk_tokens of them are
  // live.  Norm weights: both null (none), bf16, or float with normsAreFloat (the reference's
  // NormWeights of a GGUF's F32 norms).
  struct QkvBuffers final {
    const void *packed = nullptr;
    const void *queryNorm = nullptr;
    const void *keyNorm = nullptr;
    bool normsAreFloat = false;
    const float *ropeCos = nullptr;
    const float *ropeSin = nullptr;
    void *queries = nullptr;
    const uint64_t *const *pageTables = nullptr;
  };
  static void addQkvStore(void *stream, const kv::PageStorage &storage, uint32_t layer,
                          const QkvBuffers &buffers, const std::vector<kv::ChunkedPrefillParams> &chunks,
                          uint32_t queryHeads, uint32_t rows, uint32_t rowStride, uint32_t rotaryPairs,
                          bool queryGate, float eps = 0.0f, uint32_t verifyMaxRows = 0) {
    if ((buffers.queryNorm == nullptr) != (buffers.keyNorm == nullptr))
      throw std::invalid_argument("query and key norms come together");
    const kvx_qkv_shape shape{queryHeads, rotaryPairs, queryGate ? 1u : 0u,
                              !buffers.queryNorm ? 0u : buffers.normsAreFloat ? 2u : 1u, eps};
    check(kv_prepare_append(storage.handle(), layer, &shape, buffers.packed, buffers.queryNorm,
                            buffers.keyNorm, buffers.ropeCos, buffers.ropeSin, buffers.queries, rowStride,
                            buffers.pageTables, chunks.data(), static_cast<uint32_t>(chunks.size()), rows,
                            verifyMaxRows, stream));
  }
  static void addPrefill(void *stream, const kv::PageStorage &storage, uint32_t layer, const void *queries,
                         void *output, void *workspace, uint64_t workspaceBytes, const uint64_t *pageTable,
                         const kv::ChunkedPrefillParams &chunk, const PrefillAttentionPlan &plan) {
    const kv::PrefillAttentionParams p{chunk.committed_tokens, chunk.chunk_tokens, chunk.chunk_stride,
                                       chunk.page_table_entries, {}, plan.splits, plan.scoreScale};
    check(kv_attend_prefill(storage.handle(), layer, plan.queryHeads, queries, output, pageTable, &p,
                            workspace, workspaceBytes, stream));
  }
  // The chunks of several sequences in one call (no counterpart in the reference, whose
  // addPrefill takes one sequence): sequence q's queries and rows lie q x sequenceStride
  // elements after the first's; chunks of one shape share their launches.
  static void addPrefillBatch(void *stream, const kv::PageStorage &storage, uint32_t layer,
                              const void *queries, void *output, void *workspace, uint64_t workspaceBytes,
                              const uint64_t *const *pageTables,
                              const std::vector<kv::ChunkedPrefillParams> &chunks, uint64_t sequenceStride,
                              const PrefillAttentionPlan &plan) {
    std::vector<kv::PrefillAttentionParams> params;
    for (const kv::ChunkedPrefillParams &chunk : chunks)
      params.push_back({chunk.committed_tokens, chunk.chunk_tokens, chunk.chunk_stride,
                        chunk.page_table_entries, {}, plan.splits, plan.scoreScale});
    check(kv_attend_prefill_batch(storage.handle(), layer, plan.queryHeads, queries, output, pageTables,
                                  params.data(), static_cast<uint32_t>(params.size()), sequenceStride,
                                  workspace, workspaceBytes, stream));
  }
  // Stores each lane's chunk and attends its rows with the plan's split counts.
  // With gateHidden the merge also writes the out-projection's operand
  // ([lane][row capacity][query head][D]): scaled by the sigmoid of the gates in
  // gatePacked, the lanes' packed projection rows, or plainly gathered when
  // gatePacked is null, which the reference has for chain plans only
  // (ops::PagedAttention::addVerify, runtime/ops/PagedAttention.cpp:514-541).
  static void addVerify(void *stream, const kv::PageStorage &storage, uint32_t layer,
                        const PagedVerifyBuffers &buffers,
                        const std::vector<kv::ChunkedPrefillParams> &chunks, const VerifyAttentionPlan &plan,
                        const void *gatePacked = nullptr, void *gateHidden = nullptr) {
    if (chunks.size() != plan.lanes) throw std::invalid_argument("one chunk per plan lane");
    if (gateHidden && !gatePacked && buffers.treeMasks)
      throw std::invalid_argument("tree verify has no fused gather");
    const kv::Layout &layout = storage.layout();
    const uint64_t laneStride = uint64_t{layout.kvHeads} * kv::kVerifyChunkStride * layout.headDimension;
    if (plan.rowCapacity == 1) {  // a decode step: one call stores the token and attends
      std::vector<kv::VerifyAttentionParams> lanes(plan.lanes);
      for (uint32_t i = 0; i < plan.lanes; ++i) {
        if (chunks[i].chunk_tokens != 1 || chunks[i].chunk_stride != kv::kVerifyChunkStride)
          throw std::invalid_argument("a decode lane stores one token in a 32-token chunk");
        lanes[i] = {chunks[i].committed_tokens, chunks[i].page_table_entries, {}, plan.laneSplits[i],
                    plan.splits, 1, 1, plan.scoreScale};
      }
      if (gateHidden)
        check(kv_append_attend_decode_hidden(storage.handle(), layer, buffers.chunkKeys, buffers.chunkValues,
                                             laneStride, kv::kVerifyChunkStride, plan.queryHeads,
                                             buffers.queries, buffers.output, buffers.pageTables,
                                             lanes.data(), plan.lanes, 1, buffers.workspace,
                                             buffers.workspaceBytes, gatePacked, gateHidden, stream));
      else
        check(kv_append_attend_decode(storage.handle(), layer, buffers.chunkKeys, buffers.chunkValues,
                                      laneStride, kv::kVerifyChunkStride, plan.queryHeads, buffers.queries,
                                      buffers.output, buffers.pageTables, lanes.data(), plan.lanes, 1,
                                      buffers.workspace, buffers.workspaceBytes, stream));
      return;
    }
    check(kv_append(storage.handle(), layer, buffers.chunkKeys, buffers.chunkValues, buffers.pageTables,
                    chunks.data(), plan.lanes, laneStride, kv::kTreeVerifyNodes, stream));
    attend(stream, storage, layer, buffers, chunks, plan, gatePacked, gateHidden);
  }
  // The attention half of addVerify alone (rows already stored); decode plans
  // take the bandwidth-tuned one-row kernels with rows packed (row stride 1).
  static void attend(void *stream, const kv::PageStorage &storage, uint32_t layer,
                     const PagedVerifyBuffers &buffers, const std::vector<kv::ChunkedPrefillParams> &chunks,
                     const VerifyAttentionPlan &plan, const void *gatePacked = nullptr,
                     void *gateHidden = nullptr) {
    std::vector<kv::VerifyAttentionParams> lanes(plan.lanes);
    for (uint32_t i = 0; i < plan.lanes; ++i)
      lanes[i] = {chunks[i].committed_tokens, chunks[i].page_table_entries, {}, plan.laneSplits[i],
                  plan.splits, chunks[i].chunk_tokens, plan.rowCapacity, plan.scoreScale};
    if (gateHidden)
      check(kv_attend_verify_hidden(storage.handle(), layer, plan.queryHeads, buffers.queries,
                                    buffers.output, buffers.pageTables, lanes.data(), plan.lanes,
                                    buffers.treeMasks, plan.rowCapacity == 1 ? 1 : kv::kVerifyChunkStride,
                                    buffers.workspace, buffers.workspaceBytes, gatePacked, gateHidden,
                                    stream));
    else if (plan.rowCapacity == 1)
      check(kv_attend_decode(storage.handle(), layer, plan.queryHeads, buffers.queries, buffers.output,
                             buffers.pageTables, lanes.data(), plan.lanes, 1, buffers.workspace,
                             buffers.workspaceBytes, stream));
    else
      check(kv_attend_verify(storage.handle(), layer, plan.queryHeads, buffers.queries, buffers.output,
                             buffers.pageTables, lanes.data(), plan.lanes, buffers.treeMasks,
                             kv::kVerifyChunkStride, buffers.workspace, buffers.workspaceBytes, stream));
  }
  // attend() of a decode plan for callers that cannot bring a workspace or allocate one (graph
  // capture, tight serving loops): partial rows go to the library's static device array
  // (kv_attend_decode_static, at most KVX_STATIC_WORKSPACE_BYTES; no counterpart in the
  // reference).  Calls that overlap on one GPU race on that array.
  static void attendStatic(void *stream, const kv::PageStorage &storage, uint32_t layer,
                           const PagedVerifyBuffers &buffers,
                           const std::vector<kv::ChunkedPrefillParams> &chunks,
                           const VerifyAttentionPlan &plan) {
    if (plan.rowCapacity != 1 || chunks.size() != plan.lanes)
      throw std::invalid_argument("the static workspace serves decode plans, one chunk per lane");
    std::vector<kv::VerifyAttentionParams> lanes(plan.lanes);
    for (uint32_t i = 0; i < plan.lanes; ++i)
      lanes[i] = {chunks[i].committed_tokens, chunks[i].page_table_entries, {}, plan.laneSplits[i],
                  plan.splits, 1, 1, plan.scoreScale};
    check(kv_attend_decode_static(storage.handle(), layer, plan.queryHeads, buffers.queries,
                                  buffers.output, buffers.pageTables, lanes.data(), plan.lanes, 1, stream));
  }
  // One-row decode of up to 16 lanes whose page tables begin with the same sharedPages pages:
  // those pages are attended once for all of them (no counterpart in the reference, which lists
  // the case as a gap, docs/PERF_REPORT.md:250).  plan: a decode plan over the lanes' own tokens
  // (history minus the shared tokens); prefixSplits: the verify plan of one lane of plan.lanes
  // rows over the shared tokens.
  static void attendShared(void *stream, const kv::PageStorage &storage, uint32_t layer,
                           const PagedVerifyBuffers &buffers, const std::vector<kv::ChunkedPrefillParams> &chunks,
                           const VerifyAttentionPlan &plan, uint32_t sharedPages, uint32_t prefixSplits) {
    if (plan.rowCapacity != 1 || chunks.size() != plan.lanes)
      throw std::invalid_argument("shared-prefix attention takes a decode plan, one chunk per lane");
    std::vector<kv::VerifyAttentionParams> lanes(plan.lanes);
    for (uint32_t i = 0; i < plan.lanes; ++i)
      lanes[i] = {chunks[i].committed_tokens, chunks[i].page_table_entries, {}, plan.laneSplits[i],
                  plan.splits, 1, 1, plan.scoreScale};
    check(kv_attend_decode_shared(storage.handle(), layer, plan.queryHeads, buffers.queries, buffers.output,
                                  buffers.pageTables, lanes.data(), plan.lanes, sharedPages, prefixSplits, 1,
                                  buffers.workspace, buffers.workspaceBytes, stream));
  }
  static void addVerifyTreeCompact(void *stream, const kv::PageStorage &storage, uint32_t layer,
                                   const uint64_t *const *pageTables, const uint32_t *retainedPath,
                                   const uint32_t *retained,
                                   const std::vector<kv::ChunkedPrefillParams> &chunks, uint32_t lanes,
                                   uint32_t pathStride = 8) {
    if (chunks.size() < lanes) throw std::invalid_argument("one chunk per lane");
    check(kv_compact_path(storage.handle(), layer, pageTables, chunks.data(), lanes, retainedPath, retained,
                          pathStride, stream));
  }

private:
  static void requireShape(uint32_t queryHeads, const kv::Layout &layout) {
    if (!layout.valid() || !queryHeads || queryHeads % layout.kvHeads)
      throw std::invalid_argument("paged attention needs a valid layout and whole query groups");
  }
};

}  // namespace ops
}  // namespace kvx
