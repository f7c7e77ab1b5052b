/*
 * kvx.h -- C ABI of the MI355X-native paged KV-cache path.
 *
 * A drop-in for RichEngine's KV data plane: page storage in extents, page
 * tables of extent-address|index entries, quantize-on-append, paged
 * gather-dequant attention (decode / speculative verify / chunked prefill) with
 * split partials and a fixed-order merge, tree-path compaction and whole-page
 * copy, plus the page pool that owns page references.  The page format is the
 * reference's, byte for byte.  Every entry point cites the reference interface
 * it replaces (paths relative to the reference checkout).
 *
 * Conventions
 *  - Plain pointers and sizes only.  `stream` is a hipStream_t passed as void*
 *    (NULL = the default stream).  Work is enqueued on it and not waited for.
 *  - Device pointers are caller-owned HBM; the library owns extents only and
 *    allocates nothing on the launch path.
 *  - Status codes replace the reference's exceptions; nothing is enqueued when
 *    a call fails.  kvx_last_error() gives the message of the calling thread's
 *    last failure.
 *  - Lanes whose parameters fail the kernel contract write nothing (as the
 *    reference kernels do); host-side validation reports them first.
 *  - One caller thread per storage/pool (as the reference's engine thread) for
 *    what changes them: extents, pool, prefix cache, sequence records.  The kv_*
 *    entries only read the storage's description and keep nothing between
 *    calls, so several threads may call them at once over one storage, each on
 *    a stream and a workspace of its own.
 */
#ifndef KVX_H
#define KVX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status: the reference's exception classes as values ---- */
#define KVX_OK 0
#define KVX_EINVAL (-1)  /* std::invalid_argument: bad geometry / parameters  */
#define KVX_ESTATE (-2)  /* std::logic_error: lifecycle misuse                */
#define KVX_ENOMEM (-3)  /* allocation refused (metal::AllocationResult)      */
#define KVX_ERANGE (-4)  /* std::out_of_range: page / extent id past the pool */
#define KVX_EDEVICE (-5) /* a HIP call failed                                 */
const char *kvx_last_error(void);

/* ---- formats and limits ---- */
/* runtime/ops/PagedKv.hpp:16 (kv::Format), same values */
#define KVX_FMT_INT8 1u
#define KVX_FMT_BF16 2u
#define KVX_FMT_INT4 3u
#define KVX_FMT_FP8E4M3 4u
/* runtime/metal/abi/KvExtent.h:27-30 */
#define KVX_KEYS 0u
#define KVX_KEY_SCALES 1u
#define KVX_VALUES 2u
#define KVX_VALUE_SCALES 3u
/* runtime/metal/abi/ExecutionGeometry.h:7-39, abi/KvExtent.h:19 */
#define KVX_PAGE_TOKENS 32u
#define KVX_PAGE_INDEX_BITS 14u
#define KVX_PAGE_INDEX_MASK ((1u << KVX_PAGE_INDEX_BITS) - 1u)
#define KVX_VERIFY_ROWS 8u
#define KVX_TREE_NODES 16u
#define KVX_MAX_CONTEXT_TOKENS 262144u
#define KVX_MAX_PHYSICAL_TOKENS (KVX_MAX_CONTEXT_TOKENS + KVX_TREE_NODES - 1u)
#define KVX_PREFILL_TOKEN_BUDGET 2048u
#define KVX_PREFILL_TILE_ROWS 8u
#define KVX_PREFILL_MAX_SPLITS 32u
#define KVX_VERIFY_MAX_SPLITS 128u
#define KVX_VERIFY_CHUNK_STRIDE 32u
/* The reference batches at most 4 lanes (abi/ExecutionGeometry.h:22); this
   library takes any lane count and launches in groups of KVX_LANES_PER_LAUNCH. */
#define KVX_LANES_PER_LAUNCH 32u

/* runtime/ops/PagedKv.hpp:125-136 (kv::Layout) */
typedef struct kvx_layout {
  uint32_t layers;
  uint32_t kv_heads;
  uint32_t head_dim;
  uint32_t format;
  float score_scale; /* 0 selects 1/sqrt(head_dim) */
} kvx_layout;

/* runtime/metal/abi/KvExtent.h:93-96 (RichKvLayer) */
typedef struct kvx_kv_layer {
  uint32_t extent_pages;
  uint32_t offset;
} kvx_kv_layer;

/* runtime/metal/abi/PagedAttention.h:39-45 (RichChunkedPrefillParams, 24 B) */
typedef struct kvx_chunk_params {
  uint32_t committed_tokens;
  uint32_t chunk_tokens;
  uint32_t chunk_stride;
  uint32_t page_table_entries;
  kvx_kv_layer kv; /* filled by the library from `layer` */
} kvx_chunk_params;

/* runtime/metal/abi/PagedAttention.h:52-61 (RichPrefillAttentionParams, 32 B) */
typedef struct kvx_prefill_params {
  uint32_t committed_tokens;
  uint32_t rows;
  uint32_t chunk_stride;
  uint32_t page_table_entries;
  kvx_kv_layer kv;
  uint32_t split_count;
  float score_scale;
} kvx_prefill_params;

/* runtime/metal/abi/PagedAttention.h:72-84 (RichVerifyAttentionParams, 36 B) */
typedef struct kvx_verify_params {
  uint32_t committed_tokens;
  uint32_t page_table_entries;
  kvx_kv_layer kv;
  uint32_t split_count;
  uint32_t slot_splits;
  uint32_t active_rows;
  uint32_t row_capacity;
  float score_scale;
} kvx_verify_params;

/* runtime/ops/PagedKv.hpp:48-51 (kv::PageCopy) */
typedef struct kvx_page_copy {
  uint32_t from;
  uint32_t to;
} kvx_page_copy;

/* ---- layout geometry: kv::Layout members, runtime/ops/PagedKv.hpp:137-230 ---- */
int kvx_layout_valid(const kvx_layout *layout);
uint64_t kvx_layout_data_bytes_per_layer_page(const kvx_layout *layout);
uint64_t kvx_layout_scale_bytes_per_layer_page(const kvx_layout *layout);
uint64_t kvx_layout_bytes_per_layer_page(const kvx_layout *layout);
uint64_t kvx_layout_bytes_per_model_page(const kvx_layout *layout);
uint32_t kvx_layout_extent_alignment_pages(const kvx_layout *layout);
uint32_t kvx_layout_minimum_extent_pages(const kvx_layout *layout);
uint32_t kvx_layout_maximum_extent_pages(const kvx_layout *layout);
uint32_t kvx_layout_extent_pages_for(const kvx_layout *layout, uint64_t pages);
/* The largest extent the page entry and the 32-bit layer offset allow: whole
   alignment units, at most 16383 pages, below 4 GiB.  MI355X pools want few,
   large extents (fewer allocations, better TLB reach); the reference's 128 MiB
   target (extent_pages_for) stays available for parity. */
uint32_t kvx_layout_largest_extent_pages(const kvx_layout *layout);
/* runtime/metal/abi/KvExtent.h:76-89 (richengine_kv_offset) */
uint64_t kvx_kv_offset(uint32_t extent_pages, uint32_t data_bytes, uint32_t scale_bytes,
                       uint32_t layer, uint32_t tensor, uint32_t index);

/* ---- planning: runtime/ops/PagedAttention.hpp:54-95, PagedAttention.cpp:23-32,200-297 ---- */
/* kv::verifyAttentionSplits: clamp(ceil(pages/16), 32, 128) */
uint32_t kvx_verify_splits(uint32_t committed_tokens, uint32_t rows);
/* prefillSplits: clamp(32 / tiles, 1, 32) with tiles = ceil(rows / 8) */
uint32_t kvx_prefill_splits(uint32_t rows);
/* The batched-decode rule of this library: one split per
   KVX_DECODE_PAGES_PER_SPLIT visible pages, at least 1, at most 128.  Decode at
   batch 32 has enough (lane, head) parallelism that the reference's 32-split
   floor would only add partial traffic. */
#define KVX_DECODE_PAGES_PER_SPLIT 32u
uint32_t kvx_decode_splits(uint32_t committed_tokens, uint32_t rows);
/* The split counts of a whole decode batch of pages of `format`, planned launch by launch: the
   attend calls take the lanes KVX_LANES_PER_LAUNCH at a time in the caller's order, and every
   such group is planned to fill the GPU by itself.  A launch runs (sum of splits) x
   KV heads waves; the plan is a split length in pages, each lane getting
   clamp(ceil(its pages / that), 1, KVX_DECODE_MAX_SPLITS) splits.  The length starts at
   max(ceil(the launch's page-heads / 1024), 8) (at most 32 for int4, whose kernel holds two waves per
   SIMD and is fastest at 32; at least 4 instead of 8 for a launch of at most 4096 page-heads
   on int4 pages, 2048 on the others, whose longest lane has at most 512 pages: splits of 8
   pages would leave most SIMDs of such a launch empty),
   which fills the GPU when the batch is small, and grows until the
   launch has no more waves than the kernel has wave slots (2048 for int4, 1024 for the other
   formats), because waves beyond that run as a second round on a nearly empty GPU.  An int4
   batch of at most KVX_LANES_PER_LAUNCH lanes that needs two waves on most SIMDs is planned in
   two classes instead, because the two waves of a SIMD do not share it evenly: lanes from the
   longest down get splits of one length while their waves fit one per SIMD (1024), the other
   lanes splits of 0.58 of that length, and the length is the least for which the second class
   fits 1024 waves too; kv_attend_decode dispatches the lanes with the longest splits first, so
   the long splits take the first wave of every SIMD and both classes end together.  One-row
   decode lanes may use up to KVX_DECODE_MAX_SPLITS splits; every other attend entry keeps the
   reference's KVX_VERIFY_MAX_SPLITS.  KVX_EINVAL for a null argument, no lanes, no KV heads or a
   lane whose context (committed + 1) is beyond KVX_MAX_PHYSICAL_TOKENS.  No counterpart in the
   reference, whose decode shares the verify plan (runtime/ops/PagedAttention.cpp:232-262). */
#define KVX_DECODE_MAX_SPLITS 512u
int kvx_decode_plan(const uint32_t *committed_tokens, uint32_t n_lanes, uint32_t kv_heads,
                    uint32_t format, uint32_t *split_counts);
/* kvx_prefill_plan_batch by layout: head dimension 256 is that plan; at head dimensions 64 and
   128 (runtime/ops/PagedAttention.cpp:66-115), whose tiles run a workgroup each, or one for the
   four or two tiles that begin in the same page of a chunk on a page-aligned history, the fewest
   splits that make 4096 workgroups, none shorter than 4 pages, at most KVX_PREFILL_MAX_SPLITS.
   0 for an invalid layout, bad head counts or no sequences. */
uint32_t kvx_prefill_plan_for(const kvx_layout *layout, uint32_t committed_tokens, uint32_t rows,
                              uint32_t query_heads, uint32_t n_sequences);
/* The same by layout: head dimension 256 is kvx_decode_plan; head dimensions 64 and 128 (the
   reference's other layouts, runtime/ops/PagedAttention.cpp:66-115), whose one-row tiles run a
   wave each over a staged copy of their own, get the split length (at least 4 pages) that makes
   one round of those waves, 4096 (2048 at head dimension 128 over pages other than int4; half as
   many over bf16 pages), launch by launch, at most KVX_VERIFY_MAX_SPLITS per lane.  Same errors, and KVX_EINVAL
   for an invalid layout. */
int kvx_decode_plan_for(const kvx_layout *layout, const uint32_t *committed_tokens, uint32_t n_lanes,
                        uint32_t *split_counts);
/* Split counts of a verify batch (`rows` live rows per lane) sized for this GPU instead of
   the reference's clamp(ceil(pages/16), 32, 128), launch by launch like kvx_decode_plan: the
   longest split length (at least 8 pages; 4 in a launch of at most 2048 page-waves whose
   longest lane has at most 512 pages)
   for which the launch has no more waves than the GPU has SIMDs (1024; 2048 for int4 lanes of
   more than 32 fused rows in blocks of 32 from 16 lanes on, whose kernel holds two waves per
   SIMD), each lane getting
   clamp(ceil(its pages / that), 1, KVX_VERIFY_MAX_SPLITS).  A launch runs (sum of splits) x
   KV heads x ceil(rows x group / 32) waves, one per SIMD; on int4 pages ceil(rows x group / 48)
   where that is fewer by more than 1.74 (33 .. 48 fused rows among others).  No counterpart in the reference
   (its rule is kvx_verify_splits); any split count either rule gives is valid for
   kv_attend_verify.  KVX_EINVAL for a null argument, no lanes, bad head counts or a lane whose
   context (committed + rows) is beyond KVX_MAX_PHYSICAL_TOKENS. */
int kvx_verify_plan(const uint32_t *committed_tokens, uint32_t n_lanes, uint32_t rows,
                    uint32_t kv_heads, uint32_t query_heads, uint32_t format,
                    uint32_t *split_counts);
/* kv::chunkedPrefillValidationError: 0 ok, 1 chunk_tokens_out_of_range,
   2 context_out_of_range, 3 chunk_stride_invalid, 4 page_table_too_short */
int kvx_chunk_validation(const kvx_chunk_params *params);
/* Split count of one sequence's chunked prefill sized for this GPU instead of the reference's
   clamp(32 / tiles, 1, 32).  That rule gives chunks of 256 rows and more a single split, which
   is one wave per (pair of tiles, KV head, block of 32 fused rows): 192 waves for 256 rows of
   24 query heads on 4 KV heads, on a GPU with 1024 SIMDs, each walking the whole context
   alone.  The plan keeps one split while those waves fill at least half of the kernel's wave
   slots and otherwise takes the largest count (at most 32, at least 8 pages per split) whose
   launch still fits one round of slots: of the paired tiles' waves where the two tiles of
   every pair see the same number of pages (a pair is 16 rows of 32-token pages, and its two
   8-row tiles end in the same page exactly when committed_tokens mod 16 is 0 or at least 9:
   then the first tile's last row and the second tile's last row, 8 tokens later, do not
   straddle a page boundary; so every page-aligned chunk start; int4 pages: from 512 rows on), else of tiles x splits x KV heads x ceil(8 x group / 16)
   waves of single tiles.  int4 pages, chunks whose paired waves fill a quarter of the 2048
   slots or more (from 683 rows of 24 query heads on 4 KV heads): the waves of a launch
   are equally long and take the slots round by round, so the plan takes the fewest splits
   (of at least 16 pages of the average tile's history each) that leave every round at least
   nine tenths full, or failing that the fullest rounds: 4 for 2048 rows (1536 waves per
   split) once 2048 tokens are committed, 5 for 1024 rows, 1 where there is no history to cut.  bf16, fp8 and int8 pages, chunks of 64 rows and more (lanes of four tiles of
   8 x group <= 48 fused rows, or two of <= 96, one workgroup per lane, split and KV head, one
   workgroup per CU): one split where those workgroups fill three quarters of the 256 CUs, else
   the count (same bounds) that fills them, where the chunk starts on a page boundary (lanes
   of two tiles: where the tiles pair); other starts fall under the rules above.
   Returns 0 for bad head counts.  No counterpart in the reference (its rule is
   kvx_prefill_splits); any count in 1..32 is valid for kv_attend_prefill. */
uint32_t kvx_prefill_plan(uint32_t committed_tokens, uint32_t rows, uint32_t kv_heads,
                          uint32_t query_heads, uint32_t format);
/* The same for n_sequences chunks of this shape in one kv_attend_prefill_batch call, whose
   launches hold every sequence's waves (four chunks of 2048 rows: 6144 waves, three full
   rounds in one split each).  n_sequences = 1 is kvx_prefill_plan; 0 returns 0. */
uint32_t kvx_prefill_plan_batch(uint32_t committed_tokens, uint32_t rows, uint32_t kv_heads,
                                uint32_t query_heads, uint32_t format, uint32_t n_sequences);
/* ops::PagedAttention::prefillPlan(...).workspace / prefillWorkspace / verifyWorkspace.
   Bytes of partials and statistics; a workspace buffer holds partials first,
   then statistics at the next 256-byte boundary. */
int kvx_prefill_workspace(uint32_t rows, uint32_t query_heads, const kvx_layout *layout,
                          uint64_t *partials_bytes, uint64_t *statistics_bytes);
/* The same for a given split count (kvx_prefill_plan's, or any in 1..32). */
int kvx_prefill_workspace_for(uint32_t rows, uint32_t split_count, uint32_t query_heads,
                              const kvx_layout *layout, uint64_t *partials_bytes,
                              uint64_t *statistics_bytes);
int kvx_prefill_workspace_bound(uint32_t maximum_rows, uint32_t query_heads,
                                const kvx_layout *layout, uint64_t *partials_bytes,
                                uint64_t *statistics_bytes);
int kvx_verify_workspace(uint32_t lanes, uint32_t row_capacity, uint32_t query_heads,
                         const kvx_layout *layout, uint64_t *partials_bytes,
                         uint64_t *statistics_bytes);
/* Total bytes of one workspace buffer for an attend call over these lanes
   (sum over lanes of split_count * kv_heads * row_capacity * group fused rows). */
uint64_t kvx_attend_workspace_bytes(const kvx_verify_params *lanes, uint32_t n_lanes,
                                    uint32_t query_heads, const kvx_layout *layout);

/* ---- page storage: kv::PageStorage / kv::ExtentStorage,
        runtime/ops/PageStorage.hpp:27-102, runtime/ops/PagedKv.hpp:56-76 ---- */
typedef struct kvx_storage kvx_storage;
/* PageStorage::PageStorage (PageStorage.mm:12-46).  aligned != 0 enforces whole
   alignment units per extent as production does; 0 takes any extent size the
   page index allows (dev/tuning/HostKvExtents.hpp:158-169, test pools).  KVX_EINVAL beyond the
   reference's own checks: head dimensions other than 64 / 128 / 256, more than 4096 KV heads or
   65536 layers (the kernels index a page's bytes in 32 bits), more than 1048576 extents. */
int kvx_storage_create(const kvx_layout *layout, uint32_t page_count, uint32_t extent_pages,
                       int aligned, kvx_storage **out);
/* Storage with no memory behind its extents, for the page bookkeeping alone (pool,
   prefix cache, sequences): the counterpart of the reference's deterministic test
   storage (test::TestKvStorage, dev/tests/engine/TestKvPool.hpp).  Needs no GPU.  Allocation, release,
   budget and kv_page_copy validation behave as usual; page and extent reads/writes, table
   uploads and every hot-path entry answer KVX_ESTATE. */
int kvx_storage_create_accounting(const kvx_layout *layout, uint32_t page_count,
                                  uint32_t extent_pages, int aligned, kvx_storage **out);
void kvx_storage_destroy(kvx_storage *storage);
uint32_t kvx_storage_page_count(const kvx_storage *storage);
uint32_t kvx_storage_extent_pages(const kvx_storage *storage);
uint64_t kvx_storage_bytes_per_page(const kvx_storage *storage);
uint64_t kvx_storage_extent_bytes(const kvx_storage *storage);
uint64_t kvx_storage_allocated_bytes(const kvx_storage *storage);
int kvx_storage_is_allocated(const kvx_storage *storage, uint32_t page);
/* ExtentStorage::allocateExtent / releaseExtent (PageStorage.mm:64-93).
   KVX_ENOMEM when hipMalloc refuses; KVX_ESTATE for an (un)allocated extent.
   A new extent is zero-filled.  Release synchronises the device first. */
int kvx_storage_allocate_extent(kvx_storage *storage, uint32_t extent);
int kvx_storage_release_extent(kvx_storage *storage, uint32_t extent);
/* A budget in bytes past which allocate_extent answers KVX_ENOMEM (the
   reference's admission callback, runtime/metal/MetalBackend.hpp:18-45); 0 = none. */
void kvx_storage_set_budget(kvx_storage *storage, uint64_t bytes);
/* PageStorage::layers()[layer] */
int kvx_storage_layer(const kvx_storage *storage, uint32_t layer, kvx_kv_layer *out);
/* PageStorage::writeEntries (PageStorage.mm:127-141): entries [first, n) of the
   pages' table.  The first form fills a host array; the second copies them to
   a device table on `stream` (entries before `first` are left as they are). */
int kvx_storage_entries(const kvx_storage *storage, const uint32_t *pages, uint32_t n,
                        uint32_t first, uint64_t *table_host);
int kvx_storage_write_entries(const kvx_storage *storage, const uint32_t *pages, uint32_t n,
                              uint32_t first, uint64_t *table_device, uint64_t table_capacity,
                              void *stream);
/* PageStorage::spans (PageStorage.mm:143-167) for memory the host cannot map:
   the page's bytes, layer by layer as keys, key scales, values, value scales
   (bytes_per_page long), copied to / from host memory.  Synchronous. */
int kvx_storage_page_read(const kvx_storage *storage, uint32_t page, void *host_bytes);
int kvx_storage_page_write(kvx_storage *storage, uint32_t page, const void *host_bytes);
/* The same wire form for many pages at once and without a host round trip per span: page i of
   the list occupies bytes [i, i + 1) x bytes_per_page of `buffer`, which is device memory or
   pinned host memory the device can reach (hipHostMalloc), so that a host or disk tier can
   demote and restore pages byte for byte (engine::KvPageTier::demote / restore,
   runtime/engine/cache/KvPageTier.hpp:13-21, which moves PageStorage::spans to and from a slot
   file).  Enqueued on `stream`; nothing is enqueued when a page id is invalid, its extent is not
   allocated, or two imported pages share a destination. */
int kv_page_export(const kvx_storage *storage, const uint32_t *pages, uint32_t n, void *buffer,
                   void *stream);
int kv_page_import(kvx_storage *storage, const uint32_t *pages, uint32_t n, const void *buffer,
                   void *stream);
/* Raw extent bytes, for tests that compare whole extents.  Synchronous. */
int kvx_storage_extent_read(const kvx_storage *storage, uint32_t extent, uint64_t offset,
                            uint64_t bytes, void *host_bytes);
int kvx_storage_extent_write(kvx_storage *storage, uint32_t extent, uint64_t offset,
                             uint64_t bytes, const void *host_bytes);

/* ExtentStorage::copyPages (PageStorage.mm:95-114): every tensor of every layer
   of each page, on `stream`.  All-or-nothing validation first: KVX_ESTATE and no
   copy when any page sits in an unallocated extent, KVX_ERANGE past the pool,
   KVX_EINVAL when a destination is also a source of the batch (the reference
   copies in order on the host; the device copies all pages at once). */
int kv_page_copy(kvx_storage *storage, const kvx_page_copy *copies, uint32_t n, void *stream);

/* ---- page pool: engine::KvPool, runtime/engine/cache/KvPool.hpp:75-115 ---- */
typedef struct kvx_pool kvx_pool;
typedef struct kvx_pool_snapshot { /* KvPool.hpp:12-35 (KvPoolSnapshot) */
  uint32_t pages_allocated, pages_free, pages_active, pages_prefix;
  uint64_t allocated_bytes, reclaimable_bytes;
  uint64_t extent_allocations, extent_releases;
  double extent_allocate_max_ms, extent_release_max_ms;
  uint64_t extent_compactions, pages_moved;
} kvx_pool_snapshot;
/* KvPool::KvPool (KvPool.cpp:14-33): allocates the runway. */
int kvx_pool_create(kvx_storage *storage, uint32_t runway_pages, kvx_pool **out);
void kvx_pool_destroy(kvx_pool *pool);
/* KvPool::acquirePages (KvPool.cpp:35-72): `count` pages with one active
   reference each, or KVX_ENOMEM with no page held (extents allocated on the
   way stay, reclaimable). */
int kvx_pool_acquire(kvx_pool *pool, uint32_t count, uint32_t *pages);
int kvx_pool_retain(kvx_pool *pool, uint32_t page, int prefix_owner);  /* KvPool.cpp:74-91 */
int kvx_pool_release(kvx_pool *pool, uint32_t page, int prefix_owner); /* KvPool.cpp:93-105 */
int kvx_pool_page_active(const kvx_pool *pool, uint32_t page);
uint32_t kvx_pool_free_pages(const kvx_pool *pool);
/* KvPool::reclaimEmptyExtents (KvPool.cpp:125-141): bytes released via *released. */
int kvx_pool_reclaim_empty(kvx_pool *pool, int keep_runway, uint32_t limit, uint64_t *released);
/* KvPool::compactExtent (KvPool.cpp:165-230): empties the sparsest extent into
   the fullest others through kv_page_copy on `stream`.  *moved_pages = 0 when
   nothing moved; otherwise *first_page and destinations[extent_pages] say where
   each page of the emptied extent went (KvPageMoves, KvPool.hpp:39-52).
   The reference copies on the host before it returns; here the copies are only
   enqueued when the call returns, while the emptied extent's pages are already free
   and the receiving pages already held.  Whatever may write a page of the emptied
   extent (an append into a page acquired after this call) or read a receiving page
   must therefore be ordered after `stream` has passed this point: the same stream, or
   an event recorded on it.  kvx_pool_reclaim_empty frees memory with hipFree, which
   waits for the device. */
int kvx_pool_compact_extent(kvx_pool *pool, const uint32_t *fixed, uint32_t n_fixed,
                            uint32_t *first_page, uint32_t *destinations,
                            uint32_t *moved_pages, void *stream);
int kvx_pool_snapshot_get(const kvx_pool *pool, kvx_pool_snapshot *out);

/* ---- prefix page cache: engine::KvCache, resident tier
        (runtime/engine/cache/KvCache.hpp:40-241, KvCache.cpp:66-158, 227-283, 393-409, 480-484,
        515-559).  Blocks are keyed by (parent block, the page's 32 tokens, image identity) and own
        one prefix reference of their page in the pool.  The disk tier, recurrent states and
        poisoning are outside the KV data path and have no counterpart. ---- */
typedef struct kvx_prefix kvx_prefix;
#define KVX_NO_PAGE 0xffffffffu
int kvx_prefix_create(kvx_pool *pool, kvx_prefix **out);
void kvx_prefix_destroy(kvx_prefix *prefix); /* gives every block's page back (KvCache::~KvCache) */
/* KvCache::find: 1 with *block / *page when the exact key exists, else 0.  parent 0 = root. */
int kvx_prefix_find(const kvx_prefix *prefix, uint64_t parent, const uint32_t *tokens,
                    uint32_t n_tokens, uint64_t image_lo, uint64_t image_hi, uint64_t *block,
                    uint32_t *page);
/* KvCache::insert: existing content is returned as it is (*canonical_page may differ from
   `page`).  KVX_EINVAL for a partial page or an unknown parent, KVX_ERANGE for a page past the
   pool, KVX_ESTATE when the page already holds a block. */
int kvx_prefix_insert(kvx_prefix *prefix, uint64_t parent, const uint32_t *tokens,
                      uint32_t n_tokens, uint32_t page, uint64_t image_lo, uint64_t image_hi,
                      uint64_t *block, uint32_t *canonical_page);
int kvx_prefix_contains(const kvx_prefix *prefix, uint64_t block);
uint64_t kvx_prefix_generation(const kvx_prefix *prefix);
uint64_t kvx_prefix_block_count(const kvx_prefix *prefix);
/* KvCache::chain, root first; *length = KvCache::chainLength. */
int kvx_prefix_chain(const kvx_prefix *prefix, uint64_t block, uint64_t *blocks, uint32_t *pages,
                     uint32_t capacity, uint32_t *length);
int kvx_prefix_retain_active(kvx_prefix *prefix, uint64_t block);
int kvx_prefix_release_active(kvx_prefix *prefix, uint64_t block);
int kvx_prefix_touch(kvx_prefix *prefix, uint64_t block);
/* KvCache::evictionCandidate: idle leaves, least recently used first; after = 0 starts the scan.
   1 with *block, or 0 when there is no further candidate. */
int kvx_prefix_eviction_candidate(const kvx_prefix *prefix, uint64_t after, uint64_t *block);
/* KvCache::erase: KVX_ESTATE for a block with children or users. */
int kvx_prefix_erase(kvx_prefix *prefix, uint64_t block);
/* KvCache::followPages: after kvx_pool_compact_extent moved pages. */
void kvx_prefix_follow_pages(kvx_prefix *prefix, uint32_t first_page, const uint32_t *destinations,
                             uint32_t n);
/* Cache::extendMatch (runtime/engine/cache/Cache.cpp:179-199): the chain of cached blocks that
   covers the prompt's leading whole pages, leaving at least one prompt token unmatched.  Returns
   the number of pages looked up.  kvx_prefix_match is the text-only form (every block keyed
   with the zero identity); a prompt with images goes through kvx_prefix_match_images below,
   or two prompts with the same placeholder tokens and different images would share pages. */
uint64_t kvx_prefix_match(const kvx_prefix *prefix, const uint32_t *prompt, uint64_t n_tokens,
                          uint64_t *blocks, uint32_t capacity, uint32_t *matched);

/* engine::blockImageIdentity (runtime/engine/cache/KvCache.hpp:22-32, KvCache.cpp:29-52): the
   128-bit identity that the images overlapping tokens [block_begin, block_begin + block_tokens)
   of a prompt add to that block's key; both halves 0 for a text-only block.  `spans` are the
   prompt's images sorted by offset (model::ImageSpan, runtime/model/Model.hpp:130-138). */
typedef struct kvx_image_span {
  uint32_t offset, tokens;
  uint32_t grid_height, grid_width;
  uint64_t digest_lo, digest_hi;
} kvx_image_span;
void kvx_block_image_identity(uint64_t block_begin, uint32_t block_tokens,
                              const kvx_image_span *spans, uint32_t n_spans, uint64_t *lo,
                              uint64_t *hi);
/* Cache::extendMatch with the prompt's images (Cache.cpp:186-193: spansFrom, then
   blockImageIdentity per block): every block is looked up under the identity of the spans
   that overlap it.  `spans` sorted by offset and disjoint; null or none = kvx_prefix_match. */
uint64_t kvx_prefix_match_images(const kvx_prefix *prefix, const uint32_t *prompt,
                                 uint64_t n_tokens, const kvx_image_span *spans, uint32_t n_spans,
                                 uint64_t *blocks, uint32_t capacity, uint32_t *matched);

/* ---- per-sequence page lists: the Request records of engine::Cache
        (runtime/engine/cache/Cache.cpp:143-166, 284-333, 381-413, 700-731, 748-785) ---- */
typedef struct kvx_sequences kvx_sequences;
typedef struct kvx_sequence_pages { /* Cache::pageTable -> PageTableView, plus the cached blocks */
  const uint32_t *pages;
  uint32_t page_count;
  uint64_t revision;      /* bumped whenever a page id changed */
  uint32_t first_changed; /* first logical page of the latest change */
  const uint64_t *blocks;
  uint32_t block_count;
} kvx_sequence_pages;
int kvx_sequences_create(kvx_pool *pool, kvx_prefix *prefix, kvx_sequences **out);
void kvx_sequences_destroy(kvx_sequences *sequences);
int kvx_sequence_begin(kvx_sequences *sequences, uint64_t id); /* Cache::beginRequest */
int kvx_sequence_end(kvx_sequences *sequences, uint64_t id);   /* Cache::endRequest */
/* Cache::restoreRequest for a resident chain: the sequence takes the chain of `last_block` as its
   first pages (one active reference each) and becomes the block's user. */
int kvx_sequence_restore(kvx_sequences *sequences, uint64_t id, uint64_t last_block);
/* Cache::ensureTokens: pages for `tokens` tokens, or KVX_ENOMEM with nothing taken. */
int kvx_sequence_ensure_tokens(kvx_sequences *sequences, uint64_t id, uint64_t tokens);
/* Copy-on-write sharing of a prefix that does not end on a page boundary.  No counterpart in
   the reference, which shares whole published pages only (Cache.cpp:183-184, :774).
   kvx_sequence_fork: the empty sequence `id` takes the pages that hold the first `tokens`
   tokens of `source` by reference (one more active reference each, the partly filled last
   page included) and the source's blocks over them.
   kvx_sequence_ensure_writable: call before rows are stored at `token` and after.  When
   another sequence or the prefix cache also holds the page of `token`, the sequence gets a
   fresh page, kv_page_copy copies every layer of the shared page into it on `stream`, the
   sequence's list points at the copy (revision / first_changed say so) and its reference to
   the shared page is given back; *copied = 1 with the two page ids.  A page held by nobody
   else is written in place (*copied = 0).  KVX_ESTATE for a published page (its rows are
   final), KVX_EINVAL when the sequence holds no page for `token`, KVX_ENOMEM with nothing
   changed when no page is to be had.  Stores into the copy go on `stream` or after it.  The
   copy is only enqueued when the call returns, and the sequence's reference to the shared
   page is given back at once: should every other holder let go of it too, the pool can hand
   the page out again, and whoever gets it must not store into it before `stream` has passed
   the copy (an event recorded on `stream` after this call, waited for by the writer's stream;
   the same rule as after kvx_pool_compact_extent).  kvx_sequence_fork copies nothing. */
int kvx_sequence_fork(kvx_sequences *sequences, uint64_t id, uint64_t source, uint64_t tokens);
int kvx_sequence_ensure_writable(kvx_sequences *sequences, uint64_t id, uint64_t token,
                                 uint32_t *copied, uint32_t *from_page, uint32_t *to_page,
                                 void *stream);
/* Cache::publishCommittedBlocks: every newly full page becomes a block; where the content is
   cached already the sequence moves to the canonical page (copy-free dedup) and the view's
   revision / first_changed say so. */
int kvx_sequence_publish(kvx_sequences *sequences, uint64_t id, const uint32_t *tokens,
                         uint64_t n_tokens, uint32_t committed_tokens);
/* The same with the request's images (Cache.cpp:310-318): every new block is keyed with the
   identity of the spans that overlap it, so equal placeholder tokens under different images
   stay apart.  kvx_sequence_publish is the text-only form (no spans). */
int kvx_sequence_publish_images(kvx_sequences *sequences, uint64_t id, const uint32_t *tokens,
                                uint64_t n_tokens, uint32_t committed_tokens,
                                const kvx_image_span *spans, uint32_t n_spans);
/* After a speculative rollback (kv_compact_path, then the host's committed count): gives the
   pages past those that hold the first `tokens` tokens back to the pool, one active reference
   each, and says how many in *released_pages; the view's revision / first_changed say so.
   `tokens` is what the sequence keeps room for: the committed tokens plus the scratch rows of
   the next step (the reference asks ensureTokens for position + 15, Engine.cpp:1190-1193, and
   never shrinks a request; this is the other direction, for trees of 16 draft rows that can
   leave a whole page without a committed token).  A page somebody else holds too only loses
   this sequence's reference.  KVX_ESTATE when that would drop a published page. */
int kvx_sequence_truncate(kvx_sequences *sequences, uint64_t id, uint64_t tokens,
                          uint32_t *released_pages);
int kvx_sequence_view(const kvx_sequences *sequences, uint64_t id, kvx_sequence_pages *out);
/* Cache::compactExtent: kvx_pool_compact_extent (with its ordering rule for `stream`), then
   blocks and sequences follow their pages. */
int kvx_sequences_compact_extent(kvx_sequences *sequences, uint32_t *first_page,
                                 uint32_t *destinations, uint32_t *moved_pages, void *stream);

/* ---- producers of the verify inputs, host versions ---- */
/* Ancestor bitmasks of a verify tree (kernel verify_input_tree_tokens,
   runtime/metal/kernels/shared/embedding.metal:248-281): masks[row] = 1 << row | bits of its
   ancestors.  parents[row] < row; KVX_TREE_NO_PARENT marks the root (row 0) and, on any later
   row, a dead row, whose mask is 0.  KVX_EINVAL for rows > 32 or a parent that is not an
   earlier row. */
#define KVX_TREE_NO_PARENT 0xffffffffu
int kvx_tree_masks(const uint32_t *parents, uint32_t rows, uint32_t *masks);
/* The contract of a retained path (kernel decode_accept_tree,
   runtime/metal/kernels/decode/sampling.metal:1927-1989): starts at row 0, rows strictly
   increase, each row is a child of the one before.  1 valid, 0 not. */
int kvx_tree_path_valid(const uint32_t *parents, uint32_t rows, const uint32_t *path,
                        uint32_t retained);

/* ---- the hot path ---- */

/* Quantize-on-append + scatter through page tables.
   Replaces ops::PagedAttention::addPrefillStore (runtime/ops/PagedAttention.cpp:424-440;
   kernels prefill/paged_attention_store.metal:7-148) when verify_max_rows == 0,
   and the store dispatch of ops::PagedAttention::addVerify
   (PagedAttention.cpp:467-500; decode/paged_attention_store.metal:3-186) otherwise.
   chunk_keys is bf16 [lane][kv head][chunk_stride][D], chunk_values bf16
   [lane][kv head][D][chunk_stride]; lanes lie lane_stride elements apart.
   page_tables[lane] is the device address of that lane's entries.
   verify_max_rows > 0 applies the verify contract: chunk_stride == 32 and
   chunk_tokens <= verify_max_rows (15 in the reference; up to 16 here).
   Host validation follows kv::chunkedPrefillValidationError; the kernel keeps the
   contract check of common/paged_store_row.h:14-29. */
int kv_append(const kvx_storage *storage, uint32_t layer, const void *chunk_keys,
              const void *chunk_values, const uint64_t *const *page_tables,
              const kvx_chunk_params *lanes, uint32_t n_lanes, uint64_t lane_stride,
              uint32_t verify_max_rows, void *stream);

/* QKV prepare fused with quantize-on-append: what prefill_attention_qkv* / verify_attention_qkv*
   followed by the store kernels do (ops::PagedAttention::addPrefillQkv / addVerifyQkv,
   runtime/ops/PagedAttention.cpp:299-320, 351-371; kernels prefill/attention_qkv.metal:6-33,
   decode/attention_qkv.metal:6-118, common/attention_qkv_prepare.h:12-83, common/rms_inverse.h:14-31;
   then the stores kv_append replaces), without the bf16 chunk between them: the reference's own
   open item (TODO.md, item 10).
   Per live row and head: RMS norm over the head dimension with the head-type's weights, rotation
   of the first rotary_pairs dimension pairs (d, d + rotary_pairs) by the row's cos / sin, bf16
   rounding after the norm and after the rotation; queries go to `queries` in the attention
   layout, keys are quantized from the rotated bf16 row and values from the packed row as
   kv_append quantizes them, into the slots of tokens committed_tokens + row.
   packed_qkv: bf16 [lane][rows][query heads x (query_gate ? 2 : 1) x D | KV heads x D keys |
   KV heads x D values] (with query_gate each query head is its D query values, then D gate
   values, which kv_attend_verify_hidden reads later).
   q_norm / k_norm: [D] weights, bf16 (norm_type 1) or float (2); norm_type 0 runs no norm.
   rope_cos / rope_sin: float [lane][rows][rotary_pairs].
   queries: bf16 [lane][kv head][row_stride][group][D]; rows >= a lane's chunk_tokens are not
   written.  lanes[i]: committed_tokens, chunk_tokens (live rows <= rows), page_table_entries;
   chunk_stride must be a valid chunk stride (32 does) and is otherwise unused.
   verify_max_rows > 0 bounds chunk_tokens as in kv_append.  Every buffer is 16-byte aligned.
   Results depend on the inputs alone (fixed summation order, no fused multiply-add). */
typedef struct kvx_qkv_shape {
  uint32_t query_heads;
  uint32_t rotary_pairs; /* 32 for the 256-wide heads of the reference, D / 2 for full rotary */
  uint32_t query_gate;   /* 1: packed query heads are [query | gate] pairs */
  uint32_t norm_type;    /* 0 none, 1 bf16 weights, 2 float weights */
  float eps;             /* 0 selects 1e-6 (kRmsEpsilon) */
} kvx_qkv_shape;
int kv_prepare_append(const kvx_storage *storage, uint32_t layer, const kvx_qkv_shape *shape,
                      const void *packed_qkv, const void *q_norm, const void *k_norm,
                      const float *rope_cos, const float *rope_sin, void *queries,
                      uint32_t row_stride, const uint64_t *const *page_tables,
                      const kvx_chunk_params *lanes, uint32_t n_lanes, uint32_t rows,
                      uint32_t verify_max_rows, void *stream);

/* Paged attention of `active_rows` query rows per lane over committed history
   plus those rows (chain: causal; tree: row_masks).  Replaces the split and
   reduce dispatches of ops::PagedAttention::addVerify (PagedAttention.cpp:506-544;
   kernels decode/paged_attention.metal:23-464, common/paged_attention_tile.h).
   queries / output: bf16 [lane][kv head][row_stride][group][D]
   (dev/tuning/AttentionFixture.hpp:167-173; row_stride = 32 in the reference).
   row_masks: NULL, or u32 [lane][row_capacity] ancestor bitmasks
   (shared/embedding.metal:248-281).  Each lane's split_count partitions its
   pages as ceil(pages / split_count) per split.  The reference strides a lane's
   slots by slot_splits (common/paged_attention_tile.h:57-58); here slots are packed
   by split_count, and slot_splits is only checked: 0, or split_count <= slot_splits
   <= the maximum, else KVX_EINVAL.  Output rows >= active_rows up to row_capacity are
   written as zeros.  workspace: device memory of at least
   kvx_attend_workspace_bytes(). */
int kv_attend_verify(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                     const void *queries, void *output, const uint64_t *const *page_tables,
                     const kvx_verify_params *lanes, uint32_t n_lanes,
                     const uint32_t *row_masks, uint32_t row_stride, void *workspace,
                     uint64_t workspace_bytes, void *stream);

/* The two dispatches of kv_attend_verify as calls of their own, as the reference encodes them
   (ops::PagedAttention::addVerify: the *_split dispatch, runtime/ops/PagedAttention.cpp:506-513,
   then the *_reduce dispatch, :517-544).
   kv_attend_split: every split of every lane writes its fp32 partial rows and (max, sum) to the
   workspace and nothing is merged, also for a lane with one split.  The workspace holds the
   partial rows first, [fused row slot][D] floats, then, at the next 256-byte boundary, the
   statistics, [fused row slot][2]; lane i's slots start after those of lanes 0 .. i-1 (split_count x
   KV heads x row_capacity x group each) and are ordered [KV head][split][fused row], fused row =
   query row x group + head in group.
   kv_attend_merge: the fixed-order merge over a workspace filled that way, by kv_attend_split or
   by the caller (the reference pins its reduce kernels with synthetic partial rows,
   dev/tests/engine/q8_flash_attention_metal_test.mm:648-725); `lanes` as for the split (their
   committed_tokens, active_rows and split_count say which slots were written). */
int kv_attend_split(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                    const void *queries, const uint64_t *const *page_tables,
                    const kvx_verify_params *lanes, uint32_t n_lanes, const uint32_t *row_masks,
                    uint32_t row_stride, void *workspace, uint64_t workspace_bytes, void *stream);
int kv_attend_merge(const kvx_storage *storage, uint32_t query_heads, void *output,
                    const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                    void *workspace, uint64_t workspace_bytes, void *stream);

/* kv_attend_verify whose merge also hands the out-projection its operand, so that no
   elementwise gate or gather dispatch has to read the attention rows back.  Replaces
   ops::PagedAttention::addVerify with gateHidden bound (runtime/ops/PagedAttention.hpp:299-311,
   PagedAttention.cpp:514-541; kernels verify_attention_reduce_gate* and
   verify_tree_attention_reduce_gate*, decode/paged_attention.metal:266-330, 466-530, and
   verify_attention_reduce_gather*, :356-413).
   hidden: bf16 [lane][row_capacity][query head][D], query head = kv head x group + head in group.
   packed_qkv: NULL, or the lanes' packed projection rows, bf16 [lane][row_capacity][stride] with
   stride = (2 x query heads + 2 x KV heads) x D: per query head its D query values then its D gate
   values, then keys and values.
   packed_qkv given: hidden = bf16(value x sigmoid(gate)), value being the bf16 attention element
   and sigmoid(x) = 1 / (1 + 2^(-x log2 e)) (common/activation.h:14-16), what
   verify_attention_gate computes from the staged rows (decode/attention_qkv.metal:121-164).
   packed_qkv NULL: hidden = value (verify_attention_gather).
   output may be NULL; when given it receives the staged rows exactly as kv_attend_verify writes
   them.  Rows >= active_rows of hidden are zeros.  The reference has no fused gather for tree
   rows; this entry takes row_masks in both modes. */
int kv_attend_verify_hidden(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes,
                            const uint32_t *row_masks, uint32_t row_stride, void *workspace,
                            uint64_t workspace_bytes, const void *packed_qkv, void *hidden,
                            void *stream);

/* One-row decode attention of up to 16 sequences whose page tables begin with the same
   `shared_pages` pages (a cached prompt prefix, engine::KvCache chains restored by
   Cache::restoreRequest): the shared pages are read once for all of them instead of once per
   sequence.  The reference lists this as a gap (docs/PERF_REPORT.md:250, :259) and has no
   counterpart; the result is kv_attend_decode's within its tolerance (the partition into splits
   differs, so the fp32 sums are taken in another order).
   The sequences' query rows are attended together over the prefix as the rows of one lane with
   `prefix_splits` splits, each sequence's remaining pages as a decode lane of its own with
   lanes[i].split_count splits, and one merge combines both per sequence.  lanes[i] describe the
   whole sequences (committed_tokens >= shared_pages x 32; tables of all their pages).
   queries / output as kv_attend_decode.  Head dimension 256, int4 / int8 / bf16 pages.
   workspace: at least kvx_attend_shared_workspace_bytes(). */
uint64_t kvx_attend_shared_workspace_bytes(const kvx_verify_params *lanes, uint32_t n_lanes,
                                           uint32_t prefix_splits, uint32_t query_heads,
                                           const kvx_layout *layout);
int kv_attend_decode_shared(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t shared_pages,
                            uint32_t prefix_splits, uint32_t row_stride, void *workspace,
                            uint64_t workspace_bytes, void *stream);

/* One-row decode attention per lane: kv_attend_verify with active_rows =
   row_capacity = 1 on the bandwidth-tuned kernels (the reference reaches decode
   through its prefill entries with rows = 1, prefill/paged_attention.metal:7-67,
   pinned by dev/tests/engine/paged_attention_plan_test.mm:1019). */
int kv_attend_decode(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                     const void *queries, void *output, const uint64_t *const *page_tables,
                     const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                     void *workspace, uint64_t workspace_bytes, void *stream);

/* kv_attend_decode for callers that cannot allocate device memory or bring a workspace: code
   under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
   in the reference.  The partial rows and statistics go to a static device array of the library
   (KVX_STATIC_WORKSPACE_BYTES, held by every GPU the library runs on until the process ends)
   instead of a workspace argument; the call allocates nothing, on the host or on the device.
   KVX_EINVAL when kvx_attend_workspace_bytes() of the lanes exceeds the array (the headline batch
   of 32 sequences at 507 splits needs 12.6 MB), KVX_ESTATE when the storage's device is not the
   current device.  All calls on one GPU share the array: calls that overlap there (two streams,
   two threads) race on it; calls on one stream, or ordered by events, do not.
   Where the array lies on a device is looked up once per device: kvx_storage_create does it
   for the device it runs on, kvx_static_workspace_prime for a storage whose device became
   current later.  A call under stream capture on a device where neither has happened is
   refused with KVX_ESTATE instead of asking the runtime in the middle of the capture. */
#define KVX_STATIC_WORKSPACE_BYTES (32u << 20)
int kvx_static_workspace_prime(const kvx_storage *storage);
int kv_attend_decode_static(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                            void *stream);

/* One decode step of a layer in one call: kv_append of one token per lane at
   lanes[i].committed_tokens (chunk rows as for kv_append: keys [head][chunk_stride][D],
   values [head][D][chunk_stride], token 0 of each lane's chunk, lanes chunk_lane_stride
   elements apart) followed by kv_attend_decode over committed_tokens + 1 tokens.  The
   reference stores and attends in one call the same way (ops::PagedAttention::addVerify,
   runtime/ops/PagedAttention.cpp:467-544).  Same page bytes and same output as the two
   calls; for int4 pages of head dimension 256 the wave that owns a sequence's last page
   stores the token itself, which saves the append launch. */
int kv_append_attend_decode(const kvx_storage *storage, uint32_t layer, const void *chunk_keys,
                            const void *chunk_values, uint64_t chunk_lane_stride,
                            uint32_t chunk_stride, uint32_t query_heads, const void *queries,
                            void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                            void *workspace, uint64_t workspace_bytes, void *stream);
/* The same step with the merge of kv_attend_verify_hidden: the token is stored, the row attended and
   the out-projection's operand written ([lane][1][query head][D]; gated by packed_qkv when that is
   given, as described there) in one call, which is the reference's decode step with gateHidden bound
   (ops::PagedAttention::addVerify, runtime/ops/PagedAttention.cpp:467-544; kernel
   verify_attention_reduce_gate*, decode/paged_attention.metal:266-330).  output may be NULL.
   Same page bytes, output and hidden rows as kv_append followed by kv_attend_verify_hidden. */
int kv_append_attend_decode_hidden(const kvx_storage *storage, uint32_t layer, const void *chunk_keys,
                                   const void *chunk_values, uint64_t chunk_lane_stride,
                                   uint32_t chunk_stride, uint32_t query_heads, const void *queries,
                                   void *output, const uint64_t *const *page_tables,
                                   const kvx_verify_params *lanes, uint32_t n_lanes,
                                   uint32_t row_stride, void *workspace, uint64_t workspace_bytes,
                                   const void *packed_qkv, void *hidden, void *stream);

/* Chunked prefill attention of one sequence: rows in tiles of 8, each tile
   causal over committed + its rows.  Replaces ops::PagedAttention::addPrefill
   (PagedAttention.cpp:442-465; kernels prefill/paged_attention.metal:7-206).
   queries / output: bf16 [kv head][chunk_stride][group][D].  workspace: at
   least kvx_prefill_workspace() partials + statistics. */
int kv_attend_prefill(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                      const void *queries, void *output, const uint64_t *page_table,
                      const kvx_prefill_params *params, void *workspace,
                      uint64_t workspace_bytes, void *stream);
/* The chunks of several sequences in one call, as the reference records the lanes of a step in one
   command (ops::PagedAttention::addVerify's lane array, runtime/ops/PagedAttention.cpp:467-500; its
   addPrefill takes one sequence).  Sequence q has params[q] and page_tables[q]; its queries and
   output rows ([kv head][chunk_stride][group][D] as above) begin q x sequence_stride elements after
   the first sequence's.  Chunks of the same shape (rows, chunk_stride and split_count equal, and
   committed_tokens such that their tiles are paired or grouped alike: page-aligned starts always
   are) share their launches, 32 sequences at a time: every sequence's tiles are lanes of one
   launch.  Anything else runs sequence by sequence on `stream`.  Either way every sequence's
   rows are the bits kv_attend_prefill gives for it alone.  workspace: at least the sum of the
   sequences' kvx_prefill_workspace_for() bounds plus 256 bytes.  Nothing is enqueued unless every
   sequence's parameters are valid. */
int kv_attend_prefill_batch(const kvx_storage *storage, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_prefill_params *params, uint32_t n_sequences,
                            uint64_t sequence_stride, void *workspace, uint64_t workspace_bytes,
                            void *stream);

/* Tree-path compaction after acceptance: for i < retained_count[lane], the
   row at committed + retained_path[lane * path_stride + i] moves to
   committed + i.  Replaces ops::PagedAttention::addVerifyTreeCompact
   (PagedAttention.cpp:546-573; kernel decode/paged_attention_store.metal:198-309).
   retained_path / retained_count are device arrays (the acceptance kernel
   writes them, decode/sampling.metal:1927-1989); path_stride is 8 in the
   reference.  layer = UINT32_MAX compacts every layer. */
int kv_compact_path(const kvx_storage *storage, uint32_t layer,
                    const uint64_t *const *page_tables, const kvx_chunk_params *lanes,
                    uint32_t n_lanes, const uint32_t *retained_path,
                    const uint32_t *retained_count, uint32_t path_stride, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KVX_H */
