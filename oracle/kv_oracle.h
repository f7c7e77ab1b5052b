/*
 * kv_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * A scalar CPU restatement of RichEngine's paged-KV semantics (layout, codecs,
 * quantize-on-append, paged attention with split partials and fixed-order
 * merge, tree-path compaction, whole-page copy, page pool).  It is the checker
 * the HIP path is compared against; nothing in the product may link, import
 * or call it.  Only tests, the smoke check and the benchmark's CPU-baseline
 * leg use it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout).  Pinning status per function group:
 *   layout / addressing  : pinned (reference known answers + bijection)
 *   bf16 / fp8 / fp16    : pinned (reference headers via oracle/_ref, exhaustive)
 *   int8/int4/fp8 append : pinned (reference quantizer via oracle/_ref,
 *                          reference closed-form row patterns, invariants)
 *   attention            : pinned to tolerance only (fp64 dense softmax,
 *                          special cases); bit-level parity unpinned because
 *                          the reference's exp and matmul order live in Apple's
 *                          Metal runtime, which cannot run here
 *   tree verify/compact  : pinned by brute force only (the reference holds no
 *                          test of them) -- parity unpinned against reference
 *   gate / gather        : pinned by mathematics (sigmoid identities and fp64
 *                          values; the index map against an independent
 *                          transpose/reshape statement); the reference's only
 *                          check is a Metal fused-vs-unfused comparison
 *   QKV prepare          : pinned by mathematics (float64 RMS norm and rotation,
 *                          exact special cases); the simdgroup sum order and
 *                          rsqrt of the reference are Metal's -- parity of
 *                          those two unpinned (one float ulp before the bf16
 *                          rounding)
 *   pool                 : pinned (reference pool tests' exact page ids/moves)
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* runtime/ops/PagedKv.hpp:16 -- same numeric values as kv::Format. */
enum { KO_INT8 = 1, KO_BF16 = 2, KO_INT4 = 3, KO_FP8E4M3 = 4 };

/* runtime/metal/abi/KvExtent.h:27-30 */
enum { KO_KEYS = 0, KO_KEY_SCALES = 1, KO_VALUES = 2, KO_VALUE_SCALES = 3 };

#define KO_PAGE_TOKENS 32u           /* abi/ExecutionGeometry.h:28 */
#define KO_PAGE_INDEX_BITS 14u       /* abi/KvExtent.h:19 */
#define KO_PAGE_INDEX_MASK ((1u << KO_PAGE_INDEX_BITS) - 1u)
#define KO_MAX_CONTEXT 262144u       /* abi/ExecutionGeometry.h:15 */
#define KO_TREE_NODES 16u            /* abi/ExecutionGeometry.h:14 */
#define KO_VERIFY_ROWS 8u            /* abi/ExecutionGeometry.h:7 */
#define KO_MAX_PHYSICAL (KO_MAX_CONTEXT + KO_TREE_NODES - 1u)
#define KO_PREFILL_BUDGET 2048u      /* abi/ExecutionGeometry.h:23 */
#define KO_PREFILL_TILE_ROWS 8u      /* abi/ExecutionGeometry.h:32 */
#define KO_PREFILL_MAX_SPLITS 32u    /* abi/ExecutionGeometry.h:33 */
#define KO_VERIFY_MAX_SPLITS 128u    /* abi/ExecutionGeometry.h:39 */
#define KO_DECODE_MAX_SPLITS 512u    /* one-row decode lanes of the MI355X build; no reference counterpart */
#define KO_VERIFY_STRIDE 32u         /* abi/ExecutionGeometry.h:31 */

/* runtime/ops/PagedKv.hpp:125-136 */
typedef struct ko_layout {
  uint32_t layers;
  uint32_t kv_heads;
  uint32_t head_dim;
  uint32_t format;
  float score_scale;
} ko_layout;

/* runtime/metal/abi/KvExtent.h:93-96 */
typedef struct ko_kv_layer {
  uint32_t extent_pages;
  uint32_t offset;
} ko_kv_layer;

/* runtime/metal/abi/PagedAttention.h:39-45 (24 bytes) */
typedef struct ko_chunk_params {
  uint32_t committed_tokens;
  uint32_t chunk_tokens;
  uint32_t chunk_stride;
  uint32_t page_table_entries;
  ko_kv_layer kv;
} ko_chunk_params;

/* runtime/metal/abi/PagedAttention.h:52-61 (32 bytes) */
typedef struct ko_prefill_params {
  uint32_t committed_tokens;
  uint32_t rows;
  uint32_t chunk_stride;
  uint32_t page_table_entries;
  ko_kv_layer kv;
  uint32_t split_count;
  float score_scale;
} ko_prefill_params;

/* runtime/metal/abi/PagedAttention.h:72-84 (36 bytes) */
typedef struct ko_verify_params {
  uint32_t committed_tokens;
  uint32_t page_table_entries;
  ko_kv_layer kv;
  uint32_t split_count;
  uint32_t slot_splits;
  uint32_t active_rows;
  uint32_t row_capacity;
  float score_scale;
} ko_verify_params;

/* runtime/ops/PagedKv.hpp:48-51 */
typedef struct ko_page_copy {
  uint32_t from;
  uint32_t to;
} ko_page_copy;

/* ---- layout geometry: runtime/ops/PagedKv.hpp:137-230 ---- */
int ko_layout_valid(const ko_layout *l);
uint64_t ko_elements_per_layer_page(const ko_layout *l);
uint64_t ko_data_bytes_per_layer_page(const ko_layout *l);
uint64_t ko_scale_bytes_per_layer_page(const ko_layout *l);
uint64_t ko_bytes_per_layer_page(const ko_layout *l);
uint64_t ko_bytes_per_model_page(const ko_layout *l);
uint32_t ko_extent_alignment_pages(const ko_layout *l);
uint32_t ko_minimum_extent_pages(const ko_layout *l);
uint32_t ko_maximum_extent_pages(const ko_layout *l);
uint32_t ko_extent_pages_for(const ko_layout *l, uint64_t pages);

/* ---- addressing: runtime/metal/abi/KvExtent.h:45-111 ---- */
uint64_t ko_key_element(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim);
uint64_t ko_value_element(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim);
uint64_t ko_scale_element(uint32_t head, uint32_t token);
uint64_t ko_kv_offset(uint32_t extent_pages, uint32_t data_bytes, uint32_t scale_bytes,
                      uint32_t layer, uint32_t tensor, uint32_t index);
ko_kv_layer ko_kv_layer_of(uint32_t extent_pages, uint32_t data_bytes, uint32_t scale_bytes,
                           uint32_t layer);
uint64_t ko_page_entry(uint64_t extent_address, uint32_t index);

/* ---- codecs ---- */
uint16_t ko_float_to_bf16(float v);   /* dev/tests/engine/Q8PageFormatReference.hpp:66-76 */
float ko_bf16_to_float(uint16_t v);   /* Q8PageFormatReference.hpp:78-80 */
uint8_t ko_float_to_fp8e4m3(float v); /* dev/tests/engine/Fp8PageFormatReference.hpp:27-52 */
float ko_fp8e4m3_to_float(uint8_t c); /* Fp8PageFormatReference.hpp:54-63 */
float ko_round_to_f16(float v);       /* Fp8PageFormatReference.hpp:67-69 (queryStage) */

/* ---- planning: runtime/ops/PagedAttention.hpp:54-95, PagedAttention.cpp:23-32,200-297 ---- */
uint32_t ko_verify_splits(uint32_t committed_tokens, uint32_t rows);
uint32_t ko_prefill_tiles(uint32_t rows);
uint32_t ko_prefill_splits(uint32_t tiles);
/* 0 = ok, 1 chunk_tokens_out_of_range, 2 context_out_of_range,
   3 chunk_stride_invalid, 4 page_table_too_short */
int ko_chunk_validation(const ko_chunk_params *p);
uint32_t ko_chunk_required_pages(const ko_chunk_params *p);
void ko_prefill_workspace(uint32_t rows, uint32_t query_heads, uint32_t kv_heads,
                          uint32_t head_dim, uint64_t *partials_bytes,
                          uint64_t *statistics_bytes);
void ko_prefill_workspace_bound(uint32_t maximum_rows, uint32_t query_heads,
                                uint32_t head_dim, uint64_t *partials_bytes,
                                uint64_t *statistics_bytes);
void ko_verify_workspace(uint32_t lanes, uint32_t row_capacity, uint32_t query_heads,
                         uint32_t head_dim, uint64_t *partials_bytes,
                         uint64_t *statistics_bytes);

/* ---- host page storage: runtime/ops/PageStorage.mm:12-167 ---- */
typedef struct ko_store ko_store;
ko_store *ko_store_create(const ko_layout *l, uint32_t page_count, uint32_t extent_pages);
/* dev/tuning/HostKvExtents.hpp:158-169: as above without the alignment-unit rule. */
ko_store *ko_store_create_host(const ko_layout *l, uint32_t page_count, uint32_t extent_pages);
void ko_store_destroy(ko_store *s);
/* 0 ok; -1 already allocated / not allocated (std::logic_error in the reference);
   -2 out of range */
int ko_store_allocate_extent(ko_store *s, uint32_t extent);
int ko_store_release_extent(ko_store *s, uint32_t extent);
uint8_t *ko_store_extent(ko_store *s, uint32_t extent);
uint64_t ko_store_extent_bytes(const ko_store *s);
uint32_t ko_store_extent_pages(const ko_store *s);
ko_kv_layer ko_store_layer(const ko_store *s, uint32_t layer);
/* PageStorage::writeEntries: entries [first, n) are written. */
int ko_store_write_entries(const ko_store *s, const uint32_t *pages, uint32_t n,
                           uint32_t first, uint64_t *table);
/* PageStorage::copyPages: all-or-nothing validation, then every tensor span. */
int ko_store_copy_pages(ko_store *s, const ko_page_copy *copies, uint32_t n);
/* PageStorage::spans flattened: copies the page's bytes (layer-major, tensor
   order K, Kscale, V, Vscale) to/from `bytes` (bytes_per_model_page long). */
int ko_store_page_read(const ko_store *s, uint32_t page, uint8_t *bytes);
int ko_store_page_write(ko_store *s, uint32_t page, const uint8_t *bytes);

/* ---- quantize-on-append: common/paged_store_row.h:14-147, paged_store_row_fp8.h:28-78 ---- */
/* prefill/paged_attention_store.metal:7-27: one sequence. Returns 1 when the
   contract is valid and rows were written, 0 when the lane wrote nothing. */
int ko_store_chunk(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                   const uint16_t *chunk_keys, const uint16_t *chunk_values,
                   const uint64_t *page_table, const ko_chunk_params *params);
/* decode/paged_attention_store.metal:3-45: `lanes` lanes, each with its own
   table; chunk buffers are [lane][head][32][D] / [lane][head][D][32].
   max_rows is the verify bound on chunk_tokens (15 in the reference). */
int ko_store_verify(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                    const uint16_t *chunk_keys, const uint16_t *chunk_values,
                    const uint64_t *const *page_tables, const ko_chunk_params *params,
                    uint32_t lanes, uint32_t max_rows);

/* ---- attention: common/paged_attention_tile.h:85-417, paged_attention_fp8_tile.h ---- */
/* One tile (one KV head, `row_capacity` rows x `group` query heads) over one
   split.  queries point at the tile's [row][g][D] block.  Writes
   partials[slot][M][D] and statistics[slot][M]{max,sum}.  Returns 0 when the
   split owns no page (nothing written). */
int ko_attention_tile(uint32_t format, uint32_t kv_heads, uint32_t group, uint32_t head_dim,
                      uint32_t row_capacity, const uint16_t *tile_queries,
                      const uint64_t *page_table, ko_kv_layer kv, uint32_t kv_head,
                      uint32_t committed_tokens, uint32_t active_rows, uint32_t splits,
                      uint32_t split, float *partials, float *statistics, uint64_t slot,
                      const uint32_t *row_masks, float score_scale);
/* common/paged_attention_tile.h:362-417: merges one fused row. out_bf16 and
   out_f32 (either may be NULL) receive D values. */
/* Test aids.  ko_attention_flips: while fused_row >= 0, ko_attention_tile looks at the weight
   (probability x value scale) of each listed token of that fused row before it rounds it to its
   format (bf16; fp16 on fp8 pages); where the unrounded value lies within slack (relative) of the
   boundary between two neighbours of the format it takes the neighbour on the other side, and
   leaves the weight alone otherwise.  With only_row it computes that fused row alone;
   fused_row = -1 switches everything off.  ko_attention_flips_applied: bit i set when token i was
   turned since the last ko_attention_flips.  State is per thread.
   ko_attention_row_weights: softmax weight x value scale of every token a query row sees (against
   the row's maximum over all pages), weights[committed + active_rows]. */
void ko_attention_flips(int64_t fused_row, const uint32_t *tokens, uint32_t count, float slack,
                        int only_row);
uint32_t ko_attention_flips_applied(void);
/* Threads that ko_attention_tile spreads a tile's rows over and ko_attend_prefill its tiles
   (OpenMP; default 1).  Every row is computed by one thread in the same order whatever the
   number, so results do not depend on it; it only shortens the checks of the GPU suite.
   Timed baselines leave it at 1. */
void ko_set_threads(int threads);
int ko_threads(void);
void ko_attention_row_weights(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                              const uint16_t *query_row, const uint64_t *page_table, ko_kv_layer kv,
                              uint32_t kv_head, uint32_t committed, uint32_t active_rows,
                              uint32_t row, const uint32_t *row_masks, float score_scale,
                              float *weights);
void ko_attention_reduce_row(uint32_t group, uint32_t head_dim, uint32_t row_capacity,
                             const float *partials, const float *statistics,
                             uint32_t committed_tokens, uint32_t active_rows,
                             uint32_t splits, uint64_t head_slot, uint32_t fused_row,
                             uint16_t *out_bf16, float *out_f32);
/* prefill/paged_attention.metal:7-67 + reduce: whole chunk of one sequence.
   queries/output are [kv head][row (chunk_stride)][g][D] bf16.  out_f32, when
   not NULL, has the same shape and holds the value before the bf16 rounding.
   Returns 1 when valid. rows=1 is the decode step. */
int ko_attend_prefill(uint32_t format, uint32_t kv_heads, uint32_t group, uint32_t head_dim,
                      const uint16_t *queries, uint16_t *output, float *out_f32,
                      const uint64_t *page_table, const ko_prefill_params *params);
/* decode/paged_attention.metal:23-191 + reduce: `lanes` lanes of row_capacity
   rows (8 chain, 16 tree).  queries/output are
   [lane][kv head][32][g][D].  row_masks (tree) is [lane][row_capacity] or NULL
   (chain: every lane attends row_capacity rows causally). */
int ko_attend_verify(uint32_t format, uint32_t kv_heads, uint32_t group, uint32_t head_dim,
                     const uint16_t *queries, uint16_t *output, float *out_f32,
                     const uint64_t *const *page_tables, const ko_verify_params *params,
                     uint32_t lanes, const uint32_t *row_masks);

/* common/activation.h:14-16: 1 / (1 + 2^(-x log2 e)). */
float ko_sigmoid(float x);
/* The out-projection's operand from staged attention rows: verify_attention_gate /
   verify_attention_gather (decode/attention_qkv.metal:121-164), which the fused reduces
   (decode/paged_attention.metal:266-309, 356-393, 466-510) reproduce bit for bit.
   attention is [lane][kv head][row_stride][g][D] bf16, hidden [lane][rows][query head][D];
   packed_qkv (NULL = gather) is [lane][rows][(2 x query heads + 2 x kv heads) x D] with each
   query head's gate D elements after its query.  One flat element at a time, as the kernel. */
void ko_attention_hidden(uint32_t kv_heads, uint32_t group, uint32_t head_dim, uint32_t lanes,
                         uint32_t rows, uint32_t row_stride, const uint16_t *attention,
                         const uint16_t *packed_qkv, uint16_t *hidden);

/* QKV prepare of one lane: per-head RMS norm, partial rotary embedding and the layout
   change from packed projection rows to attention queries and bf16 chunk rows
   (common/attention_qkv_prepare.h:12-83, common/rms_inverse.h:14-31; entries
   prefill_attention_qkv*, prefill/attention_qkv.metal:6-33, and verify_attention_qkv*,
   decode/attention_qkv.metal:6-118, which call it per lane).
   packed: bf16 [tokens][query heads x (query_gate ? 2 : 1) x D, kv heads x D keys, kv heads x D
   values]; norms: NULL (none), bf16 (norm_f32 = 0) or float (norm_f32 = 1) [D]; rope_cos /
   rope_sin: float [tokens][rotary_pairs]; queries: bf16 [kv head][stride][g][D]; chunk_keys
   [kv head][stride][D], chunk_values [kv head][D][stride].
   Two operations are implementation-defined in Metal and fixed here: simd_sum over a
   simdgroup of 32 is the xor butterfly (offsets 16, 8, 4, 2, 1), and rsqrt(x) is the
   correctly rounded 1 / sqrt(x).  Every other operation is a single rounded fp32 product,
   sum or quotient in the source's order. */
void ko_qkv_prepare(uint32_t kv_heads, uint32_t group, uint32_t head_dim, uint32_t rotary_pairs,
                    int query_gate, int norm_f32, float eps, uint32_t tokens, uint32_t stride,
                    const uint16_t *packed, const void *q_norm, const void *k_norm,
                    const float *rope_cos, const float *rope_sin, uint16_t *queries,
                    uint16_t *chunk_keys, uint16_t *chunk_values);

/* ---- tree path compaction: decode/paged_attention_store.metal:198-278 ---- */
int ko_compact_tree(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                    const uint64_t *const *page_tables, const ko_chunk_params *params,
                    const uint32_t *retained_path, const uint32_t *retained_count,
                    uint32_t lanes, uint32_t path_stride);

/* ---- page pool: runtime/engine/cache/KvPool.cpp ---- */
typedef struct ko_pool ko_pool;
/* An accounting-only storage like the reference tests' TestKvStorage
   (dev/tests/engine/TestKvPool.hpp:27-113): growth is refused past
   budget_pages or while blocked. */
ko_pool *ko_pool_create(uint32_t page_count, uint64_t bytes_per_page, uint32_t extent_pages,
                        uint32_t runway_pages, uint32_t budget_pages);
void ko_pool_destroy(ko_pool *p);
void ko_pool_set_growth_blocked(ko_pool *p, int blocked);
void ko_pool_set_refused_extent(ko_pool *p, int64_t extent); /* -1 = none */
void ko_pool_set_budget_pages(ko_pool *p, uint32_t pages);  /* the storage's budget moves */
/* returns count granted (== count) or -1 denied, -2 ids ran out */
int ko_pool_acquire(ko_pool *p, uint32_t count, uint32_t *pages);
int ko_pool_retain(ko_pool *p, uint32_t page, int prefix_owner);   /* 0 ok, -1 logic error */
int ko_pool_release(ko_pool *p, uint32_t page, int prefix_owner);
int ko_pool_page_active(const ko_pool *p, uint32_t page);
uint64_t ko_pool_reclaim_empty(ko_pool *p, int keep_runway, uint32_t limit);
/* Returns moves count (extent_pages) or 0 when nothing moved; first_page and
   destinations[extent_pages] filled; copies (pairs) appended to copies_out
   (up to extent_pages) with *n_copies. */
int ko_pool_compact_extent(ko_pool *p, const uint32_t *fixed, uint32_t n_fixed,
                           uint32_t *first_page, uint32_t *destinations,
                           ko_page_copy *copies_out, uint32_t *n_copies);
typedef struct ko_pool_snapshot {
  uint32_t pages_allocated, pages_free, pages_active, pages_prefix;
  uint64_t allocated_bytes, reclaimable_bytes;
  uint64_t extent_allocations, extent_releases, extent_compactions, pages_moved;
} ko_pool_snapshot;
void ko_pool_snapshot_get(const ko_pool *p, ko_pool_snapshot *out);
uint64_t ko_pool_content(const ko_pool *p, uint32_t page);
void ko_pool_set_content(ko_pool *p, uint32_t page, uint64_t value);
int ko_pool_extent_allocated(const ko_pool *p, uint32_t extent);

#ifdef __cplusplus
}
#endif
