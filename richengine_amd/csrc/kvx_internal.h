// Internal definitions shared by the host side and the kernels of libkvx.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>
#include <vector>

#include "kvx.h"

namespace kvx {

// ---- errors -----------------------------------------------------------------
int fail(int code, const std::string &message);
// Looks up, once per device, where the static workspace of kv_attend_decode_static lies
// on `device` (the current one).
int prime_static_workspace(int device);
int hip_fail(hipError_t error, const char *what);
#define KVX_HIP(call)                                     \
  do {                                                    \
    hipError_t kvx_e_ = (call);                           \
    if (kvx_e_ != hipSuccess) return ::kvx::hip_fail(kvx_e_, #call); \
  } while (0)

// ---- geometry (host and device) --------------------------------------------
__host__ __device__ inline bool quantized(uint32_t format) { return format != KVX_FMT_BF16; }

__host__ __device__ inline uint32_t data_bytes_of(uint32_t format, uint32_t kv_heads,
                                                  uint32_t head_dim) {
  const uint32_t elements = KVX_PAGE_TOKENS * kv_heads * head_dim;
  return format == KVX_FMT_BF16 ? elements * 2 : format == KVX_FMT_INT4 ? elements / 2 : elements;
}
__host__ __device__ inline uint32_t scale_bytes_of(uint32_t format, uint32_t kv_heads) {
  return quantized(format) ? KVX_PAGE_TOKENS * kv_heads * 4 : 0;
}

// Where the four tensors of a layer start inside the layer's region of an
// extent, in bytes: keys | key scales | values | value scales, each holding
// every page of the extent (reference: abi/KvExtent.h:76-89).
struct RegionOffsets {
  uint64_t key_scales;
  uint64_t values;
  uint64_t value_scales;
};
__host__ __device__ inline RegionOffsets region_offsets(uint32_t extent_pages, uint32_t db,
                                                        uint32_t sb) {
  RegionOffsets r;
  r.key_scales = uint64_t(extent_pages) * db;
  r.values = uint64_t(extent_pages) * (uint64_t(db) + sb);
  r.value_scales = uint64_t(extent_pages) * (2ull * db + sb);
  return r;
}

// One KV head's slab of each tensor of a page in one layer.
struct Slab {
  uint8_t *keys;
  uint8_t *values;
  float *key_scales;
  float *value_scales;
};
__device__ inline Slab slab_of(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                               kvx_kv_layer kv, uint32_t head, uint64_t entry) {
  const uint32_t index = uint32_t(entry) & KVX_PAGE_INDEX_MASK;
  uint8_t *region = reinterpret_cast<uint8_t *>(entry - index) + kv.offset;
  const uint32_t db = data_bytes_of(format, kv_heads, head_dim);
  const uint32_t sb = scale_bytes_of(format, kv_heads);
  const RegionOffsets r = region_offsets(kv.extent_pages, db, sb);
  const uint32_t head_bytes = db / kv_heads;
  Slab s;
  s.keys = region + uint64_t(index) * db + head * head_bytes;
  s.values = region + r.values + uint64_t(index) * db + head * head_bytes;
  const uint64_t scale_index = (uint64_t(index) * kv_heads + head) * KVX_PAGE_TOKENS;
  s.key_scales = reinterpret_cast<float *>(region + r.key_scales) + scale_index;
  s.value_scales = reinterpret_cast<float *>(region + r.value_scales) + scale_index;
  return s;
}

// ---- attention epilogue -----------------------------------------------------
// What an attend call writes beside (or instead of) its staging rows: `hidden`,
// the out-projection's operand, bf16 [lane][row capacity][query head][D]
// (reference: the reduce/gather fusion, decode/paged_attention.metal:356-393).
// With `packed_qkv`, the lanes' packed projection rows, bf16 [lane][row capacity]
// [(query | gate) x query heads, (key | value) x KV heads][D], each element is
// first scaled by the sigmoid of its gate (the reduce/gate fusion,
// decode/paged_attention.metal:266-309, 466-510).
// With `partials_only` nothing is merged at all: every split writes its partial rows and
// statistics, and the caller combines them (kv_attend_split; attention over a shared
// prefix merges the prefix's splits with each sequence's own).  With `merge_only` no
// split kernel runs: the workspace holds every split's rows already (kv_attend_merge).
struct Epilogue {
  const uint16_t *packed_qkv;
  uint16_t *hidden;
  bool partials_only = false;
  bool merge_only = false;
};

// Regular lanes of a launch (the tiles of chunked prefill): `rows` > 0 says that the lanes
// passed are `sequences` runs of equally many lanes, lane i of a run being its first lane
// moved on by i x rows query rows and committed tokens over the run's one page table; the
// runs' queries and rows lie sequence_stride elements apart.  rows = 0: ordinary lanes.
struct Tiles {
  uint32_t rows = 0;
  uint32_t sequences = 1;
  uint64_t sequence_stride = 0;
  Tiles(uint32_t tile_rows = 0) : rows(tile_rows) {}
  Tiles(uint32_t tile_rows, uint32_t runs, uint64_t stride)
      : rows(tile_rows), sequences(runs), sequence_stride(stride) {}
  operator uint32_t() const { return rows; }
};

// ---- storage ----------------------------------------------------------------
struct Storage {
  kvx_layout layout;
  uint32_t page_count = 0;
  uint32_t extent_pages = 0;
  uint32_t data_bytes = 0;
  uint32_t scale_bytes = 0;
  uint64_t budget_bytes = 0;
  int device = 0;
  bool accounting = false;  // no memory behind the extents: page bookkeeping only
  std::vector<void *> extents;      // 16 KiB-aligned base; nullptr while not allocated
  std::vector<void *> allocations;  // what hipMalloc returned for each extent
  uint64_t extent_bytes() const;
  uint64_t bytes_per_page() const;
  uint32_t allocated_extents() const;
};

// Fused query rows one wave of a verify launch covers: the matrix-core kernels
// hold 32 per wave (16 when there are no more); the int4 kernels also have a
// 48-row form, which reads and expands every page once for all three blocks of
// 16 but keeps its accumulators where rescaling them costs three times as much:
// per page a wave of the 48-row form costs about 1.74 waves of the 32-row form
// (5040 against 2900 cycles), and it is used where it leaves fewer waves by
// more than that (48 fused rows: one wave against two; 96: two against three,
// which is not enough).
inline uint32_t verify_block_rows(uint32_t format, uint32_t fused_rows) {
  if (fused_rows <= 16) return 16;
  const uint32_t by32 = (fused_rows + 31) / 32, by48 = (fused_rows + 47) / 48;
  if (format == KVX_FMT_INT4 && 26 * by48 < 15 * by32) return 48;
  return 32;
}
// Whether tiles 2i and 2i + 1 of a chunked prefill that starts after `committed`
// tokens see the same number of pages, for every i: tile 2i sees committed + 16 i
// + 8 tokens, its neighbour 8 more, and no page boundary lies in between exactly
// when committed mod 16 is 0 or at least 9 (page-aligned chunk starts among them).
// Such pairs cut their pages into the same splits, whatever the split count.
inline bool prefill_tiles_pair(uint32_t committed) {
  const uint32_t r = committed % 16;
  return r == 0 || r >= 9;
}
// Waves of a chunked prefill whose tiles run in pairs (lanes of 16 rows on the
// kernels with two blocks of 16 fused rows per wave), per split, and the wave
// slots those kernels have (int4: two waves per SIMD).
inline uint32_t prefill_paired_waves(uint32_t tiles, uint32_t kv_heads, uint32_t group) {
  return (tiles + 1) / 2 * kv_heads * ((2 * KVX_PREFILL_TILE_ROWS * group + 31) / 32);
}
inline uint32_t prefill_paired_slots(uint32_t format) { return format == KVX_FMT_INT4 ? 2048 : 1024; }
// Whether a prefill with several splits runs its tiles in pairs: the pairs must
// cut their pages alike, and the paired launch must fill at least half of its
// wave slots (half as many waves, each twice as long, lose on an emptier GPU).
// int4 pages: only from 64 tiles on; below, the one-tile kernel with its two
// register sets of pages is faster per page than sharing saves.
inline bool prefill_pairs_with_splits(uint32_t format, uint32_t committed, uint32_t tiles,
                                      uint32_t splits, uint32_t kv_heads, uint32_t group) {
  if (tiles < 2 || !prefill_tiles_pair(committed)) return false;
  if (format == KVX_FMT_INT4 && tiles < 64) return false;
  return 2ull * prefill_paired_waves(tiles, kv_heads, group) * splits >= prefill_paired_slots(format);
}
// bf16, fp8 and int8 pages of head dimension 256: chunks from kGroupedPrefillRows rows on run
// in lanes of four (or two) tiles, for a workgroup of four waves that fetches every page
// once for all of them and shares it through LDS, where the lane's fused rows fit three
// blocks of 16 per wave (192).  Measured from 64-row chunks up (two lanes per KV head, under
// the plan's 32 splits): 0.085 against 0.12 ms on bf16 pages after 16 K tokens.
// 0 = no such lanes for this shape.
constexpr uint32_t kGroupedPrefillRows = 64;
inline uint32_t prefill_group_width(uint32_t format, uint32_t head_dim, uint32_t rows, uint32_t group) {
  if (format == KVX_FMT_INT4 || head_dim != 256 || rows < kGroupedPrefillRows) return 0;
  const uint32_t tile_fused = KVX_PREFILL_TILE_ROWS * group;
  const uint32_t width = 4 * tile_fused <= 192 ? 4u : 2 * tile_fused <= 192 ? 2u : 0u;
  // Groups of one or two query heads would leave three quarters of every wave's rows empty.
  return width * tile_fused >= 96 ? width : 0u;
}
// Whether the tiles of every such lane see the same number of pages, so that a lane cut into
// splits is each of its tiles cut into splits: lanes of four tiles (32 rows) when the chunk
// starts on a page boundary, lanes of two as for pairs.
inline bool prefill_group_splits_alike(uint32_t width, uint32_t committed) {
  return width == 4 ? committed % KVX_PAGE_TOKENS == 0 : prefill_tiles_pair(committed);
}
// Waves (row blocks) per (lane, split, KV head) of a verify launch.
inline uint32_t verify_row_blocks(uint32_t format, uint32_t fused_rows) {
  // bf16, fp8, int8 pages: 65 .. 128 fused rows run as four waves that share their pages
  // (bf16 up to 96 rows: as two waves of 48).
  if (format == KVX_FMT_BF16 && fused_rows > 64 && fused_rows <= 96) return 2;
  if (format != KVX_FMT_INT4 && fused_rows > 64 && fused_rows <= 128) return 4;
  const uint32_t rows = verify_block_rows(format, fused_rows);
  return (fused_rows + rows - 1) / rows;
}

// How many consecutive tiles of a chunked prefill at head dimension 64 or 128 share a workgroup
// and a staged page (prefill_group_small_kernel): 1 = tile by tile.  A history that ends on a
// page boundary is what gives the tiles that begin in the same 32 (or 16) rows of the chunk the
// same pages under the same splits.  As many tiles as keep four waves to a SIMD: a wave then
// holds the accumulators of two blocks of 16 fused rows at head dimension 64 and of one at 128
// (two at 128, on two waves a SIMD: 2048 rows over 16 384 tokens at 2 x 8 x 128 took 789 us
// against 742 tile by tile on int4 pages, 596 against 550 on bf16).  Groups make a launch
// of fewer workgroups, so a small launch stays tile by tile: where a tile alone leaves waves
// without a block the groups win from 256 workgroups on (8 x 4 x 64, 512 rows over 16 384 tokens,
// int4: 504 us against 484 at 256, 311 against 467 at 512), where it does not, from 1024
// (2 x 8 x 64, 2048 rows: 647 against 593 at 512, 454 against 562 at 1024).
inline uint32_t small_prefill_tiles_together(uint32_t D, uint32_t H, uint32_t G, uint32_t committed,
                                             uint32_t rows, uint32_t splits) {
  if ((D != 64 && D != 128) || committed % KVX_PAGE_TOKENS) return 1;
  const uint32_t blocks = (KVX_PREFILL_TILE_ROWS * G + 15) / 16, most = D == 64 ? 8u : 4u;
  const uint32_t together = 4 * blocks <= most ? 4u : 2 * blocks <= most ? 2u : 1u;
  const uint64_t tiles = (rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  if (together == 1 || tiles < 2) return 1;
  const uint64_t workgroups = (tiles + together - 1) / together * H * splits;
  return workgroups >= (blocks < 4 ? 256u : 1024u) ? together : 1u;
}

}  // namespace kvx

struct kvx_storage : kvx::Storage {};
