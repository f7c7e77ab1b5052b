// Host side of libkvx: layout geometry, planning rules, extent storage and the
// page pool.  No kernels here; device memory is reached through the HIP runtime.
#include "kvx_internal.h"

#include <algorithm>
#include <vector>
#include <chrono>
#include <cstring>
#include <limits>
#include <numeric>

namespace kvx {

static thread_local std::string g_last_error;

int fail(int code, const std::string &message) {
  g_last_error = message;
  return code;
}
int hip_fail(hipError_t error, const char *what) {
  g_last_error = std::string(what) + ": " + hipGetErrorString(error);
  (void)hipGetLastError();
  return KVX_EDEVICE;
}

uint64_t Storage::extent_bytes() const { return uint64_t(extent_pages) * bytes_per_page(); }
uint64_t Storage::bytes_per_page() const {
  return uint64_t(layout.layers) * 2 * (uint64_t(data_bytes) + scale_bytes);
}
uint32_t Storage::allocated_extents() const {
  uint32_t n = 0;
  for (void *e : extents) n += e != nullptr;
  return n;
}

namespace {

constexpr uint64_t kRegionAlignment = 64 * 1024;            // PagedKv.hpp:89
constexpr uint64_t kExtentTargetBytes = 128ull << 20;       // PagedKv.hpp:94

uint64_t gcd(uint64_t a, uint64_t b) { return b ? gcd(b, a % b) : a; }
uint64_t lcm(uint64_t a, uint64_t b) { return a && b ? a / gcd(a, b) * b : 0; }
uint64_t aligned_region_pages(uint64_t bytes) {
  return bytes ? kRegionAlignment / gcd(kRegionAlignment, bytes) : 0;
}
bool valid_format(uint32_t f) { return f >= KVX_FMT_INT8 && f <= KVX_FMT_FP8E4M3; }

}  // namespace
}  // namespace kvx

using namespace kvx;

// The page's spans in the reference's order: layer by layer, keys, key scales,
// values, value scales.
template <class F>
static int for_each_span(const kvx_storage *s, uint32_t page, F &&f) {
  if (page >= s->page_count) return fail(KVX_ERANGE, "invalid KV page id");
  auto *extent = static_cast<uint8_t *>(s->extents[page / s->extent_pages]);
  if (!extent)
    return fail(KVX_ESTATE,
                "KV page " + std::to_string(page) + " is in an extent that is not allocated");
  const uint32_t index = page % s->extent_pages;
  for (uint32_t layer = 0; layer < s->layout.layers; ++layer)
    for (uint32_t tensor = KVX_KEYS; tensor <= KVX_VALUE_SCALES; ++tensor) {
      const uint32_t bytes = (tensor & 1) ? s->scale_bytes : s->data_bytes;
      if (!bytes) continue;
      if (int rc = f(extent + kvx_kv_offset(s->extent_pages, s->data_bytes, s->scale_bytes, layer,
                                            tensor, index),
                     bytes))
        return rc;
    }
  return KVX_OK;
}
extern "C" {

const char *kvx_last_error(void) { return g_last_error.c_str(); }

// ---------------------------------------------------------------- layout ---
int kvx_layout_valid(const kvx_layout *l) {
  return l && l->layers && l->kv_heads && l->head_dim && valid_format(l->format);
}
// In 64 bits: the device-side forms (data_bytes_of, scale_bytes_of) hold for the layouts a
// storage accepts, these for whatever a caller asks about.
uint64_t kvx_layout_data_bytes_per_layer_page(const kvx_layout *l) {
  const uint64_t elements = uint64_t(KVX_PAGE_TOKENS) * l->kv_heads * l->head_dim;
  return l->format == KVX_FMT_BF16 ? elements * 2 : l->format == KVX_FMT_INT4 ? elements / 2 : elements;
}
uint64_t kvx_layout_scale_bytes_per_layer_page(const kvx_layout *l) {
  return quantized(l->format) ? uint64_t(KVX_PAGE_TOKENS) * l->kv_heads * 4 : 0;
}
uint64_t kvx_layout_bytes_per_layer_page(const kvx_layout *l) {
  return 2 * (kvx_layout_data_bytes_per_layer_page(l) + kvx_layout_scale_bytes_per_layer_page(l));
}
uint64_t kvx_layout_bytes_per_model_page(const kvx_layout *l) {
  return uint64_t(l->layers) * kvx_layout_bytes_per_layer_page(l);
}
uint32_t kvx_layout_extent_alignment_pages(const kvx_layout *l) {
  const uint64_t data = aligned_region_pages(kvx_layout_data_bytes_per_layer_page(l));
  if (l->format == KVX_FMT_BF16) return uint32_t(data);
  return uint32_t(lcm(data, aligned_region_pages(kvx_layout_scale_bytes_per_layer_page(l))));
}
uint32_t kvx_layout_minimum_extent_pages(const kvx_layout *l) {
  const uint64_t align = kvx_layout_extent_alignment_pages(l);
  const uint64_t unit = align * kvx_layout_bytes_per_model_page(l);
  if (!unit) return 0;
  const uint64_t units = std::max<uint64_t>(1, (kExtentTargetBytes / 2 + unit - 1) / unit);
  return uint32_t(units * align);
}
uint32_t kvx_layout_maximum_extent_pages(const kvx_layout *l) {
  const uint64_t align = kvx_layout_extent_alignment_pages(l);
  const uint64_t unit = align * kvx_layout_bytes_per_model_page(l);
  if (!unit) return 0;
  const uint64_t units = kExtentTargetBytes * 3 / 2 / unit;
  return std::max(uint32_t(units * align), kvx_layout_minimum_extent_pages(l));
}
uint32_t kvx_layout_extent_pages_for(const kvx_layout *l, uint64_t pages) {
  const uint32_t step = kvx_layout_extent_alignment_pages(l);
  const uint64_t smallest = kvx_layout_minimum_extent_pages(l);
  if (!smallest || pages < smallest) return 0;
  const uint64_t largest = std::min<uint64_t>(kvx_layout_maximum_extent_pages(l), pages);
  const uint64_t page_bytes = kvx_layout_bytes_per_model_page(l);
  uint64_t best = 0, best_left = 0, best_distance = 0;
  for (uint64_t candidate = smallest; candidate <= largest; candidate += step) {
    const uint64_t bytes = candidate * page_bytes;
    const uint64_t distance =
        bytes > kExtentTargetBytes ? bytes - kExtentTargetBytes : kExtentTargetBytes - bytes;
    const uint64_t left = pages % candidate;
    if (!best || left < best_left || (left == best_left && distance < best_distance)) {
      best = candidate;
      best_left = left;
      best_distance = distance;
    }
  }
  return uint32_t(best);
}
uint32_t kvx_layout_largest_extent_pages(const kvx_layout *l) {
  const uint64_t align = kvx_layout_extent_alignment_pages(l);
  const uint64_t page_bytes = kvx_layout_bytes_per_model_page(l);
  if (!align || !page_bytes) return 0;
  uint64_t pages = std::min<uint64_t>(KVX_PAGE_INDEX_MASK,
                                      std::numeric_limits<uint32_t>::max() / page_bytes);
  pages = pages / align * align;
  return uint32_t(pages);
}
uint64_t kvx_kv_offset(uint32_t extent_pages, uint32_t db, uint32_t sb, uint32_t layer,
                       uint32_t tensor, uint32_t index) {
  const RegionOffsets r = region_offsets(extent_pages, db, sb);
  const uint64_t region = uint64_t(layer) * extent_pages * 2 * (uint64_t(db) + sb);
  const uint64_t start[4] = {0, r.key_scales, r.values, r.value_scales};
  return region + start[tensor & 3] + uint64_t(index) * ((tensor & 1) ? sb : db);
}

// -------------------------------------------------------------- planning ---
static uint32_t pages_of(uint64_t tokens) {
  return uint32_t((tokens + KVX_PAGE_TOKENS - 1) / KVX_PAGE_TOKENS);
}
uint32_t kvx_verify_splits(uint32_t committed, uint32_t rows) {
  const uint32_t scaled = (pages_of(uint64_t(committed) + rows) + 15) / 16;
  return std::min(std::max(32u, scaled), KVX_VERIFY_MAX_SPLITS);
}
uint32_t kvx_prefill_splits(uint32_t rows) {
  const uint32_t tiles = (rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  if (!tiles) return KVX_PREFILL_MAX_SPLITS;
  return std::min(std::max(KVX_PREFILL_MAX_SPLITS / tiles, 1u), KVX_PREFILL_MAX_SPLITS);
}
uint32_t kvx_prefill_plan(uint32_t committed, uint32_t rows, uint32_t kv_heads, uint32_t query_heads,
                          uint32_t format) {
  return kvx_prefill_plan_batch(committed, rows, kv_heads, query_heads, format, 1);
}
uint32_t kvx_prefill_plan_batch(uint32_t committed, uint32_t rows, uint32_t kv_heads,
                                uint32_t query_heads, uint32_t format, uint32_t sequences) {
  if (!kv_heads || !query_heads || query_heads % kv_heads || !sequences) return 0;
  const uint32_t tiles = uint32_t((uint64_t(rows) + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS);
  if (!tiles) return 1;
  // wave counts saturate instead of wrapping (no shape the kernels take comes near)
  const auto times = [](uint64_t a, uint64_t b) {
    return b && a > std::numeric_limits<uint64_t>::max() / b ? std::numeric_limits<uint64_t>::max() : a * b;
  };
  const uint32_t group = query_heads / kv_heads, tile_fused = KVX_PREFILL_TILE_ROWS * group;
  const uint32_t pages = pages_of(uint64_t(committed) + rows);
  constexpr uint32_t kSimds = 1024;
  const uint32_t by_pages = std::max(1u, pages / 8);
  // bf16, fp8 and int8 pages, long chunks: lanes of several tiles, one workgroup per lane,
  // split and KV head, one workgroup per CU.  One split where that fills three quarters of
  // the CUs; else as many as fill them, where the lanes' tiles cut their pages alike.
  if (const uint32_t width = kvx::prefill_group_width(format, 256, rows, group)) {
    constexpr uint32_t kCus = 256;
    const uint64_t workgroups = times(times((tiles + width - 1) / width, kv_heads), sequences);
    if (workgroups >= 3 * kCus / 4) return 1;
    if (kvx::prefill_group_splits_alike(width, committed))
      return std::max(1u, std::min({uint32_t((kCus + workgroups - 1) / workgroups), by_pages,
                                    KVX_PREFILL_MAX_SPLITS}));
  }
  // One split: neighbouring tiles share a walk as lanes of 16 rows on the kernels
  // with two blocks of 16 fused rows per wave (int4: two waves per SIMD).
  const uint64_t paired_waves =
      times(times(times((uint64_t(tiles) + 1) / 2, kv_heads), (2 * uint64_t(tile_fused) + 31) / 32), sequences);
  const uint32_t paired_slots = kvx::prefill_paired_slots(format);
  if (tile_fused <= 16) return 1;
  // int4 pages, chunks whose paired waves fill a quarter of the slots or more: the waves of a
  // launch are equally long and take their slots round by round, so a last round that is
  // partly empty costs as much as a full one (2048 rows, one split: 1536 waves, 4.97 ms after
  // 65536 tokens; four splits, three full rounds: 3.84 ms; 1024 rows: 2.45 -> 1.9 ms).  The
  // fewest splits that leave every round at least nine tenths full, of at least 16 pages of
  // the average tile's history each (shorter ones cost more in set-up and partial rows than
  // the rounds win: 1024 rows with no history, 77 us in one split, 90 in two); failing that,
  // the fullest rounds.
  if (format == KVX_FMT_INT4 && paired_waves >= paired_slots / 4) {
    const uint32_t seen = pages_of(uint64_t(committed) + rows / 2);
    const uint32_t most = std::max(1u, std::min(seen / 16, KVX_PREFILL_MAX_SPLITS));
    uint32_t best = 1;
    uint64_t best_waves = 0, best_room = 1;
    for (uint32_t s = 1; s <= most; ++s) {
      if (s > 1 && !kvx::prefill_pairs_with_splits(format, committed, tiles, s, kv_heads, group)) continue;
      const uint64_t waves = times(paired_waves, s);
      if (waves > (1ull << 30)) return s;  // thousands of rounds: full by any count
      const uint64_t room = (waves + paired_slots - 1) / paired_slots * paired_slots;
      if (10 * waves >= 9 * room) return s;
      if (waves * best_room > best_waves * room) best = s, best_waves = waves, best_room = room;
    }
    return best;
  }
  if (paired_waves >= paired_slots / 2) return 1;
  // Tiles that pair under any split count keep their shared walks: as many
  // splits as fit one round of the paired kernels' slots.
  const uint32_t paired_splits =
      std::max(1u, std::min({uint32_t(paired_slots / paired_waves), by_pages, KVX_PREFILL_MAX_SPLITS}));
  if (paired_splits >= 2 &&
      kvx::prefill_pairs_with_splits(format, committed, tiles, paired_splits, kv_heads, group))
    return paired_splits;
  // Several splits: one lane per tile on the kernels with one block per wave
  // (two waves per SIMD except for bf16 pages).
  const uint32_t slots = format == KVX_FMT_BF16 ? kSimds : 2 * kSimds;
  const uint64_t per_split = times(times(times(tiles, kv_heads), (uint64_t(tile_fused) + 15) / 16), sequences);
  const uint32_t fit = uint32_t(slots / per_split);
  const uint32_t splits = std::min({fit, by_pages, KVX_PREFILL_MAX_SPLITS});
  return splits >= 2 ? splits : 1;
}
uint32_t kvx_decode_splits(uint32_t committed, uint32_t rows) {
  const uint32_t pages = pages_of(uint64_t(committed) + rows);
  const uint32_t wanted = (pages + KVX_DECODE_PAGES_PER_SPLIT - 1) / KVX_DECODE_PAGES_PER_SPLIT;
  return std::min(std::max(1u, wanted), KVX_VERIFY_MAX_SPLITS);
}
// The decode plan of the lanes of one launch (at most KVX_LANES_PER_LAUNCH).
static void decode_plan_of_launch(const uint32_t *committed, uint32_t n_lanes, uint32_t kv_heads,
                                  uint32_t format, uint32_t *split_counts) {
  // A launch runs (sum of splits) x KV heads waves.  One per SIMD of 256 CUs x 4
  // is the least that fills the GPU; shorter splits than 8 pages cost more in
  // set-up and partial rows than they win, except in a launch so small that splits of 8
  // pages leave half of the SIMDs empty (three quarters where the kernel runs one wave per
  // SIMD): there splits go down to 4 pages, unless that gives a lane more than 128 of them
  // to merge (one sequence of 8192 tokens: int4 21.1 -> 16.1, int8 24.0 -> 17.9, bf16 21.6 ->
  // 16.8 us; 2048 tokens, batches of 1 to 4: 19 -> 15, 22 -> 16, 19 -> 15 us; one sequence
  // of 32768 tokens loses 5 % to the longer merge).  What must not happen is a launch
  // with more waves than the kernel has wave slots: the overflow runs as a second
  // round on a nearly empty GPU (measured on 530 K tokens: int4 146 -> 115 us,
  // bf16 397 -> 350 us once the waves fit).  The int4 kernel holds two waves per
  // SIMD; the other formats' kernels are fastest with one wave per SIMD.
  constexpr uint64_t kSimds = 1024;
  const uint64_t slots = format == KVX_FMT_INT4 ? 2 * kSimds : kSimds;
  std::vector<uint32_t> pages(n_lanes);
  uint64_t page_heads = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) {
    pages[i] = pages_of(uint64_t(committed[i]) + 1);
    page_heads += uint64_t(pages[i]) * kv_heads;
  }
  uint32_t longest_lane = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) longest_lane = std::max(longest_lane, pages[i]);
  const uint64_t small_launch = format == KVX_FMT_INT4 ? 4 * kSimds : 2 * kSimds;  // page-heads
  const uint64_t shortest = (page_heads <= small_launch && longest_lane <= 512) ? 4 : 8;
  constexpr uint64_t kMostPages = KVX_MAX_PHYSICAL_TOKENS / KVX_PAGE_TOKENS + 1;  // one split per lane by then
  uint32_t per = uint32_t(std::min(std::max<uint64_t>((page_heads + kSimds - 1) / kSimds, shortest), kMostPages));
  if (format == KVX_FMT_INT4) per = std::min(per, KVX_DECODE_PAGES_PER_SPLIT);
  uint64_t waves = 0;
  for (;; ++per) {
    waves = 0;
    bool single = true;
    for (uint32_t i = 0; i < n_lanes; ++i) {
      split_counts[i] = std::min(std::max(1u, (pages[i] + per - 1) / per), KVX_DECODE_MAX_SPLITS);
      waves += uint64_t(split_counts[i]) * kv_heads;
      single = single && split_counts[i] == 1;
    }
    if (waves <= slots || single) break;  // one split per lane is the fewest waves there can be
  }
  if (format != KVX_FMT_INT4 || waves <= kSimds) return;
  // int4, a launch with two waves on most SIMDs.  The two do not share their SIMD evenly:
  // the wave that was dispatched first runs ahead of the other (measured on splits of equal
  // length: 2.05 against 3.9 us per page while both run), ends a quarter of the launch early
  // and leaves the other alone, and a lone wave of this kernel cannot keep its share of the
  // memory system busy.  So the lanes are planned in two classes: long splits for exactly the
  // first wave of every SIMD (the launch dispatches the lanes with the longest splits first,
  // the heads of a work item side by side), and splits of kPairedShortShare of that length
  // for the second, which then end together (same batch and GPU: 104 -> 100 us per launch, 1.83 -> 1.76 ms per
  // step; shares of 0.52 / 0.56 / 0.60 / 0.64 gave 1.80 / 1.767 / 1.761 / 1.785 ms).  Lanes
  // go to the long class from the longest down while their waves fit one per SIMD, lanes that
  // do not fit to the short class; the long length is the least whose short class fits the
  // second waves.
  constexpr double kPairedShortShare = 0.58;
  std::vector<uint32_t> order(n_lanes);
  for (uint32_t i = 0; i < n_lanes; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return pages[x] > pages[y]; });
  std::vector<uint32_t> paired(n_lanes);
  for (uint32_t longer = 8; longer <= KVX_MAX_PHYSICAL_TOKENS / KVX_PAGE_TOKENS; ++longer) {
    const uint32_t shorter = std::max(4u, uint32_t(kPairedShortShare * longer));
    uint64_t first_waves = 0, second_waves = 0;
    bool capped = false;
    for (uint32_t i : order) {
      const uint32_t as_long = (pages[i] + longer - 1) / longer;
      if (first_waves + uint64_t(as_long) * kv_heads <= kSimds) {
        paired[i] = as_long;
        first_waves += uint64_t(as_long) * kv_heads;
      } else {
        paired[i] = (pages[i] + shorter - 1) / shorter;
        second_waves += uint64_t(paired[i]) * kv_heads;
      }
      capped = capped || paired[i] > KVX_DECODE_MAX_SPLITS;
    }
    if (second_waves <= kSimds && !capped) {
      std::copy(paired.begin(), paired.end(), split_counts);
      break;
    }
  }
}
int kvx_decode_plan(const uint32_t *committed, uint32_t n_lanes, uint32_t kv_heads, uint32_t format,
                    uint32_t *split_counts) {
  if (!committed || !split_counts || !n_lanes || !kv_heads)
    return fail(KVX_EINVAL, "kvx_decode_plan: null argument or empty batch");
  for (uint32_t i = 0; i < n_lanes; ++i)
    if (uint64_t(committed[i]) + 1 > KVX_MAX_PHYSICAL_TOKENS)
      return fail(KVX_EINVAL, "kvx_decode_plan: context_out_of_range");
  // The attend calls take the lanes KVX_LANES_PER_LAUNCH at a time, in the caller's order,
  // and the launches follow one another: every launch is planned to fill the GPU by itself
  // (a batch of 128 sequences of 8192 tokens planned as one: 341 us; launch by launch: 220).
  for (uint32_t first = 0; first < n_lanes; first += KVX_LANES_PER_LAUNCH)
    decode_plan_of_launch(committed + first, std::min(KVX_LANES_PER_LAUNCH, n_lanes - first), kv_heads,
                          format, split_counts + first);
  return KVX_OK;
}
uint32_t kvx_prefill_plan_for(const kvx_layout *layout, uint32_t committed, uint32_t rows,
                              uint32_t query_heads, uint32_t sequences) {
  if (!kvx_layout_valid(layout) || !query_heads || query_heads % layout->kv_heads || !sequences) return 0;
  if (layout->head_dim != 64 && layout->head_dim != 128)
    return kvx_prefill_plan_batch(committed, rows, layout->kv_heads, query_heads, layout->format, sequences);
  // Head dimensions 64 and 128: a workgroup of four waves per (tile or group of tiles, KV head,
  // split), four of them to a CU at a time.  The fewest splits that make four rounds of them
  // (4096 workgroups), none shorter than 4 pages (2048 rows over 16 384 tokens, int4, in 1 / 2 /
  // 4 / 8 splits: 8 x 4 x 64 1562 / 1173 / 1092 / 1051 us, 2 x 8 x 128 1311 / 963 / 887 / 833;
  // 256 rows over 8192 tokens in 4 / 8 / 16 / 32: 173 / 116 / 96 / 102 and 132 / 97 / 82 / 88).
  // The sequences of a batch run one after the other at these head dimensions.
  const uint64_t tiles = (uint64_t(rows) + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  if (!tiles) return 1;
  const uint64_t seen = pages_of(uint64_t(committed) + rows / 2);
  const uint32_t most = uint32_t(std::max<uint64_t>(1, std::min<uint64_t>(seen / 4, KVX_PREFILL_MAX_SPLITS)));
  const uint32_t group = query_heads / layout->kv_heads;
  for (uint32_t s = 1; s < most; ++s) {
    const uint32_t together =
        kvx::small_prefill_tiles_together(layout->head_dim, layout->kv_heads, group, committed, rows, s);
    if ((tiles + together - 1) / together * layout->kv_heads * s >= 4096) return s;
  }
  return most;
}
int kvx_decode_plan_for(const kvx_layout *layout, const uint32_t *committed, uint32_t n_lanes,
                        uint32_t *split_counts) {
  if (!kvx_layout_valid(layout)) return fail(KVX_EINVAL, "kvx_decode_plan_for: invalid layout");
  if (layout->head_dim != 64 && layout->head_dim != 128)
    return kvx_decode_plan(committed, n_lanes, layout->kv_heads, layout->format, split_counts);
  if (!committed || !split_counts || !n_lanes)
    return fail(KVX_EINVAL, "kvx_decode_plan_for: null argument or empty batch");
  for (uint32_t i = 0; i < n_lanes; ++i)
    if (uint64_t(committed[i]) + 1 > KVX_MAX_PHYSICAL_TOKENS)
      return fail(KVX_EINVAL, "kvx_decode_plan_for: context_out_of_range");
  // Head dimensions 64 and 128: a wave per (lane, KV head, split) over a staged copy of the
  // page's values of its own, sixteen waves to a CU (eight at head dimension 128 over pages
  // other than int4, whose raw bytes take more registers); one round of them, splits of at
  // least 4 pages (32 sequences of 8192 tokens, int4, 2 x 8 x 128: 48 us at 64 splits, 51 at
  // 32, 60 at 128; 8 x 4 x 64: 83 us at 16, 82 at 32, 85 at 64; int8 2 x 8 x 128: 44 us at 32,
  // 49 at 64).  bf16 pages are read at close to the memory's rate with half as many waves, and
  // the other half only adds partial rows (2 x 8 x 128: 54 us at 16 splits, 55 at 32; 8 x 4 x 64:
  // 106 at 8, 110 at 16).
  const bool sixteen = layout->head_dim == 64 || layout->format == KVX_FMT_INT4;
  const uint64_t slots = (sixteen ? 4096 : 2048) / (layout->format == KVX_FMT_BF16 ? 2 : 1);
  for (uint32_t first = 0; first < n_lanes; first += KVX_LANES_PER_LAUNCH) {
    const uint32_t count = std::min(KVX_LANES_PER_LAUNCH, n_lanes - first);
    uint64_t page_heads = 0;
    for (uint32_t i = 0; i < count; ++i)
      page_heads += uint64_t(pages_of(uint64_t(committed[first + i]) + 1)) * layout->kv_heads;
    const uint64_t per = std::max<uint64_t>((page_heads + slots - 1) / slots, 4);
    for (uint32_t i = 0; i < count; ++i) {
      const uint64_t pages = pages_of(uint64_t(committed[first + i]) + 1);
      split_counts[first + i] =
          uint32_t(std::min<uint64_t>(std::max<uint64_t>(1, (pages + per - 1) / per), KVX_VERIFY_MAX_SPLITS));
    }
  }
  return KVX_OK;
}
// The verify plan of the lanes of one launch (at most KVX_LANES_PER_LAUNCH).
static void verify_plan_of_launch(const uint32_t *committed, uint32_t n_lanes, uint32_t rows,
                                  uint32_t kv_heads, uint32_t query_heads, uint32_t format,
                                  uint32_t *split_counts) {
  // The verify kernels keep 32 fused rows (16 when there are no more; all of 33 .. 48
  // on int4 pages) per wave and run one wave per SIMD, so a launch is (sum of splits) x KV heads x row blocks
  // waves: the plan is the longest split length that still gives every SIMD of
  // 256 CUs x 4 a wave, but no more waves than SIMDs, so that no second round of
  // waves starts on a nearly empty GPU; splits shorter than 8 pages cost more in
  // set-up and partial rows than they win.
  const uint32_t fused = rows * (query_heads / kv_heads);
  const uint32_t blocks = kvx::verify_row_blocks(format, fused);
  // The int4 kernel for lanes of more than 32 fused rows in blocks of 32 is built for two
  // waves per SIMD, and from 16 lanes on a launch is faster with them (16 lanes of 8192
  // tokens, 16 rows: 134 -> 118 us; 32 lanes of 4096: 152 -> 123 us); with fewer, longer
  // lanes the second wave's partial rows cost what it gains (4 lanes of 32768: 114 -> 131).
  const bool two_per_simd = format == KVX_FMT_INT4 && fused > 32 &&
                            kvx::verify_block_rows(format, fused) == 32 && n_lanes >= 16;
  const uint64_t kSimds = two_per_simd ? 2048 : 1024;
  uint64_t page_waves = 0;
  for (uint32_t i = 0; i < n_lanes; ++i)
    page_waves += uint64_t(pages_of(uint64_t(committed[i]) + rows)) * kv_heads * blocks;
  // A launch that splits of 8 pages would spread over a quarter of the SIMDs takes splits of 4
  // (one lane of 2048 tokens, 4 / 8 / 16 rows: 35 -> 26, 39 -> 30, 30 -> 25 us), unless that
  // gives a lane more than 128 splits.
  uint32_t longest_lane = 0;
  for (uint32_t i = 0; i < n_lanes; ++i)
    longest_lane = std::max(longest_lane, pages_of(uint64_t(committed[i]) + rows));
  const uint64_t shortest = (page_waves <= 2048 && longest_lane <= 512) ? 4 : 8;
  constexpr uint64_t kMostPages = KVX_MAX_PHYSICAL_TOKENS / KVX_PAGE_TOKENS + 1;  // one split per lane by then
  uint32_t per = uint32_t(std::min(std::max<uint64_t>((page_waves + kSimds - 1) / kSimds, shortest), kMostPages));
  for (;; ++per) {
    uint64_t waves = 0;
    for (uint32_t i = 0; i < n_lanes; ++i) {
      const uint32_t pages = pages_of(uint64_t(committed[i]) + rows);
      split_counts[i] = std::min(std::max(1u, (pages + per - 1) / per), KVX_VERIFY_MAX_SPLITS);
      waves += uint64_t(split_counts[i]) * kv_heads * blocks;
    }
    // One split per lane is the fewest waves there can be.
    if (waves <= kSimds || per >= KVX_MAX_PHYSICAL_TOKENS / KVX_PAGE_TOKENS) break;
    bool single = true;
    for (uint32_t i = 0; i < n_lanes; ++i) single = single && split_counts[i] == 1;
    if (single) break;
  }
}
int kvx_verify_plan(const uint32_t *committed, uint32_t n_lanes, uint32_t rows, uint32_t kv_heads,
                    uint32_t query_heads, uint32_t format, uint32_t *split_counts) {
  if (!committed || !split_counts || !n_lanes || !kv_heads || !rows || !query_heads ||
      query_heads % kv_heads)
    return fail(KVX_EINVAL, "kvx_verify_plan: null argument, empty batch or bad head counts");
  for (uint32_t i = 0; i < n_lanes; ++i)
    if (uint64_t(committed[i]) + rows > KVX_MAX_PHYSICAL_TOKENS)
      return fail(KVX_EINVAL, "kvx_verify_plan: context_out_of_range");
  // launch by launch, as kvx_decode_plan
  for (uint32_t first = 0; first < n_lanes; first += KVX_LANES_PER_LAUNCH)
    verify_plan_of_launch(committed + first, std::min(KVX_LANES_PER_LAUNCH, n_lanes - first), rows,
                          kv_heads, query_heads, format, split_counts + first);
  return KVX_OK;
}
int kvx_chunk_validation(const kvx_chunk_params *p) {
  if (!p->chunk_tokens || p->chunk_tokens > KVX_PREFILL_TOKEN_BUDGET) return 1;
  if (uint64_t(p->committed_tokens) + p->chunk_tokens > KVX_MAX_PHYSICAL_TOKENS) return 2;
  if (p->chunk_stride < p->chunk_tokens || p->chunk_stride > KVX_PREFILL_TOKEN_BUDGET ||
      p->chunk_stride % KVX_PAGE_TOKENS)
    return 3;
  if (p->page_table_entries < pages_of(uint64_t(p->committed_tokens) + p->chunk_tokens)) return 4;
  return 0;
}
static int geometry_ok(uint32_t query_heads, const kvx_layout *l) {
  if (!kvx_layout_valid(l) || !query_heads || query_heads % l->kv_heads)
    return fail(KVX_EINVAL, "query heads are not a multiple of the layout's KV heads");
  return KVX_OK;
}
static void workspace_rows(uint64_t rows, uint32_t head_dim, uint64_t *pb, uint64_t *sb) {
  if (pb) *pb = rows * head_dim * sizeof(float);
  if (sb) *sb = rows * 2 * sizeof(float);
}
int kvx_prefill_workspace(uint32_t rows, uint32_t query_heads, const kvx_layout *l, uint64_t *pb,
                          uint64_t *sb) {
  if (int rc = geometry_ok(query_heads, l)) return rc;
  if (!rows || rows > KVX_PREFILL_TOKEN_BUDGET)
    return fail(KVX_EINVAL, "invalid paged prefill attention geometry");
  const uint64_t tiles = (rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  workspace_rows(tiles * kvx_prefill_splits(rows) * KVX_PREFILL_TILE_ROWS * query_heads,
                 l->head_dim, pb, sb);
  return KVX_OK;
}
int kvx_prefill_workspace_for(uint32_t rows, uint32_t split_count, uint32_t query_heads,
                              const kvx_layout *l, uint64_t *pb, uint64_t *sb) {
  if (int rc = geometry_ok(query_heads, l)) return rc;
  if (!rows || rows > KVX_PREFILL_TOKEN_BUDGET || !split_count ||
      split_count > KVX_PREFILL_MAX_SPLITS)
    return fail(KVX_EINVAL, "invalid paged prefill attention geometry");
  const uint64_t tiles = (rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  workspace_rows(tiles * split_count * KVX_PREFILL_TILE_ROWS * query_heads, l->head_dim, pb, sb);
  return KVX_OK;
}
int kvx_prefill_workspace_bound(uint32_t maximum_rows, uint32_t query_heads, const kvx_layout *l,
                                uint64_t *pb, uint64_t *sb) {
  if (int rc = geometry_ok(query_heads, l)) return rc;
  if (!maximum_rows || maximum_rows > KVX_PREFILL_TOKEN_BUDGET)
    return fail(KVX_EINVAL, "invalid attention workspace rows");
  uint64_t slots = 0;
  for (uint32_t rows = 1; rows <= maximum_rows; rows += KVX_PREFILL_TILE_ROWS) {
    const uint64_t tiles = (rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
    slots = std::max(slots, tiles * kvx_prefill_splits(rows));
  }
  workspace_rows(slots * KVX_PREFILL_TILE_ROWS * query_heads, l->head_dim, pb, sb);
  return KVX_OK;
}
int kvx_verify_workspace(uint32_t lanes, uint32_t row_capacity, uint32_t query_heads,
                         const kvx_layout *l, uint64_t *pb, uint64_t *sb) {
  if (int rc = geometry_ok(query_heads, l)) return rc;
  if (!lanes || !row_capacity) return fail(KVX_EINVAL, "invalid attention workspace batch width");
  workspace_rows(uint64_t(lanes) * row_capacity * KVX_VERIFY_MAX_SPLITS * query_heads, l->head_dim,
                 pb, sb);
  return KVX_OK;
}
uint64_t kvx_attend_workspace_bytes(const kvx_verify_params *lanes, uint32_t n, uint32_t query_heads,
                                    const kvx_layout *l) {
  uint64_t rows = 0;
  for (uint32_t i = 0; i < n; ++i)
    rows += uint64_t(lanes[i].split_count) * lanes[i].row_capacity * query_heads;
  const uint64_t partials = (rows * l->head_dim * sizeof(float) + 255) / 256 * 256;
  return partials + rows * 2 * sizeof(float);
}

// --------------------------------------------------------------- storage ---
static int storage_create(const kvx_layout *layout, uint32_t page_count, uint32_t extent_pages,
                          int aligned, bool accounting, kvx_storage **out) {
  if (!out) return fail(KVX_EINVAL, "null output");
  *out = nullptr;
  if (!kvx_layout_valid(layout)) return fail(KVX_EINVAL, "KV page storage layout is invalid");
  if (layout->head_dim != 64 && layout->head_dim != 128 && layout->head_dim != 256)
    return fail(KVX_EINVAL, "head dimension must be 64, 128 or 256");
  // The kernels index a page's bytes in 32 bits.
  if (layout->kv_heads > 4096 || layout->layers > 65536)
    return fail(KVX_EINVAL, "more than 4096 KV heads or 65536 layers");
  const uint64_t extent_bytes = uint64_t(extent_pages) * kvx_layout_bytes_per_model_page(layout);
  if (!extent_pages || (aligned && extent_pages % kvx_layout_extent_alignment_pages(layout)) ||
      extent_pages > KVX_PAGE_INDEX_MASK ||
      extent_bytes > std::numeric_limits<uint32_t>::max())
    return fail(KVX_EINVAL, "KV extent geometry is invalid");
  if (!page_count || page_count % extent_pages)
    return fail(KVX_EINVAL, "KV page pool is not a whole number of extents");
  if (page_count / extent_pages > (1u << 20))
    return fail(KVX_EINVAL, "KV page pool of more than 1048576 extents");
  auto *s = new kvx_storage;
  s->layout = *layout;
  s->page_count = page_count;
  s->extent_pages = extent_pages;
  s->data_bytes = uint32_t(kvx_layout_data_bytes_per_layer_page(layout));
  s->scale_bytes = uint32_t(kvx_layout_scale_bytes_per_layer_page(layout));
  s->extents.assign(page_count / extent_pages, nullptr);
  s->allocations.assign(page_count / extent_pages, nullptr);
  s->accounting = accounting;
  if (!accounting && hipGetDevice(&s->device) != hipSuccess) {
    delete s;
    return fail(KVX_EDEVICE, "no HIP device: the paged KV path needs a GPU");
  }
  // The static workspace's address on this device, asked here so that no launch has to
  // (a launch may be under stream capture).  A refusal only matters to the entry that
  // uses the workspace, which then reports it.
  if (!accounting && kvx::prime_static_workspace(s->device) != KVX_OK) (void)hipGetLastError();
  *out = s;
  return KVX_OK;
}
int kvx_storage_create(const kvx_layout *layout, uint32_t page_count, uint32_t extent_pages,
                       int aligned, kvx_storage **out) {
  return storage_create(layout, page_count, extent_pages, aligned, false, out);
}
int kvx_storage_create_accounting(const kvx_layout *layout, uint32_t page_count,
                                  uint32_t extent_pages, int aligned, kvx_storage **out) {
  return storage_create(layout, page_count, extent_pages, aligned, true, out);
}
void kvx_storage_destroy(kvx_storage *s) {
  if (!s) return;
  if (!s->accounting) (void)hipDeviceSynchronize();
  for (void *raw : s->allocations)
    if (raw) (void)hipFree(raw);
  delete s;
}
uint32_t kvx_storage_page_count(const kvx_storage *s) { return s->page_count; }
uint32_t kvx_storage_extent_pages(const kvx_storage *s) { return s->extent_pages; }
uint64_t kvx_storage_bytes_per_page(const kvx_storage *s) { return s->bytes_per_page(); }
uint64_t kvx_storage_extent_bytes(const kvx_storage *s) { return s->extent_bytes(); }
uint64_t kvx_storage_allocated_bytes(const kvx_storage *s) {
  return uint64_t(s->allocated_extents()) * s->extent_bytes();
}
int kvx_storage_is_allocated(const kvx_storage *s, uint32_t page) {
  return page < s->page_count && s->extents[page / s->extent_pages] != nullptr;
}
void kvx_storage_set_budget(kvx_storage *s, uint64_t bytes) { s->budget_bytes = bytes; }

int kvx_storage_allocate_extent(kvx_storage *s, uint32_t extent) {
  if (extent >= s->extents.size()) return fail(KVX_ERANGE, "KV extent is past the pool");
  if (s->extents[extent])
    return fail(KVX_ESTATE, "KV extent " + std::to_string(extent) + " is already allocated");
  const uint64_t bytes = s->extent_bytes();
  if (s->budget_bytes && kvx_storage_allocated_bytes(s) + bytes > s->budget_bytes)
    return fail(KVX_ENOMEM, "KV extent refused by the storage budget");
  // Page entries keep the page index in the low 14 bits of the extent address.
  // Large allocations come back aligned far beyond that; a small test extent
  // may not, and is then allocated again with room to align inside it.
  constexpr uint64_t kAlign = uint64_t(KVX_PAGE_INDEX_MASK) + 1;
  if (s->accounting) {  // a distinct, aligned, never dereferenced address per extent
    s->extents[extent] = reinterpret_cast<void *>(uint64_t(extent + 1) << 32);
    return KVX_OK;
  }
  void *raw = nullptr;
  if (hipMalloc(&raw, bytes) != hipSuccess || !raw) {
    (void)hipGetLastError();
    return fail(KVX_ENOMEM, "hipMalloc refused a KV extent of " + std::to_string(bytes) + " bytes");
  }
  if (reinterpret_cast<uint64_t>(raw) & KVX_PAGE_INDEX_MASK) {
    (void)hipFree(raw);
    raw = nullptr;
    if (hipMalloc(&raw, bytes + kAlign) != hipSuccess || !raw) {
      (void)hipGetLastError();
      return fail(KVX_ENOMEM, "hipMalloc refused a KV extent of " + std::to_string(bytes) + " bytes");
    }
  }
  void *p = reinterpret_cast<void *>((reinterpret_cast<uint64_t>(raw) + kAlign - 1) & ~(kAlign - 1));
  if (hipMemset(p, 0, bytes) != hipSuccess) {
    (void)hipFree(raw);
    return hip_fail(hipGetLastError(), "hipMemset(extent)");
  }
  s->extents[extent] = p;
  s->allocations[extent] = raw;
  return KVX_OK;
}
int kvx_storage_release_extent(kvx_storage *s, uint32_t extent) {
  if (extent >= s->extents.size()) return fail(KVX_ERANGE, "KV extent is past the pool");
  if (!s->extents[extent])
    return fail(KVX_ESTATE, "KV extent " + std::to_string(extent) + " is not allocated");
  if (s->accounting) {
    s->extents[extent] = nullptr;
    return KVX_OK;
  }
  // Kernels reach extents through page tables without retaining them: wait for
  // everything in flight before the memory goes away.
  KVX_HIP(hipDeviceSynchronize());
  KVX_HIP(hipFree(s->allocations[extent]));
  s->extents[extent] = nullptr;
  s->allocations[extent] = nullptr;
  return KVX_OK;
}
int kvx_storage_layer(const kvx_storage *s, uint32_t layer, kvx_kv_layer *out) {
  if (layer >= s->layout.layers) return fail(KVX_ERANGE, "KV layer is outside the layout");
  out->extent_pages = s->extent_pages;
  out->offset = uint32_t(kvx_kv_offset(s->extent_pages, s->data_bytes, s->scale_bytes, layer,
                                       KVX_KEYS, 0));
  return KVX_OK;
}
int kvx_storage_entries(const kvx_storage *s, const uint32_t *pages, uint32_t n, uint32_t first,
                        uint64_t *table) {
  if (first > n)
    return fail(KVX_EINVAL, "KV page table entries start past the end of its pages");
  for (uint32_t i = first; i < n; ++i) {
    if (pages[i] >= s->page_count) return fail(KVX_ERANGE, "invalid KV page id");
    const uint32_t extent = pages[i] / s->extent_pages;
    if (!s->extents[extent])
      return fail(KVX_ESTATE, "KV page " + std::to_string(pages[i]) +
                                  " is in an extent that is not allocated");
  }
  for (uint32_t i = first; i < n; ++i) {
    const uint32_t extent = pages[i] / s->extent_pages;
    table[i] = reinterpret_cast<uint64_t>(s->extents[extent]) | (pages[i] - extent * s->extent_pages);
  }
  return KVX_OK;
}
int kvx_storage_write_entries(const kvx_storage *s, const uint32_t *pages, uint32_t n,
                              uint32_t first, uint64_t *table_device, uint64_t capacity,
                              void *stream) {
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory");
  if (!table_device || capacity < n)
    return fail(KVX_ESTATE, "KV page table is missing or too small for its entries");
  std::vector<uint64_t> host(n);
  if (int rc = kvx_storage_entries(s, pages, n, first, host.data())) return rc;
  if (first == n) return KVX_OK;
  // The staging vector dies with this call, so the copy completes here.
  KVX_HIP(hipMemcpyAsync(table_device + first, host.data() + first, (n - first) * sizeof(uint64_t),
                         hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
  KVX_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return KVX_OK;
}

int kvx_storage_page_read(const kvx_storage *s, uint32_t page, void *host) {
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory");
  auto *out = static_cast<uint8_t *>(host);
  KVX_HIP(hipDeviceSynchronize());
  return for_each_span(s, page, [&](uint8_t *device, uint32_t bytes) -> int {
    KVX_HIP(hipMemcpy(out, device, bytes, hipMemcpyDeviceToHost));
    out += bytes;
    return KVX_OK;
  });
}
int kvx_storage_page_write(kvx_storage *s, uint32_t page, const void *host) {
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory");
  auto *in = static_cast<const uint8_t *>(host);
  KVX_HIP(hipDeviceSynchronize());
  return for_each_span(s, page, [&](uint8_t *device, uint32_t bytes) -> int {
    KVX_HIP(hipMemcpy(device, in, bytes, hipMemcpyHostToDevice));
    in += bytes;
    return KVX_OK;
  });
}
static int extent_range(const kvx_storage *s, uint32_t extent, uint64_t offset, uint64_t bytes) {
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory");
  if (extent >= s->extents.size()) return fail(KVX_ERANGE, "KV extent is past the pool");
  if (!s->extents[extent]) return fail(KVX_ESTATE, "KV extent is not allocated");
  if (offset > s->extent_bytes() || bytes > s->extent_bytes() - offset)
    return fail(KVX_ERANGE, "range is outside the extent");
  return KVX_OK;
}
int kvx_storage_extent_read(const kvx_storage *s, uint32_t extent, uint64_t offset, uint64_t bytes,
                            void *host) {
  if (int rc = extent_range(s, extent, offset, bytes)) return rc;
  KVX_HIP(hipDeviceSynchronize());
  KVX_HIP(hipMemcpy(host, static_cast<uint8_t *>(s->extents[extent]) + offset, bytes,
                    hipMemcpyDeviceToHost));
  return KVX_OK;
}
int kvx_storage_extent_write(kvx_storage *s, uint32_t extent, uint64_t offset, uint64_t bytes,
                             const void *host) {
  if (int rc = extent_range(s, extent, offset, bytes)) return rc;
  KVX_HIP(hipDeviceSynchronize());
  KVX_HIP(hipMemcpy(static_cast<uint8_t *>(s->extents[extent]) + offset, host, bytes,
                    hipMemcpyHostToDevice));
  return KVX_OK;
}

int kvx_tree_masks(const uint32_t *parents, uint32_t rows, uint32_t *masks) {
  if (!parents || !masks || rows > 32) return kvx::fail(KVX_EINVAL, "verify tree has at most 32 rows");
  for (uint32_t row = 0; row < rows; ++row) {
    const uint32_t parent = parents[row];
    if (parent != KVX_TREE_NO_PARENT && parent >= row)
      return kvx::fail(KVX_EINVAL, "a tree row's parent must be an earlier row");
    // Row 0 is the anchor; a later row without a parent is dead.
    if (row && parent == KVX_TREE_NO_PARENT) {
      masks[row] = 0;
      continue;
    }
    uint32_t mask = 1u << row;
    for (uint32_t above = parent; above != KVX_TREE_NO_PARENT; above = parents[above])
      mask |= 1u << above;
    masks[row] = mask;
  }
  return KVX_OK;
}

int kvx_tree_path_valid(const uint32_t *parents, uint32_t rows, const uint32_t *path,
                        uint32_t retained) {
  if (!parents || !path || !retained || path[0] != 0) return 0;
  for (uint32_t i = 1; i < retained; ++i)
    if (path[i] >= rows || path[i] <= path[i - 1] || parents[path[i]] != path[i - 1]) return 0;
  return 1;
}

}  // extern "C"
