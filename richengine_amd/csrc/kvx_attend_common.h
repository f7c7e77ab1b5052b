// Shared by the matrix-core (MFMA) attention kernels: lane arguments, the
// per-row visibility rule, the merge kernel and the launch sequence.
#pragma once

#include <algorithm>

#include "kvx_device.h"

namespace kvx {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
#define KVX_GLOBAL __attribute__((address_space(1)))

// Loads through pointers rebuilt from page entries: say they are global memory
// so the compiler emits global_load rather than flat_load.
// Page bytes.  REUSED = false: read once by the launch (decode, verify), so the
// load carries the non-temporal hint and does not displace anything in the
// caches.  REUSED = true: the tiles of a chunked prefill walk the same pages
// hundreds of times, and with the hint every one of those walks went past the L2
// (bf16 prefill 4.0 -> 2.9 ms once the pages were allowed to stay).
template <class T, bool REUSED = false>
__device__ __forceinline__ T load_streaming(const uint8_t *p) {
  if constexpr (REUSED)
    return *reinterpret_cast<const KVX_GLOBAL T *>(reinterpret_cast<uintptr_t>(p));
  else
    return __builtin_nontemporal_load(reinterpret_cast<const KVX_GLOBAL T *>(
        reinterpret_cast<uintptr_t>(p)));
}
template <class T>
__device__ __forceinline__ T load_global(const void *p) {
  return *reinterpret_cast<const KVX_GLOBAL T *>(reinterpret_cast<uintptr_t>(p));
}

// A page-table entry through the scalar unit: the table pointer and the slot are the
// same in every lane, and a table is not written while a launch reads it, so the entry
// can come through the constant path (s_load) into scalar registers.  A vector load
// would return in order behind every page load in flight, and the wait for it would
// drain them; a scalar load waits on its own counter.
__device__ __forceinline__ uint64_t scalar_entry(const uint64_t *table, uint32_t slot) {
  typedef __attribute__((address_space(4))) const uint64_t ConstantEntry;
  return *reinterpret_cast<ConstantEntry *>(reinterpret_cast<uintptr_t>(table + slot));
}

// Stores through pointers rebuilt from page entries, as global memory.  A flat
// store would do, but while one is pending the compiler has to assume that memory
// operations complete out of order, and every wait for a page load after it, the
// ones in the page loop included, becomes a wait for all loads in flight.
template <class T>
__device__ __forceinline__ void store_global(void *p, T value) {
  *reinterpret_cast<KVX_GLOBAL T *>(reinterpret_cast<uintptr_t>(p)) = value;
}

constexpr uint32_t kPage = KVX_PAGE_TOKENS;
constexpr uint32_t kLanes = KVX_LANES_PER_LAUNCH;
constexpr uint32_t kD = 256;
constexpr float kLog2e = 1.4426950408889634f;

struct DecodeLane {
  const uint64_t *table;
  const uint32_t *masks;  // tree verify: ancestor bitmask per row; null = causal chain
  uint32_t committed;
  uint32_t active_rows;   // query rows attended (1 for decode)
  uint32_t split_count;
  uint32_t first_item;  // first (lane, split) work item of this lane
  float score_scale;
  uint32_t source;      // the lane's place among the launch's lanes as the caller passed them
  uint64_t row_base;    // first fused row of the lane's slots in the workspace
  uint64_t q_offset;    // element offset of the lane's queries
};
struct DecodeArgs {
  // First work item of every lane again, side by side (unused lanes hold the largest
  // value): a wave finds its lane from these with a few wide scalar loads instead of
  // walking the lane records, whose loads would follow one another.
  uint32_t item_base[kLanes];
  DecodeLane lane[kLanes];
  uint32_t n_lanes;
  uint32_t kv_heads;
  uint32_t group;
  uint32_t row_stride;
  uint32_t fused_rows;  // row capacity x group: fused query rows per (lane, KV head)
  kvx_kv_layer kv;
  // One-row decode with the step's token appended by the kernel itself: the
  // bf16 chunk rows of the launch's first lane ([head][stride][D] keys,
  // [head][D][stride] values, token 0 of each lane's chunk); null = the rows are
  // in the pages already.
  const uint16_t *chunk_keys;
  const uint16_t *chunk_values;
  uint64_t chunk_lane_stride;
  uint32_t chunk_stride;
  // Regular lanes (the tiles of a chunked prefill): tile_lanes > 0 means lane[0]
  // describes the first of that many lanes over one page table, each tile_rows
  // query rows and committed tokens after the one before, its queries
  // tile_lane_stride elements further on; the last holds tile_last_rows rows.
  // Any number of them fits one launch.  With tile_per_sequence < tile_lanes the
  // lanes are runs of tile_per_sequence lanes, one run per sequence of a batch of equal
  // chunks: lane[s] describes the first lane of run s.
  uint32_t tile_lanes;
  uint32_t tile_rows;
  uint32_t tile_last_rows;
  uint32_t tile_per_sequence;
  uint64_t tile_lane_stride;
  // The merge's second output (see Epilogue): hidden rows of the launch's first
  // lane onwards, and the packed rows their gates come from (null = no gate).
  // With `hidden` every split writes partials, the only split of a short lane
  // too, so that the merge produces every row.
  uint16_t *hidden;
  const uint16_t *packed_qkv;
  uint32_t all_partials;
  // Work items in the grid's y and KV heads in its x (the heads of an item are dispatched
  // side by side and the items in the order of the lane records) instead of items in x.
  uint32_t item_major;
};

// The lane with this index of a launch: read from the arguments, or derived
// from the first for regular lanes.
__device__ __forceinline__ DecodeLane lane_at(const DecodeArgs &a, uint32_t index) {
  // Field by field from a reference into the kernel arguments: a copy of a whole
  // lane record picked by a run-time index would make the compiler move the
  // argument block to scratch memory.
  uint32_t tile = 0, record = index;
  if (a.tile_lanes) {
    record = a.tile_per_sequence < a.tile_lanes ? index / a.tile_per_sequence : 0u;
    tile = index - record * a.tile_per_sequence;
  }
  const DecodeLane &from = a.lane[record];
  DecodeLane l;
  l.table = from.table;
  l.masks = from.masks;
  l.committed = from.committed + tile * a.tile_rows;
  l.active_rows =
      (a.tile_lanes && tile + 1 == a.tile_per_sequence) ? a.tile_last_rows : from.active_rows;
  l.split_count = from.split_count;
  l.first_item = a.tile_lanes ? index * from.split_count : from.first_item;
  l.score_scale = from.score_scale;
  l.source = a.tile_lanes ? index : from.source;
  l.row_base = from.row_base + uint64_t(tile) * from.split_count * a.kv_heads * a.fused_rows;
  l.q_offset = from.q_offset + tile * a.tile_lane_stride;
  return l;
}
// The lane that owns work item `item` (a lane's items are its splits), and its index.
__device__ __forceinline__ DecodeLane lane_of_item(const DecodeArgs &a, uint32_t item, uint32_t &index) {
  index = 0;
  if (a.tile_lanes) {
    index = item / a.lane[0].split_count;
  } else {
    // item_base is non-decreasing: the lane is the number of later lanes that
    // start at or before the item.
#pragma unroll
    for (uint32_t i = 1; i < kLanes; ++i) index += item >= a.item_base[i] ? 1u : 0u;
  }
  return lane_at(a, index);
}
// What a fused append brings to a launch (host side).
struct FusedAppend {
  const void *keys, *values;
  uint64_t lane_stride;
  uint32_t stride;
};

// Which tokens one fused query row (an MFMA column) may see
// (reference: common/paged_attention_tile.h:141-143).
struct Sight {
  uint32_t committed;
  uint32_t visible;  // committed + active rows
  uint32_t limit;    // chain: first token the row may not see
  uint32_t mask;     // tree: the row's ancestor bits over tokens committed + i
  bool tree;
  __device__ __forceinline__ bool sees(uint32_t token) const {
    if (tree)
      return token < committed || (token < visible && ((mask >> ((token - committed) & 31u)) & 1u));
    return token < limit;
  }
};

// Merge of one fused query row over the splits of its (sequence, KV head)
// (reference: common/paged_attention_tile.h:362-417).  Each lane owns four
// consecutive dimensions.  The statistics of up to 64 splits are fetched at
// once, one split per lane, so the maximum and the weights cost one load
// latency; the partial rows then stream with several loads in flight.
//
// The order of the sums is fixed, which keeps the result a function of the
// inputs and the split count alone: up to kMergeSequential splits are summed
// in split order by one wave, as the reference does; longer lists (small
// batches over long contexts) are cut into kMergeWaves consecutive ranges, one
// per wave, each summed in split order, and the ranges are then added in range
// order.  Eight ranges (two waves per SIMD, so a wave may hold 20 partial rows in
// registers): a range of a list of up to 160 splits is requested at once, statistics
// and partial rows together, and the merge costs little more than one round trip to
// memory; longer lists take one more per 20 splits of a range.
constexpr uint32_t kMergeSequential = 32;
constexpr uint32_t kMergeWaves = 8;
// Partial rows a wave has in flight at a time.  One wave per row (lists of up to
// kMergeSequential splits): 16, the average list of a mixed batch at 32 pages per split.
// A wave of the ranged form: 20, which is what two waves per SIMD leave registers for.
constexpr uint32_t kMergeAhead = 16;
constexpr uint32_t kMergeAheadRanged = 20;

struct MergeSums {
  f32x4 numerator;
  float denominator;
};

// Sums splits [first, last) of the row in split order; `maximum` is the row's
// maximum over all splits.  `early` holds the partial rows of the range's first
// kMergeAhead splits (clamped to the last) and `early_stat` the statistics of split
// first + lane, loaded before the caller waited for anything.
template <uint32_t AHEAD>
__device__ __forceinline__ MergeSums merge_range(const float *__restrict__ partials,
                                                 const float *__restrict__ statistics,
                                                 uint64_t first_row, uint32_t first, uint32_t last,
                                                 uint32_t M, float maximum, uint32_t lane,
                                                 const f32x4 (&early)[AHEAD], f32x2 early_stat) {
  MergeSums sums{{0.0f, 0.0f, 0.0f, 0.0f}, 0.0f};
  // One batch of up to AHEAD splits from `base + i` on, in split order; the weights
  // and terms of the 64 splits from `base` on sit one per lane.
  const auto add_batch = [&](const f32x4 (&part)[AHEAD], uint32_t i, uint32_t count,
                             float my_weight, float my_term) {
#pragma unroll
    for (uint32_t u = 0; u < AHEAD; ++u) {
      if (i + u < count) {
        const float weight = __shfl(my_weight, i + u);
#pragma unroll
        for (uint32_t c = 0; c < 4; ++c)
          sums.numerator[c] = __fadd_rn(sums.numerator[c], __fmul_rn(weight, part[u][c]));
        sums.denominator = __fadd_rn(sums.denominator, __shfl(my_term, i + u));
      }
    }
  };
  for (uint32_t base = first; base < last; base += 64) {
    const uint32_t mine = base + lane;
    f32x2 stat = {-INFINITY, 0.0f};
    if (base == first) {
      stat = early_stat;
    } else if (mine < last) {
      stat = load_global<f32x2>(statistics + (first_row + uint64_t(mine) * M) * 2);
    }
    const float my_weight = expf(__fsub_rn(stat[0], maximum));
    const float my_term = __fmul_rn(my_weight, stat[1]);
    const uint32_t count = min(64u, last - base);
    uint32_t i = 0;
    if (base == first) {  // the batch that was requested ahead
      add_batch(early, 0, count, my_weight, my_term);
      i = AHEAD;
    }
    for (; i < count; i += AHEAD) {
      f32x4 part[AHEAD];
#pragma unroll
      for (uint32_t u = 0; u < AHEAD; ++u) {
        const uint64_t row = first_row + uint64_t(base + min(i + u, count - 1)) * M;
        part[u] = load_global<f32x4>(partials + row * kD + 4 * lane);
      }
      add_batch(part, i, count, my_weight, my_term);
    }
  }
  return sums;
}

// grid (fused query row, KV head, lane), WAVES waves per row: one for launches whose
// longest list has at most kMergeSequential splits, else kMergeWaves.  Lanes whose pages
// fit one split were written by the split kernel itself.
template <uint32_t WAVES, uint32_t AHEAD>
__global__ __launch_bounds__(64 * WAVES) void matrix_merge_kernel(
    uint16_t *__restrict__ output, const float *__restrict__ partials,
    const float *__restrict__ statistics, DecodeArgs a) {
  const uint32_t j = blockIdx.x, head = blockIdx.y;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const DecodeLane l = lane_at(a, blockIdx.z);
  const uint32_t pages = (l.committed + l.active_rows + kPage - 1) / kPage;
  const uint32_t per = (pages + l.split_count - 1) / l.split_count;
  const uint32_t written = (pages + per - 1) / per;
  if (written <= 1 && !a.all_partials) return;
  const uint32_t G = a.group, M = a.fused_rows;
  uint16_t *out_row =
      output ? output + l.q_offset + uint64_t(head) * a.row_stride * G * kD + uint64_t(j) * kD
             : nullptr;
  // The row's place in the out-projection's operand and in the packed rows:
  // [lane][row][query head], the gate D elements after the head's query.
  const uint64_t hidden_row = uint64_t(l.source) * (M / G) + j / G;
  const uint32_t query_head = head * G + j % G;
  uint16_t *hidden_out =
      a.hidden ? a.hidden + (hidden_row * a.kv_heads * G + query_head) * kD + 4 * lane : nullptr;
  if (j / G >= l.active_rows) {  // rows past the live ones read as zeros
    if (wave == 0) {
      if (out_row) *reinterpret_cast<u32x2 *>(out_row + 4 * lane) = u32x2{0u, 0u};
      if (hidden_out) *reinterpret_cast<u32x2 *>(hidden_out) = u32x2{0u, 0u};
    }
    return;
  }
  u32x2 gates = {0u, 0u};
  if (a.packed_qkv && wave == 0)
    gates = load_global<u32x2>(a.packed_qkv +
                               hidden_row * (2ull * a.kv_heads * G + 2ull * a.kv_heads) * kD +
                               uint64_t(query_head) * 2 * kD + kD + 4 * lane);
  const uint64_t first_row = l.row_base + uint64_t(head) * l.split_count * M + j;
  const bool sequential = WAVES == 1 || written <= kMergeSequential;
  if (sequential && wave) return;
  // A wave's range of the list: all of it for the sequential case (at most kMergeSequential
  // splits), else one of kMergeWaves consecutive shares (at most 32 splits of 512).  Its
  // statistics and its first kMergeAhead partial rows are requested together, before
  // anything waits.
  const uint32_t share = sequential ? written : (written + WAVES - 1) / WAVES;
  const uint32_t first = min(written, wave * share), last = min(written, first + share);
  const uint32_t count = last - first;
  f32x4 early[AHEAD];
  f32x2 early_stat = {-INFINITY, 0.0f};
  if (lane < count)
    early_stat = load_global<f32x2>(statistics + (first_row + uint64_t(first + lane) * M) * 2);
#pragma unroll
  for (uint32_t u = 0; u < AHEAD; ++u)
    early[u] = count ? load_global<f32x4>(partials +
                                          (first_row + uint64_t(first + min(u, count - 1)) * M) * kD +
                                          4 * lane)
                     : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  float maximum = early_stat[0];
  for (int offset = 32; offset; offset >>= 1) maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
  __shared__ float maxima[WAVES];
  __shared__ f32x4 numerators[WAVES][64];
  __shared__ float denominators[WAVES][64];
  if (!sequential) {  // the row's maximum is the largest of the ranges' maxima
    if (lane == 0) maxima[wave] = maximum;
    __syncthreads();
#pragma unroll
    for (uint32_t w = 0; w < WAVES; ++w) maximum = fmaxf(maximum, maxima[w]);
  }
  MergeSums sums{{0.0f, 0.0f, 0.0f, 0.0f}, 0.0f};
  if (count)
    sums = merge_range<AHEAD>(partials, statistics, first_row, first, last, M, maximum, lane, early,
                              early_stat);
  if (!sequential) {
    numerators[wave][lane] = sums.numerator;
    denominators[wave][lane] = sums.denominator;
    __syncthreads();
    if (wave) return;
#pragma unroll
    for (uint32_t w = 1; w < WAVES; ++w) {
      const f32x4 other = numerators[w][lane];
#pragma unroll
      for (uint32_t c = 0; c < 4; ++c) sums.numerator[c] = __fadd_rn(sums.numerator[c], other[c]);
      sums.denominator = __fadd_rn(sums.denominator, denominators[w][lane]);
    }
  }
  u32x2 packed;
#pragma unroll
  for (uint32_t i = 0; i < 2; ++i) {
    const float lo = sums.denominator > 0.0f ? __fdiv_rn(sums.numerator[2 * i], sums.denominator) : 0.0f;
    const float hi =
        sums.denominator > 0.0f ? __fdiv_rn(sums.numerator[2 * i + 1], sums.denominator) : 0.0f;
    packed[i] = uint32_t(f32_to_bf16(lo)) | (uint32_t(f32_to_bf16(hi)) << 16);
  }
  if (out_row) *reinterpret_cast<u32x2 *>(out_row + 4 * lane) = packed;
  if (!hidden_out) return;
  if (a.packed_qkv) {
    // hidden = bf16(value x sigmoid(gate)) with the bf16 value just written
    // (reference: decode/paged_attention.metal:302-308, common/activation.h:14-16).
#pragma unroll
    for (uint32_t i = 0; i < 2; ++i) {
      const float lo = __fmul_rn(bf16_to_f32(uint16_t(packed[i])), sigmoid(bf16_to_f32(uint16_t(gates[i]))));
      const float hi = __fmul_rn(bf16_to_f32(uint16_t(packed[i] >> 16)),
                                 sigmoid(bf16_to_f32(uint16_t(gates[i] >> 16))));
      packed[i] = uint32_t(f32_to_bf16(lo)) | (uint32_t(f32_to_bf16(hi)) << 16);
    }
  }
  *reinterpret_cast<u32x2 *>(hidden_out) = packed;
}

// Launches a split kernel over (work items, KV heads, column blocks) and then
// the merge of the lanes that have more than one split.  `columns` is how many
// fused query rows one workgroup of the split kernel covers (one wave of it where a
// workgroup is waves_per_group independent waves, each a work item).  Returns 1
// (declined) when the workspace cannot hold the aligned layout, 0 when
// enqueued, or a negative status.
template <class SplitKernel>
int launch_matrix_attention(SplitKernel split_kernel, const char *name, uint32_t columns,
                            uint32_t threads, const kvx_storage *s, kvx_kv_layer kv,
                            uint32_t query_heads, const void *queries, void *output,
                            const uint64_t *const *page_tables, const kvx_verify_params *lanes,
                            uint32_t n_lanes, const uint32_t *row_masks, uint32_t row_stride,
                            uint64_t lane_stride, void *workspace, uint64_t workspace_bytes,
                            hipStream_t stream, const FusedAppend *fused = nullptr,
                            Tiles tile_rows = 0, const Epilogue *epilogue = nullptr,
                            bool longest_first = false, uint32_t waves_per_group = 1) {
  const bool run_split = !(epilogue && epilogue->merge_only);
  const bool run_merge = !(epilogue && epilogue->partials_only);
  const kvx_layout &l = s->layout;
  const uint32_t H = l.kv_heads, G = query_heads / H;
  const uint32_t capacity = lanes[0].row_capacity, M = capacity * G;
  uint64_t total_rows = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) total_rows += uint64_t(lanes[i].split_count) * H * M;
  const uint64_t statistics_offset = (total_rows * kD * sizeof(float) + 255) / 256 * 256;
  if (workspace_bytes < statistics_offset + total_rows * 2 * sizeof(float)) return 1;
  float *partials = static_cast<float *>(workspace);
  float *statistics = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + statistics_offset);
  uint64_t row_base = 0;
  // Regular lanes (tile_rows > 0: lane i is lane 0 moved on by i x tile_rows rows
  // and tokens, all full but perhaps the last) go out in one launch whatever
  // their number; others 32 to a launch.
  const uint32_t lanes_per_launch = tile_rows ? n_lanes : kLanes;
  for (uint32_t first = 0; first < n_lanes; first += lanes_per_launch) {
    DecodeArgs a{};
    a.n_lanes = std::min(lanes_per_launch, n_lanes - first);
    if (tile_rows) {
      a.tile_lanes = n_lanes;
      a.tile_per_sequence = n_lanes / tile_rows.sequences;
      a.tile_rows = tile_rows;
      a.tile_last_rows = lanes[n_lanes - 1].active_rows;
      a.tile_lane_stride = lane_stride;
    }
    a.kv_heads = H;
    a.group = G;
    a.row_stride = row_stride;
    a.fused_rows = M;
    a.kv = kv;
    if (fused) {
      a.chunk_keys = static_cast<const uint16_t *>(fused->keys) + uint64_t(first) * fused->lane_stride;
      a.chunk_values = static_cast<const uint16_t *>(fused->values) + uint64_t(first) * fused->lane_stride;
      a.chunk_lane_stride = fused->lane_stride;
      a.chunk_stride = fused->stride;
    }
    uint32_t items = 0, max_splits = 0;
    for (uint32_t i = 0; i < kLanes; ++i) a.item_base[i] = UINT32_MAX;
    // Where each lane's rows lie in the workspace follows the caller's order of lanes; the
    // order of the lane records, which is the order the work items are dispatched in, may
    // differ: longest_first puts the lanes with the longest splits first (a plan that pairs
    // long and short splits on a SIMD counts on the long ones taking the first wave slots).
    // Regular lanes: one record per run, that of the run's first lane.
    const uint32_t recorded = tile_rows ? tile_rows.sequences : a.n_lanes;
    const uint32_t run = tile_rows ? n_lanes / tile_rows.sequences : 1u;
    uint64_t lane_row_base[kLanes];
    uint32_t order[kLanes];
    for (uint32_t i = 0; i < recorded; ++i) {
      order[i] = i * run;
      lane_row_base[i] = row_base;
      row_base += uint64_t(lanes[first + i * run].split_count) * H * M * run;
    }
    if (longest_first && !tile_rows) {
      const auto split_pages = [&](uint32_t k) {
        const kvx_verify_params &p = lanes[first + k];
        const uint32_t pages = (p.committed_tokens + p.active_rows + kPage - 1) / kPage;
        return (pages + p.split_count - 1) / p.split_count;
      };
      std::stable_sort(order, order + recorded,
                       [&](uint32_t x, uint32_t y) { return split_pages(x) > split_pages(y); });
      a.item_major = 1;
    }
    for (uint32_t i = 0; i < recorded; ++i) {
      const uint32_t source = order[i];  // index of the lane (of the run's first lane)
      const kvx_verify_params &p = lanes[first + source];
      DecodeLane &dl = a.lane[i];
      dl.table = page_tables ? page_tables[first + source] : nullptr;
      dl.masks = row_masks ? row_masks + uint64_t(first + source) * capacity : nullptr;
      dl.committed = p.committed_tokens;
      dl.active_rows = p.active_rows;
      dl.split_count = p.split_count;
      dl.first_item = items;
      a.item_base[i] = items;
      dl.score_scale = p.score_scale != 0.0f ? p.score_scale : l.score_scale;
      dl.source = source;
      dl.row_base = lane_row_base[tile_rows ? i : source];
      dl.q_offset = tile_rows ? uint64_t(i) * tile_rows.sequence_stride
                              : uint64_t(first + source) * lane_stride;
      items += p.split_count;
      max_splits = std::max(max_splits, p.split_count);
    }
    if (tile_rows) items = n_lanes * lanes[0].split_count;
    if (epilogue && !epilogue->hidden) {
      a.all_partials = 1;
    } else if (epilogue) {
      a.hidden = epilogue->hidden + uint64_t(first) * capacity * query_heads * kD;
      a.packed_qkv = epilogue->packed_qkv
                         ? epilogue->packed_qkv +
                               uint64_t(first) * capacity * (2ull * query_heads + 2ull * H) * kD
                         : nullptr;
      a.all_partials = 1;
    }
    if (run_split) {
      const uint32_t column_blocks = (M + columns - 1) / columns;
      hipLaunchKernelGGL(split_kernel,
                         a.item_major
                             ? (waves_per_group > 1
                                    ? dim3((H * items + waves_per_group - 1) / waves_per_group, 1, column_blocks)
                                    : dim3(H, items, column_blocks))
                             : dim3((items + waves_per_group - 1) / waves_per_group, H, column_blocks),
                         dim3(threads), 0, stream, static_cast<const uint16_t *>(queries),
                         static_cast<uint16_t *>(output), partials, statistics, a);
      const hipError_t e = hipGetLastError();
      if (e != hipSuccess) return hip_fail(e, name);
    }
    if ((max_splits > 1 || epilogue) && run_merge) {
      // One wave per row where every list of the launch is short; else the ranged form,
      // whose first wave alone sums the short lists among them.
      if (max_splits <= kMergeSequential)
        hipLaunchKernelGGL((matrix_merge_kernel<1, kMergeAhead>), dim3(M, H, a.n_lanes), dim3(64), 0,
                           stream, static_cast<uint16_t *>(output), partials, statistics, a);
      else
        hipLaunchKernelGGL((matrix_merge_kernel<kMergeWaves, kMergeAheadRanged>), dim3(M, H, a.n_lanes),
                           dim3(64 * kMergeWaves), 0, stream, static_cast<uint16_t *>(output), partials,
                           statistics, a);
      const hipError_t e = hipGetLastError();
      if (e != hipSuccess) return hip_fail(e, "matrix_merge_kernel");
    }
  }
  return 0;
}

// The shapes every matrix-core kernel of this library covers: head dimension
// 256, a group of at most 16 query heads, at most KVX_TREE_NODES rows per lane,
// every lane with the row capacity of the first.
inline bool matrix_attention_covers(const kvx_storage *s, uint32_t query_heads,
                                    const kvx_verify_params *lanes, uint32_t n_lanes) {
  const kvx_layout &l = s->layout;
  if (l.head_dim != kD) return false;
  const uint32_t G = query_heads / l.kv_heads, capacity = lanes[0].row_capacity;
  // up to 16 rows per lane (a verify tree), or the 32 rows of four prefill tiles
  if (G > 16 || !capacity || capacity > 2 * KVX_TREE_NODES) return false;
  for (uint32_t i = 0; i < n_lanes; ++i) {
    const kvx_verify_params &p = lanes[i];
    if (p.row_capacity != capacity || !p.active_rows || p.active_rows > capacity) return false;
  }
  return true;
}

}  // namespace
}  // namespace kvx
