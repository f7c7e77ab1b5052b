// kv_oracle.cpp -- TEST INFRASTRUCTURE ONLY (see kv_oracle.h).
//
// Scalar restatement of the reference's paged-KV semantics.  Written for
// clarity and for agreement with the reference's arithmetic order, not speed.
// All arithmetic is fp32 round-to-nearest unless a comment says otherwise.
#include "kv_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <numeric>
#include <vector>

namespace {

constexpr uint32_t kPage = KO_PAGE_TOKENS;
constexpr float kInf = std::numeric_limits<float>::infinity();

inline float bits_to_float(uint32_t b) {
  float f;
  std::memcpy(&f, &b, 4);
  return f;
}
inline uint32_t float_to_bits(float f) {
  uint32_t b;
  std::memcpy(&b, &f, 4);
  return b;
}

uint64_t gcd64(uint64_t a, uint64_t b) {
  while (b) {
    uint64_t r = a % b;
    a = b;
    b = r;
  }
  return a;
}
uint64_t lcm64(uint64_t a, uint64_t b) { return a && b ? a / gcd64(a, b) * b : 0; }

// runtime/ops/PagedKv.hpp:89-94
constexpr uint64_t kRegionAlign = 64 * 1024;
constexpr uint64_t kExtentTarget = 128ull * 1024 * 1024;

// runtime/ops/PagedKv.hpp:113-120
uint64_t pages_for_aligned_region(uint64_t bytes_per_page) {
  return bytes_per_page ? kRegionAlign / gcd64(kRegionAlign, bytes_per_page) : 0;
}

bool quantized(uint32_t format) { return format != KO_BF16; }
bool valid_format(uint32_t f) {
  return f == KO_INT8 || f == KO_BF16 || f == KO_INT4 || f == KO_FP8E4M3;
}

// Bytes one (head, token) row of D elements takes, and bytes per element pair.
uint32_t data_bytes(uint32_t format, uint32_t kv_heads, uint32_t head_dim) {
  const uint64_t elements = uint64_t{kPage} * kv_heads * head_dim;
  if (format == KO_BF16) return uint32_t(elements * 2);
  if (format == KO_INT4) return uint32_t(elements / 2);
  return uint32_t(elements);
}
uint32_t scale_bytes(uint32_t format, uint32_t kv_heads) {
  return quantized(format) ? kPage * kv_heads * 4 : 0;
}

// One KV head's slab of each tensor of one page in one layer.
// runtime/metal/kernels/common/kv_extent.h:63-112 (and :119-156 for int4)
struct Slab {
  uint8_t *keys;
  uint8_t *values;
  float *key_scales;
  float *value_scales;
};

Slab slab_of(uint32_t format, uint32_t kv_heads, uint32_t head_dim, ko_kv_layer kv,
             uint32_t head, uint64_t entry) {
  const uint32_t index = uint32_t(entry) & KO_PAGE_INDEX_MASK;
  uint8_t *extent = reinterpret_cast<uint8_t *>(uintptr_t(entry - index));
  uint8_t *region = extent + kv.offset;
  const uint32_t db = data_bytes(format, kv_heads, head_dim);
  const uint32_t sb = scale_bytes(format, kv_heads);
  const uint64_t key_scales_off = ko_kv_offset(kv.extent_pages, db, sb, 0, KO_KEY_SCALES, 0);
  const uint64_t values_off = ko_kv_offset(kv.extent_pages, db, sb, 0, KO_VALUES, 0);
  const uint64_t value_scales_off =
      ko_kv_offset(kv.extent_pages, db, sb, 0, KO_VALUE_SCALES, 0);
  const uint64_t head_bytes = uint64_t{db} / kv_heads;
  Slab s{};
  s.keys = region + uint64_t{index} * db + head * head_bytes;
  s.values = region + values_off + uint64_t{index} * db + head * head_bytes;
  if (quantized(format)) {
    const uint64_t scale_index = uint64_t{index} * kPage * kv_heads + head * kPage;
    s.key_scales = reinterpret_cast<float *>(region + key_scales_off) + scale_index;
    s.value_scales = reinterpret_cast<float *>(region + value_scales_off) + scale_index;
  }
  return s;
}

int nibble_code(uint8_t byte, uint32_t hi) {
  const int code = int(byte >> (hi * 4)) & 0xF;
  return code - ((code & 0x8) ? 16 : 0);
}

// The decoded (un-scaled) code of key element (token, d) in a head's slab.
float key_code(uint32_t format, const Slab &s, uint32_t head_dim, uint32_t token, uint32_t d) {
  const uint64_t e = uint64_t{token} * head_dim + d;  // abi/KvExtent.h:45-51 at head 0
  switch (format) {
  case KO_INT8: return float(reinterpret_cast<const int8_t *>(s.keys)[e]);
  case KO_INT4: return float(nibble_code(s.keys[e / 2], uint32_t(e & 1)));
  case KO_FP8E4M3: return ko_fp8e4m3_to_float(s.keys[e]);
  default: return ko_bf16_to_float(reinterpret_cast<const uint16_t *>(s.keys)[e]);
  }
}

float value_code(uint32_t format, const Slab &s, uint32_t head_dim, uint32_t token,
                 uint32_t d) {
  if (format == KO_INT4) {
    // common/kv_extent.h:25-30: packed values are token-major like the keys.
    const uint64_t e = uint64_t{token} * head_dim + d;
    return float(nibble_code(s.values[e / 2], uint32_t(e & 1)));
  }
  const uint64_t e = uint64_t{d} * kPage + token;  // abi/KvExtent.h:53-59 at head 0
  switch (format) {
  case KO_INT8: return float(reinterpret_cast<const int8_t *>(s.values)[e]);
  case KO_FP8E4M3: return ko_fp8e4m3_to_float(s.values[e]);
  default: return ko_bf16_to_float(reinterpret_cast<const uint16_t *>(s.values)[e]);
  }
}

// common/paged_store_row.h:14-29
bool chunk_contract_valid(const ko_chunk_params &p) {
  const uint64_t required =
      (uint64_t{p.committed_tokens} + p.chunk_tokens + kPage - 1) / kPage;
  return p.committed_tokens <= KO_MAX_PHYSICAL && p.chunk_tokens > 0 &&
         p.chunk_tokens <= KO_PREFILL_BUDGET &&
         uint64_t{p.committed_tokens} + p.chunk_tokens <= KO_MAX_PHYSICAL &&
         p.chunk_stride >= p.chunk_tokens && p.chunk_stride <= KO_PREFILL_BUDGET &&
         p.chunk_stride % kPage == 0 && p.page_table_entries >= required &&
         p.kv.extent_pages > 0;
}

// common/paged_attention_tile.h:28-42
bool prefill_contract_valid(const ko_prefill_params &p) {
  return p.rows > 0 && p.rows <= KO_PREFILL_BUDGET && p.chunk_stride >= p.rows &&
         p.chunk_stride <= KO_PREFILL_BUDGET && p.chunk_stride % kPage == 0 &&
         p.page_table_entries >= (uint64_t{p.committed_tokens} + p.rows + kPage - 1) / kPage &&
         p.kv.extent_pages > 0 && p.split_count > 0 &&
         p.split_count <= KO_PREFILL_MAX_SPLITS &&
         uint64_t{p.committed_tokens} + p.rows <= uint64_t{KO_MAX_PHYSICAL};
}

// common/paged_attention_tile.h:44-59.  One-row decode lanes may use up to
// KO_DECODE_MAX_SPLITS splits (a rule of the MI355X build for small batches, not
// of the reference, whose bound is KO_VERIFY_MAX_SPLITS).
bool verify_contract_valid(const ko_verify_params &p) {
  const uint32_t max_splits = p.row_capacity == 1 ? KO_DECODE_MAX_SPLITS : KO_VERIFY_MAX_SPLITS;
  return p.active_rows > 0 && p.active_rows <= p.row_capacity &&
         p.page_table_entries >=
             (uint64_t{p.committed_tokens} + p.active_rows + kPage - 1) / kPage &&
         p.kv.extent_pages > 0 &&
         uint64_t{p.committed_tokens} + p.active_rows <= uint64_t{KO_MAX_PHYSICAL} &&
         p.split_count > 0 && p.split_count <= max_splits &&
         p.slot_splits >= p.split_count && p.slot_splits <= max_splits;
}

// common/paged_store_row.h:47-147 and paged_store_row_fp8.h:28-78: one row of
// one tensor of one head goes to its final page slot.
void store_row(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
               const uint16_t *chunk_keys, const uint16_t *chunk_values,
               const uint64_t *page_table, const ko_chunk_params &p, bool value_tensor,
               uint32_t head, uint32_t chunk_token) {
  const uint32_t logical = p.committed_tokens + chunk_token;
  const Slab s = slab_of(format, kv_heads, head_dim, p.kv, head, page_table[logical / kPage]);
  const uint32_t slot = logical % kPage;
  std::vector<uint16_t> source(head_dim);
  for (uint32_t d = 0; d < head_dim; ++d) {
    // common/paged_store_row.h:31-41: keys token-major, values dimension-major.
    source[d] = value_tensor
                    ? chunk_values[(uint64_t{head} * head_dim + d) * p.chunk_stride + chunk_token]
                    : chunk_keys[(uint64_t{head} * p.chunk_stride + chunk_token) * head_dim + d];
  }
  uint8_t *data = value_tensor ? s.values : s.keys;
  if (format == KO_BF16) {
    uint16_t *out = reinterpret_cast<uint16_t *>(data);
    for (uint32_t d = 0; d < head_dim; ++d)
      out[value_tensor ? uint64_t{d} * kPage + slot : uint64_t{slot} * head_dim + d] = source[d];
    return;
  }
  float maximum = 0.0f;
  for (uint32_t d = 0; d < head_dim; ++d)
    maximum = std::max(maximum, std::fabs(ko_bf16_to_float(source[d])));
  const float qmax = format == KO_INT4 ? 7.0f : format == KO_INT8 ? 127.0f : 448.0f;
  const float scale = maximum == 0.0f ? 0.0f : maximum / qmax;
  (value_tensor ? s.value_scales : s.key_scales)[slot] = scale;
  for (uint32_t d = 0; d < head_dim; ++d) {
    const float v = ko_bf16_to_float(source[d]);
    if (format == KO_FP8E4M3) {
      const uint8_t code = maximum == 0.0f ? 0 : ko_float_to_fp8e4m3(v * 448.0f / maximum);
      data[value_tensor ? uint64_t{d} * kPage + slot : uint64_t{slot} * head_dim + d] = code;
      continue;
    }
    const int limit = format == KO_INT4 ? 7 : 127;
    int code = 0;
    if (maximum != 0.0f) {
      // Clamped as a float first: a product that overflowed to infinity must
      // saturate like the GPU's float-to-int conversion, not wrap.
      const float rounded = std::nearbyint(v * qmax / maximum);
      code = rounded != rounded ? 0 : int(std::min(std::max(rounded, float(-limit)), float(limit)));
    }
    if (format == KO_INT8) {
      reinterpret_cast<int8_t *>(
          data)[value_tensor ? uint64_t{d} * kPage + slot : uint64_t{slot} * head_dim + d] =
          int8_t(code);
    } else {
      // common/paged_store_row.h:93-111: even element in the low nibble, both
      // tensors token-major.
      uint8_t &byte = data[(uint64_t{slot} * head_dim + d) / 2];
      const uint8_t nibble = uint8_t(code) & 0xF;
      byte = (d & 1) ? uint8_t((byte & 0x0F) | (nibble << 4)) : uint8_t((byte & 0xF0) | nibble);
    }
  }
}

float default_score_scale(uint32_t head_dim, float requested) {
  // common/paged_attention_tile.h:122-126
  if (requested != 0.0f) return requested;
  return head_dim == 64 ? 0.125f : head_dim == 128 ? 0.08838834764831845f : 0.0625f;
}

}  // namespace

extern "C" {

// ---------------------------------------------------------------- layout ---
int ko_layout_valid(const ko_layout *l) {
  return l->layers && l->kv_heads && l->head_dim && valid_format(l->format);
}
uint64_t ko_elements_per_layer_page(const ko_layout *l) {
  return uint64_t{kPage} * l->kv_heads * l->head_dim;
}
uint64_t ko_data_bytes_per_layer_page(const ko_layout *l) {
  const uint64_t e = ko_elements_per_layer_page(l);
  if (l->format == KO_BF16) return e * 2;
  if (l->format == KO_INT4) return e / 2;
  return e;
}
uint64_t ko_scale_bytes_per_layer_page(const ko_layout *l) {
  return quantized(l->format) ? uint64_t{kPage} * l->kv_heads * 4 : 0;
}
uint64_t ko_bytes_per_layer_page(const ko_layout *l) {
  return 2 * (ko_data_bytes_per_layer_page(l) + ko_scale_bytes_per_layer_page(l));
}
uint64_t ko_bytes_per_model_page(const ko_layout *l) {
  return uint64_t{l->layers} * ko_bytes_per_layer_page(l);
}
// runtime/ops/PagedKv.hpp:172-180
uint32_t ko_extent_alignment_pages(const ko_layout *l) {
  if (l->format == KO_BF16)
    return uint32_t(pages_for_aligned_region(ko_data_bytes_per_layer_page(l)));
  return uint32_t(lcm64(pages_for_aligned_region(ko_data_bytes_per_layer_page(l)),
                        pages_for_aligned_region(ko_scale_bytes_per_layer_page(l))));
}
// runtime/ops/PagedKv.hpp:184-202
uint32_t ko_minimum_extent_pages(const ko_layout *l) {
  const uint64_t unit = uint64_t{ko_extent_alignment_pages(l)} * ko_bytes_per_model_page(l);
  if (!unit) return 0;
  const uint64_t units = std::max<uint64_t>(1, (kExtentTarget / 2 + unit - 1) / unit);
  return uint32_t(units * ko_extent_alignment_pages(l));
}
uint32_t ko_maximum_extent_pages(const ko_layout *l) {
  const uint64_t unit = uint64_t{ko_extent_alignment_pages(l)} * ko_bytes_per_model_page(l);
  if (!unit) return 0;
  const uint64_t units = kExtentTarget * 3 / 2 / unit;
  return std::max(uint32_t(units * ko_extent_alignment_pages(l)), ko_minimum_extent_pages(l));
}
// runtime/ops/PagedKv.hpp:209-229
uint32_t ko_extent_pages_for(const ko_layout *l, uint64_t pages) {
  const uint32_t step = ko_extent_alignment_pages(l);
  const uint64_t smallest = ko_minimum_extent_pages(l);
  if (!smallest || pages < smallest) return 0;
  const uint64_t largest = std::min<uint64_t>(ko_maximum_extent_pages(l), pages);
  uint64_t best = 0, best_left = 0, best_distance = 0;
  for (uint64_t extent = smallest; extent <= largest; extent += step) {
    const uint64_t bytes = extent * ko_bytes_per_model_page(l);
    const uint64_t distance = bytes > kExtentTarget ? bytes - kExtentTarget : kExtentTarget - bytes;
    const uint64_t left = pages % extent;
    if (!best || left < best_left || (left == best_left && distance < best_distance)) {
      best = extent;
      best_left = left;
      best_distance = distance;
    }
  }
  return uint32_t(best);
}

// ------------------------------------------------------------ addressing ---
uint64_t ko_key_element(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim) {
  return (uint64_t{head} * kPage + token) * head_dim + dim;
}
uint64_t ko_value_element(uint32_t head, uint32_t token, uint32_t dim, uint32_t head_dim) {
  return (uint64_t{head} * head_dim + dim) * kPage + token;
}
uint64_t ko_scale_element(uint32_t head, uint32_t token) { return uint64_t{head} * kPage + token; }

uint64_t ko_kv_offset(uint32_t extent_pages, uint32_t db, uint32_t sb, uint32_t layer,
                      uint32_t tensor, uint32_t index) {
  // abi/KvExtent.h:76-89: per layer a region of keys | key scales | values |
  // value scales, each holding every page of the extent.
  const uint64_t region = uint64_t{layer} * extent_pages * 2 * (uint64_t{db} + sb);
  const uint64_t tensors_before_data = (tensor + 1) / 2;  // 0,1,1,2
  const uint64_t tensors_before_scale = tensor / 2;       // 0,0,1,1
  const uint64_t before = tensors_before_data * db + tensors_before_scale * sb;
  const uint64_t page_bytes = (tensor % 2) ? sb : db;
  return region + uint64_t{extent_pages} * before + uint64_t{index} * page_bytes;
}
ko_kv_layer ko_kv_layer_of(uint32_t extent_pages, uint32_t db, uint32_t sb, uint32_t layer) {
  return {extent_pages, uint32_t(ko_kv_offset(extent_pages, db, sb, layer, KO_KEYS, 0))};
}
uint64_t ko_page_entry(uint64_t extent_address, uint32_t index) { return extent_address | index; }

// ---------------------------------------------------------------- codecs ---
uint16_t ko_float_to_bf16(float v) {
  const uint32_t bits = float_to_bits(v);
  if ((bits & 0x7f800000u) == 0x7f800000u) {
    // Inf/NaN keep their top half; a NaN whose payload sits only in the low
    // half keeps a set mantissa bit so it stays a NaN.
    uint16_t upper = uint16_t(bits >> 16);
    if ((bits & 0x007fffffu) && !(upper & 0x007fu)) upper |= 1;
    return upper;
  }
  return uint16_t((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);  // RNE
}
float ko_bf16_to_float(uint16_t v) { return bits_to_float(uint32_t{v} << 16); }

uint8_t ko_float_to_fp8e4m3(float v) {
  // RNE, saturating at 448; subnormal step 2^-9.
  const uint8_t sign = std::signbit(v) ? 0x80 : 0;
  const float a = std::fabs(v);
  if (!std::isfinite(a)) return uint8_t(sign | 0x7F);
  if (a >= 512.0f) return uint8_t(sign | 0x7E);
  if (a < 0.015625f) {  // below 2^-6: subnormal codes, 8 is the first normal
    const long m = std::lrintf(a * 512.0f);
    return uint8_t(sign | uint8_t(std::min<long>(m, 8)));
  }
  int e = std::ilogb(a);
  long m = std::lrintf(std::ldexp(a, 3 - e));  // in [8,16]
  if (m == 16) {
    ++e;
    m = 8;
  }
  if (e > 8 || (e == 8 && m - 8 > 6)) return uint8_t(sign | 0x7E);
  return uint8_t(sign | uint8_t(((e + 7) << 3) | (m - 8)));
}
static float fp8e4m3_value(uint8_t c) {
  const float sign = (c & 0x80) ? -1.0f : 1.0f;
  const int e = (c >> 3) & 0xF, m = c & 7;
  if (e == 0) return sign * std::ldexp(float(m), -9);
  if (e == 15 && m == 7) return std::numeric_limits<float>::quiet_NaN();
  return sign * std::ldexp(1.0f + float(m) / 8.0f, e - 7);
}
float ko_fp8e4m3_to_float(uint8_t c) {
  // The 256 values of the formula above, computed once: the attention restatement decodes a
  // code per key and value element of every row, and ldexp per element is most of its time.
  static const struct Table {
    float value[256];
    Table() {
      for (int i = 0; i < 256; ++i) value[i] = fp8e4m3_value(uint8_t(i));
    }
  } table;
  return table.value[c];
}
float ko_round_to_f16(float v) {
  // IEEE binary16 round-to-nearest-even, returned widened to fp32.
  if (std::isnan(v)) return v;
  const float a = std::fabs(v);
  const float sign = std::signbit(v) ? -1.0f : 1.0f;
  if (a >= 65520.0f) return sign * kInf;  // rounds past the largest finite half
  if (a < 6.103515625e-05f) {             // below 2^-14: subnormal step 2^-24
    return sign * std::ldexp(std::nearbyint(std::ldexp(a, 24)), -24);
  }
  const int e = std::ilogb(a);
  return sign * std::ldexp(std::nearbyint(std::ldexp(a, 10 - e)), e - 10);
}

// -------------------------------------------------------------- planning ---
uint32_t ko_verify_splits(uint32_t committed, uint32_t rows) {
  // runtime/ops/PagedAttention.hpp:54-63
  const uint64_t visible = uint64_t{committed} + rows;
  const uint64_t pages = (visible + kPage - 1) / kPage;
  const uint64_t scaled = (pages + 15) / 16;
  return uint32_t(std::min<uint64_t>(std::max<uint64_t>(32, scaled), KO_VERIFY_MAX_SPLITS));
}
uint32_t ko_prefill_tiles(uint32_t rows) {
  return (rows + KO_PREFILL_TILE_ROWS - 1) / KO_PREFILL_TILE_ROWS;
}
uint32_t ko_prefill_splits(uint32_t tiles) {
  // runtime/ops/PagedAttention.cpp:23-26
  return std::clamp(KO_PREFILL_MAX_SPLITS / tiles, 1u, KO_PREFILL_MAX_SPLITS);
}
uint32_t ko_chunk_required_pages(const ko_chunk_params *p) {
  return (p->committed_tokens + p->chunk_tokens + kPage - 1) / kPage;
}
int ko_chunk_validation(const ko_chunk_params *p) {
  // runtime/ops/PagedAttention.hpp:80-95
  if (!p->chunk_tokens || p->chunk_tokens > KO_PREFILL_BUDGET) return 1;
  if (uint64_t{p->committed_tokens} + p->chunk_tokens > KO_MAX_PHYSICAL) return 2;
  if (p->chunk_stride < p->chunk_tokens || p->chunk_stride > KO_PREFILL_BUDGET ||
      p->chunk_stride % kPage)
    return 3;
  if (p->page_table_entries < ko_chunk_required_pages(p)) return 4;
  return 0;
}
static void workspace_of(uint64_t rows, uint32_t head_dim, uint64_t *pb, uint64_t *sb) {
  // runtime/ops/PagedAttention.cpp:29-32
  *pb = rows * head_dim * 4;
  *sb = rows * 2 * 4;
}
void ko_prefill_workspace(uint32_t rows, uint32_t query_heads, uint32_t kv_heads,
                          uint32_t head_dim, uint64_t *pb, uint64_t *sb) {
  // runtime/ops/PagedAttention.cpp:223-244
  const uint32_t tiles = ko_prefill_tiles(rows);
  const uint32_t fused = KO_PREFILL_TILE_ROWS * (query_heads / kv_heads);
  workspace_of(uint64_t{tiles} * ko_prefill_splits(tiles) * kv_heads * fused, head_dim, pb, sb);
}
void ko_prefill_workspace_bound(uint32_t maximum_rows, uint32_t query_heads, uint32_t head_dim,
                                uint64_t *pb, uint64_t *sb) {
  // runtime/ops/PagedAttention.cpp:200-213
  uint64_t slots = 0;
  for (uint32_t tiles = 1; tiles <= ko_prefill_tiles(maximum_rows); ++tiles)
    slots = std::max(slots, uint64_t{tiles} * ko_prefill_splits(tiles));
  workspace_of(slots * KO_PREFILL_TILE_ROWS * query_heads, head_dim, pb, sb);
}
void ko_verify_workspace(uint32_t lanes, uint32_t row_capacity, uint32_t query_heads,
                         uint32_t head_dim, uint64_t *pb, uint64_t *sb) {
  // runtime/ops/PagedAttention.cpp:215-226, :268-271
  workspace_of(uint64_t{lanes} * row_capacity * KO_VERIFY_MAX_SPLITS * query_heads, head_dim, pb,
               sb);
}

// --------------------------------------------------------------- storage ---
struct ko_store {
  ko_layout layout;
  uint32_t page_count;
  uint32_t extent_pages;
  std::vector<uint8_t *> extents;
};

static ko_store *store_create(const ko_layout *l, uint32_t page_count, uint32_t extent_pages,
                              bool aligned) {
  if (!ko_layout_valid(l)) return nullptr;
  const uint64_t bytes = uint64_t{extent_pages} * ko_bytes_per_model_page(l);
  if (!extent_pages || (aligned && extent_pages % ko_extent_alignment_pages(l)) ||
      extent_pages > KO_PAGE_INDEX_MASK || bytes > std::numeric_limits<uint32_t>::max())
    return nullptr;
  if (!page_count || page_count % extent_pages) return nullptr;
  auto *s = new ko_store{*l, page_count, extent_pages, {}};
  s->extents.assign(page_count / extent_pages, nullptr);
  return s;
}
ko_store *ko_store_create(const ko_layout *l, uint32_t page_count, uint32_t extent_pages) {
  // runtime/ops/PageStorage.mm:12-46: extents hold whole alignment units.
  return store_create(l, page_count, extent_pages, true);
}
ko_store *ko_store_create_host(const ko_layout *l, uint32_t page_count, uint32_t extent_pages) {
  // dev/tuning/HostKvExtents.hpp:158-169: test pools take any extent size the
  // page index allows (alignment units only matter for speed).
  return store_create(l, page_count, extent_pages, false);
}
void ko_store_destroy(ko_store *s) {
  if (!s) return;
  for (uint8_t *e : s->extents) std::free(e);
  delete s;
}
uint64_t ko_store_extent_bytes(const ko_store *s) {
  return uint64_t{s->extent_pages} * ko_bytes_per_model_page(&s->layout);
}
uint32_t ko_store_extent_pages(const ko_store *s) { return s->extent_pages; }
int ko_store_allocate_extent(ko_store *s, uint32_t extent) {
  if (extent >= s->extents.size()) return -2;
  if (s->extents[extent]) return -1;
  const uint64_t bytes = ko_store_extent_bytes(s);
  const uint64_t align = uint64_t{KO_PAGE_INDEX_MASK} + 1;
  void *p = std::aligned_alloc(align, (bytes + align - 1) / align * align);
  if (!p) return -3;
  std::memset(p, 0, bytes);
  s->extents[extent] = static_cast<uint8_t *>(p);
  return 0;
}
int ko_store_release_extent(ko_store *s, uint32_t extent) {
  if (extent >= s->extents.size()) return -2;
  if (!s->extents[extent]) return -1;
  std::free(s->extents[extent]);
  s->extents[extent] = nullptr;
  return 0;
}
uint8_t *ko_store_extent(ko_store *s, uint32_t extent) {
  return extent < s->extents.size() ? s->extents[extent] : nullptr;
}
ko_kv_layer ko_store_layer(const ko_store *s, uint32_t layer) {
  return ko_kv_layer_of(s->extent_pages, uint32_t(ko_data_bytes_per_layer_page(&s->layout)),
                        uint32_t(ko_scale_bytes_per_layer_page(&s->layout)), layer);
}
int ko_store_write_entries(const ko_store *s, const uint32_t *pages, uint32_t n, uint32_t first,
                           uint64_t *table) {
  // runtime/ops/PageStorage.mm:116-141
  if (first > n) return -4;
  for (uint32_t i = first; i < n; ++i) {
    if (pages[i] >= s->page_count) return -2;
    const uint32_t extent = pages[i] / s->extent_pages;
    if (!s->extents[extent]) return -1;
    table[i] = ko_page_entry(uint64_t(uintptr_t(s->extents[extent])),
                             pages[i] - extent * s->extent_pages);
  }
  return 0;
}
static int page_spans(const ko_store *s, uint32_t page, std::vector<std::pair<uint8_t *, uint32_t>> &out) {
  // runtime/ops/PageStorage.mm:143-167
  if (page >= s->page_count) return -2;
  uint8_t *extent = s->extents[page / s->extent_pages];
  if (!extent) return -1;
  const uint32_t db = uint32_t(ko_data_bytes_per_layer_page(&s->layout));
  const uint32_t sb = uint32_t(ko_scale_bytes_per_layer_page(&s->layout));
  const uint32_t index = page % s->extent_pages;
  for (uint32_t layer = 0; layer < s->layout.layers; ++layer)
    for (uint32_t tensor = KO_KEYS; tensor <= KO_VALUE_SCALES; ++tensor)
      if (const uint32_t bytes = (tensor % 2) ? sb : db)
        out.emplace_back(extent + ko_kv_offset(s->extent_pages, db, sb, layer, tensor, index),
                         bytes);
  return 0;
}
int ko_store_copy_pages(ko_store *s, const ko_page_copy *copies, uint32_t n) {
  // runtime/ops/PageStorage.mm:95-114: validate all, then copy all.
  for (uint32_t i = 0; i < n; ++i) {
    if (copies[i].from >= s->page_count || copies[i].to >= s->page_count) return -2;
    if (!s->extents[copies[i].from / s->extent_pages] ||
        !s->extents[copies[i].to / s->extent_pages])
      return -1;
  }
  for (uint32_t i = 0; i < n; ++i) {
    std::vector<std::pair<uint8_t *, uint32_t>> from, to;
    page_spans(s, copies[i].from, from);
    page_spans(s, copies[i].to, to);
    for (size_t t = 0; t < from.size(); ++t) std::memmove(to[t].first, from[t].first, from[t].second);
  }
  return 0;
}
int ko_store_page_read(const ko_store *s, uint32_t page, uint8_t *bytes) {
  std::vector<std::pair<uint8_t *, uint32_t>> spans;
  if (int rc = page_spans(s, page, spans)) return rc;
  for (auto &sp : spans) {
    std::memcpy(bytes, sp.first, sp.second);
    bytes += sp.second;
  }
  return 0;
}
int ko_store_page_write(ko_store *s, uint32_t page, const uint8_t *bytes) {
  std::vector<std::pair<uint8_t *, uint32_t>> spans;
  if (int rc = page_spans(s, page, spans)) return rc;
  for (auto &sp : spans) {
    std::memcpy(sp.first, bytes, sp.second);
    bytes += sp.second;
  }
  return 0;
}

// ---------------------------------------------------------------- append ---
int ko_store_chunk(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                   const uint16_t *chunk_keys, const uint16_t *chunk_values,
                   const uint64_t *page_table, const ko_chunk_params *params) {
  // prefill/paged_attention_store.metal:7-27
  if (!chunk_contract_valid(*params)) return 0;
  for (int tensor = 0; tensor < 2; ++tensor)
    for (uint32_t head = 0; head < kv_heads; ++head)
      for (uint32_t token = 0; token < params->chunk_tokens; ++token)
        store_row(format, kv_heads, head_dim, chunk_keys, chunk_values, page_table, *params,
                  tensor == 1, head, token);
  return 1;
}

int ko_store_verify(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                    const uint16_t *chunk_keys, const uint16_t *chunk_values,
                    const uint64_t *const *page_tables, const ko_chunk_params *params,
                    uint32_t lanes, uint32_t max_rows) {
  // decode/paged_attention_store.metal:3-45
  int written = 0;
  const uint64_t lane_stride = uint64_t{kv_heads} * KO_VERIFY_STRIDE * head_dim;
  for (uint32_t lane = 0; lane < lanes; ++lane) {
    const ko_chunk_params &p = params[lane];
    if (!chunk_contract_valid(p) || p.chunk_tokens > max_rows ||
        p.chunk_stride != KO_VERIFY_STRIDE)
      continue;
    ko_store_chunk(format, kv_heads, head_dim, chunk_keys + lane * lane_stride,
                   chunk_values + lane * lane_stride, page_tables[lane], &p);
    ++written;
  }
  return written;
}

// ------------------------------------------------------------- attention ---
namespace {
// A test's question to the oracle: "had the rounding of these probabilities fallen the
// other way, what would the row be?"  While set, the tile looks at the weight
// (probability x value scale) of each listed token of one fused row before it is rounded
// to its format (bf16; fp16 on the fp8 path): where that value lies within `slack`
// (relative) of the boundary between two neighbours of the format, the tile takes the
// neighbour on the other side.  A weight that is not that close to a boundary is left
// alone, so only roundings that a perturbation of `slack` in the score could have turned
// are turned.  With only_row the tile computes that fused row alone.
struct Flips {
  int64_t fused_row = -1;
  bool only_row = false;
  float slack = 0.0f;
  uint32_t count = 0;
  uint32_t tokens[32] = {};
  uint32_t applied = 0;  // bit i: token i was close to a boundary and was turned
};
thread_local Flips g_flips;

float next_up(float r, bool f16) {
  // the neighbour above a non-negative value of the format
  if (!f16) return ko_bf16_to_float(uint16_t(ko_float_to_bf16(r) + 1));
  const int e = r < 6.103515625e-05f ? -14 : std::ilogb(r);
  return r + std::ldexp(1.0f, e - 10);
}
float next_down(float r, bool f16) {
  if (r == 0.0f) return 0.0f;
  if (!f16) return ko_bf16_to_float(uint16_t(ko_float_to_bf16(r) - 1));
  const int e = r < 6.103515625e-05f ? -14 : std::ilogb(r);
  const float step = std::ldexp(1.0f, e - 10);
  return r - ((e > -14 && r == std::ldexp(1.0f, e)) ? 0.5f * step : step);
}
// `rounded` is `w` rounded to the format; the value on the other side of the nearest
// rounding boundary if w is within slack * w of it, else `rounded`.
float turned(float w, float rounded, bool f16, float slack, bool *did) {
  const float lo = rounded <= w ? rounded : next_down(rounded, f16);
  const float hi = rounded <= w ? next_up(rounded, f16) : rounded;
  const float boundary = 0.5f * (lo + hi);
  if (!(std::fabs(w - boundary) <= slack * w)) return rounded;
  *did = true;
  return rounded == lo ? hi : lo;
}
}  // namespace

void ko_attention_flips(int64_t fused_row, const uint32_t *tokens, uint32_t count, float slack,
                        int only_row) {
  g_flips = Flips{};
  g_flips.fused_row = fused_row;
  g_flips.only_row = only_row != 0;
  g_flips.slack = slack;
  g_flips.count = std::min<uint32_t>(count, 32);
  for (uint32_t i = 0; i < g_flips.count; ++i) g_flips.tokens[i] = tokens[i];
}
uint32_t ko_attention_flips_applied(void) { return g_flips.applied; }

void ko_attention_row_weights(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                              const uint16_t *query_row, const uint64_t *page_table, ko_kv_layer kv,
                              uint32_t kv_head, uint32_t committed, uint32_t active_rows,
                              uint32_t row, const uint32_t *row_masks, float score_scale_param,
                              float *weights) {
  // softmax weight x value scale of every token the row sees, against the row's
  // maximum over all pages; tokens it does not see get 0.
  const uint32_t D = head_dim, visible = committed + active_rows;
  const bool fp8 = format == KO_FP8E4M3, quant = quantized(format);
  const float score_scale = default_score_scale(D, score_scale_param);
  const uint32_t limit = std::min(visible, committed + std::min(row, active_rows - 1) + 1);
  const uint32_t mask = row_masks ? row_masks[row] : 0u;
  std::vector<float> q(D), score(visible, -kInf);
  for (uint32_t d = 0; d < D; ++d) {
    const float v = ko_bf16_to_float(query_row[d]);
    q[d] = fp8 ? ko_round_to_f16(v) : v;
  }
  float maximum = -kInf;
  for (uint32_t t = 0; t < visible; ++t) {
    const bool admitted = !row_masks ? t < limit
                                     : (t < committed) || ((mask >> (t - committed)) & 1u);
    if (!admitted) continue;
    const Slab s = slab_of(format, kv_heads, D, kv, kv_head, page_table[t / kPage]);
    float dot = 0.0f;
    for (uint32_t d = 0; d < D; ++d) dot += q[d] * key_code(format, s, D, t % kPage, d);
    if (quant) dot *= s.key_scales[t % kPage];
    score[t] = dot * score_scale;
    maximum = std::max(maximum, score[t]);
  }
  for (uint32_t t = 0; t < visible; ++t) {
    if (score[t] == -kInf) {
      weights[t] = 0.0f;
      continue;
    }
    const Slab s = slab_of(format, kv_heads, D, kv, kv_head, page_table[t / kPage]);
    weights[t] = std::exp(score[t] - maximum) * (quant ? s.value_scales[t % kPage] : 1.0f);
  }
}

// Threads the attention functions may spread independent rows and tiles over (the checks of
// the GPU suite; 1, the default, for anything that is timed as a one-thread baseline).  Every
// row is still computed by one thread in the reference's order, so the results do not depend
// on the number.
static int g_threads = 1;
void ko_set_threads(int threads) { g_threads = threads > 1 ? threads : 1; }
int ko_threads(void) { return g_threads; }

int ko_attention_tile(uint32_t format, uint32_t kv_heads, uint32_t group, uint32_t head_dim,
                      uint32_t row_capacity, const uint16_t *tile_queries,
                      const uint64_t *page_table, ko_kv_layer kv, uint32_t kv_head,
                      uint32_t committed, uint32_t active_rows, uint32_t splits, uint32_t split,
                      float *partials, float *statistics, uint64_t slot,
                      const uint32_t *row_masks, float score_scale_param) {
  // common/paged_attention_tile.h:208-349 with the page softmax of :85-189;
  // fp8: paged_attention_fp8_tile.h:34-265.
  const uint32_t M = row_capacity * group, D = head_dim;
  const uint32_t visible = committed + active_rows;
  const uint32_t pages = (visible + kPage - 1) / kPage;
  const uint32_t per = (pages + splits - 1) / splits;
  const uint32_t begin = split * per;
  if (begin >= pages) return 0;
  const uint32_t end = std::min(pages, begin + per);
  const bool fp8 = format == KO_FP8E4M3;
  const bool quant = quantized(format);
  const float score_scale = default_score_scale(D, score_scale_param);
  // The question is the calling thread's (thread_local); the worker threads of the loop below
  // read this copy of it and report into `turned_tokens`.
  const Flips flips = g_flips;
  uint32_t turned_tokens = 0;

#pragma omp parallel for schedule(dynamic, 1) num_threads(g_threads) if (g_threads > 1)
  for (uint32_t r = 0; r < M; ++r) {
    std::vector<float> q(D), acc(D);
    const uint32_t query_row = r / group;
    // Rows past the live ones are never read by the merge (it writes zeros
    // for them), so the oracle leaves their partials untouched.
    if (query_row >= active_rows) continue;
    if (flips.only_row && flips.fused_row >= 0 && int64_t(r) != flips.fused_row) continue;
    for (uint32_t d = 0; d < D; ++d) {
      const float v = ko_bf16_to_float(tile_queries[uint64_t{r} * D + d]);
      q[d] = fp8 ? ko_round_to_f16(v) : v;  // fp8 tile stages queries as fp16
    }
    const uint32_t causal_end = committed + std::min(query_row, active_rows - 1) + 1;
    const uint32_t limit = std::min(visible, causal_end);
    const uint32_t mask = row_masks ? row_masks[query_row] : 0u;
    float row_max = -kInf, row_sum = 0.0f;
    std::fill(acc.begin(), acc.end(), 0.0f);

    for (uint32_t page = begin; page < end; ++page) {
      const Slab s = slab_of(format, kv_heads, D, kv, kv_head, page_table[page]);
      const uint32_t token_start = page * kPage;
      bool admitted[kPage];
      float score[kPage], prob[kPage];
      float local_max = -kInf;
      for (uint32_t j = 0; j < kPage; ++j) {
        const uint32_t t = token_start + j;
        admitted[j] = !row_masks ? t < limit
                                 : (t < committed) ||
                                       (t < visible && ((mask >> (t - committed)) & 1u));
        score[j] = -kInf;
        if (!admitted[j]) continue;
        float dot = 0.0f;
        for (uint32_t d = 0; d < D; ++d) dot += q[d] * key_code(format, s, D, j, d);
        if (quant) dot *= s.key_scales[j];  // :129-135: key scale, then score scale
        dot *= score_scale;
        score[j] = dot;
        local_max = std::max(local_max, dot);
      }
      const float next_max = std::max(row_max, local_max);
      // :159-169: four lanes of eight tokens each sum their own tokens, then
      // two xor-shuffle steps combine them.
      float lane_sum[4] = {0, 0, 0, 0};
      for (uint32_t j = 0; j < kPage; ++j) {
        prob[j] = admitted[j] ? std::exp(score[j] - next_max) : 0.0f;
        lane_sum[j / 8] += prob[j];
      }
      const float local_sum = (lane_sum[0] + lane_sum[1]) + (lane_sum[2] + lane_sum[3]);
      const float rescale =
          (next_max == -kInf || next_max == row_max) ? 1.0f : std::exp(row_max - next_max);
      row_sum = row_sum * rescale + local_sum;
      row_max = next_max;
      if (rescale != 1.0f)
        for (uint32_t d = 0; d < D; ++d) acc[d] *= rescale;
      // :175-188: probability x value scale, rounded to bf16 (fp16 on fp8).
      float weight[kPage];
      for (uint32_t j = 0; j < kPage; ++j) {
        float w = 0.0f;
        if (admitted[j] && score[j] > -kInf) w = prob[j] * (quant ? s.value_scales[j] : 1.0f);
        weight[j] = fp8 ? ko_round_to_f16(w) : ko_bf16_to_float(ko_float_to_bf16(w));
        if (flips.fused_row == int64_t(r))
          for (uint32_t f = 0; f < flips.count; ++f)
            if (flips.tokens[f] == token_start + j) {
              bool did = false;
              weight[j] = turned(w, weight[j], fp8, flips.slack, &did);
              if (did) {
#pragma omp atomic
                turned_tokens |= 1u << f;
              }
            }
      }
      for (uint32_t d = 0; d < D; ++d) {
        float sum = 0.0f;
        for (uint32_t j = 0; j < kPage; ++j)
          if (admitted[j]) sum += weight[j] * value_code(format, s, D, j, d);
        acc[d] += sum;
      }
    }
    std::memcpy(partials + (slot * M + r) * D, acc.data(), size_t{D} * 4);
    statistics[(slot * M + r) * 2] = row_max;
    statistics[(slot * M + r) * 2 + 1] = row_sum;
  }
  g_flips.applied |= turned_tokens;
  return 1;
}

void ko_attention_reduce_row(uint32_t group, uint32_t head_dim, uint32_t row_capacity,
                             const float *partials, const float *statistics, uint32_t committed,
                             uint32_t active_rows, uint32_t splits, uint64_t head_slot,
                             uint32_t fused_row, uint16_t *out_bf16, float *out_f32) {
  // common/paged_attention_tile.h:362-417
  const uint32_t M = row_capacity * group, D = head_dim;
  if (fused_row / group >= active_rows) {
    for (uint32_t d = 0; d < D; ++d) {
      if (out_bf16) out_bf16[d] = 0;
      if (out_f32) out_f32[d] = 0.0f;
    }
    return;
  }
  const uint32_t pages = (committed + active_rows + kPage - 1) / kPage;
  const uint32_t per = (pages + splits - 1) / splits;
  const uint32_t written = (pages + per - 1) / per;
  float maximum = -kInf;
  for (uint32_t s = 0; s < written; ++s)
    maximum = std::max(maximum, statistics[((head_slot + s) * M + fused_row) * 2]);
  std::vector<float> weights(written);
  for (uint32_t s = 0; s < written; ++s)
    weights[s] = std::exp(statistics[((head_slot + s) * M + fused_row) * 2] - maximum);
  float denominator = 0.0f;
  for (uint32_t s = 0; s < written; ++s)
    denominator += weights[s] * statistics[((head_slot + s) * M + fused_row) * 2 + 1];
  for (uint32_t d = 0; d < D; ++d) {
    float numerator = 0.0f;
    for (uint32_t s = 0; s < written; ++s)  // split order is part of the contract
      numerator += weights[s] * partials[((head_slot + s) * M + fused_row) * D + d];
    const float value = denominator > 0.0f ? numerator / denominator : 0.0f;
    if (out_f32) out_f32[d] = value;
    if (out_bf16) out_bf16[d] = ko_float_to_bf16(value);
  }
}

int ko_attend_prefill(uint32_t format, uint32_t kv_heads, uint32_t group, uint32_t head_dim,
                      const uint16_t *queries, uint16_t *output, float *out_f32,
                      const uint64_t *page_table, const ko_prefill_params *p) {
  // prefill/paged_attention.metal:7-67 and the reduce entries of :105-206
  if (!prefill_contract_valid(*p)) return 0;
  const uint32_t D = head_dim, R = KO_PREFILL_TILE_ROWS, M = R * group;
  const uint32_t tiles = ko_prefill_tiles(p->rows);
  const uint64_t slots = uint64_t{tiles} * kv_heads * p->split_count;
  std::vector<float> partials(slots * M * D, 0.0f), statistics(slots * M * 2, 0.0f);
#pragma omp parallel for schedule(dynamic, 1) num_threads(g_threads) if (g_threads > 1)
  for (uint32_t tile = 0; tile < tiles; ++tile) {
    const uint32_t tile_start = tile * R;
    const uint32_t active = std::min(R, p->rows - tile_start);
    for (uint32_t head = 0; head < kv_heads; ++head) {
      const uint64_t tile_offset = (uint64_t{head} * p->chunk_stride + tile_start) * group * D;
      const uint64_t head_slot = (uint64_t{tile} * kv_heads + head) * p->split_count;
      for (uint32_t split = 0; split < p->split_count; ++split)
        ko_attention_tile(format, kv_heads, group, D, R, queries + tile_offset, page_table, p->kv,
                          head, p->committed_tokens + tile_start, active, p->split_count, split,
                          partials.data(), statistics.data(), head_slot + split, nullptr,
                          p->score_scale);
      for (uint32_t fused = 0; fused < M; ++fused)
        ko_attention_reduce_row(group, D, R, partials.data(), statistics.data(),
                                p->committed_tokens + tile_start, active, p->split_count,
                                head_slot, fused, output ? output + tile_offset + fused * D : nullptr,
                                out_f32 ? out_f32 + tile_offset + fused * D : nullptr);
    }
  }
  return 1;
}

int ko_attend_verify(uint32_t format, uint32_t kv_heads, uint32_t group, uint32_t head_dim,
                     const uint16_t *queries, uint16_t *output, float *out_f32,
                     const uint64_t *const *page_tables, const ko_verify_params *params,
                     uint32_t lanes, const uint32_t *row_masks) {
  // decode/paged_attention.metal:23-191 (split) and :226-464 (reduce)
  const uint32_t D = head_dim;
  int attended = 0;
  const uint64_t group_stride = uint64_t{KO_VERIFY_STRIDE} * group * D;
  for (uint32_t lane = 0; lane < lanes; ++lane) {
    const ko_verify_params &p = params[lane];
    if (!verify_contract_valid(p)) continue;
    const uint32_t R = p.row_capacity, M = R * group;
    std::vector<float> partials(uint64_t{kv_heads} * p.slot_splits * M * D, 0.0f);
    std::vector<float> statistics(uint64_t{kv_heads} * p.slot_splits * M * 2, 0.0f);
    const uint32_t *masks = row_masks ? row_masks + uint64_t{lane} * R : nullptr;
    for (uint32_t head = 0; head < kv_heads; ++head) {
      const uint64_t offset = (uint64_t{lane} * kv_heads + head) * group_stride;
      const uint64_t head_slot = uint64_t{head} * p.slot_splits;
      for (uint32_t split = 0; split < p.split_count; ++split)
        ko_attention_tile(format, kv_heads, group, D, R, queries + offset, page_tables[lane], p.kv,
                          head, p.committed_tokens, p.active_rows, p.split_count, split,
                          partials.data(), statistics.data(), head_slot + split, masks,
                          p.score_scale);
      for (uint32_t fused = 0; fused < M; ++fused)
        ko_attention_reduce_row(group, D, R, partials.data(), statistics.data(),
                                p.committed_tokens, p.active_rows, p.split_count, head_slot,
                                fused, output ? output + offset + fused * D : nullptr,
                                out_f32 ? out_f32 + offset + fused * D : nullptr);
    }
    ++attended;
  }
  return attended;
}

float ko_sigmoid(float x) {
  // common/activation.h:14-16
  return 1.0f / (1.0f + exp2f(-1.44269504089f * x));
}

void ko_attention_hidden(uint32_t kv_heads, uint32_t group, uint32_t head_dim, uint32_t lanes,
                         uint32_t rows, uint32_t row_stride, const uint16_t *attention,
                         const uint16_t *packed_qkv, uint16_t *hidden) {
  // decode/attention_qkv.metal:121-164 (full_attention_gate_value and its loop)
  const uint32_t D = head_dim, q_heads = kv_heads * group;
  const uint64_t q_stride = packed_qkv ? 2ull * D : D;
  const uint64_t packed_stride = q_heads * q_stride + 2ull * kv_heads * D;
  const uint64_t per_lane = uint64_t{rows} * q_heads * D;
  for (uint64_t element = 0; element < per_lane * lanes; ++element) {
    const uint64_t batch = element / per_lane, lane_element = element % per_lane;
    const uint64_t row = lane_element / (uint64_t{q_heads} * D);
    const uint64_t remainder = lane_element % (uint64_t{q_heads} * D);
    const uint64_t query_head = remainder / D, dim = remainder % D;
    float gate_scale = 1.0f;
    if (packed_qkv)
      gate_scale = ko_sigmoid(ko_bf16_to_float(
          packed_qkv[(batch * rows + row) * packed_stride + query_head * q_stride + D + dim]));
    const uint64_t kv_head = query_head / group, local_head = query_head % group;
    const uint64_t at = (((batch * kv_heads + kv_head) * row_stride + row) * group + local_head) * D + dim;
    hidden[element] = ko_float_to_bf16(ko_bf16_to_float(attention[at]) * gate_scale);
  }
}

// ----------------------------------------------------------- QKV prepare ---
namespace {
// common/rms_inverse.h:14-31: simd_sum per 32 lanes (the xor butterfly), the
// simdgroups' sums added in order by thread 0, rsqrt(total / width + eps).
float rms_inverse_of_sums(const float *squares, uint32_t width, float eps) {
  float total = 0.0f;
  for (uint32_t base = 0; base < width; base += 32) {
    float lane[32];
    for (uint32_t i = 0; i < 32; ++i) lane[i] = squares[base + i];
    for (uint32_t offset = 16; offset; offset >>= 1) {
      float next[32];
      for (uint32_t i = 0; i < 32; ++i) next[i] = lane[i] + lane[i ^ offset];
      std::memcpy(lane, next, sizeof lane);
    }
    total += lane[0];
  }
  return 1.0f / std::sqrt(total / float(width) + eps);
}
}  // namespace

void ko_qkv_prepare(uint32_t kv_heads, uint32_t group, uint32_t head_dim, uint32_t rotary_pairs,
                    int query_gate, int norm_f32, float eps, uint32_t tokens, uint32_t stride,
                    const uint16_t *packed, const void *q_norm, const void *k_norm,
                    const float *rope_cos, const float *rope_sin, uint16_t *queries,
                    uint16_t *chunk_keys, uint16_t *chunk_values) {
  // common/attention_qkv_prepare.h:12-83, one task per (row, head), D threads
  const uint32_t D = head_dim, q_heads = kv_heads * group;
  const uint32_t q_stride = query_gate ? 2 * D : D;
  const uint64_t packed_stride = uint64_t{q_heads} * q_stride + 2ull * kv_heads * D;
  const uint32_t q_width = q_heads * q_stride, k_width = kv_heads * D;
  const bool norms = q_norm && k_norm;
  std::vector<float> element(D), squares(D);
  std::vector<uint16_t> normalized(D);
  const uint32_t tasks = tokens * (q_heads + kv_heads);
  for (uint32_t task = 0; task < tasks; ++task) {
    const bool query = task < tokens * q_heads;
    const uint32_t local_task = query ? task : task - tokens * q_heads;
    const uint32_t heads = query ? q_heads : kv_heads;
    const uint32_t row = local_task / heads, head_index = local_task % heads;
    const uint16_t *source = query ? packed + row * packed_stride + uint64_t{head_index} * q_stride
                                   : packed + row * packed_stride + q_width + uint64_t{head_index} * D;
    const void *weight = query ? q_norm : k_norm;
    uint16_t *destination;
    if (query) {
      const uint32_t kv_head = head_index / group, local_head = head_index % group;
      destination = queries + ((uint64_t{kv_head} * stride + row) * group + local_head) * D;
    } else {
      destination = chunk_keys + (uint64_t{head_index} * stride + row) * D;
    }
    for (uint32_t d = 0; d < D; ++d) {
      element[d] = ko_bf16_to_float(source[d]);
      squares[d] = element[d] * element[d];
    }
    const float inverse = norms ? rms_inverse_of_sums(squares.data(), D, eps) : 1.0f;
    for (uint32_t d = 0; d < D; ++d) {
      float scale = 1.0f;
      if (norms)
        scale = norm_f32 ? static_cast<const float *>(weight)[d]
                         : ko_bf16_to_float(static_cast<const uint16_t *>(weight)[d]);
      normalized[d] = ko_float_to_bf16(element[d] * inverse * scale);
      if (!query) chunk_values[(uint64_t{head_index} * D + d) * stride + row] = source[k_width + d];
    }
    for (uint32_t d = 0; d < D; ++d) {
      if (d < rotary_pairs) {
        const float first = ko_bf16_to_float(normalized[d]);
        const float second = ko_bf16_to_float(normalized[d + rotary_pairs]);
        const float cosine = rope_cos[uint64_t{row} * rotary_pairs + d];
        const float sine = rope_sin[uint64_t{row} * rotary_pairs + d];
        destination[d] = ko_float_to_bf16(first * cosine - second * sine);
        destination[d + rotary_pairs] = ko_float_to_bf16(second * cosine + first * sine);
      } else if (d >= 2 * rotary_pairs) {
        destination[d] = normalized[d];
      }
    }
  }
}

// ------------------------------------------------------------ compaction ---
int ko_compact_tree(uint32_t format, uint32_t kv_heads, uint32_t head_dim,
                    const uint64_t *const *page_tables, const ko_chunk_params *params,
                    const uint32_t *retained_path, const uint32_t *retained_count,
                    uint32_t lanes, uint32_t path_stride) {
  // decode/paged_attention_store.metal:198-278: forward order over the path.
  const uint32_t D = head_dim;
  const uint32_t element = format == KO_BF16 ? 2 : 1;
  const uint32_t key_row_bytes = format == KO_INT4 ? D / 2 : D * element;
  int moved = 0;
  for (uint32_t lane = 0; lane < lanes; ++lane) {
    const ko_chunk_params &p = params[lane];
    const uint32_t count = retained_count[lane];
    for (uint32_t head = 0; head < kv_heads; ++head) {
      for (uint32_t i = 0; i < count; ++i) {
        const uint32_t src_row = retained_path[uint64_t{lane} * path_stride + i];
        if (src_row == i) continue;
        const uint32_t src_token = p.committed_tokens + src_row;
        const uint32_t dst_token = p.committed_tokens + i;
        const Slab src = slab_of(format, kv_heads, D, p.kv, head, page_tables[lane][src_token / kPage]);
        const Slab dst = slab_of(format, kv_heads, D, p.kv, head, page_tables[lane][dst_token / kPage]);
        const uint32_t so = src_token % kPage, dof = dst_token % kPage;
        std::vector<uint8_t> row(key_row_bytes);
        std::memcpy(row.data(), src.keys + uint64_t{so} * key_row_bytes, key_row_bytes);
        std::memcpy(dst.keys + uint64_t{dof} * key_row_bytes, row.data(), key_row_bytes);
        if (format == KO_INT4) {
          std::memcpy(row.data(), src.values + uint64_t{so} * key_row_bytes, key_row_bytes);
          std::memcpy(dst.values + uint64_t{dof} * key_row_bytes, row.data(), key_row_bytes);
        } else {
          for (uint32_t d = 0; d < D; ++d)
            std::memcpy(dst.values + (uint64_t{d} * kPage + dof) * element,
                        src.values + (uint64_t{d} * kPage + so) * element, element);
        }
        if (quantized(format)) {
          dst.key_scales[dof] = src.key_scales[so];
          dst.value_scales[dof] = src.value_scales[so];
        }
        ++moved;
      }
    }
  }
  return moved;
}

// ------------------------------------------------------------------ pool ---
// runtime/engine/cache/KvPool.cpp restated over an accounting-only storage.
struct ko_pool {
  static constexpr uint32_t none = 0xffffffffu;
  struct Page {
    uint32_t active = 0;
    uint32_t prev = none, next = none;
    bool prefix = false, listed = false;
  };
  struct Extent {
    uint32_t used = 0;
    uint32_t free_head = none, free_count = 0;
    bool allocated = false;
    uint64_t reclaim_stamp = 0;  // order in which it became reclaimable
    bool reclaimable = false;
  };
  uint64_t bytes_per_page;
  uint32_t extent_pages;
  uint32_t budget_pages;
  bool growth_blocked = false;
  int64_t refused_extent = -1;
  std::vector<Page> pages;
  std::vector<Extent> extents;
  std::vector<uint64_t> content;
  uint32_t free_pages = 0, active_pages = 0, prefix_pages = 0, allocated_extents = 0;
  uint32_t packing = none;
  uint64_t stamp = 0;
  uint64_t allocations = 0, releases = 0, compactions = 0, moved = 0;

  bool page_free(uint32_t p) const { return !pages[p].active && !pages[p].prefix; }
  uint32_t extent_of(uint32_t p) const { return p / extent_pages; }

  void insert_free(uint32_t p) {  // KvPool.cpp:258-272: pushed at the head
    Page &r = pages[p];
    Extent &e = extents[extent_of(p)];
    r.prev = none;
    r.next = e.free_head;
    r.listed = true;
    if (e.free_head != none) pages[e.free_head].prev = p;
    e.free_head = p;
    ++e.free_count;
    ++free_pages;
    packing = none;
  }
  void remove_free(uint32_t p) {
    Page &r = pages[p];
    Extent &e = extents[extent_of(p)];
    if (r.prev == none) e.free_head = r.next;
    else pages[r.prev].next = r.next;
    if (r.next != none) pages[r.next].prev = r.prev;
    r.prev = r.next = none;
    r.listed = false;
    --e.free_count;
    --free_pages;
  }
  void set_reclaimable(uint32_t x, bool on) {
    Extent &e = extents[x];
    if (e.reclaimable == on) return;
    e.reclaimable = on;
    if (on) e.reclaim_stamp = ++stamp;  // newest first in the reference's list
  }
  void mark_used(uint32_t p) {  // KvPool.cpp:326-338
    const uint32_t x = extent_of(p);
    if (pages[p].listed) {
      remove_free(p);
      if (x != packing) packing = none;
    }
    if (!extents[x].used) set_reclaimable(x, false);
    ++extents[x].used;
  }
  void mark_free(uint32_t p) {  // KvPool.cpp:340-349
    const uint32_t x = extent_of(p);
    --extents[x].used;
    insert_free(p);
    if (!extents[x].used) set_reclaimable(x, true);
  }
  bool storage_allocate(uint32_t x) {  // TestKvPool.hpp:41-52
    if (growth_blocked || refused_extent == int64_t(x) ||
        uint64_t{allocated_extents} * extent_pages + extent_pages > budget_pages)
      return false;
    return true;
  }
  bool allocate_extent(uint32_t x) {  // KvPool.cpp:143-153, :354-366
    if (!storage_allocate(x)) return false;
    ++allocations;
    Extent &e = extents[x];
    e.allocated = true;
    ++allocated_extents;
    const uint32_t first = x * extent_pages;
    for (uint32_t p = first + extent_pages; p > first;) insert_free(--p);  // lowest page ends at the head
    set_reclaimable(x, true);
    return true;
  }
  void release_extent(uint32_t x) {  // KvPool.cpp:155-163, :368-376
    ++releases;
    set_reclaimable(x, false);
    const uint32_t first = x * extent_pages;
    for (uint32_t p = first; p < first + extent_pages; ++p) remove_free(p);
    extents[x].allocated = false;
    --allocated_extents;
  }
  uint32_t packing_extent() {  // KvPool.cpp:309-324
    if (packing != none && extents[packing].free_count) return packing;
    uint32_t best = none;
    for (uint32_t i = 0; i < extents.size(); ++i)
      if (extents[i].free_count && (best == none || extents[i].used > extents[best].used)) best = i;
    packing = best;
    return best;
  }
};

ko_pool *ko_pool_create(uint32_t page_count, uint64_t bytes_per_page, uint32_t extent_pages,
                        uint32_t runway_pages, uint32_t budget_pages) {
  // KvPool.cpp:14-33
  if (!page_count || !bytes_per_page || !extent_pages || page_count % extent_pages) return nullptr;
  if (runway_pages > page_count) return nullptr;
  auto *p = new ko_pool;
  p->bytes_per_page = bytes_per_page;
  p->extent_pages = extent_pages;
  p->budget_pages = budget_pages;
  p->pages.resize(page_count);
  p->content.assign(page_count, 0);
  p->extents.resize(page_count / extent_pages);
  for (uint32_t x = 0; x * extent_pages < runway_pages; ++x)
    if (!p->allocate_extent(x)) {
      delete p;
      return nullptr;
    }
  return p;
}
void ko_pool_destroy(ko_pool *p) { delete p; }
void ko_pool_set_growth_blocked(ko_pool *p, int blocked) { p->growth_blocked = blocked != 0; }
void ko_pool_set_refused_extent(ko_pool *p, int64_t extent) { p->refused_extent = extent; }
void ko_pool_set_budget_pages(ko_pool *p, uint32_t pages) { p->budget_pages = pages; }

int ko_pool_acquire(ko_pool *p, uint32_t count, uint32_t *out) {
  // KvPool.cpp:35-72
  std::vector<uint32_t> selected;
  while (selected.size() < count) {
    if (p->free_pages) {
      const uint32_t page = p->extents[p->packing_extent()].free_head;
      p->remove_free(page);
      selected.push_back(page);
      continue;
    }
    uint32_t x = ko_pool::none;
    for (uint32_t i = 0; i < p->extents.size(); ++i)
      if (!p->extents[i].allocated) {
        x = i;
        break;
      }
    if (x == ko_pool::none) {
      for (auto it = selected.rbegin(); it != selected.rend(); ++it) p->insert_free(*it);
      return -2;
    }
    if (!p->allocate_extent(x)) {
      for (auto it = selected.rbegin(); it != selected.rend(); ++it) p->insert_free(*it);
      return -1;
    }
  }
  for (uint32_t page : selected) {
    p->mark_used(page);
    p->pages[page].active = 1;
    ++p->active_pages;
  }
  std::copy(selected.begin(), selected.end(), out);
  return int(count);
}
int ko_pool_retain(ko_pool *p, uint32_t page, int prefix_owner) {
  // KvPool.cpp:74-91
  if (page >= p->pages.size() || !p->extents[p->extent_of(page)].allocated) return -1;
  ko_pool::Page &r = p->pages[page];
  if (prefix_owner && r.prefix) return -1;
  if (p->page_free(page)) p->mark_used(page);
  if (prefix_owner) {
    r.prefix = true;
    ++p->prefix_pages;
  } else if (!r.active++) {
    ++p->active_pages;
  }
  return 0;
}
int ko_pool_release(ko_pool *p, uint32_t page, int prefix_owner) {
  // KvPool.cpp:93-105
  if (page >= p->pages.size()) return -1;
  ko_pool::Page &r = p->pages[page];
  if (prefix_owner ? !r.prefix : !r.active) return -1;
  if (prefix_owner) {
    r.prefix = false;
    --p->prefix_pages;
  } else if (!--r.active) {
    --p->active_pages;
  }
  if (p->page_free(page)) p->mark_free(page);
  return 0;
}
int ko_pool_page_active(const ko_pool *p, uint32_t page) { return p->pages[page].active != 0; }
uint64_t ko_pool_reclaim_empty(ko_pool *p, int keep_runway, uint32_t limit) {
  // KvPool.cpp:125-141: newest reclaimable first; the first is kept as runway.
  std::vector<uint32_t> order;
  for (uint32_t x = 0; x < p->extents.size(); ++x)
    if (p->extents[x].reclaimable) order.push_back(x);
  std::sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) {
    return p->extents[a].reclaim_stamp > p->extents[b].reclaim_stamp;
  });
  uint32_t reclaimed = 0;
  bool kept = false;
  for (uint32_t x : order) {
    if (reclaimed >= limit) break;
    if (keep_runway && !kept) {
      kept = true;
      continue;
    }
    p->release_extent(x);
    ++reclaimed;
  }
  return uint64_t{reclaimed} * p->extent_pages * p->bytes_per_page;
}
int ko_pool_compact_extent(ko_pool *p, const uint32_t *fixed, uint32_t n_fixed,
                           uint32_t *first_page, uint32_t *destinations,
                           ko_page_copy *copies_out, uint32_t *n_copies) {
  // KvPool.cpp:165-230
  constexpr uint32_t none = ko_pool::none;
  *n_copies = 0;
  uint32_t free_in_use = 0;
  for (const auto &e : p->extents)
    if (e.allocated && e.used) free_in_use += e.free_count;
  uint32_t emptied = none;
  for (uint32_t i = 0; i < p->extents.size(); ++i) {
    const auto &e = p->extents[i];
    if (!e.allocated || !e.used || e.used > free_in_use - e.free_count ||
        (emptied != none && e.used >= p->extents[emptied].used))
      continue;
    bool holds_fixed = false;
    for (uint32_t f = 0; f < n_fixed; ++f) holds_fixed |= p->extent_of(fixed[f]) == i;
    if (!holds_fixed) emptied = i;
  }
  if (emptied == none) return 0;
  std::vector<uint32_t> receivers;
  for (uint32_t i = 0; i < p->extents.size(); ++i) {
    const auto &e = p->extents[i];
    if (i != emptied && e.allocated && e.used && e.free_count) receivers.push_back(i);
  }
  std::stable_sort(receivers.begin(), receivers.end(),
                   [&](uint32_t a, uint32_t b) { return p->extents[a].used > p->extents[b].used; });
  const uint32_t first = emptied * p->extent_pages;
  std::vector<ko_page_copy> copies;
  size_t receiver = 0;
  uint32_t to = p->extents[receivers[receiver]].free_head;
  for (uint32_t page = first; page < first + p->extent_pages; ++page) {
    if (p->page_free(page)) continue;
    while (to == none) to = p->extents[receivers[++receiver]].free_head;
    copies.push_back({page, to});
    to = p->pages[to].next;
  }
  for (const auto &c : copies) p->content[c.to] = p->content[c.from];  // storage copyPages
  *first_page = first;
  for (uint32_t i = 0; i < p->extent_pages; ++i) destinations[i] = first + i;
  for (const auto &c : copies) {
    p->mark_used(c.to);
    p->pages[c.to].active = p->pages[c.from].active;
    p->pages[c.from].active = 0;
    p->pages[c.to].prefix = p->pages[c.from].prefix;
    p->pages[c.from].prefix = false;
    p->mark_free(c.from);
    destinations[c.from - first] = c.to;
  }
  ++p->compactions;
  p->moved += copies.size();
  if (copies_out) std::copy(copies.begin(), copies.end(), copies_out);
  *n_copies = uint32_t(copies.size());
  return int(p->extent_pages);
}
void ko_pool_snapshot_get(const ko_pool *p, ko_pool_snapshot *out) {
  // KvPool.cpp:232-248
  uint32_t reclaimable = 0;
  for (const auto &e : p->extents) reclaimable += e.reclaimable;
  out->pages_allocated = p->allocated_extents * p->extent_pages;
  out->pages_free = p->free_pages;
  out->pages_active = p->active_pages;
  out->pages_prefix = p->prefix_pages;
  out->allocated_bytes = uint64_t{p->allocated_extents} * p->extent_pages * p->bytes_per_page;
  out->reclaimable_bytes = uint64_t{reclaimable} * p->extent_pages * p->bytes_per_page;
  out->extent_allocations = p->allocations;
  out->extent_releases = p->releases;
  out->extent_compactions = p->compactions;
  out->pages_moved = p->moved;
}
uint64_t ko_pool_content(const ko_pool *p, uint32_t page) { return p->content[page]; }
void ko_pool_set_content(ko_pool *p, uint32_t page, uint64_t v) { p->content[page] = v; }
int ko_pool_extent_allocated(const ko_pool *p, uint32_t extent) {
  return p->extents[extent].allocated;
}

}  // extern "C"
