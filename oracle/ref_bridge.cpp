// ref_bridge.cpp -- TEST INFRASTRUCTURE ONLY.
//
// A thin extern "C" face over the reference's own headers, compiled from the
// reference checkout where it lies (never copied into this repository).  The
// resulting oracle/_ref/libkvref.so lets the tests compare the restated oracle
// with the reference's real code for everything that is host-only C++:
// layout geometry, addressing, codecs, the int8/fp8 page quantizers, the split
// rule and the chunk validation.  The Metal kernels, MetalBuffer-backed
// operators and KvPool (macOS clock) cannot be built here and are not wrapped.
#include "metal/abi/ExecutionGeometry.h"
#include "metal/abi/KvExtent.h"
#include "metal/abi/PagedAttention.h"
#include "ops/PagedAttention.hpp"
#include "ops/PagedKv.hpp"

#include "Fp8PageFormatReference.hpp"
#include "Q8PageFormatReference.hpp"

#include <cstring>
#include <memory>
#include <span>
#include <string_view>

using namespace richengine;

namespace {
kv::Layout layout_of(uint32_t layers, uint32_t heads, uint32_t dim, uint32_t format) {
  return kv::Layout{layers, heads, dim, static_cast<kv::Format>(format)};
}
}  // namespace

extern "C" {

// out[0..7]: data bytes, scale bytes, model page bytes, alignment pages,
// minimum pages, maximum pages, valid, elements per layer page
void ref_layout(uint32_t layers, uint32_t heads, uint32_t dim, uint32_t format, uint64_t *out) {
  const kv::Layout l = layout_of(layers, heads, dim, format);
  out[0] = l.dataBytesPerLayerPage();
  out[1] = l.scaleBytesPerLayerPage();
  out[2] = l.bytesPerModelPage();
  out[3] = l.extentAlignmentPages();
  out[4] = l.minimumExtentPages();
  out[5] = l.maximumExtentPages();
  out[6] = l.valid();
  out[7] = l.elementsPerLayerPage();
}
uint32_t ref_extent_pages_for(uint32_t layers, uint32_t heads, uint32_t dim, uint32_t format,
                              uint64_t pages) {
  return layout_of(layers, heads, dim, format).extentPagesFor(pages);
}
uint64_t ref_key_element(uint32_t head, uint32_t token, uint32_t d, uint32_t head_dim) {
  return richengine_kv_key_element_dim(head, token, d, head_dim);
}
uint64_t ref_value_element(uint32_t head, uint32_t token, uint32_t d, uint32_t head_dim) {
  return richengine_kv_value_element_dim(head, token, d, head_dim);
}
uint64_t ref_scale_element(uint32_t head, uint32_t token) {
  return richengine_kv_scale_element(head, token);
}
uint64_t ref_kv_offset(uint32_t extent_pages, uint32_t db, uint32_t sb, uint32_t layer,
                       uint32_t tensor, uint32_t index) {
  return richengine_kv_offset(extent_pages, db, sb, layer, tensor, index);
}
uint64_t ref_kv_layer(uint32_t extent_pages, uint32_t db, uint32_t sb, uint32_t layer) {
  const RichKvLayer l = richengine_kv_layer(extent_pages, db, sb, layer);
  return (uint64_t{l.offset} << 32) | l.extent_pages;
}
uint64_t ref_page_entry(uint64_t address, uint32_t index) {
  return richengine_kv_page_entry(address, index);
}
uint16_t ref_float_to_bf16(float v) { return kv::floatToBFloat16(v); }
float ref_bf16_to_float(uint16_t v) { return kv::bfloat16ToFloat(v); }
uint8_t ref_float_to_fp8(float v) { return kv::floatToFp8E4m3(v); }
float ref_fp8_to_float(uint8_t c) { return kv::fp8E4m3ToFloat(c); }
float ref_query_stage(float v) { return kv::queryStage(v); }
uint32_t ref_verify_splits(uint32_t committed, uint32_t rows) {
  return kv::verifyAttentionSplits(committed, rows);
}
uint32_t ref_prefill_tiles(uint32_t rows) { return kv::prefillAttentionTiles(rows); }
// 0 ok, 1..4 in the order the reference checks.
int ref_chunk_validation(uint32_t committed, uint32_t tokens, uint32_t stride, uint32_t entries) {
  const kv::ChunkedPrefillParams p{committed, tokens, stride, entries, {}};
  const std::string_view e = kv::chunkedPrefillValidationError(p);
  if (e.empty()) return 0;
  if (e == "chunk_tokens_out_of_range") return 1;
  if (e == "context_out_of_range") return 2;
  if (e == "chunk_stride_invalid") return 3;
  if (e == "page_table_too_short") return 4;
  return -1;
}
uint32_t ref_chunk_required_pages(uint32_t committed, uint32_t tokens) {
  const kv::ChunkedPrefillParams p{committed, tokens, 0, 0, {}};
  return kv::chunkedPrefillRequiredPages(p);
}
uint32_t ref_param_sizes(uint32_t which) {
  switch (which) {
  case 0: return sizeof(RichChunkedPrefillParams);
  case 1: return sizeof(RichPrefillAttentionParams);
  case 2: return sizeof(RichVerifyAttentionParams);
  case 3: return sizeof(RichKvLayer);
  default: return 0;
  }
}

// The reference's whole-page quantizers (4 KV heads x 256, one layer page):
// logical inputs are [token][head][d] fp32; the page is the packed
// keys | key scales | values | value scales struct of the reference header.
// Returns 0, or -1 when the reference rejected the input.
int ref_quantize_q8_page(const float *keys, const float *values, uint32_t valid_tokens,
                         uint8_t *page_bytes) {
  auto page = std::make_unique<kv::Q8LayerPage>();
  const size_t n = size_t{valid_tokens} * kv::kKvHeads * kv::kHeadDimension;
  try {
    kv::quantizeLayerPage(std::span<const float>(keys, n), std::span<const float>(values, n),
                          valid_tokens, *page);
  } catch (const std::exception &) {
    return -1;
  }
  std::memcpy(page_bytes, page.get(), sizeof(kv::Q8LayerPage));
  return 0;
}
int ref_quantize_fp8_page(const float *keys, const float *values, uint32_t valid_tokens,
                          uint8_t *page_bytes) {
  auto page = std::make_unique<kv::Fp8LayerPage>();
  const size_t n = size_t{valid_tokens} * kv::kFp8KvHeads * kv::kFp8HeadDimension;
  try {
    kv::quantizeFp8LayerPage(std::span<const float>(keys, n), std::span<const float>(values, n),
                             valid_tokens, *page);
  } catch (const std::exception &) {
    return -1;
  }
  std::memcpy(page_bytes, page.get(), sizeof(kv::Fp8LayerPage));
  return 0;
}
uint64_t ref_q8_page_bytes() { return sizeof(kv::Q8LayerPage); }

}  // extern "C"
