// ref_bridge_cache.cpp -- TEST INFRASTRUCTURE ONLY.
//
// An extern "C" face over the reference's own blockImageIdentity
// (runtime/engine/cache/KvCache.cpp:29-52), compiled together with that source file
// where it lies in the reference checkout (never copied into this repository).  Only
// this one function is kept: everything else of KvCache.cpp needs the page pool, whose
// source cannot be built here (a macOS-only clock), and is dropped by the linker
// (hidden visibility, a section per function, --gc-sections).
#include "engine/cache/KvCache.hpp"

#include <cstdint>
#include <span>
#include <vector>

using namespace richengine;

extern "C" __attribute__((visibility("default"))) void ref_image_identity(
    uint64_t block_begin, uint32_t block_tokens, const uint64_t *spans, uint32_t n_spans,
    uint64_t *lo, uint64_t *hi) {
  // spans: six 64-bit words per span: offset, tokens, grid height, grid width, digest lo, digest hi
  std::vector<ImageSpan> list(n_spans);
  for (uint32_t i = 0; i < n_spans; ++i) {
    const uint64_t *s = spans + 6 * size_t{i};
    list[i].offset = static_cast<uint32_t>(s[0]);
    list[i].tokens = static_cast<uint32_t>(s[1]);
    list[i].gridHeight = static_cast<uint32_t>(s[2]);
    list[i].gridWidth = static_cast<uint32_t>(s[3]);
    list[i].digestLo = s[4];
    list[i].digestHi = s[5];
  }
  const engine::ImageIdentity identity =
      engine::blockImageIdentity(block_begin, block_tokens, std::span<const ImageSpan>(list));
  *lo = identity.lo;
  *hi = identity.hi;
}
