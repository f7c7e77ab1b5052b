// Tests of the C++ host mirror (include/kvx.hpp) written the way the
// reference's own host tests are: known answers first, then behaviour.
//   kvx_host_test host    -- no GPU needed (layout, planning, validation)
//   kvx_host_test device  -- storage, pool, append, decode on the GPU
// Known answers come from the reference's tests:
//   dev/tests/engine/q8_paged_kv_test.cc:17-61 (byte accounting),
//   dev/tests/engine/q8_flash_attention_metal_test.mm:53-56 (verify splits),
//   dev/tests/engine/paged_attention_plan_test.mm:104-176 (plans, validation).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <numeric>
#include <vector>

#include "kvx.hpp"

using namespace kvx;
using kv::Format;
using kv::Layout;

namespace {

int failures = 0;
#define EXPECT(condition)                                                          \
  do {                                                                             \
    if (!(condition)) {                                                            \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #condition);           \
      ++failures;                                                                  \
    }                                                                              \
  } while (0)

template <class Exception> bool throws(const std::function<void()> &f) {
  try {
    f();
  } catch (const Exception &) {
    return true;
  } catch (...) {
    return false;
  }
  return false;
}

void hip(hipError_t e) {
  if (e != hipSuccess) {
    std::printf("HIP error: %s\n", hipGetErrorString(e));
    std::exit(2);
  }
}

uint16_t bf16(float f) {
  uint32_t bits;
  std::memcpy(&bits, &f, 4);
  return static_cast<uint16_t>((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}
float f32(uint16_t h) {
  const uint32_t bits = uint32_t{h} << 16;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

constexpr Layout kOracleLayout{16, 4, 256, Format::Int8};

void testByteAccounting() {
  const Layout bf16Layout{16, 4, 256, Format::BFloat16};
  EXPECT(bf16Layout.valid());
  EXPECT(bf16Layout.bytesPerModelPage() == 2'097'152);
  EXPECT(bf16Layout.extentAlignmentPages() == 1);
  EXPECT(bf16Layout.minimumExtentPages() == 32 && bf16Layout.maximumExtentPages() == 96);
  EXPECT(bf16Layout.scaleBytesPerLayerPage() == 0);
  const Layout compact{10, 2, 256, Format::BFloat16};
  EXPECT(compact.bytesPerModelPage() == 655'360);
  EXPECT(compact.extentAlignmentPages() == 2);
  EXPECT(compact.minimumExtentPages() == 104 && compact.maximumExtentPages() == 306);
  EXPECT(kOracleLayout.extentAlignmentPages() == 128);
  EXPECT(kOracleLayout.minimumExtentPages() == 128 && kOracleLayout.maximumExtentPages() == 128);
  EXPECT(kOracleLayout.extentPagesFor(127) == 0 && kOracleLayout.extentPagesFor(128) == 128 &&
         kOracleLayout.extentPagesFor(1000) == 128);
  const Layout compactInt8{10, 2, 256, Format::Int8};
  EXPECT(compactInt8.bytesPerModelPage() == 332'800);
  EXPECT(compactInt8.extentAlignmentPages() == 256);
  EXPECT(compactInt8.minimumExtentPages() == 256 && compactInt8.maximumExtentPages() == 512);
  EXPECT(compactInt8.extentPagesFor(255) == 0 && compactInt8.extentPagesFor(511) == 256);
  EXPECT(compactInt8.extentPagesFor(10'240) == 512);
  EXPECT(compactInt8.extentPagesFor(10'496) == 256);
  EXPECT(bf16Layout.extentPagesFor(31) == 0 && bf16Layout.extentPagesFor(448) == 64 &&
         bf16Layout.extentPagesFor(97) == 48);
  EXPECT(!(Layout{16, 4, 256, static_cast<Format>(0)}.valid()));
  EXPECT(kOracleLayout.bytesPerModelPage() == 1'064'960);
  EXPECT(4608 * kOracleLayout.bytesPerModelPage() == 4'907'335'680ULL);
  const Layout int4{16, 4, 256, Format::Int4};
  EXPECT(int4.dataBytesPerLayerPage() == 16'384 && int4.scaleBytesPerLayerPage() == 512);
  EXPECT(int4.bytesPerModelPage() == 540'672);
  // The largest extent stays a whole number of alignment units, indexable in
  // 14 bits and below 4 GiB.
  EXPECT(int4.largestExtentPages() % int4.extentAlignmentPages() == 0);
  EXPECT(int4.largestExtentPages() <= 16383);
  EXPECT(uint64_t{int4.largestExtentPages()} * int4.bytesPerModelPage() < (1ULL << 32));
}

void testPlans() {
  EXPECT(kv::verifyAttentionSplits(0) == 32);
  EXPECT(kv::verifyAttentionSplits(16384) == 33);
  EXPECT(kv::verifyAttentionSplits(131072) == 128);
  const Layout layout{16, 4, 256, Format::Int8};
  const auto one = ops::PagedAttention::prefillPlan(1, 24, layout);
  EXPECT(one.splits == 32);
  const auto full = ops::PagedAttention::prefillPlan(2048, 24, layout);
  EXPECT(full.splits == 1);
  // rows * D * 4 partial bytes and rows * 2 * 4 statistic bytes per slot
  // (runtime/ops/PagedAttention.cpp:29-32); slots = tiles * kv heads * splits,
  // rows per slot = 8 * group.
  EXPECT(full.workspace.partialsBytes == uint64_t{256} * 4 * 1 * 48 * 256 * 4);
  EXPECT(full.workspace.statisticsBytes == uint64_t{256} * 4 * 1 * 48 * 2 * 4);
  const auto sized = ops::PagedAttention::prefillPlan(16384, 256, 24, layout);
  EXPECT(sized.splits > 1 && sized.splits <= 32);
  EXPECT(sized.workspace.partialsBytes == uint64_t(32) * sized.splits * 8 * 24 * 256 * 4);
  // int4 pages: 2048 rows alone take four splits (three full rounds of wave slots), four such
  // chunks in one batched call fill them in one split each
  const Layout int4Layout{16, 4, 256, Format::Int4};
  EXPECT(ops::PagedAttention::prefillPlan(16384, 2048, 24, int4Layout).splits == 4);
  EXPECT(ops::PagedAttention::prefillPlan(16384, 2048, 24, int4Layout, 4).splits == 1);
  EXPECT(throws<std::invalid_argument>(
      [&] { (void)ops::PagedAttention::prefillPlan(16384, 2048, 24, int4Layout, 0); }));
  const auto bound = ops::PagedAttention::prefillWorkspace(2048, 24, layout);
  EXPECT(bound.partialsBytes >= full.workspace.partialsBytes);
  const auto verify = ops::PagedAttention::verifyPlan(2, 24, layout, {0, 131072});
  EXPECT(verify.laneSplits[0] == 32 && verify.laneSplits[1] == 128 && verify.splits == 128);
  EXPECT(verify.rowCapacity == kv::kVerifyRows);
  const auto decode = ops::PagedAttention::verifyPlan(2, 24, layout, {31, 32 * 64}, false, true);
  EXPECT(decode.laneSplits[0] == 1 && decode.laneSplits[1] == 3 && decode.rowCapacity == 1);
  EXPECT(throws<std::invalid_argument>([&] { (void)ops::PagedAttention::prefillPlan(0, 24, layout); }));
  EXPECT(throws<std::invalid_argument>([&] { (void)ops::PagedAttention::prefillPlan(2049, 24, layout); }));
  EXPECT(throws<std::invalid_argument>([&] { (void)ops::PagedAttention::prefillPlan(8, 25, layout); }));
  EXPECT(throws<std::invalid_argument>(
      [&] { (void)ops::PagedAttention::verifyPlan(1, 24, {16, 4, 256, Format::Float8E4M3}, {0}, true); }));
}

// dev/tests/engine/kv_page_cache_test.cpp:44-69: what images add to a block's key.
void testImageIdentity() {
  using engine::ImageSpan;
  const ImageSpan red{8, 16, 8, 8, 0x1111, 0x2222}, blue{8, 16, 8, 8, 0x3333, 0x4444};
  const ImageSpan redLater{40, 16, 8, 8, 0x1111, 0x2222}, first{0, 8, 4, 8, 0x5555, 0x6666};
  const engine::ImageIdentity none;
  EXPECT(engine::blockImageIdentity(0, 32, {}) == none);              // text only
  EXPECT(engine::blockImageIdentity(32, 32, {red}) == none);          // a block after the image
  const auto r = engine::blockImageIdentity(0, 32, {red}), b = engine::blockImageIdentity(0, 32, {blue});
  EXPECT(!(r == none) && !(r == b));                                  // the content digest counts
  EXPECT(!(engine::blockImageIdentity(32, 32, {redLater}) == r));     // so does the block's alignment
  const std::vector<ImageSpan> three{first, blue, redLater};          // only overlapping spans count
  EXPECT(engine::blockImageIdentity(32, 32, three) == engine::blockImageIdentity(32, 32, {redLater}));
  EXPECT(engine::blockImageIdentity(0, 8, three) == engine::blockImageIdentity(0, 8, {first}));
  EXPECT(!(engine::blockImageIdentity(0, 32, three) == engine::blockImageIdentity(0, 32, {first})));
}

void testParams() {
  const auto p = ops::PagedAttention::prefillParams(4093, 77, 96, 131);
  EXPECT(p.committed_tokens == 4093 && p.chunk_tokens == 77 && p.chunk_stride == 96);
  EXPECT(sizeof(kv::ChunkedPrefillParams) == 24 && sizeof(kv::PrefillAttentionParams) == 32 &&
         sizeof(kv::VerifyAttentionParams) == 36);
  // chunk_tokens 0 or past the stride, stride not a page multiple, table too
  // short, context past the limit: each is refused before anything runs.
  EXPECT(throws<std::invalid_argument>([] { (void)ops::PagedAttention::prefillParams(0, 0, 32, 1); }));
  EXPECT(throws<std::invalid_argument>([] { (void)ops::PagedAttention::prefillParams(0, 33, 32, 2); }));
  EXPECT(throws<std::invalid_argument>([] { (void)ops::PagedAttention::prefillParams(0, 8, 24, 1); }));
  EXPECT(throws<std::invalid_argument>([] { (void)ops::PagedAttention::prefillParams(32, 1, 32, 1); }));
  EXPECT(throws<std::invalid_argument>(
      [] { (void)ops::PagedAttention::prefillParams(KVX_MAX_PHYSICAL_TOKENS, 1, 32, 1 << 14); }));
  const auto v = ops::PagedAttention::verifyParams(100, 4);
  EXPECT(v.chunk_tokens == kv::kVerifyRows && v.chunk_stride == kv::kVerifyChunkStride);
  const auto t = ops::PagedAttention::verifyTreeParams(100, 4);
  EXPECT(t.chunk_tokens == 15);
}

// ---- device ------------------------------------------------------------------

void testStorageLifecycle() {
  const Layout layout{2, 2, 64, Format::Int8};
  kv::PageStorage storage(layout, 12, 4, /*aligned=*/false);
  EXPECT(storage.pageCount() == 12 && storage.extentPages() == 4);
  EXPECT(storage.bytesPerPage() == layout.bytesPerModelPage());
  EXPECT(!storage.allocated(0));
  EXPECT(storage.allocateExtent(0) == kv::AllocationFailure::None);
  EXPECT(storage.allocated(3) && !storage.allocated(4));
  EXPECT(throws<std::logic_error>([&] { (void)storage.allocateExtent(0); }));
  EXPECT(throws<std::logic_error>([&] { storage.releaseExtent(1); }));
  EXPECT(throws<std::out_of_range>([&] { (void)storage.allocateExtent(3); }));
  // copying a page of an unallocated extent copies nothing
  EXPECT(throws<std::logic_error>([&] { storage.copyPages({{0, 4}}); }));
  // a refused allocation is a value and leaves nothing allocated
  storage.setBudget(storage.extentBytes());
  EXPECT(storage.allocateExtent(1) == kv::AllocationFailure::EngineBudget);
  EXPECT(!storage.allocated(4) && storage.allocatedBytes() == storage.extentBytes());
  storage.setBudget(0);
  EXPECT(storage.allocateExtent(1) == kv::AllocationFailure::None);
  // a new extent reads as zeros; page bytes round-trip; copies are byte-identical
  std::vector<uint8_t> zero = storage.readPage(5);
  EXPECT(std::all_of(zero.begin(), zero.end(), [](uint8_t b) { return b == 0; }));
  std::vector<uint8_t> bytes(storage.bytesPerPage());
  for (size_t i = 0; i < bytes.size(); ++i) bytes[i] = static_cast<uint8_t>(i * 131 + 7);
  storage.writePage(1, bytes);
  storage.copyPages({{1, 6}});
  hip(hipDeviceSynchronize());
  EXPECT(storage.readPage(6) == bytes && storage.readPage(1) == bytes);
  // a destination that is also a source of the batch is refused
  EXPECT(throws<std::invalid_argument>([&] { storage.copyPages({{1, 2}, {2, 3}}); }));
  // entries decode to (extent base, index)
  std::vector<uint64_t> table(3);
  storage.entries({0, 3, 5}, 0, table.data());
  EXPECT((table[0] & KVX_PAGE_INDEX_MASK) == 0 && (table[1] & KVX_PAGE_INDEX_MASK) == 3 &&
         (table[2] & KVX_PAGE_INDEX_MASK) == 1);
  EXPECT((table[0] & ~uint64_t{KVX_PAGE_INDEX_MASK}) == (table[1] & ~uint64_t{KVX_PAGE_INDEX_MASK}));
  EXPECT((table[0] & ~uint64_t{KVX_PAGE_INDEX_MASK}) != (table[2] & ~uint64_t{KVX_PAGE_INDEX_MASK}));
  storage.releaseExtent(1);
  EXPECT(!storage.allocated(4));
}

void testPoolCompaction() {
  const Layout layout{2, 2, 64, Format::Int4};
  kv::PageStorage storage(layout, 12, 4, /*aligned=*/false);
  engine::KvPool pool(storage, 4);
  EXPECT(pool.freePageCount() == 4);
  auto got = pool.acquirePages(10);
  EXPECT(got.granted() && got.pages.size() == 10);
  // every page gets its own content
  std::vector<std::vector<uint8_t>> content(12);
  for (uint32_t page : got.pages) {
    content[page].resize(storage.bytesPerPage());
    for (size_t i = 0; i < content[page].size(); ++i)
      content[page][i] = static_cast<uint8_t>(page * 37 + i * 11);
    storage.writePage(page, content[page]);
  }
  // leave one extent with a single held page and the others with room for it
  std::vector<uint32_t> byExtent[3];
  for (uint32_t page : got.pages) byExtent[page / 4].push_back(page);
  uint32_t sparse = 0;
  for (uint32_t e = 1; e < 3; ++e)
    if (byExtent[e].size() < byExtent[sparse].size()) sparse = e;
  std::vector<uint32_t> held;
  for (uint32_t e = 0; e < 3; ++e)
    for (size_t i = 0; i < byExtent[e].size(); ++i) {
      const bool keep = e == sparse ? i == 0 : i + 1 < byExtent[e].size();
      if (keep) held.push_back(byExtent[e][i]);
      else pool.releasePage(byExtent[e][i], false);
    }
  const auto moves = pool.compactExtent();
  hip(hipDeviceSynchronize());
  EXPECT(!moves.empty() && moves.firstPage == sparse * 4);
  for (uint32_t page : held) {
    const uint32_t now = moves.follow(page);
    EXPECT(pool.pageActive(now));
    EXPECT(storage.readPage(now) == content[page]);
    if (page / 4 == sparse) EXPECT(now / 4 != sparse);
    else EXPECT(now == page);
  }
  EXPECT(pool.snapshot().extent_compactions == 1 && pool.snapshot().pages_moved == 1);
  EXPECT(pool.reclaimEmptyExtents(false, 8) == storage.extentBytes());
  EXPECT(throws<std::out_of_range>([&] { pool.retainPage(12, false); }));
  EXPECT(throws<std::logic_error>([&] { pool.releasePage(moves.firstPage, false); }));
}

template <class T> T *toDevice(const std::vector<T> &host) {
  T *device = nullptr;
  hip(hipMalloc(&device, host.size() * sizeof(T)));
  hip(hipMemcpy(device, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
  return device;
}

// One appended token attended by one decode row: the probability is exactly 1,
// so every query head's output is the dequantised value row, bf16(scale * code).
void testAppendDecodeSingleToken() {
  const Layout layout{2, 4, 256, Format::Int4};
  const uint32_t H = 4, G = 6, D = 256, QH = H * G;
  kv::PageStorage storage(layout, 8, 4, /*aligned=*/false);
  engine::KvPool pool(storage, 8);
  const auto got = pool.acquirePages(2);
  std::vector<uint64_t> table(2);
  storage.entries(got.pages, 0, table.data());
  uint64_t *tableDevice = toDevice(table);
  const uint64_t *tables[1] = {tableDevice};

  std::vector<uint16_t> keys(H * 32 * D, 0), values(H * D * 32, 0), queries(H * G * D);
  for (uint32_t h = 0; h < H; ++h)
    for (uint32_t d = 0; d < D; ++d) {
      keys[(h * 32 + 0) * D + d] = bf16(std::sin(0.37f * d + h));
      // codes d % 15 - 7 with scale 0.5 * (h + 1): exactly representable
      values[(h * D + d) * 32 + 0] = bf16(0.5f * (h + 1) * (float(d % 15) - 7.0f));
    }
  for (size_t i = 0; i < queries.size(); ++i) queries[i] = bf16(std::cos(0.11f * i));
  uint16_t *keysDevice = toDevice(keys), *valuesDevice = toDevice(values), *queriesDevice = toDevice(queries);
  uint16_t *outputDevice = nullptr;
  hip(hipMalloc(&outputDevice, queries.size() * 2));

  for (uint32_t layer = 0; layer < 2; ++layer) {
    const auto chunk = ops::PagedAttention::prefillParams(0, 1, 32, 2);
    ops::PagedAttention::addPrefillStore(nullptr, storage, layer, keysDevice, valuesDevice, tableDevice, chunk);
    const auto plan = ops::PagedAttention::verifyPlan(1, QH, layout, {0}, false, true);
    void *workspace = nullptr;
    hip(hipMalloc(&workspace, plan.workspace.bytes() + 256));
    ops::PagedVerifyBuffers buffers;
    buffers.queries = queriesDevice;
    buffers.output = outputDevice;
    buffers.workspace = workspace;
    buffers.workspaceBytes = plan.workspace.bytes() + 256;
    buffers.pageTables = tables;
    hip(hipMemset(outputDevice, 0xff, queries.size() * 2));
    ops::PagedAttention::attend(nullptr, storage, layer, buffers, {chunk}, plan);
    hip(hipDeviceSynchronize());
    std::vector<uint16_t> output(queries.size());
    hip(hipMemcpy(output.data(), outputDevice, output.size() * 2, hipMemcpyDeviceToHost));
    uint32_t wrong = 0;
    for (uint32_t h = 0; h < H; ++h)
      for (uint32_t g = 0; g < G; ++g)
        for (uint32_t d = 0; d < D; ++d)
          wrong += f32(output[(h * G + g) * D + d]) != 0.5f * (h + 1) * (float(d % 15) - 7.0f);
    EXPECT(wrong == 0);
    hip(hipFree(workspace));
  }
  // A second token: addVerify with a decode plan stores it and attends in one
  // call (layer 0); the store and the attention as two calls on layer 1, which
  // holds the same first token, must give the same bits.
  {
    for (uint32_t h = 0; h < H; ++h)
      for (uint32_t d = 0; d < D; ++d) {
        keys[(h * 32 + 0) * D + d] = bf16(std::cos(0.21f * d - h));
        values[(h * D + d) * 32 + 0] = bf16(std::sin(0.05f * d + 0.3f * h));
      }
    hip(hipMemcpy(keysDevice, keys.data(), keys.size() * 2, hipMemcpyHostToDevice));
    hip(hipMemcpy(valuesDevice, values.data(), values.size() * 2, hipMemcpyHostToDevice));
    const auto chunk = ops::PagedAttention::verifyParams(1, 2, 1);
    const auto plan = ops::PagedAttention::verifyPlan(1, QH, layout, {1}, false, true, /*sizedForGpu=*/true);
    EXPECT(plan.laneSplits.size() == 1 && plan.laneSplits[0] == 1);
    void *workspace = nullptr;
    hip(hipMalloc(&workspace, plan.workspace.bytes() + 256));
    ops::PagedVerifyBuffers buffers;
    buffers.chunkKeys = keysDevice;
    buffers.chunkValues = valuesDevice;
    buffers.queries = queriesDevice;
    buffers.output = outputDevice;
    buffers.workspace = workspace;
    buffers.workspaceBytes = plan.workspace.bytes() + 256;
    buffers.pageTables = tables;
    std::vector<uint16_t> one(queries.size()), two(queries.size());
    ops::PagedAttention::addVerify(nullptr, storage, 0, buffers, {chunk}, plan);
    hip(hipDeviceSynchronize());
    hip(hipMemcpy(one.data(), outputDevice, one.size() * 2, hipMemcpyDeviceToHost));
    ops::PagedAttention::addPrefillStore(nullptr, storage, 1, keysDevice, valuesDevice, tableDevice, chunk);
    ops::PagedAttention::attend(nullptr, storage, 1, buffers, {chunk}, plan);
    hip(hipDeviceSynchronize());
    hip(hipMemcpy(two.data(), outputDevice, two.size() * 2, hipMemcpyDeviceToHost));
    EXPECT(one == two);
    // the same attention over the library's static workspace, no buffer of the caller's
    {
      std::vector<uint16_t> three(queries.size());
      ops::PagedVerifyBuffers bare = buffers;
      bare.workspace = nullptr;
      bare.workspaceBytes = 0;
      hip(hipMemset(outputDevice, 0x5A, three.size() * 2));
      ops::PagedAttention::attendStatic(nullptr, storage, 1, bare, {chunk}, plan);
      hip(hipDeviceSynchronize());
      hip(hipMemcpy(three.data(), outputDevice, three.size() * 2, hipMemcpyDeviceToHost));
      EXPECT(three == two);
    }
    bool moved = false;  // and the second token did change the result
    for (size_t i = 0; i < one.size(); ++i) moved = moved || f32(one[i]) != 0.5f * (i / (G * D) + 1) * (float(i % D % 15) - 7.0f);
    EXPECT(moved);
    // The merge's second output.  One-row lanes with packed rows: the gathered
    // operand [lane][row][query head][D] has the staged rows' order, and a zero
    // gate halves every element exactly.
    void *hiddenDevice = nullptr, *packedDevice = nullptr;
    hip(hipMalloc(&hiddenDevice, two.size() * 2));
    hip(hipMalloc(&packedDevice, size_t{2 * QH + 2 * H} * D * 2));
    hip(hipMemset(packedDevice, 0, size_t{2 * QH + 2 * H} * D * 2));
    std::vector<uint16_t> hidden(two.size());
    ops::PagedAttention::attend(nullptr, storage, 1, buffers, {chunk}, plan, nullptr, hiddenDevice);
    hip(hipDeviceSynchronize());
    hip(hipMemcpy(hidden.data(), hiddenDevice, hidden.size() * 2, hipMemcpyDeviceToHost));
    EXPECT(hidden == two);
    ops::PagedAttention::attend(nullptr, storage, 1, buffers, {chunk}, plan, packedDevice, hiddenDevice);
    hip(hipDeviceSynchronize());
    hip(hipMemcpy(hidden.data(), hiddenDevice, hidden.size() * 2, hipMemcpyDeviceToHost));
    uint32_t unhalved = 0;
    for (size_t i = 0; i < hidden.size(); ++i) unhalved += f32(hidden[i]) != 0.5f * f32(two[i]);
    EXPECT(unhalved == 0);
    // The decode step as one call with the second output: the token stored again (the same
    // bytes), the row attended and the gathered operand written.
    hip(hipMemset(hiddenDevice, 0x3C, hidden.size() * 2));
    ops::PagedAttention::addVerify(nullptr, storage, 1, buffers, {chunk}, plan, nullptr, hiddenDevice);
    hip(hipDeviceSynchronize());
    hip(hipMemcpy(hidden.data(), hiddenDevice, hidden.size() * 2, hipMemcpyDeviceToHost));
    EXPECT(hidden == two);
    buffers.treeMasks = static_cast<const uint32_t *>(packedDevice);  // any non-null masks: a tree plan
    EXPECT(throws<std::invalid_argument>([&] {
      ops::PagedAttention::addVerify(nullptr, storage, 1, buffers, {chunk}, plan, nullptr, hiddenDevice);
    }));
    buffers.treeMasks = nullptr;
    hip(hipFree(hiddenDevice));
    hip(hipFree(packedDevice));
    hip(hipFree(workspace));
  }
  // an invalid chunk is refused before anything is enqueued
  kv::ChunkedPrefillParams bad{0, 1, 32, 0, {}};
  EXPECT(throws<std::invalid_argument>(
      [&] { ops::PagedAttention::addPrefillStore(nullptr, storage, 0, keysDevice, valuesDevice, tableDevice, bad); }));
  EXPECT(throws<std::out_of_range>([&] {  // a layer past the layout
    ops::PagedAttention::addPrefillStore(nullptr, storage, 2, keysDevice, valuesDevice, tableDevice,
                                         ops::PagedAttention::prefillParams(0, 1, 32, 2));
  }));
  hip(hipFree(tableDevice));
  hip(hipFree(keysDevice));
  hip(hipFree(valuesDevice));
  hip(hipFree(queriesDevice));
  hip(hipFree(outputDevice));
}

// The fused QKV prepare + store without norms and with an identity rotation is the
// layout change alone: the pages must hold what addPrefillStore writes from the same
// rows, and the queries the packed query values.
void testQkvStoreIsPrepareThenStore() {
  const Layout layout{1, 4, 256, Format::Int8};
  const uint32_t H = 4, G = 6, D = 256, QH = H * G, T = 5, packedStride = (2 * QH + 2 * H) * D;
  kv::PageStorage plain(layout, 4, 4, /*aligned=*/false), fused(layout, 4, 4, /*aligned=*/false);
  plain.allocateExtent(0);
  fused.allocateExtent(0);
  const std::vector<uint32_t> pages{2, 1};
  std::vector<uint64_t> plainTable(2), fusedTable(2);
  plain.entries(pages, 0, plainTable.data());
  fused.entries(pages, 0, fusedTable.data());
  uint64_t *plainDevice = toDevice(plainTable), *fusedDevice = toDevice(fusedTable);
  std::vector<uint16_t> packed(T * packedStride), keys(H * 32 * D, 0), values(H * D * 32, 0);
  for (size_t i = 0; i < packed.size(); ++i) packed[i] = bf16(std::sin(0.013f * float(i % 7919)));
  for (uint32_t t = 0; t < T; ++t)
    for (uint32_t h = 0; h < H; ++h)
      for (uint32_t d = 0; d < D; ++d) {
        keys[(h * 32 + t) * D + d] = packed[t * packedStride + 2 * QH * D + h * D + d];
        values[(h * D + d) * 32 + t] = packed[t * packedStride + 2 * QH * D + H * D + h * D + d];
      }
  std::vector<float> ones(T * 32, 1.0f), zeros(T * 32, 0.0f);
  uint16_t *packedDevice = toDevice(packed), *keysDevice = toDevice(keys), *valuesDevice = toDevice(values);
  float *cosDevice = toDevice(ones), *sinDevice = toDevice(zeros);
  uint16_t *queriesDevice = nullptr;
  hip(hipMalloc(&queriesDevice, size_t{H} * 32 * G * D * 2));
  hip(hipMemset(queriesDevice, 0, size_t{H} * 32 * G * D * 2));
  const auto chunk = ops::PagedAttention::prefillParams(30, T, 32, 2);  // crosses a page boundary
  ops::PagedAttention::addPrefillStore(nullptr, plain, 0, keysDevice, valuesDevice, plainDevice, chunk);
  const uint64_t *tables[1] = {fusedDevice};
  ops::PagedAttention::QkvBuffers buffers;
  buffers.packed = packedDevice;
  buffers.ropeCos = cosDevice;
  buffers.ropeSin = sinDevice;
  buffers.queries = queriesDevice;
  buffers.pageTables = tables;
  ops::PagedAttention::addQkvStore(nullptr, fused, 0, buffers, {chunk}, QH, T, 32, 32, /*queryGate=*/true);
  hip(hipDeviceSynchronize());
  EXPECT(plain.readPage(2) == fused.readPage(2) && plain.readPage(1) == fused.readPage(1));
  std::vector<uint16_t> queries(size_t{H} * 32 * G * D);
  hip(hipMemcpy(queries.data(), queriesDevice, queries.size() * 2, hipMemcpyDeviceToHost));
  uint32_t wrong = 0;
  for (uint32_t t = 0; t < T; ++t)
    for (uint32_t q = 0; q < QH; ++q)
      for (uint32_t d = 0; d < D; ++d)
        wrong += queries[(((q / G) * 32 + t) * G + q % G) * D + d] != packed[t * packedStride + q * 2 * D + d];
  EXPECT(wrong == 0);
  buffers.keyNorm = packedDevice;  // one norm without the other
  EXPECT(throws<std::invalid_argument>([&] {
    ops::PagedAttention::addQkvStore(nullptr, fused, 0, buffers, {chunk}, QH, T, 32, 32, true);
  }));
  for (void *p : {static_cast<void *>(plainDevice), static_cast<void *>(fusedDevice), static_cast<void *>(packedDevice),
                  static_cast<void *>(keysDevice), static_cast<void *>(valuesDevice), static_cast<void *>(cosDevice),
                  static_cast<void *>(sinDevice), static_cast<void *>(queriesDevice)})
    hip(hipFree(p));
}

}  // namespace

int main(int argc, char **argv) {
  const std::string mode = argc > 1 ? argv[1] : "host";
  testByteAccounting();
  testPlans();
  testParams();
  testImageIdentity();
  if (mode == "device") {
    testStorageLifecycle();
    testPoolCompaction();
    testAppendDecodeSingleToken();
    testQkvStoreIsPrepareThenStore();
  }
  if (failures) {
    std::printf("kvx_host_test (%s): %d failure(s)\n", mode.c_str(), failures);
    return 1;
  }
  std::printf("kvx_host_test (%s): ok\n", mode.c_str());
  return 0;
}
