// int4 paged attention for gfx950: the split and merge kernels of
// kv_attend_decode, kv_attend_verify (chain and tree) and kv_attend_prefill for
// packed-nibble pages with head dimension 256.
//
// One wave per (sequence or prefill tile, split, KV head, block of 16 fused
// query rows) streams the split's pages once:
// coalesced 128-bit key loads and 64-bit value loads, the page's fp32 scales,
// bf16 MFMA (16x16x32) for q.k and p.v with the GQA group as the 16-wide N
// side, page-granular online softmax in registers.  The arithmetic follows the
// reference tile (common/paged_attention_tile.h:85-349): scores are the raw
// code dot product times the key scale times the score scale, the running
// maximum moves once per 32-token page, and probability x value scale is
// rounded to bf16 before it meets the value codes.
//
// Nibble -> bf16 without a table: OR-ing a 4-bit field into the mantissa of
// 0x4300 gives 128 + field exactly.  With the stored two's-complement code c,
// field = (c & 15) ^ 8 = c + 8 gives 136 + c and field = (c & 15) ^ 7 = 7 - c
// gives 135 - c.  Even positions use the first form, odd positions the second
// with the other operand negated, so the products are q.c + 136 q and
// q.c - 135 q: the constant parts largely cancel pairwise and what is left is
// tracked in fp32 and subtracted (keys: once per q row; values: per page,
// rescaled with the accumulator).  Positions are dimensions for q.k and tokens
// for p.v.
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
template <class T>
__device__ __forceinline__ T load_streaming(const uint8_t *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const KVX_GLOBAL T *>(
      reinterpret_cast<uintptr_t>(p)));
}
template <class T>
__device__ __forceinline__ T load_global(const void *p) {
  return *reinterpret_cast<const KVX_GLOBAL T *>(reinterpret_cast<uintptr_t>(p));
}

constexpr uint32_t kPage = KVX_PAGE_TOKENS;
constexpr uint32_t kLanes = KVX_LANES_PER_LAUNCH;
constexpr uint32_t kD = 256;
constexpr uint32_t kRowBytes = kD / 2;                // one token's packed row
constexpr uint32_t kHeadSlabBytes = kPage * kRowBytes;  // 4 KiB per (head, page, tensor)
constexpr float kLog2e = 1.4426950408889634f;
constexpr uint32_t kTableSlots = 1024;  // page entries of one split staged in LDS

struct DecodeLane {
  const uint64_t *table;
  const uint32_t *masks;  // tree verify: ancestor bitmask per row; null = causal chain
  uint32_t committed;
  uint32_t active_rows;   // query rows attended (1 for decode)
  uint32_t split_count;
  uint32_t first_item;  // first (lane, split) work item of this lane
  float score_scale;
  uint64_t row_base;    // first fused row of the lane's slots in the workspace
  uint64_t q_offset;    // element offset of the lane's queries
};
struct DecodeArgs {
  DecodeLane lane[kLanes];
  uint32_t n_lanes;
  uint32_t kv_heads;
  uint32_t group;
  uint32_t row_stride;
  uint32_t fused_rows;  // row capacity x group: fused query rows per (lane, KV head)
  kvx_kv_layer kv;
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

// What one lane holds of one page.
struct PageRegs {
  u32x4 k[4];   // [token block * 2 + half row]: 16 bytes of the lane's key token
  u32x2 v[8];   // [token slot]: 8 bytes (16 dims) of each of the lane's 8 tokens
  f32x4 ks[2];  // key scales of the lane's score tokens, per token block
  f32x4 vs[2];  // value scales, same tokens
};

__device__ __forceinline__ f32x4 mfma_bf16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// Lane geometry: t = lane & 15, g = lane >> 4.
//  q.k : A = keys, row t = token 16*tb + t of the page; k-slots = the 8 nibbles
//        of one dword of that token's row.  B = queries, column t = q head.
//        Output column t = q head, rows 4g..4g+3 = tokens 16*tb + 4g + r.
//  p.v : A = values, row t = dims 16t..16t+15 (one MFMA per nibble position),
//        k-slots = the lane group's 8 tokens 4g..4g+3, 16+4g..16+4g+3.
//        B = probabilities, column t = q head: exactly the q.k output registers.
__device__ __forceinline__ void load_page(PageRegs &r, uint64_t entry, uint32_t head,
                                          uint32_t kv_heads, uint32_t layer_offset,
                                          uint64_t key_scales_off, uint64_t values_off,
                                          uint64_t value_scales_off, uint32_t t, uint32_t g) {
  const uint32_t index = uint32_t(entry) & KVX_PAGE_INDEX_MASK;
  const uint8_t *region = reinterpret_cast<const uint8_t *>(entry - index) + layer_offset;
  const uint64_t slab = (uint64_t(index) * kv_heads + head) * kHeadSlabBytes;
  const uint8_t *keys = region + slab;
  const uint8_t *values = region + values_off + slab;
  const uint64_t scale_index = (uint64_t(index) * kv_heads + head) * kPage;
  const float *key_scales = reinterpret_cast<const float *>(region + key_scales_off) + scale_index;
  const float *value_scales =
      reinterpret_cast<const float *>(region + value_scales_off) + scale_index;
#pragma unroll
  for (uint32_t tb = 0; tb < 2; ++tb)
#pragma unroll
    for (uint32_t half = 0; half < 2; ++half)
      r.k[tb * 2 + half] =
          load_streaming<u32x4>(keys + (16 * tb + t) * kRowBytes + 64 * half + 16 * g);
#pragma unroll
  for (uint32_t s = 0; s < 8; ++s) {
    const uint32_t token = (s < 4 ? 0 : 16) + 4 * g + (s & 3);
    r.v[s] = load_streaming<u32x2>(values + token * kRowBytes + 8 * t);
  }
#pragma unroll
  for (uint32_t tb = 0; tb < 2; ++tb) {
    r.ks[tb] = load_global<f32x4>(key_scales + 16 * tb + 4 * g);
    r.vs[tb] = load_global<f32x4>(value_scales + 16 * tb + 4 * g);
  }
}

// Four bf16 pairs from one dword of eight nibbles: register p holds nibble p
// (low half) and nibble p + 4 (high half).  Even nibbles become 136 + c, odd
// ones 135 - c.
__device__ __forceinline__ u32x4 expand_key_dword(uint32_t x) {
  u32x4 out;
  out[0] = (x & 0x000F000Fu) ^ 0x43084308u;
  out[1] = ((x >> 4) & 0x000F000Fu) ^ 0x43074307u;
  out[2] = ((x >> 8) & 0x000F000Fu) ^ 0x43084308u;
  out[3] = ((x >> 12) & 0x000F000Fu) ^ 0x43074307u;
  return out;
}

struct State {
  f32x4 acc[16];  // [nibble position m]: dims 16*(4g + r) + m of q head t
  float row_max;
  float row_sum;   // this lane's tokens only; lanes of a q head are summed at the end
  float bias;      // constant part carried by acc, this lane's tokens only
};

// MASKED: the page may hold tokens some row does not see (only the last two
// pages of a sequence can); other pages skip the per-token test.
template <bool MASKED>
__device__ __forceinline__ void attend_page(const PageRegs &r, const u32x4 *q_lds, float q_bias,
                                            float score_scale, uint32_t first_token,
                                            const Sight &sight, uint32_t lane, uint32_t g,
                                            State &st) {
#ifdef KVX_PROBE_STREAM_ONLY
  // Measurement build: consume every loaded register with almost no arithmetic,
  // to see what the memory system delivers for this access pattern.
  uint32_t x = 0;
  for (uint32_t i = 0; i < 4; ++i) x ^= r.k[i][0] ^ r.k[i][1] ^ r.k[i][2] ^ r.k[i][3];
  for (uint32_t i = 0; i < 8; ++i) x ^= r.v[i][0] ^ r.v[i][1];
  st.row_sum += r.ks[0][0] + r.ks[1][3] + r.vs[0][1] + r.vs[1][2] + __uint_as_float(x & 0xffu);
  return;
#endif
  // ---- q.k ----
  f32x4 s[2];
  s[0] = s[1] = f32x4{-q_bias, -q_bias, -q_bias, -q_bias};
#pragma unroll
  for (uint32_t kb = 0; kb < 8; ++kb) {
    const u32x4 q = q_lds[kb * 64 + lane];
#pragma unroll
    for (uint32_t tb = 0; tb < 2; ++tb)
      s[tb] = mfma_bf16(expand_key_dword(r.k[tb * 2 + (kb >> 2)][kb & 3]), q, s[tb]);
  }
  // ---- page softmax ----
  float score[8], local_max = -INFINITY;
  bool live[8];
#pragma unroll
  for (uint32_t i = 0; i < 8; ++i) {
    const uint32_t tb = i >> 2, rr = i & 3;
    float v = s[tb][rr] * r.ks[tb][rr];
    v *= score_scale;
    live[i] = !MASKED || sight.sees(first_token + 16 * tb + 4 * g + rr);
    score[i] = live[i] ? v : -INFINITY;
    local_max = fmaxf(local_max, score[i]);
  }
  local_max = fmaxf(local_max, __shfl_xor(local_max, 16));
  local_max = fmaxf(local_max, __shfl_xor(local_max, 32));
  const float next_max = fmaxf(st.row_max, local_max);
  // A row that has seen nothing yet keeps -inf; its rescale is 1, not exp(nan).
  const float rescale = next_max == st.row_max
                            ? 1.0f
                            : __builtin_amdgcn_exp2f((st.row_max - next_max) * kLog2e);
  float weight[8], page_sum = 0.0f;
#pragma unroll
  for (uint32_t i = 0; i < 8; ++i) {
    // The difference first, so the page's maximum gets exactly 1.
    float p = __builtin_amdgcn_exp2f((score[i] - next_max) * kLog2e);
    if (MASKED) p = live[i] ? p : 0.0f;
    page_sum += p;
    const float w = p * r.vs[i >> 2][i & 3];
    weight[i] = live[i] ? w : 0.0f;
  }
  st.row_sum = fmaf(st.row_sum, rescale, page_sum);
  st.row_max = next_max;
  // bf16 probabilities (round to nearest even): even tokens as they are, odd
  // tokens negated (their value codes are expanded as 135 - c).
  u32x4 pb;
  float page_bias = 0.0f;
#pragma unroll
  for (uint32_t p = 0; p < 4; ++p) {
    const f32x2 pair = {weight[2 * p], weight[2 * p + 1]};
    const uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
    page_bias = fmaf(136.0f, __uint_as_float(bits << 16), page_bias);
    page_bias = fmaf(-135.0f, __uint_as_float(bits & 0xffff0000u), page_bias);
    pb[p] = bits ^ 0x80000000u;
  }
  st.bias = fmaf(st.bias, rescale, page_bias);
  if (__builtin_amdgcn_ballot_w64(rescale != 1.0f)) {
#pragma unroll
    for (uint32_t m = 0; m < 16; ++m) st.acc[m] *= rescale;
  }
  // ---- p.v ----
#pragma unroll
  for (uint32_t half = 0; half < 2; ++half) {
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {  // nibbles 0..3, then 4..7 of the dword
      u32x4 vop[4];
#pragma unroll
      for (uint32_t p = 0; p < 4; ++p) {
        const uint32_t even = r.v[2 * p][half], odd = r.v[2 * p + 1][half];
        const uint32_t both =
            __builtin_amdgcn_perm(odd, even, part ? 0x07060302u : 0x05040100u);
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i)
          vop[i][p] = ((both >> (4 * i)) & 0x000F000Fu) ^ 0x43074308u;
      }
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t m = 8 * half + 4 * part + i;
        st.acc[m] = mfma_bf16(vop[i], pb, st.acc[m]);
      }
    }
  }
}

#ifndef KVX_DECODE_DEPTH
#define KVX_DECODE_DEPTH 2
#endif
#ifndef KVX_DECODE_WAVES
#define KVX_DECODE_WAVES 2
#endif
constexpr uint32_t kDepth = KVX_DECODE_DEPTH;

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
// order.
constexpr uint32_t kMergeSequential = 32;
constexpr uint32_t kMergeWaves = 4;

struct MergeSums {
  f32x4 numerator;
  float denominator;
};

// Sums splits [first, last) of the row in split order; `maximum` is the row's
// maximum over all splits.
__device__ __forceinline__ MergeSums merge_range(const float *__restrict__ partials,
                                                 const float *__restrict__ statistics,
                                                 uint64_t first_row, uint32_t first, uint32_t last,
                                                 uint32_t M, float maximum, uint32_t lane) {
  MergeSums sums{{0.0f, 0.0f, 0.0f, 0.0f}, 0.0f};
  for (uint32_t base = first; base < last; base += 64) {
    const uint32_t mine = base + lane;
    f32x2 stat = {-INFINITY, 0.0f};
    if (mine < last) stat = load_global<f32x2>(statistics + (first_row + uint64_t(mine) * M) * 2);
    const float my_weight = expf(__fsub_rn(stat[0], maximum));
    const float my_term = __fmul_rn(my_weight, stat[1]);
    const uint32_t count = min(64u, last - base);
    for (uint32_t i = 0; i < count; i += 8) {
      f32x4 part[8];
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u) {
        const uint64_t row = first_row + uint64_t(base + min(i + u, count - 1)) * M;
        part[u] = load_global<f32x4>(partials + row * kD + 4 * lane);
      }
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u) {
        if (i + u < count) {
          const float weight = __shfl(my_weight, i + u);
#pragma unroll
          for (uint32_t c = 0; c < 4; ++c)
            sums.numerator[c] = __fadd_rn(sums.numerator[c], __fmul_rn(weight, part[u][c]));
          sums.denominator = __fadd_rn(sums.denominator, __shfl(my_term, i + u));
        }
      }
    }
  }
  return sums;
}

// grid (fused query row, KV head, lane), kMergeWaves waves per row.  Lanes whose
// pages fit one split were written by the split kernel itself.
__global__ __launch_bounds__(64 * kMergeWaves) void decode_int4_merge_kernel(
    uint16_t *__restrict__ output, const float *__restrict__ partials,
    const float *__restrict__ statistics, DecodeArgs a) {
  const uint32_t j = blockIdx.x, head = blockIdx.y;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const DecodeLane &l = a.lane[blockIdx.z];
  const uint32_t pages = (l.committed + l.active_rows + kPage - 1) / kPage;
  const uint32_t per = (pages + l.split_count - 1) / l.split_count;
  const uint32_t written = (pages + per - 1) / per;
  if (written <= 1) return;
  const uint32_t G = a.group, M = a.fused_rows;
  uint16_t *out_row =
      output + l.q_offset + uint64_t(head) * a.row_stride * G * kD + uint64_t(j) * kD;
  if (j / G >= l.active_rows) {  // rows past the live ones read as zeros
    if (wave == 0) *reinterpret_cast<u32x2 *>(out_row + 4 * lane) = u32x2{0u, 0u};
    return;
  }
  const uint64_t first_row = l.row_base + uint64_t(head) * l.split_count * M + j;
  const bool sequential = written <= kMergeSequential;
  if (sequential && wave) return;
  float maximum = -INFINITY;
  for (uint32_t base = 0; base < written; base += 64) {
    const uint32_t s = base + lane;
    float m = s < written ? load_global<float>(statistics + (first_row + uint64_t(s) * M) * 2)
                          : -INFINITY;
#pragma unroll
    for (uint32_t step = 32; step > 0; step >>= 1) m = fmaxf(m, __shfl_xor(m, step));
    maximum = fmaxf(maximum, m);
  }
  MergeSums sums;
  if (sequential) {
    sums = merge_range(partials, statistics, first_row, 0, written, M, maximum, lane);
  } else {
    const uint32_t share = (written + kMergeWaves - 1) / kMergeWaves;
    const uint32_t first = min(written, wave * share), last = min(written, first + share);
    const MergeSums mine = merge_range(partials, statistics, first_row, first, last, M, maximum, lane);
    __shared__ f32x4 numerators[kMergeWaves][64];
    __shared__ float denominators[kMergeWaves][64];
    numerators[wave][lane] = mine.numerator;
    denominators[wave][lane] = mine.denominator;
    __syncthreads();
    if (wave) return;
    sums = mine;
#pragma unroll
    for (uint32_t w = 1; w < kMergeWaves; ++w) {
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
  *reinterpret_cast<u32x2 *>(out_row + 4 * lane) = packed;
}

__global__ __launch_bounds__(64)
__attribute__((amdgpu_waves_per_eu(KVX_DECODE_WAVES, KVX_DECODE_WAVES))) void decode_int4_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  const uint32_t item = blockIdx.x, head = blockIdx.y;
  uint32_t li = 0;
  for (uint32_t i = 1; i < a.n_lanes; ++i)
    if (item >= a.lane[i].first_item) li = i;
  const DecodeLane &l = a.lane[li];
  const uint32_t split = item - l.first_item;
  if (split >= l.split_count) return;
  const uint32_t visible = l.committed + l.active_rows;
  const uint32_t pages = (visible + kPage - 1) / kPage;
  const uint32_t per = (pages + l.split_count - 1) / l.split_count;
  const uint32_t written = (pages + per - 1) / per;  // splits that own a page
  const uint32_t begin = split * per;
  if (begin >= pages) return;
  const uint32_t end = min(pages, begin + per);

  const uint32_t lane = threadIdx.x, t = lane & 15, g = lane >> 4;
  const uint32_t H = a.kv_heads, G = a.group, M = a.fused_rows;
  // This wave's MFMA columns are fused rows 16 z .. 16 z + 15 of the tile; a fused
  // row is (query row, head in group) = (m / G, m % G).
  const uint32_t m = 16 * blockIdx.z + t, query_row = m / G;
  const bool in_tile = m < M, live_row = in_tile && query_row < l.active_rows;
  Sight sight;
  sight.committed = l.committed;
  sight.visible = visible;
  sight.limit = live_row ? min(visible, l.committed + min(query_row, l.active_rows - 1) + 1) : visible;
  sight.tree = live_row && l.masks != nullptr;
  sight.mask = sight.tree ? l.masks[query_row] : 0u;
  const uint32_t db = kPage * H * kRowBytes, sb = kPage * H * 4;
  const RegionOffsets ro = region_offsets(a.kv.extent_pages, db, sb);
  const float score_scale = default_score_scale(kD, l.score_scale);

  // Queries of this KV head: [row][g][D] bf16, fused row m.  Their loads go out
  // first; everything behind them returns later, so the wait for the queries
  // leaves the page loads in flight.  Columns without a live row carry zeros.
  const uint16_t *q_head = queries + l.q_offset + uint64_t(head) * a.row_stride * G * kD;
  const uint16_t *q_row = q_head + uint64_t(live_row ? m : 0) * kD;
  u32x4 q_raw[8];
#pragma unroll
  for (uint32_t kb = 0; kb < 8; ++kb)
    q_raw[kb] = load_global<u32x4>(q_row + 8 * (16 * (kb >> 2) + 4 * g + (kb & 3)));

  // The split's page entries (at most kTableSlots; the launcher declines longer
  // splits) go through LDS and are read back with uniform LDS loads.  (Fetched from memory one by one they would be
  // vector loads in the steady loop, and since loads return in order the wait for
  // an entry would drain every page load in flight.)
  __shared__ uint64_t table_lds[kTableSlots];
  for (uint32_t i = lane; i < end - begin; i += 64)
    table_lds[i] = load_global<uint64_t>(l.table + begin + i);
  __syncthreads();
  // kDepth register sets rotate: a set is refilled with the page kDepth ahead as
  // soon as its page has been consumed, so up to kDepth pages are in flight.
  PageRegs r[kDepth];
  auto fill = [&](PageRegs &set, uint32_t slot) {
#ifdef KVX_PROBE_SAME_PAGE
    // Measurement build: every refill is the split's first page, so loads hit the
    // caches and the time left is the kernel's own arithmetic.
    slot = 0;
#endif
    // The empty asm statements pin the loads of one fill together and in place:
    // moved up into the arithmetic that still reads the set they would need a
    // second copy of its registers, and interleaved with another fill's loads
    // they would make every wait cover both.
    asm volatile("");
    load_page(set, table_lds[slot], head, H, a.kv.offset, ro.key_scales, ro.values,
              ro.value_scales, t, g);
    asm volatile("");
  };
  // The first fills are unconditional too (a split shorter than kDepth pages
  // loads its last page again): the steady loop must be entered with the same
  // loads in flight, in the same order, as its own iterations leave behind.
#pragma unroll
  for (uint32_t d = 0; d < kDepth; ++d) fill(r[d], min(d, end - begin - 1));

  // Register kb of the staged queries holds the 8 dims of dword
  // w = 16*(kb>>2) + 4g + (kb&3) of a key row in expansion order; odd dims are
  // negated.  q_bias is the constant part of every score.
  __shared__ u32x4 q_lds[8 * 64];
  float q_bias = 0.0f;
#pragma unroll
  for (uint32_t kb = 0; kb < 8; ++kb) {
    // dims 8w .. 8w+7 as four bf16 pairs, regrouped to (p, p+4) pairs
    const u32x4 raw = q_raw[kb];
    u32x4 q_reg;
    q_reg[0] = __builtin_amdgcn_perm(raw[2], raw[0], 0x05040100u);
    q_reg[1] = __builtin_amdgcn_perm(raw[2], raw[0], 0x07060302u) ^ 0x80008000u;
    q_reg[2] = __builtin_amdgcn_perm(raw[3], raw[1], 0x05040100u);
    q_reg[3] = __builtin_amdgcn_perm(raw[3], raw[1], 0x07060302u) ^ 0x80008000u;
    if (!live_row) q_reg = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (uint32_t p = 0; p < 4; ++p) {
      // even dims carry +136 q, odd dims (stored negated) -135 q = +135 stored
      const float pair_sum =
          __uint_as_float(q_reg[p] << 16) + __uint_as_float(q_reg[p] & 0xffff0000u);
      q_bias = fmaf((p & 1) ? 135.0f : 136.0f, pair_sum, q_bias);
    }
    q_lds[kb * 64 + lane] = q_reg;
  }
  q_bias += __shfl_xor(q_bias, 16);
  q_bias += __shfl_xor(q_bias, 32);

  State st;
#pragma unroll
  for (uint32_t m = 0; m < 16; ++m) st.acc[m] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  st.row_max = -INFINITY;
  st.row_sum = 0.0f;
  st.bias = 0.0f;

  // Steady state: every refill is unconditional, so the loop body is straight
  // line code and the wait for a set counts exactly the loads issued after it;
  // a refill under a branch would make each wait cover the newest loads too.
  // The last page of the split is never consumed here, so no token test.
  uint32_t page = begin;
  for (; page + 2 * kDepth <= end; page += kDepth) {
#pragma unroll
    for (uint32_t d = 0; d < kDepth; ++d) {
      attend_page<false>(r[d], q_lds, q_bias, score_scale, (page + d) * kPage, sight, lane, g,
                         st);
      fill(r[d], page + d + kDepth - begin);
    }
  }
  // Tail: at most 2 * kDepth - 1 pages are left, the first kDepth of them loaded.
#pragma unroll
  for (uint32_t k = 0; k < 2 * kDepth - 1; ++k) {
    const uint32_t d = k % kDepth;
    if (page + k < end) {
      attend_page<true>(r[d], q_lds, q_bias, score_scale, (page + k) * kPage, sight, lane, g,
                        st);
      if (k + kDepth < 2 * kDepth - 1 && page + k + kDepth < end)
        fill(r[d], page + k + kDepth - begin);
    }
  }

  // Lanes of one q head hold disjoint tokens: combine their sums and the
  // constant part, then take the constant part out of the accumulators.
  float row_sum = st.row_sum, bias = st.bias;
  row_sum += __shfl_xor(row_sum, 16);
  row_sum += __shfl_xor(row_sum, 32);
  bias += __shfl_xor(bias, 16);
  bias += __shfl_xor(bias, 32);
  uint16_t *out_head = output + l.q_offset + uint64_t(head) * a.row_stride * G * kD;

  if (written == 1) {
    // One split: the merge's weights are exp(0) = 1, so the row is acc / sum.
    // Rows of the tile past the live ones read as zeros (row_sum is 0 there).
    if (in_tile) {
      const float denominator = live_row ? row_sum : 0.0f;
#pragma unroll
      for (uint32_t rr = 0; rr < 4; ++rr)
#pragma unroll
        for (uint32_t m4 = 0; m4 < 4; ++m4) {
          u32x2 packed;
#pragma unroll
          for (uint32_t i = 0; i < 2; ++i) {
            const float lo = st.acc[4 * m4 + 2 * i][rr] - bias;
            const float hi = st.acc[4 * m4 + 2 * i + 1][rr] - bias;
            const float qlo = denominator > 0.0f ? __fdiv_rn(lo, denominator) : 0.0f;
            const float qhi = denominator > 0.0f ? __fdiv_rn(hi, denominator) : 0.0f;
            packed[i] = uint32_t(f32_to_bf16(qlo)) | (uint32_t(f32_to_bf16(qhi)) << 16);
          }
          *reinterpret_cast<u32x2 *>(out_head + uint64_t(m) * kD + 16 * (4 * g + rr) + 4 * m4) =
              packed;
        }
    }
    return;
  }

  const uint64_t head_row = l.row_base + uint64_t(head) * l.split_count * M;
  if (live_row) {
    const uint64_t row = head_row + uint64_t(split) * M + m;
    float *out = partials + row * kD;
#pragma unroll
    for (uint32_t rr = 0; rr < 4; ++rr)
#pragma unroll
      for (uint32_t m4 = 0; m4 < 4; ++m4) {
        f32x4 v;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) v[i] = st.acc[4 * m4 + i][rr] - bias;
        *reinterpret_cast<f32x4 *>(out + 16 * (4 * g + rr) + 4 * m4) = v;
      }
    if (g == 0) {
      statistics[row * 2] = st.row_max;
      statistics[row * 2 + 1] = row_sum;
    }
  }
}

}  // namespace
}  // namespace kvx

using namespace kvx;

uint32_t kvx_attend_phases();  // bit 0 = split kernel, bit 1 = merge kernel

// Runs paged attention (split kernel, then the merge of multi-split lanes) for
// int4 pages of head dimension 256; returns 1 (declined) for shapes it does not
// cover so the caller runs the format-generic kernels, 0 when enqueued, or a
// negative status.  Lane i reads its queries and writes its rows at element
// offset i * lane_stride; the rows of one KV head lie row_stride * group * 256
// elements apart.  row_masks: null, or one ancestor bitmask per (lane, row of
// capacity).  Every lane has the row capacity of the first.
int kvx_attend_int4_launch(const kvx_storage *s, kvx_kv_layer kv, uint32_t query_heads,
                           const void *queries, void *output, const uint64_t *const *page_tables,
                           const kvx_verify_params *lanes, uint32_t n_lanes,
                           const uint32_t *row_masks, uint32_t row_stride, uint64_t lane_stride,
                           void *workspace, uint64_t workspace_bytes, hipStream_t stream) {
  const kvx_layout &l = s->layout;
  if (l.format != KVX_FMT_INT4 || l.head_dim != kD) return 1;
  const uint32_t H = l.kv_heads, G = query_heads / H;
  const uint32_t capacity = lanes[0].row_capacity, M = capacity * G;
  if (G > 16 || !capacity || capacity > KVX_TREE_NODES) return 1;
  uint64_t total_rows = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) {
    const kvx_verify_params &p = lanes[i];
    if (p.row_capacity != capacity || !p.active_rows || p.active_rows > capacity) return 1;
    const uint32_t pages = (p.committed_tokens + p.active_rows + kPage - 1) / kPage;
    const uint32_t splits = std::max(1u, p.split_count);
    if ((pages + splits - 1) / splits > kTableSlots) return 1;
    total_rows += uint64_t(p.split_count) * H * M;
  }
  const uint64_t statistics_offset = (total_rows * kD * sizeof(float) + 255) / 256 * 256;
  if (workspace_bytes < statistics_offset + total_rows * 2 * sizeof(float)) return 1;
  float *partials = static_cast<float *>(workspace);
  float *statistics = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + statistics_offset);
  uint64_t row_base = 0;
  for (uint32_t first = 0; first < n_lanes; first += kLanes) {
    DecodeArgs a{};
    a.n_lanes = std::min(kLanes, n_lanes - first);
    a.kv_heads = H;
    a.group = G;
    a.row_stride = row_stride;
    a.fused_rows = M;
    a.kv = kv;
    uint32_t items = 0;
    for (uint32_t i = 0; i < a.n_lanes; ++i) {
      const kvx_verify_params &p = lanes[first + i];
      DecodeLane &dl = a.lane[i];
      dl.table = page_tables[first + i];
      dl.masks = row_masks ? row_masks + uint64_t(first + i) * capacity : nullptr;
      dl.committed = p.committed_tokens;
      dl.active_rows = p.active_rows;
      dl.split_count = p.split_count;
      dl.first_item = items;
      dl.score_scale = p.score_scale != 0.0f ? p.score_scale : l.score_scale;
      dl.row_base = row_base;
      dl.q_offset = uint64_t(first + i) * lane_stride;
      items += p.split_count;
      row_base += uint64_t(p.split_count) * H * M;
    }
    uint32_t max_splits = 0;
    for (uint32_t i = 0; i < a.n_lanes; ++i) max_splits = std::max(max_splits, a.lane[i].split_count);
    const uint32_t phases = kvx_attend_phases();
    hipError_t e = hipSuccess;
    if (phases & 1u) {
      hipLaunchKernelGGL(decode_int4_kernel, dim3(items, H, (M + 15) / 16), dim3(64), 0, stream,
                         static_cast<const uint16_t *>(queries), static_cast<uint16_t *>(output),
                         partials, statistics, a);
      e = hipGetLastError();
      if (e != hipSuccess) return hip_fail(e, "decode_int4_kernel");
    }
    if (max_splits > 1 && (phases & 2u)) {
      hipLaunchKernelGGL(decode_int4_merge_kernel, dim3(M, H, a.n_lanes), dim3(64 * kMergeWaves), 0,
                         stream,
                         static_cast<uint16_t *>(output), partials, statistics, a);
      e = hipGetLastError();
      if (e != hipSuccess) return hip_fail(e, "decode_int4_merge_kernel");
    }
  }
  return 0;
}
