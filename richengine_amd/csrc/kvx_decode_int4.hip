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
// Nibble -> bf16 without a table: a 4-bit field OR-ed into the mantissa of a
// power of two 2^e, at the place whose weight is 1, gives 2^e + field exactly:
// 0x4300 | field = 128 + field, 0x4180 | field << 3 = 16 + field.  With the stored
// two's-complement code c, field = (c & 15) ^ 8 = c + 8 and field = (c & 15) ^ 7 =
// 7 - c.  Even positions use the first form, odd positions the second with the other
// operand negated, so the products are q.c plus a constant times q; the constant
// parts are tracked in fp32 and subtracted (keys: once per q row; values: per page,
// rescaled with the accumulator).  Positions are dimensions for q.k and tokens for p.v.
// Keys use 16 + field (24 + c, 23 - c): what the fp32 accumulator of q.k carries
// beside q.c decides how exact a score is, and a score that is off in its fifth
// digit turns the bf16 rounding of a probability now and then; with 128 + field that
// happened to one output row in two hundred, each then up to a bf16 place from the
// scalar result.  The field's place costs one shift per dword.  Values use 128 +
// field (136 + c, 135 - c): nothing is rounded after p.v but the result.
#include "kvx_attend_common.h"
#include "kvx_debug.h"

namespace kvx {
namespace {

constexpr uint32_t kRowBytes = kD / 2;                // one token's packed row
constexpr uint32_t kHeadSlabBytes = kPage * kRowBytes;  // 4 KiB per (head, page, tensor)

// What one lane holds of one page.
struct PageRegs {
  u32x4 k[4];   // [token block * 2 + half row]: 16 bytes of the lane's key token
  u32x2 v[8];   // [token slot]: 8 bytes (16 dims) of each of the lane's 8 tokens
  float scale;  // lane i < 32: key scale of token i; lane 32 + i: value scale of token i
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
// Byte offsets of this lane inside a (head, page) slab and inside the page's
// two scale rows; the same for every page, so the page's own part of an address
// is uniform and the loads take a scalar base plus one of these.
struct LaneOffsets {
  uint32_t keys;    // token t, bytes 16g.. of the row's first half
  uint32_t values;  // token 4g, bytes 8t..
  uint32_t scale;   // lane i < 32: key scale i; lane 32 + i: value scale i (from the key scales)
};
__device__ __forceinline__ LaneOffsets lane_offsets(uint32_t t, uint32_t g, uint32_t scale_rows_apart) {
  const uint32_t lane = 16 * g + t;
  return {t * kRowBytes + 16 * g, 4 * g * kRowBytes + 8 * t,
          (lane < kPage ? 0u : scale_rows_apart) + 4u * (lane & (kPage - 1))};
}

// PARTS: bit 0 the keys, bit 1 the values, bit 2 the scale lines.
template <uint32_t PARTS, bool REUSED>
__device__ __forceinline__ void load_page(PageRegs &r, uint64_t entry, uint32_t head,
                                          uint32_t kv_heads, uint32_t layer_offset,
                                          uint64_t key_scales_off, uint64_t values_off,
                                          const LaneOffsets &at) {
  // The entry is the same in every lane; saying so keeps the address arithmetic
  // on the scalar unit.
  const uint32_t entry_lo = __builtin_amdgcn_readfirstlane(uint32_t(entry));
  const uint32_t entry_hi = __builtin_amdgcn_readfirstlane(uint32_t(entry >> 32));
  const uint32_t index = entry_lo & KVX_PAGE_INDEX_MASK;
  const uint8_t *region =
      reinterpret_cast<const uint8_t *>((uint64_t(entry_hi) << 32) | (entry_lo - index)) + layer_offset;
  const uint64_t head_page = uint64_t(index) * kv_heads + head;
  const uint8_t *keys = region + head_page * kHeadSlabBytes;
  if constexpr (PARTS & 1u) {
#pragma unroll
    for (uint32_t tb = 0; tb < 2; ++tb)
#pragma unroll
      for (uint32_t half = 0; half < 2; ++half)
        r.k[tb * 2 + half] =
            load_streaming<u32x4, REUSED>(keys + at.keys + (16 * tb * kRowBytes + 64 * half));
  }
  if constexpr (PARTS & 2u) {
    const uint8_t *values = keys + values_off;
#pragma unroll
    for (uint32_t s = 0; s < 8; ++s)
      r.v[s] = load_streaming<u32x2, REUSED>(values + at.values + ((s < 4 ? 0 : 16) + (s & 3)) * kRowBytes);
  }
  // One scale per lane instead of the sixteen a lane multiplies with: they
  // are fetched from the owning lanes when the page is attended, which keeps
  // a register set at 33 registers.
  if constexpr (PARTS & 4u)
    r.scale = load_global<float>(region + key_scales_off + head_page * (kPage * 4u) + at.scale);
}

// x of this lane and x of the lane 16 (32) away, without the address register a
// shuffle through the LDS crossbar needs: the swaps exchange the odd rows of 16
// (the upper 32 lanes) of one operand with the even rows (lower lanes) of the
// other, so the two results hold x[l] and x[l ^ 16] (x[l ^ 32]) in some order.
struct LanePair {
  float a, b;
};
__device__ __forceinline__ LanePair across16(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return {__uint_as_float(r[0]), __uint_as_float(r[1])};
}
__device__ __forceinline__ LanePair across32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return {__uint_as_float(r[0]), __uint_as_float(r[1])};
}
// Maximum / sum over the four lanes of a column (lanes l, l^16, l^32, l^48).
__device__ __forceinline__ float column_max(float x) {
  LanePair p = across16(x);
  x = fmaxf(p.a, p.b);
  p = across32(x);
  return fmaxf(p.a, p.b);
}
__device__ __forceinline__ float column_sum(float x) {
  LanePair p = across16(x);
  x = p.a + p.b;
  p = across32(x);
  return p.a + p.b;
}

// Four bf16 pairs from one dword of eight nibbles: register p holds nibble p
// (low half) and nibble p + 4 (high half).  Even nibbles become 24 + c, odd
// ones 23 - c: the field sits at mantissa bits 3..6 of 16.0 (0x4180).
__device__ __forceinline__ u32x4 expand_key_dword(uint32_t x) {
  u32x4 out;
  out[0] = ((x << 3) & 0x00780078u) ^ 0x41C041C0u;
  out[1] = ((x >> 1) & 0x00780078u) ^ 0x41B841B8u;
  out[2] = ((x >> 5) & 0x00780078u) ^ 0x41C041C0u;
  out[3] = ((x >> 9) & 0x00780078u) ^ 0x41B841B8u;
  return out;
}

// Softmax state and accumulators of one block of 16 fused query rows.
struct State {
  // [nibble position m]: register r holds dim 16 (4g + r) + m of fused row t; in the kernels
  // that hold the tiles transposed (the probabilities as the A operand of p.v), dim
  // 16 t + m of fused row 4g + r.
  f32x4 acc[16];
  float row_max;
  float row_sum;   // this lane's tokens only; lanes of a column are summed at the end
  float bias;      // constant part carried by acc, this lane's tokens only
};

// Where a page's operands come from.  key(tb, kb): the A operand of q.k for token
// block tb and dims block kb; scales(ks, vs): key and value scales of the lane's
// eight score tokens; values(half, part, vop): the four A operands of p.v for nibble
// positions 8 half + 4 part + i.
//
// A page held in the wave's own registers as it was loaded, expanded on use.
struct RegisterPage {
  const PageRegs &r;
  uint32_t g;
  __device__ __forceinline__ u32x4 key(uint32_t tb, uint32_t kb) const {
    return expand_key_dword(r.k[tb * 2 + (kb >> 2)][kb & 3]);
  }
  // The scales come from the lanes that hold them (lane i: key scale of token i;
  // lane 32 + i: value scale of token i).  One base address per lane and the
  // token's place as the instruction's constant offset; written out because the
  // compiler would spend a register on every address.  The data comes back through
  // the LDS return path, hence the wait inside the block.
  __device__ __forceinline__ void scales(float (&ks)[8], float (&vs)[8]) const {
    const uint32_t own = 16 * g;
    asm volatile(
        "ds_bpermute_b32 %0, %16, %17\n\t"
        "ds_bpermute_b32 %1, %16, %17 offset:4\n\t"
        "ds_bpermute_b32 %2, %16, %17 offset:8\n\t"
        "ds_bpermute_b32 %3, %16, %17 offset:12\n\t"
        "ds_bpermute_b32 %4, %16, %17 offset:64\n\t"
        "ds_bpermute_b32 %5, %16, %17 offset:68\n\t"
        "ds_bpermute_b32 %6, %16, %17 offset:72\n\t"
        "ds_bpermute_b32 %7, %16, %17 offset:76\n\t"
        "ds_bpermute_b32 %8, %16, %17 offset:128\n\t"
        "ds_bpermute_b32 %9, %16, %17 offset:132\n\t"
        "ds_bpermute_b32 %10, %16, %17 offset:136\n\t"
        "ds_bpermute_b32 %11, %16, %17 offset:140\n\t"
        "ds_bpermute_b32 %12, %16, %17 offset:192\n\t"
        "ds_bpermute_b32 %13, %16, %17 offset:196\n\t"
        "ds_bpermute_b32 %14, %16, %17 offset:200\n\t"
        "ds_bpermute_b32 %15, %16, %17 offset:204\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(ks[0]), "=&v"(ks[1]), "=&v"(ks[2]), "=&v"(ks[3]), "=&v"(ks[4]), "=&v"(ks[5]),
          "=&v"(ks[6]), "=&v"(ks[7]), "=&v"(vs[0]), "=&v"(vs[1]), "=&v"(vs[2]), "=&v"(vs[3]),
          "=&v"(vs[4]), "=&v"(vs[5]), "=&v"(vs[6]), "=&v"(vs[7])
        : "v"(own), "v"(r.scale));
  }
  __device__ __forceinline__ void values(uint32_t half, uint32_t part, u32x4 (&vop)[4]) const {
#pragma unroll
    for (uint32_t p = 0; p < 4; ++p) {
      const uint32_t even = r.v[2 * p][half], odd = r.v[2 * p + 1][half];
      const uint32_t both = __builtin_amdgcn_perm(odd, even, part ? 0x07060302u : 0x05040100u);
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) vop[i][p] = ((both >> (4 * i)) & 0x000F000Fu) ^ 0x43074308u;
    }
  }
};

// One page against NB blocks of 16 fused query rows; every key and value
// operand is made once and used by all blocks.
// MASKED: the page may hold tokens some row does not see (only the last pages of a
// lane can); other pages skip the per-token test.
// keys_consumed() runs when the page's keys have been read for the last time:
// the steady loop refills them from there, half a page ahead of the rest.
// queries(nb, kb) yields the B operand of block nb for dims block kb.
// PINNED: the kernel runs one wave per SIMD and its accumulators live in the second
// register file (see the rescaling below).
// ROWS_DOWN: the accumulator tiles are held transposed (State::acc); for kernels whose
// accumulators live in the first register file, where one register of a tile can be
// multiplied alone.
template <bool MASKED, uint32_t NB, bool PINNED, bool ROWS_DOWN, class Page, class Queries,
          class KeysConsumed>
__device__ __forceinline__ void attend_page(const Page &source, Queries queries,
                                            const float *q_bias, float score_scale,
                                            uint32_t first_token, const Sight *sight,
                                            uint32_t g, State *st, KeysConsumed keys_consumed) {
  // ---- q.k ----
  f32x4 s[NB][2];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb)
    s[nb][0] = s[nb][1] = f32x4{-q_bias[nb], -q_bias[nb], -q_bias[nb], -q_bias[nb]};
#pragma unroll
  for (uint32_t kb = 0; kb < 8; ++kb) {
    u32x4 q[NB];
#pragma unroll
    for (uint32_t nb = 0; nb < NB; ++nb) q[nb] = queries(nb, kb);
#pragma unroll
    for (uint32_t tb = 0; tb < 2; ++tb) {
      const u32x4 k = source.key(tb, kb);
#pragma unroll
      for (uint32_t nb = 0; nb < NB; ++nb) s[nb][tb] = mfma_bf16(k, q[nb], s[nb][tb]);
    }
  }
  keys_consumed();
  float ks[8], vs[8];
  source.scales(ks, vs);
  // ---- page softmax, per block ----
  u32x4 pb[NB];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    float score[8], local_max = -INFINITY;
    bool live[8];
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
      const uint32_t tb = i >> 2, rr = i & 3;
      float v = s[nb][tb][rr] * ks[i];
      v *= score_scale;
      live[i] = !MASKED || sight[nb].sees(first_token + 16 * tb + 4 * g + rr);
      score[i] = live[i] ? v : -INFINITY;
      local_max = fmaxf(local_max, score[i]);
    }
    local_max = column_max(local_max);
    const float next_max = fmaxf(st[nb].row_max, local_max);
    // A row that has seen nothing yet keeps -inf; its rescale is 1, not exp(nan).
    const float rescale = next_max == st[nb].row_max
                              ? 1.0f
                              : __builtin_amdgcn_exp2f((st[nb].row_max - next_max) * kLog2e);
    float weight[8], page_sum = 0.0f;
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
      // The difference first, so the page's maximum gets exactly 1.
      float p = __builtin_amdgcn_exp2f((score[i] - next_max) * kLog2e);
      if (MASKED) p = live[i] ? p : 0.0f;
      page_sum += p;
      const float w = p * vs[i];
      weight[i] = live[i] ? w : 0.0f;
    }
    st[nb].row_sum = fmaf(st[nb].row_sum, rescale, page_sum);
    st[nb].row_max = next_max;
    // bf16 probabilities (round to nearest even): even tokens as they are, odd
    // tokens negated (their value codes are expanded as 135 - c).
    float page_bias = 0.0f;
#pragma unroll
    for (uint32_t p = 0; p < 4; ++p) {
      const f32x2 pair = {weight[2 * p], weight[2 * p + 1]};
      const uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
      page_bias = fmaf(136.0f, __uint_as_float(bits << 16), page_bias);
      page_bias = fmaf(-135.0f, __uint_as_float(bits & 0xffff0000u), page_bias);
      pb[nb][p] = bits ^ 0x80000000u;
    }
    st[nb].bias = fmaf(st[nb].bias, rescale, page_bias);
    const uint64_t grown = __builtin_amdgcn_ballot_w64(rescale != 1.0f);
    if constexpr (ROWS_DOWN) {
      // Register j of a lane holds fused row 4g + j, so the registers j need the multiply
      // only when one of the four rows j, 4 + j, 8 + j, 12 + j has a new maximum: over a
      // split of 64 pages that happens on about 15 pages, where some row of all sixteen
      // grows on about 38.  The factors of those four rows come out of the lanes that hold
      // them (lane t holds row t's).
      if (grown) {
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
          if (uint32_t(grown) & (0x1111u << j)) {
            const auto factor_of = [&](uint32_t row) {
              return __uint_as_float(
                  uint32_t(__builtin_amdgcn_readlane(int(__float_as_uint(rescale)), int(row))));
            };
            const float f0 = factor_of(j), f1 = factor_of(4 + j), f2 = factor_of(8 + j),
                        f3 = factor_of(12 + j);
            const float factor = g == 0 ? f0 : g == 1 ? f1 : g == 2 ? f2 : f3;
#pragma unroll
            for (uint32_t m = 0; m < 16; ++m) st[nb].acc[m][j] *= factor;
          }
        }
      }
    } else if (grown) {
#pragma unroll
      for (uint32_t m = 0; m < 16; ++m) {
        // Accumulators in the second register file are named there on the way in, so that
        // the moves out of it that a multiply needs stay inside this branch; left to itself
        // the compiler moves every accumulator out on every page.
        if constexpr (PINNED) asm volatile("" : "+a"(st[nb].acc[m]));
        st[nb].acc[m] *= rescale;
      }
    }
  }
  // ---- p.v ----
#pragma unroll
  for (uint32_t half = 0; half < 2; ++half) {
#pragma unroll
    for (uint32_t part = 0; part < 2; ++part) {  // nibbles 0..3, then 4..7 of the dword
      u32x4 vop[4];
      source.values(half, part, vop);
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t m = 8 * half + 4 * part + i;
#pragma unroll
        for (uint32_t nb = 0; nb < NB; ++nb)
          st[nb].acc[m] = ROWS_DOWN ? mfma_bf16(pb[nb], vop[i], st[nb].acc[m])
                                    : mfma_bf16(vop[i], pb[nb], st[nb].acc[m]);
      }
    }
  }
}

// The launch-wide arguments a wave works with, in registers.  The kernels read them out
// of DecodeArgs once; the kernel argument block itself is only ever read where this is
// filled in, because the compiler prefers fetching an argument again where it is used
// (one more trip to memory in a wave's set-up) to keeping it.
struct LaunchArgs {
  uint32_t kv_heads, group, fused_rows, row_stride;
  kvx_kv_layer kv;
  const uint16_t *chunk_keys, *chunk_values;
  uint64_t chunk_lane_stride;
  uint32_t chunk_stride;
  uint32_t all_partials;
};
__device__ __forceinline__ LaunchArgs launch_args_of(const DecodeArgs &a) {
  return {a.kv_heads,   a.group,        a.fused_rows,        a.row_stride,   a.kv,
          a.chunk_keys, a.chunk_values, a.chunk_lane_stride, a.chunk_stride, a.all_partials};
}

// One-token append done by the wave that owns the sequence's last page, for its
// own KV head: quantizes the token's key row and value row (bf16 -> int4 codes and
// one fp32 scale each, the arithmetic of append_kernel: reference
// common/paged_store_row.h:47-147) and stores them at slot committed % 32 of the
// page.  Each lane owns four consecutive dims.  The stores are complete before
// the caller loads the page: the wave waits for them, and no cache of this CU can
// hold the lines yet because only this wave reads this head of this page.
__device__ __forceinline__ void append_decode_token(const LaunchArgs &a, const DecodeLane &l,
                                                    uint32_t li, uint32_t head, uint32_t lane) {
  const uint32_t H = a.kv_heads;
  const uint32_t slot = l.committed % kPage;
  const uint64_t entry = l.table[l.committed / kPage];
  const Slab slab = slab_of(KVX_FMT_INT4, H, kD, a.kv, head, entry);
  const uint16_t *key_row =
      a.chunk_keys + li * a.chunk_lane_stride + uint64_t(head) * a.chunk_stride * kD + 4 * lane;
  const uint16_t *value_column =
      a.chunk_values + li * a.chunk_lane_stride + (uint64_t(head) * kD + 4 * lane) * a.chunk_stride;
  const u32x2 key_bits = load_global<u32x2>(key_row);
  float row[2][4];
  row[0][0] = __uint_as_float(key_bits[0] << 16);
  row[0][1] = __uint_as_float(key_bits[0] & 0xffff0000u);
  row[0][2] = __uint_as_float(key_bits[1] << 16);
  row[0][3] = __uint_as_float(key_bits[1] & 0xffff0000u);
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i)
    row[1][i] = bf16_to_f32(load_global<uint16_t>(value_column + uint64_t(i) * a.chunk_stride));
#pragma unroll
  for (uint32_t tensor = 0; tensor < 2; ++tensor) {
    float maximum = fmaxf(fmaxf(fabsf(row[tensor][0]), fabsf(row[tensor][1])),
                          fmaxf(fabsf(row[tensor][2]), fabsf(row[tensor][3])));
    for (int offset = 32; offset; offset >>= 1) maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
    uint32_t packed = 0;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      const float scaled =
          maximum == 0.0f ? 0.0f : __fdiv_rn(__fmul_rn(row[tensor][i], 7.0f), maximum);
      int code = int(rintf(scaled));
      code = code < -7 ? -7 : code > 7 ? 7 : code;
      if (maximum == 0.0f) code = 0;
      packed |= (uint32_t(code) & 0xfu) << (4 * i);
    }
    uint8_t *data = tensor ? slab.values : slab.keys;
    store_global<uint16_t>(data + slot * kRowBytes + 2 * lane, uint16_t(packed));
    if (lane == 0)
      store_global<float>((tensor ? slab.value_scales : slab.key_scales) + slot,
                          maximum == 0.0f ? 0.0f : __fdiv_rn(maximum, 7.0f));
  }
  // The stores are complete before the page is loaded: vmcnt(0), with the other
  // counters left alone.  The builtin, so that the compiler's own count of what is
  // in flight sees the wait.
  __builtin_amdgcn_s_waitcnt(0x0F70);
}

// Register sets of pages per wave: two rotate in the one-block decode kernel
// (two waves per SIMD), one in the three-block verify kernel.
constexpr uint32_t kDecodeDepth = 2;
constexpr uint32_t kVerify48Depth = 1;

// Writes what a wave has accumulated for its NB blocks: the finished bf16 rows
// when the lane has a single split, else fp32 partial rows and (max, sum).
template <uint32_t NB, bool ROWS_DOWN>
__device__ __forceinline__ void write_blocks(const State *st, const uint32_t *m, const bool *in_tile,
                                             const bool *live_row, const DecodeLane &l,
                                             const LaunchArgs &a, uint32_t head, uint32_t split,
                                             uint32_t written, uint32_t g,
                                             uint16_t *__restrict__ output,
                                             float *__restrict__ partials,
                                             float *__restrict__ statistics) {
  const uint32_t G = a.group, M = a.fused_rows;
  uint16_t *out_head = output + l.q_offset + uint64_t(head) * a.row_stride * G * kD;
  const uint64_t first_row = l.row_base + uint64_t(head) * l.split_count * M + uint64_t(split) * M;
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    // Lanes of one column hold disjoint tokens: combine their sums and the
    // constant part, then take the constant part out of the accumulators.
    float row_sum = st[nb].row_sum, bias = st[nb].bias;
    row_sum = column_sum(row_sum);
    bias = column_sum(bias);
    if (written != 1 && live_row[nb] && g == 0) {
      statistics[(first_row + m[nb]) * 2] = st[nb].row_max;
      statistics[(first_row + m[nb]) * 2 + 1] = row_sum;
    }
    if constexpr (ROWS_DOWN) {
      // Register rr of this lane holds fused row 4g + rr of the block, dims 16 t + 0 .. 15
      // over the sixteen accumulators; the row's sum and constant part sit in lane 4g + rr.
      const uint32_t t = threadIdx.x & 15;
#pragma unroll
      for (uint32_t rr = 0; rr < 4; ++rr) {
        const uint32_t fused = m[nb] - t + 4 * g + rr;
        const bool row_in_tile = fused < M, row_live = row_in_tile && fused / G < l.active_rows;
        const float sum_of_row = __shfl(row_sum, int(4 * g + rr));
        const float bias_of_row = __shfl(bias, int(4 * g + rr));
        if (written == 1) {
          // One split: the merge's weights are exp(0) = 1, so the row is acc / sum.
          // Rows of the tile past the live ones read as zeros.
          if (row_in_tile) {
            const float denominator = row_live ? sum_of_row : 0.0f;
#pragma unroll
            for (uint32_t m8 = 0; m8 < 2; ++m8) {
              u32x4 packed;
#pragma unroll
              for (uint32_t i = 0; i < 4; ++i) {
                const float lo = st[nb].acc[8 * m8 + 2 * i][rr] - bias_of_row;
                const float hi = st[nb].acc[8 * m8 + 2 * i + 1][rr] - bias_of_row;
                const float qlo = denominator > 0.0f ? __fdiv_rn(lo, denominator) : 0.0f;
                const float qhi = denominator > 0.0f ? __fdiv_rn(hi, denominator) : 0.0f;
                packed[i] = uint32_t(f32_to_bf16(qlo)) | (uint32_t(f32_to_bf16(qhi)) << 16);
              }
              *reinterpret_cast<u32x4 *>(out_head + uint64_t(fused) * kD + 16 * t + 8 * m8) = packed;
            }
          }
        } else if (row_live) {
          float *out = partials + (first_row + fused) * kD + 16 * t;
#pragma unroll
          for (uint32_t m4 = 0; m4 < 4; ++m4) {
            f32x4 v;
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) v[i] = st[nb].acc[4 * m4 + i][rr] - bias_of_row;
            *reinterpret_cast<f32x4 *>(out + 4 * m4) = v;
          }
        }
      }
      continue;
    }
    if (written == 1) {
      // One split: the merge's weights are exp(0) = 1, so the row is acc / sum.
      // Rows of the tile past the live ones read as zeros (row_sum is 0 there).
      if (in_tile[nb]) {
        const float denominator = live_row[nb] ? row_sum : 0.0f;
#pragma unroll
        for (uint32_t rr = 0; rr < 4; ++rr)
#pragma unroll
          for (uint32_t m4 = 0; m4 < 4; ++m4) {
            u32x2 packed;
#pragma unroll
            for (uint32_t i = 0; i < 2; ++i) {
              const float lo = st[nb].acc[4 * m4 + 2 * i][rr] - bias;
              const float hi = st[nb].acc[4 * m4 + 2 * i + 1][rr] - bias;
              const float qlo = denominator > 0.0f ? __fdiv_rn(lo, denominator) : 0.0f;
              const float qhi = denominator > 0.0f ? __fdiv_rn(hi, denominator) : 0.0f;
              packed[i] = uint32_t(f32_to_bf16(qlo)) | (uint32_t(f32_to_bf16(qhi)) << 16);
            }
            *reinterpret_cast<u32x2 *>(out_head + uint64_t(m[nb]) * kD + 16 * (4 * g + rr) +
                                       4 * m4) = packed;
          }
      }
      continue;
    }
    if (live_row[nb]) {
      float *out = partials + (first_row + m[nb]) * kD;
#pragma unroll
      for (uint32_t rr = 0; rr < 4; ++rr)
#pragma unroll
        for (uint32_t m4 = 0; m4 < 4; ++m4) {
          f32x4 v;
#pragma unroll
          for (uint32_t i = 0; i < 4; ++i) v[i] = st[nb].acc[4 * m4 + i][rr] - bias;
          *reinterpret_cast<f32x4 *>(out + 16 * (4 * g + rr) + 4 * m4) = v;
        }
    }
  }
}

// The split kernel's body for NB blocks of 16 fused query rows per wave, with
// kDepth register sets of pages.
// kItemMajor: the launch has its work items in the grid's y and the KV heads in x
// (DecodeArgs::item_major), and its lanes are plain lane records, never the regular tiles of a
// prefill.
// kQuad: workgroups of four waves, each wave a work item of its own (items 4 x .. 4 x + 3); the
// waves share nothing.  A kernel built for two waves per SIMD but launched with at most one
// wave per SIMD is not always given one SIMD per wave: after another kernel the dispatcher has
// put two single-wave workgroups on one SIMD of a CU and none on its neighbour (38 of 960
// SIMDs, the launch 157 instead of 121 us).  The four waves of one workgroup go to the four
// SIMDs of its CU.
template <uint32_t NB, uint32_t kDepth, bool kReused = false, bool kItemMajor = false, bool kQuad = false>
__device__ __forceinline__ void attend_int4(const uint16_t *__restrict__ queries,
                                            uint16_t *__restrict__ output,
                                            float *__restrict__ partials,
                                            float *__restrict__ statistics, const DecodeArgs &args) {
  // The forms that have a SIMD to themselves: three blocks, or two with two page sets.
  constexpr bool kPinned = NB == 3 || (NB == 2 && kDepth >= 2);
  // Two blocks with one page set run two waves per SIMD with every accumulator in the first
  // register file: they hold their tiles transposed, which needs the rescaling for a quarter
  // of a tile's registers on a fifth of the pages instead of all of them on half.
  constexpr bool kRowsDown = NB == 2 && kDepth == 1;
  const uint32_t wave = kQuad ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0u;
  // item-major workgroups of four waves: (item, head) pairs in dispatch order, heads fastest
  const uint32_t flat = 4 * blockIdx.x + wave;
  uint32_t item = kItemMajor ? (kQuad ? 0u : blockIdx.y) : kQuad ? flat : blockIdx.x;
  uint32_t head = kItemMajor ? (kQuad ? 0u : blockIdx.x) : blockIdx.y;
  uint32_t li;
  DecodeLane l;
  LaunchArgs a;
  if constexpr (kItemMajor) {
    // Every wave of the launch pays the way from its first instruction to its first page
    // load at the same time, so that way is kept to three trips to memory: the launch-wide
    // arguments with the first items of all lanes, the wave's lane record, its first page
    // entries.  Left to itself the compiler fetches each field where it is first used, behind
    // the branch before it, and fetches it again rather than keep it: ten trips one after the
    // other, 5.6 us of a 100 us launch.  The empty statements below take in everything one
    // trip brings and hand it out again as values the compiler cannot fetch anew, so the
    // loads of a trip go out together and are waited for once.
    uint32_t base[kLanes];
#pragma unroll
    for (uint32_t i = 0; i < kLanes; ++i) base[i] = args.item_base[i];
    uint32_t kv_heads = args.kv_heads, group = args.group, fused_rows = args.fused_rows,
             row_stride = args.row_stride, extent_pages = args.kv.extent_pages,
             kv_offset = args.kv.offset, all_partials = args.all_partials,
             chunk_stride = args.chunk_stride;
    uint64_t chunk_keys = reinterpret_cast<uint64_t>(args.chunk_keys),
             chunk_values = reinterpret_cast<uint64_t>(args.chunk_values),
             chunk_lane_stride = args.chunk_lane_stride;
    asm volatile("" : "+s"(base[0]), "+s"(base[1]), "+s"(base[2]), "+s"(base[3]), "+s"(base[4]),
                      "+s"(base[5]), "+s"(base[6]), "+s"(base[7]), "+s"(base[8]), "+s"(base[9]),
                      "+s"(base[10]), "+s"(base[11]), "+s"(base[12]), "+s"(base[13]),
                      "+s"(base[14]), "+s"(base[15]));
    asm volatile("" : "+s"(base[16]), "+s"(base[17]), "+s"(base[18]), "+s"(base[19]),
                      "+s"(base[20]), "+s"(base[21]), "+s"(base[22]), "+s"(base[23]),
                      "+s"(base[24]), "+s"(base[25]), "+s"(base[26]), "+s"(base[27]),
                      "+s"(base[28]), "+s"(base[29]), "+s"(base[30]), "+s"(base[31]));
    asm volatile("" : "+s"(kv_heads), "+s"(group), "+s"(fused_rows), "+s"(row_stride),
                      "+s"(extent_pages), "+s"(kv_offset), "+s"(all_partials), "+s"(chunk_stride),
                      "+s"(chunk_keys), "+s"(chunk_values), "+s"(chunk_lane_stride));
    a = {kv_heads, group, fused_rows, row_stride, {extent_pages, kv_offset},
         reinterpret_cast<const uint16_t *>(chunk_keys),
         reinterpret_cast<const uint16_t *>(chunk_values), chunk_lane_stride, chunk_stride,
         all_partials};
    if constexpr (kQuad) {
      item = flat / kv_heads;
      head = flat - item * kv_heads;
    }
    // base is non-decreasing: the lane is the number of later lanes that start at or
    // before the item.
    uint32_t index = 0;
#pragma unroll
    for (uint32_t i = 1; i < kLanes; ++i) index += item >= base[i] ? 1u : 0u;
    const DecodeLane &from = args.lane[index];
    uint64_t table = reinterpret_cast<uint64_t>(from.table),
             masks = reinterpret_cast<uint64_t>(from.masks), row_base = from.row_base,
             q_offset = from.q_offset;
    uint32_t committed = from.committed, active_rows = from.active_rows,
             split_count = from.split_count, first_item = from.first_item, source = from.source;
    float lane_scale = from.score_scale;
    asm volatile("" : "+s"(table), "+s"(masks), "+s"(row_base), "+s"(q_offset), "+s"(committed),
                      "+s"(active_rows), "+s"(split_count), "+s"(first_item), "+s"(source),
                      "+s"(lane_scale));
    l.table = reinterpret_cast<const uint64_t *>(table);
    l.masks = reinterpret_cast<const uint32_t *>(masks);
    l.committed = committed;
    l.active_rows = active_rows;
    l.split_count = split_count;
    l.first_item = first_item;
    l.score_scale = lane_scale;
    l.source = source;
    l.row_base = row_base;
    l.q_offset = q_offset;
  } else {
    l = lane_of_item(args, item, li);
    a = launch_args_of(args);
  }
  li = l.source;  // the step's token rows lie in the caller's order of lanes
  const uint32_t split = item - l.first_item;
  if (split >= l.split_count) return;
  const uint32_t visible = l.committed + l.active_rows;
  const uint32_t pages = (visible + kPage - 1) / kPage;
  const uint32_t per = (pages + l.split_count - 1) / l.split_count;
  const uint32_t written = (pages + per - 1) / per;  // splits that own a page
  const uint32_t begin = split * per;
  if (begin >= pages) return;
  const uint32_t end = min(pages, begin + per);

  const uint32_t lane = kQuad ? threadIdx.x & 63u : threadIdx.x, t = lane & 15, g = lane >> 4;
  const uint32_t H = a.kv_heads, G = a.group, M = a.fused_rows;
  // The wave that owns the sequence's last page stores the step's token: before
  // anything else when that page is among the first fills, otherwise behind them,
  // where its latency hides under the loads already in flight.
  const bool appends = a.chunk_keys != nullptr && end == pages;
  const bool appends_first = appends && end - begin <= kDepth;
  if (appends_first) append_decode_token(a, l, li, head, lane);
  // This wave's MFMA columns are fused rows 16 NB z .. of the tile, 16 per block;
  // a fused row is (query row, head in group) = (m / G, m % G).
  uint32_t m[NB];
  bool in_tile[NB], live_row[NB];
  Sight sight[NB];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    m[nb] = 16 * (NB * blockIdx.z + nb) + t;
    const uint32_t query_row = m[nb] / G;
    in_tile[nb] = m[nb] < M;
    live_row[nb] = in_tile[nb] && query_row < l.active_rows;
    sight[nb].committed = l.committed;
    sight[nb].visible = visible;
    sight[nb].limit =
        live_row[nb] ? min(visible, l.committed + min(query_row, l.active_rows - 1) + 1) : visible;
    sight[nb].tree = live_row[nb] && l.masks != nullptr;
    sight[nb].mask = sight[nb].tree ? l.masks[query_row] : 0u;
  }
  const uint32_t db = kPage * H * kRowBytes, sb = kPage * H * 4;
  const RegionOffsets ro = region_offsets(a.kv.extent_pages, db, sb);
  const float score_scale = default_score_scale(kD, l.score_scale);

  // The split's first page entries, one per lane (lane i: slot i mod 2 kDepth, clamped), as
  // one vector load ahead of everything else.  Every wave of a launch wants its first entries
  // at the same moment, from cache lines nobody has touched yet: through the scalar cache,
  // which a few CUs share and which takes few misses at a time, that trip took 3 to 4 us of
  // the 5 a wave needs to issue its first page load; the vector path takes them all at once.
  const uint64_t *const entries = l.table + begin;
  const uint32_t last_slot = end - begin - 1;
  const u32x2 first_entries = load_global<u32x2>(entries + min(lane & (2 * kDepth - 1), last_slot));
  const auto first_entry = [&](uint32_t slot) {
    // the builtin returns a signed int: through uint32_t, or the low half's top bit
    // would spread over the high half
    const uint32_t lo = uint32_t(__builtin_amdgcn_readlane(int(first_entries[0]), int(slot)));
    const uint32_t hi = uint32_t(__builtin_amdgcn_readlane(int(first_entries[1]), int(slot)));
    return uint64_t(lo) | uint64_t(hi) << 32;
  };

  // Queries of this KV head: [row][g][D] bf16, fused row m.  Their loads go out
  // ahead of the page loads; everything behind them returns later, so the wait for the
  // queries leaves the page loads in flight.  Columns without a live row carry zeros.
  const uint16_t *q_head = queries + l.q_offset + uint64_t(head) * a.row_stride * G * kD;
  u32x4 q_raw[NB][8];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    const uint16_t *q_row = q_head + uint64_t(live_row[nb] ? m[nb] : 0) * kD;
#pragma unroll
    for (uint32_t kb = 0; kb < 8; ++kb)
      q_raw[nb][kb] = load_global<u32x4>(q_row + 8 * (16 * (kb >> 2) + 4 * g + (kb & 3)));
  }

  // The later page entries come through the scalar unit, each set's next entry
  // fetched a whole page period before the refill that uses it.
  // kDepth register sets rotate: a set is refilled with the page kDepth ahead as
  // soon as its page has been consumed, so up to kDepth pages are in flight.
  PageRegs r[kDepth];
  uint64_t upcoming[kDepth];  // upcoming[d]: the entry of set d's next refill
  const LaneOffsets at = lane_offsets(t, g, uint32_t(ro.value_scales - ro.key_scales));
  // The empty asm statements pin the loads of one fill together and in place:
  // moved up into the arithmetic that still reads the set they would need a
  // second copy of its registers, and interleaved with another fill's loads
  // they would make every wait cover both.
  auto fill = [&](PageRegs &set, uint64_t entry) {
    asm volatile("");
    load_page<7, kReused>(set, entry, head, H, a.kv.offset, ro.key_scales, ro.values, at);
    asm volatile("");
  };
  // The same in two steps for the steady loop: the keys as soon as the page that
  // held the set has multiplied its last key, the rest when the page is done.
  auto fill_keys = [&](PageRegs &set, uint64_t entry) {
    asm volatile("");
    load_page<1, kReused>(set, entry, head, H, a.kv.offset, ro.key_scales, ro.values, at);
    asm volatile("");
  };
  auto fill_rest = [&](PageRegs &set, uint64_t entry) {
    asm volatile("");
    load_page<6, kReused>(set, entry, head, H, a.kv.offset, ro.key_scales, ro.values, at);
    asm volatile("");
  };
  // The first fills are unconditional too (a split shorter than kDepth pages
  // loads its last page again): the steady loop must be entered with the same
  // loads in flight, in the same order, as its own iterations leave behind.
#pragma unroll
  for (uint32_t d = 0; d < kDepth; ++d) {
    fill(r[d], first_entry(d));
    upcoming[d] = first_entry(d + kDepth);
  }
  if (appends && !appends_first) append_decode_token(a, l, li, head, lane);

  // Register kb of the staged queries holds the 8 dims of dword
  // w = 16*(kb>>2) + 4g + (kb&3) of a key row in expansion order; odd dims are
  // negated.  q_bias is the constant part of every score.
  __shared__ u32x4 q_lds_all[kQuad ? 4 : 1][NB][8 * 64];
  u32x4 (&q_lds)[NB][8 * 64] = q_lds_all[wave];
  float q_bias[NB];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    q_bias[nb] = 0.0f;
#pragma unroll
    for (uint32_t kb = 0; kb < 8; ++kb) {
      // dims 8w .. 8w+7 as four bf16 pairs, regrouped to (p, p+4) pairs
      const u32x4 raw = q_raw[nb][kb];
      u32x4 q_reg;
      q_reg[0] = __builtin_amdgcn_perm(raw[2], raw[0], 0x05040100u);
      q_reg[1] = __builtin_amdgcn_perm(raw[2], raw[0], 0x07060302u) ^ 0x80008000u;
      q_reg[2] = __builtin_amdgcn_perm(raw[3], raw[1], 0x05040100u);
      q_reg[3] = __builtin_amdgcn_perm(raw[3], raw[1], 0x07060302u) ^ 0x80008000u;
      if (!live_row[nb]) q_reg = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
      for (uint32_t p = 0; p < 4; ++p) {
        // even dims carry +24 q, odd dims (stored negated) -23 q = +23 stored
        const float pair_sum =
            __uint_as_float(q_reg[p] << 16) + __uint_as_float(q_reg[p] & 0xffff0000u);
        q_bias[nb] = fmaf((p & 1) ? 23.0f : 24.0f, pair_sum, q_bias[nb]);
      }
      q_lds[nb][kb * 64 + lane] = q_reg;
    }
    q_bias[nb] = column_sum(q_bias[nb]);
  }

  State st[NB];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i) st[nb].acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    st[nb].row_max = -INFINITY;
    st[nb].row_sum = 0.0f;
    st[nb].bias = 0.0f;
  }
  auto staged_queries = [&](uint32_t nb, uint32_t kb) { return q_lds[nb][kb * 64 + lane]; };

  // Steady state: every refill is unconditional, so the loop body is straight
  // line code and the wait for a set counts exactly the loads issued after it;
  // a refill under a branch would make each wait cover the newest loads too.
  // The last page of the split is never consumed here, so no token test.
  // Nor is the page before it: the rows of a lane may see different parts of the
  // last two pages of a sequence (a chain of 8 rows or a pair of prefill tiles
  // that begins shortly before a page boundary), so both take the masked path.
  constexpr uint32_t kUnmaskedStop = 2 * kDepth > kDepth + 2 ? 2 * kDepth : kDepth + 2;
  uint32_t page = begin;
  for (; page + kUnmaskedStop <= end; page += kDepth) {
#pragma unroll
    for (uint32_t d = 0; d < kDepth; ++d) {
      // upcoming[d] is the entry of slot page + d + kDepth - begin, this set's refill
      attend_page<false, NB, kPinned, kRowsDown>(RegisterPage{r[d], g}, staged_queries, q_bias, score_scale,
                             (page + d) * kPage, sight, g, st, [&] { fill_keys(r[d], upcoming[d]); });
      fill_rest(r[d], upcoming[d]);
      upcoming[d] = scalar_entry(entries, min(page + d + 2 * kDepth - begin, last_slot));
    }
  }
  // Tail: at most kUnmaskedStop - 1 pages are left, the first kDepth of them loaded.
#pragma unroll
  for (uint32_t k = 0; k < kUnmaskedStop - 1; ++k) {
    const uint32_t d = k % kDepth;
    if (page + k < end) {
      attend_page<true, NB, kPinned, kRowsDown>(RegisterPage{r[d], g}, staged_queries, q_bias, score_scale,
                            (page + k) * kPage, sight, g, st, [] {});
      if (k + kDepth < kUnmaskedStop - 1 && page + k + kDepth < end) {
        fill(r[d], upcoming[d]);  // slot page + k + kDepth - begin, and d = k here
        upcoming[d] = scalar_entry(entries, min(page + k + 2 * kDepth - begin, last_slot));
      }
    }
  }

  write_blocks<NB, kRowsDown>(st, m, in_tile, live_row, l, a, head, split, a.all_partials ? 2u : written,
                              g, output, partials, statistics);
}

// One block of 16 fused rows per wave, two waves per SIMD: one-row decode, where
// the group's query heads are the only rows and memory latency is what to hide.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) void decode_int4_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  attend_int4<1, kDecodeDepth, false, true>(queries, output, partials, statistics, a);
}
// The same as workgroups of four waves, (work item, KV head) pairs in dispatch order: for
// launches with two waves on most SIMDs, whose plan counts on the lanes with the longest
// splits taking the first wave of every SIMD.  Single-wave workgroups get that placement only
// while the dispatcher starts from a clean state (16 lanes of 32 768 tokens after a merge
// kernel: 127 us, against 112 us for this form and 111 for its parts alone); a launch that
// leaves SIMDs empty is better off with single waves spread over all CUs (one sequence of
// 32 768 tokens: 15.5 against 16.6 us).
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void decode_int4_quad_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  attend_int4<1, kDecodeDepth, false, true, true>(queries, output, partials, statistics, a);
}

// The same for the 8-row tiles of a chunked prefill with several splits: every
// tile of the chunk walks the same pages, so the loads may stay in the caches.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) void decode_int4_tiles_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  attend_int4<1, kDecodeDepth, true>(queries, output, partials, statistics, a);
}

// Two blocks per wave share every expanded key and value operand (verify, tree
// verify, prefill tiles); the accumulators of both take the register file of a
// whole SIMD lane, so one wave per SIMD.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(1, 1))) void verify_int4_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  attend_int4<2, 2>(queries, output, partials, statistics, a);
}

// The same two blocks with one register set of pages, which fits two waves per
// SIMD: for the paired tiles of a chunked prefill, whose 1536 waves per 2048-row
// chunk then all run at once instead of in a full round and a half-empty one
// (2.0 -> 1.5 ms on 2048 rows over 16K tokens); its page loads may stay in the
// caches, because every tile of the chunk walks the same pages.  Verify batches, sized to one
// wave per SIMD by their plan, are faster with two sets and the SIMD to
// themselves.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) void prefill_int4_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  attend_int4<2, 1, true>(queries, output, partials, statistics, a);
}

// Two blocks with one register set of pages, for lanes of more than 32 fused rows that fill
// blocks of 32 better than blocks of 48 (a tree of 16 nodes for a group of 6: three waves of
// 32 rows).  Built for two waves per SIMD, so that every accumulator lives in the first
// register file, where its rescaling costs one instruction a register instead of three;
// per block and page it issues 235 vector instructions where the three-block kernel
// issues 268, and a wave's vector instructions are what these kernels wait for.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void verify32_int4_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  attend_int4<2, 1, false, false, true>(queries, output, partials, statistics, a);
}

// Three blocks (48 fused rows: a chain of 8 rows for a group of 6 query heads, half
// of a 16-node tree) read and expand every page once for all of them; one register set of pages,
// one wave per SIMD.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(1, 1))) void verify48_int4_kernel(
    const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
    float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  attend_int4<3, kVerify48Depth>(queries, output, partials, statistics, a);
}

// Calibration, not part of any attention path: the page loads of decode_int4_kernel
// (same instructions, same two register sets, two waves per SIMD) with nothing but an
// exclusive-or behind them.  What it streams at is what this access pattern can reach
// before any arithmetic.  Workgroup (x, y) reads entries x * per .. of the table; its waves
// take consecutive KV heads from y * (waves per workgroup) on.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void stream_int4_kernel(
    const uint64_t *__restrict__ entries, uint32_t n_entries, uint32_t per, kvx_kv_layer kv,
    uint32_t kv_heads, uint32_t *__restrict__ sink) {
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t head = blockIdx.y * (blockDim.x >> 6) + wave;
  const uint32_t lane = threadIdx.x & 63u, t = lane & 15, g = lane >> 4;
  const uint32_t begin = blockIdx.x * per;
  if (begin >= n_entries) return;
  const uint32_t count = min(per, n_entries - begin), last_slot = count - 1;
  const uint32_t db = kPage * kv_heads * kRowBytes, sb = kPage * kv_heads * 4;
  const RegionOffsets ro = region_offsets(kv.extent_pages, db, sb);
  const LaneOffsets at = lane_offsets(t, g, uint32_t(ro.value_scales - ro.key_scales));
  const uint64_t *const table = entries + begin;
  PageRegs r[2];
  uint32_t x = 0;
#pragma unroll
  for (uint32_t d = 0; d < 2; ++d)
    load_page<7, false>(r[d], scalar_entry(table, min(d, last_slot)), head, kv_heads, kv.offset,
                        ro.key_scales, ro.values, at);
  for (uint32_t slot = 0; slot < count; slot += 2) {
#pragma unroll
    for (uint32_t d = 0; d < 2; ++d) {
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) x ^= r[d].k[i][0] ^ r[d].k[i][1] ^ r[d].k[i][2] ^ r[d].k[i][3];
#pragma unroll
      for (uint32_t i = 0; i < 8; ++i) x ^= r[d].v[i][0] ^ r[d].v[i][1];
      x ^= __float_as_uint(r[d].scale);
      asm volatile("");
      load_page<7, false>(r[d], scalar_entry(table, min(slot + d + 2, last_slot)), head, kv_heads,
                          kv.offset, ro.key_scales, ro.values, at);
      asm volatile("");
    }
  }
  if (x == 0x9e3779b9u) sink[0] = x;  // keeps the loads alive
}

}  // namespace
}  // namespace kvx

using namespace kvx;

// Runs paged attention (split kernel, then the merge of multi-split lanes) for
// int4 pages of head dimension 256; returns 1 (declined) for shapes it does not
// cover so the caller runs the format-generic kernels, 0 when enqueued, or a
// negative status.  Lane i reads its queries and writes its rows at element
// offset i * lane_stride; the rows of one KV head lie row_stride * group * 256
// elements apart.  row_masks: null, or one ancestor bitmask per (lane, row of
// capacity).  Every lane has the row capacity of the first.  many_tiles: the
// lanes are the 8-row tiles of a chunked prefill.
int kvx_attend_int4_launch(const kvx_storage *s, kvx_kv_layer kv, uint32_t query_heads,
                           const void *queries, void *output, const uint64_t *const *page_tables,
                           const kvx_verify_params *lanes, uint32_t n_lanes,
                           const uint32_t *row_masks, uint32_t row_stride, uint64_t lane_stride,
                           void *workspace, uint64_t workspace_bytes, int many_tiles,
                           hipStream_t stream, const void *append_keys, const void *append_values,
                           uint64_t append_lane_stride, uint32_t append_stride, Tiles tile_rows,
                           const Epilogue *epilogue) {
  if (s->layout.format != KVX_FMT_INT4 || !matrix_attention_covers(s, query_heads, lanes, n_lanes))
    return 1;
  const FusedAppend appended{append_keys, append_values, append_lane_stride, append_stride};
  const FusedAppend *fused = append_keys ? &appended : nullptr;
  const uint32_t fused_rows = lanes[0].row_capacity * (query_heads / s->layout.kv_heads);
  // The kernel appends the step's token itself only where one wave owns a
  // (sequence, KV head, split): one-row decode.
  if (fused && (fused_rows > 16 || lanes[0].row_capacity != 1)) return 1;
  // Sharing the expanded operands between two blocks pays where the lanes are few
  // and long (verify: 13% on 4 x 65536 tokens x 16 tree rows); chunked prefill has
  // hundreds of tiles of 48 fused rows, where a half-empty second wave and one
  // wave per SIMD cost more than the sharing saves.
  if (fused_rows > 16 && !many_tiles && tile_rows)
    return launch_matrix_attention(prefill_int4_kernel, "prefill_int4_kernel", 32, 64, s, kv,
                                   query_heads, queries, output, page_tables, lanes, n_lanes,
                                   row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                   stream, nullptr, tile_rows, epilogue);
  // 48 fused rows per wave where that leaves clearly fewer waves: the pages are
  // read and expanded once per 48 rows instead of once per 32.
  if (verify_block_rows(KVX_FMT_INT4, fused_rows) == 48 && !many_tiles)
    return launch_matrix_attention(verify48_int4_kernel, "verify48_int4_kernel", 48, 64, s, kv,
                                   query_heads, queries, output, page_tables, lanes, n_lanes,
                                   row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                   stream, nullptr, tile_rows, epilogue);
  if (fused_rows > 32 && !many_tiles)
    return launch_matrix_attention(verify32_int4_kernel, "verify32_int4_kernel", 32, 256, s, kv,
                                   query_heads, queries, output, page_tables, lanes, n_lanes,
                                   row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                   stream, nullptr, tile_rows, epilogue, false, /*waves_per_group=*/4);
  if (fused_rows > 16 && !many_tiles)
    return launch_matrix_attention(verify_int4_kernel, "verify_int4_kernel", 32, 64, s, kv,
                                   query_heads, queries, output, page_tables, lanes, n_lanes,
                                   row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                   stream, nullptr, tile_rows, epilogue);
  if (tile_rows && !fused)
    return launch_matrix_attention(decode_int4_tiles_kernel, "decode_int4_tiles_kernel", 16, 64, s,
                                   kv, query_heads, queries, output, page_tables, lanes, n_lanes,
                                   row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                   stream, nullptr, tile_rows, epilogue);
  // two waves on most SIMDs (of the first launch's lanes): the form whose placement holds
  uint64_t first_waves = 0;
  for (uint32_t i = 0; i < std::min(n_lanes, kLanes); ++i)
    first_waves += uint64_t(lanes[i].split_count) * s->layout.kv_heads;
  if (first_waves > 1024)
    return launch_matrix_attention(decode_int4_quad_kernel, "decode_int4_quad_kernel", 16, 256, s, kv,
                                   query_heads, queries, output, page_tables, lanes, n_lanes,
                                   row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                   stream, fused, tile_rows, epilogue, /*longest_first=*/true,
                                   /*waves_per_group=*/4);
  return launch_matrix_attention(decode_int4_kernel, "decode_int4_kernel", 16, 64, s, kv,
                                 query_heads, queries, output, page_tables, lanes, n_lanes,
                                 row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                 stream, fused, tile_rows, epilogue, /*longest_first=*/true);
}

extern "C" int kvx_calibrate_stream(const kvx_storage *s, uint32_t layer, const uint64_t *page_table,
                                    uint32_t n_pages, uint32_t pages_per_wave,
                                    uint32_t heads_per_workgroup, uint32_t *sink, void *stream) {
  if (!s || !page_table || !sink || !n_pages || !pages_per_wave) return KVX_EINVAL;
  if (heads_per_workgroup < 1 || heads_per_workgroup > 4 || s->layout.kv_heads % heads_per_workgroup)
    return KVX_EINVAL;
  if (s->layout.format != KVX_FMT_INT4 || s->layout.head_dim != kD) return KVX_EINVAL;
  kvx_kv_layer kv;
  if (const int status = kvx_storage_layer(s, layer, &kv)) return status;
  const dim3 grid((n_pages + pages_per_wave - 1) / pages_per_wave, s->layout.kv_heads / heads_per_workgroup);
  hipLaunchKernelGGL(stream_int4_kernel, grid, dim3(64 * heads_per_workgroup), 0, static_cast<hipStream_t>(stream), page_table,
                     n_pages, pages_per_wave, kv, s->layout.kv_heads, sink);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? KVX_OK : hip_fail(e, "stream_int4_kernel");
}
