// bf16, fp8-e4m3 and int8 paged attention for gfx950: the split kernel of
// kv_attend_decode, kv_attend_verify and kv_attend_prefill for pages whose
// elements are two bytes (bf16) or one byte (fp8, int8) wide, head dimension 256.
//
// One wave per (sequence or prefill tile, split, KV head, group of NB blocks of
// 16 fused query rows).  The wave streams the split's pages once; keys and
// values are the A operands of 16x16x32 MFMAs as they lie in the page (bf16) or
// after an exact byte -> fp16 expansion (fp8, int8), and all NB row blocks reuse
// them.  The arithmetic follows the reference tiles
// (common/paged_attention_tile.h:85-349 for bf16,
// common/paged_attention_fp8_tile.h:34-265 for fp8): page-granular online
// softmax, scores = raw dot x key scale x score scale, probabilities x value
// scale rounded to bf16 (bf16 pages) or fp16 (fp8 pages, whose queries are
// staged as fp16) before they meet the values.
//
// fp8 -> fp16: gfx950 converts two e4m3 (OCP) bytes to two halves in one
// instruction (v_cvt_scalef32_pk_f16_fp8); every e4m3 value, subnormals included,
// is a normal fp16 number, so the conversion is exact (half a VALU instruction per
// byte; a shift-and-mask construction of the same halves took 2.5).
//
// int8 -> fp16 without a table: the code's byte with its top bit flipped is
// u = c + 128 in 1..255, 0x6400 | u is the fp16 number 1024 + u exactly, and a
// packed fp16 subtraction of 1152 leaves the code itself, exactly.  Queries and
// probabilities meet the codes as fp16: a bf16 query, or a probability already
// rounded to bf16 as the reference tile rounds it, converts without loss unless
// its magnitude is below 2^-14, far under the tolerance.
#include "kvx_attend_common.h"

namespace kvx {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <uint32_t FMT>
struct Wide {
  static constexpr bool kFp8 = FMT == KVX_FMT_FP8E4M3;
  static constexpr bool kInt8 = FMT == KVX_FMT_INT8;
  static constexpr bool kByte = kFp8 || kInt8;                       // one byte per element, scaled
  static constexpr uint32_t kBytes = kByte ? 1 : 2;                  // per element
  static constexpr uint32_t kSlab = kPage * kD * kBytes;             // per (head, page, tensor)
  static constexpr uint32_t kDwords = kByte ? 2 : 4;                 // raw dwords per MFMA operand
};

template <uint32_t FMT>
__device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (Wide<FMT>::kByte)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// Two e4m3 bytes (the low or the high half of x) to two fp16 halves holding their
// values: one v_cvt_scalef32_pk_f16_fp8 with scale 1.
template <bool HIGH>
__device__ __forceinline__ uint32_t fp8_pair(uint32_t x) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(x, 1.0f, HIGH));
}
// Eight consecutive bytes (two dwords) to eight fp16 in order.
__device__ __forceinline__ u32x4 fp8_operand(uint32_t first, uint32_t second) {
  return u32x4{fp8_pair<false>(first), fp8_pair<true>(first), fp8_pair<false>(second),
               fp8_pair<true>(second)};
}

// Two int8 codes (bytes of x flipped in the top bit, selected by the perm
// pattern under the constant byte 0x64) to two fp16 halves holding the codes.
__device__ __forceinline__ uint32_t int8_pair(uint32_t flipped, uint32_t select) {
  const uint32_t biased = __builtin_amdgcn_perm(0x64646464u, flipped, select);  // 1024 + u each
  const f16x2 codes = __builtin_bit_cast(f16x2, biased) - f16x2{_Float16(1152.0f), _Float16(1152.0f)};
  return __builtin_bit_cast(uint32_t, codes);
}
// Eight consecutive int8 codes (two dwords) to eight fp16 in order.
__device__ __forceinline__ u32x4 int8_operand(uint32_t first, uint32_t second) {
  const uint32_t a = first ^ 0x80808080u, b = second ^ 0x80808080u;
  return u32x4{int8_pair(a, 0x04010400u), int8_pair(a, 0x04030402u), int8_pair(b, 0x04010400u),
               int8_pair(b, 0x04030402u)};
}

// What one lane holds of one page's keys / values.  Which token sits in which
// MFMA row and which dims in which k-slots is free as long as both operands
// agree; both are chosen so that every load instruction reads long contiguous
// runs (a load that touches sixteen lines for 16 or 32 bytes each is bound by
// the number of requests, not by bytes).
//  q.k : A = keys, row t of token block tb = token 8*(t/4) + 4*tb + t%4; the
//        k-slots of step kb are 8 dims at key_dims(kb, g).  B = queries, column
//        t = fused query row, same dims.  Output column t, rows 4g..4g+3 =
//        tokens 8g + 4*tb + r: a lane holds the scores of tokens 8g..8g+7.
//  p.v : A = values (stored dimension-major), row t = dim 16*mb + t, k-slots =
//        tokens 8g..8g+7, contiguous in the page: exactly the tokens whose scores
//        the lane holds, so the probabilities are the B operand as they are.
// First dim of the 8 dims lane group g multiplies in step kb: two-byte elements
// take 16 bytes per step, one-byte elements take two steps out of one 16-byte load.
template <uint32_t FMT>
__device__ __forceinline__ uint32_t key_dims(uint32_t kb, uint32_t g) {
  if constexpr (Wide<FMT>::kByte) return 64 * (kb >> 1) + 16 * g + 8 * (kb & 1);
  else return 32 * kb + 8 * g;
}
template <uint32_t FMT>
struct KeyRegs {
  uint32_t raw[2][8][Wide<FMT>::kDwords];  // [token block][dim block]
};
template <uint32_t FMT>
struct ValueRegs {
  uint32_t raw[16][Wide<FMT>::kDwords];  // [dim block]: tokens 8g .. 8g+7
};

struct PagePlace {
  const uint8_t *keys, *values;
  const float *key_scales, *value_scales;
};
template <uint32_t FMT>
__device__ __forceinline__ PagePlace place_page(uint64_t entry, uint32_t head, uint32_t kv_heads,
                                                uint32_t layer_offset, const RegionOffsets &ro) {
  const uint32_t index = uint32_t(entry) & KVX_PAGE_INDEX_MASK;
  const uint8_t *region = reinterpret_cast<const uint8_t *>(entry - index) + layer_offset;
  const uint64_t slab = (uint64_t(index) * kv_heads + head) * Wide<FMT>::kSlab;
  const uint64_t scale_index = (uint64_t(index) * kv_heads + head) * kPage;
  PagePlace p;
  p.keys = region + slab;
  p.values = region + ro.values + slab;
  p.key_scales = reinterpret_cast<const float *>(region + ro.key_scales) + scale_index;
  p.value_scales = reinterpret_cast<const float *>(region + ro.value_scales) + scale_index;
  return p;
}

template <uint32_t FMT, bool REUSED>
__device__ __forceinline__ void load_keys(KeyRegs<FMT> &k, const PagePlace &p, uint32_t t,
                                          uint32_t g) {
  constexpr uint32_t B = Wide<FMT>::kBytes;
#pragma unroll
  for (uint32_t tb = 0; tb < 2; ++tb) {
    const uint8_t *row = p.keys + (8 * (t >> 2) + 4 * tb + (t & 3)) * kD * B;
    if constexpr (Wide<FMT>::kByte) {
#pragma unroll
      for (uint32_t j = 0; j < 4; ++j) {  // 16 tokens x 64 contiguous bytes per instruction
        const u32x4 v = load_streaming<u32x4, REUSED>(row + 64 * j + 16 * g);
        k.raw[tb][2 * j][0] = v[0];
        k.raw[tb][2 * j][1] = v[1];
        k.raw[tb][2 * j + 1][0] = v[2];
        k.raw[tb][2 * j + 1][1] = v[3];
      }
    } else {
#pragma unroll
      for (uint32_t kb = 0; kb < 8; ++kb) {
        const u32x4 v = load_streaming<u32x4, REUSED>(row + key_dims<FMT>(kb, g) * B);
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) k.raw[tb][kb][i] = v[i];
      }
    }
  }
}
template <uint32_t FMT, bool REUSED>
__device__ __forceinline__ void load_values(ValueRegs<FMT> &v, const PagePlace &p, uint32_t t,
                                            uint32_t g) {
  constexpr uint32_t B = Wide<FMT>::kBytes;
#pragma unroll
  for (uint32_t mb = 0; mb < 16; ++mb) {  // 16 dims x 32 tokens, contiguous, per instruction
    const uint8_t *at = p.values + ((16 * mb + t) * kPage + 8 * g) * B;
    if constexpr (Wide<FMT>::kByte) {
      const u32x2 x = load_streaming<u32x2, REUSED>(at);
      v.raw[mb][0] = x[0];
      v.raw[mb][1] = x[1];
    } else {
      const u32x4 x = load_streaming<u32x4, REUSED>(at);
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) v.raw[mb][i] = x[i];
    }
  }
}
template <uint32_t FMT>
__device__ __forceinline__ u32x4 key_operand(const KeyRegs<FMT> &k, uint32_t tb, uint32_t kb) {
  if constexpr (Wide<FMT>::kFp8) return fp8_operand(k.raw[tb][kb][0], k.raw[tb][kb][1]);
  else if constexpr (Wide<FMT>::kInt8) return int8_operand(k.raw[tb][kb][0], k.raw[tb][kb][1]);
  else return u32x4{k.raw[tb][kb][0], k.raw[tb][kb][1], k.raw[tb][kb][2], k.raw[tb][kb][3]};
}
template <uint32_t FMT>
__device__ __forceinline__ u32x4 value_operand(const ValueRegs<FMT> &v, uint32_t mb) {
  if constexpr (Wide<FMT>::kFp8) return fp8_operand(v.raw[mb][0], v.raw[mb][1]);
  else if constexpr (Wide<FMT>::kInt8) return int8_operand(v.raw[mb][0], v.raw[mb][1]);
  else return u32x4{v.raw[mb][0], v.raw[mb][1], v.raw[mb][2], v.raw[mb][3]};
}

// WAVES: waves per SIMD the kernel is compiled for (1 or 2).
template <uint32_t FMT, uint32_t NB, uint32_t WAVES, bool REUSED>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) void attend_wide_kernel(const uint16_t *__restrict__ queries,
                                                         uint16_t *__restrict__ output,
                                                         float *__restrict__ partials,
                                                         float *__restrict__ statistics,
                                                         DecodeArgs a) {
  constexpr bool kFp8 = Wide<FMT>::kFp8, kInt8 = Wide<FMT>::kInt8, kByte = Wide<FMT>::kByte;
  const uint32_t item = blockIdx.x, head = blockIdx.y;
  uint32_t li;
  const DecodeLane l = lane_of_item(a, item, li);
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
  const uint32_t db = Wide<FMT>::kSlab * H, sb = kByte ? kPage * H * 4 : 0;
  const RegionOffsets ro = region_offsets(a.kv.extent_pages, db, sb);
  const float score_scale = default_score_scale(kD, l.score_scale);

  // Column t of block nb is fused row m = (query row, head in group).
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

  // Queries: [row][g][D] bf16, fused row m; register kb of a column holds the 8
  // dims from key_dims(kb, g).  fp8 and int8 pages stage them as fp16.  Columns without a
  // live row carry zeros.
  const uint16_t *q_head = queries + l.q_offset + uint64_t(head) * a.row_stride * G * kD;
  __shared__ u32x4 q_lds[NB][8][64];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    const uint16_t *q_row = q_head + uint64_t(live_row[nb] ? m[nb] : 0) * kD;
#pragma unroll
    for (uint32_t kb = 0; kb < 8; ++kb) {
      u32x4 q = load_global<u32x4>(q_row + key_dims<FMT>(kb, g));
      if constexpr (kByte) {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
          const f16x2 pair = {_Float16(__uint_as_float(q[i] << 16)),
                              _Float16(__uint_as_float(q[i] & 0xffff0000u))};
          q[i] = __builtin_bit_cast(uint32_t, pair);
        }
      }
      if (!live_row[nb]) q = u32x4{0u, 0u, 0u, 0u};
      q_lds[nb][kb][lane] = q;
    }
  }
  __syncthreads();  // the staged queries
  // The split's page entries come through the scalar unit, each set's next entry
  // fetched a whole page period before the refill that uses it.
  const uint64_t *const entries = l.table + begin;
  const uint32_t last_slot = end - begin - 1;

  // kSets register sets rotate: a set's keys are refilled with the page kSets
  // ahead as soon as the page has multiplied its last key, its values when the
  // page is done, so more than one page is always in flight.
  // Two sets when the wave has a SIMD's registers to itself and the elements are
  // one byte wide.  With two waves per SIMD each has one set, which overlaps one
  // wave's expansion arithmetic with the other's loads better than one wave with
  // two sets (int8 decode 262 -> 246 us).  A page of two-byte elements is 128 registers per lane:
  // with two of them the compiler spills (and a spill reload waits behind every
  // page load in flight), and one set already streams bf16 decode at 5.5 TB/s
  // (two sets with spills: 4.7).
  constexpr uint32_t kSets = (kByte && WAVES == 1) ? 2 : 1;
  struct PageSet {
    KeyRegs<FMT> keys;
    ValueRegs<FMT> values;
    f32x4 ks[2], vs[2];  // fp8, int8: scales of the lane's score tokens, per token block
  };
  PageSet set[kSets];
  // The empty asm statements keep the loads of one fetch together and in place.
  auto fetch_keys = [&](PageSet &r, uint64_t entry) {
    const PagePlace p = place_page<FMT>(entry, head, H, a.kv.offset, ro);
    asm volatile("");
    load_keys<FMT, REUSED>(r.keys, p, t, g);
    if constexpr (kByte) {
      r.ks[0] = load_global<f32x4>(p.key_scales + 8 * g);
      r.ks[1] = load_global<f32x4>(p.key_scales + 8 * g + 4);
    }
    asm volatile("");
  };
  auto fetch_values = [&](PageSet &r, uint64_t entry) {
    const PagePlace p = place_page<FMT>(entry, head, H, a.kv.offset, ro);
    asm volatile("");
    load_values<FMT, REUSED>(r.values, p, t, g);
    if constexpr (kByte) {
      r.vs[0] = load_global<f32x4>(p.value_scales + 8 * g);
      r.vs[1] = load_global<f32x4>(p.value_scales + 8 * g + 4);
    }
    asm volatile("");
  };
  // The first fills are unconditional (a split shorter than kSets pages loads its
  // last page again), so the steady loop is entered with the loads in flight that
  // its own iterations leave behind.
  uint64_t upcoming[kSets];  // upcoming[d]: the entry of set d's next refill
#pragma unroll
  for (uint32_t d = 0; d < kSets; ++d) upcoming[d] = scalar_entry(entries, min(d, last_slot));
#pragma unroll
  for (uint32_t d = 0; d < kSets; ++d) {
    fetch_keys(set[d], upcoming[d]);
    fetch_values(set[d], upcoming[d]);
    upcoming[d] = scalar_entry(entries, min(d + kSets, last_slot));
  }

  f32x4 acc[NB][16];  // [block][dim block]: dims 16*mb + 4g + r of column t
  float row_max[NB], row_sum[NB];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
#pragma unroll
    for (uint32_t mb = 0; mb < 16; ++mb) acc[nb][mb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    row_max[nb] = -INFINITY;
    row_sum[nb] = 0.0f;
  }
  constexpr float kUnscale = 1.0f;  // every format's MFMA operands hold the values themselves

  // One page out of set r; keys_consumed() runs when its keys have been read for
  // the last time.
  // Pages that lie wholly inside the committed tokens are seen whole by every row; only
  // from this page on does a token have to be tested (one copy of the page code serves
  // both, the test itself is skipped).  The one-block forms wait for memory, not for this
  // arithmetic, and two of them spill with the branch: they test every token.
  const uint32_t first_masked = l.committed / kPage;
  auto attend_page = [&](PageSet &r, uint32_t page, auto keys_consumed) {
      const bool check_tokens = page >= first_masked;
      // ---- q.k ----
      f32x4 s[NB][2];
#pragma unroll
      for (uint32_t nb = 0; nb < NB; ++nb) s[nb][0] = s[nb][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (uint32_t kb = 0; kb < 8; ++kb)
#pragma unroll
        for (uint32_t tb = 0; tb < 2; ++tb) {
          const u32x4 k = key_operand<FMT>(r.keys, tb, kb);
#pragma unroll
          for (uint32_t nb = 0; nb < NB; ++nb) s[nb][tb] = mfma<FMT>(k, q_lds[nb][kb][lane], s[nb][tb]);
        }
      f32x4 page_ks[2];
      if constexpr (kByte) {
        page_ks[0] = r.ks[0];
        page_ks[1] = r.ks[1];
      }
      keys_consumed();
      // ---- page softmax, per column block ----
      const uint32_t first_token = page * kPage;
      u32x4 pb[NB];
      f32x4 page_vs[2];
      if constexpr (kByte) {
        page_vs[0] = r.vs[0];
        page_vs[1] = r.vs[1];
      }
#pragma unroll
      for (uint32_t nb = 0; nb < NB; ++nb) {
        float score[8], local_max = -INFINITY;
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) {
          const uint32_t tb = i >> 2, rr = i & 3;
          float v = s[nb][tb][rr] * kUnscale;
          if constexpr (kByte) v *= page_ks[tb][rr];
          score[i] = v * score_scale;
        }
        // A token the row does not see scores -inf, and its weight below comes out as
        // exp(-inf) = 0 by itself.  (The one-block forms, which run two waves per SIMD on the
        // byte formats, spill with this form of it and select per token instead.)
        bool live[8];
        if constexpr (NB == 1) {
#pragma unroll
          for (uint32_t i = 0; i < 8; ++i) {
            live[i] = sight[nb].sees(first_token + 8 * g + 4 * (i >> 2) + (i & 3));
            score[i] = live[i] ? score[i] : -INFINITY;
          }
        } else if (check_tokens) {
#pragma unroll
          for (uint32_t i = 0; i < 8; ++i)
            if (!sight[nb].sees(first_token + 8 * g + 4 * (i >> 2) + (i & 3))) score[i] = -INFINITY;
        }
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) local_max = fmaxf(local_max, score[i]);
        local_max = fmaxf(local_max, __shfl_xor(local_max, 16));
        local_max = fmaxf(local_max, __shfl_xor(local_max, 32));
        const float next_max = fmaxf(row_max[nb], local_max);
        // A row that has seen nothing yet keeps -inf; its rescale is 1, not exp(nan).
        const float rescale = next_max == row_max[nb]
                                  ? 1.0f
                                  : __builtin_amdgcn_exp2f((row_max[nb] - next_max) * kLog2e);
        // A row that still has seen nothing measures from 0: -inf - -inf is no number.
        const float reference = (NB == 1 || next_max != -INFINITY) ? next_max : 0.0f;
        float weight[8], page_sum = 0.0f;
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) {
          // The difference first, so the page's maximum gets exactly 1.
          float p = __builtin_amdgcn_exp2f((score[i] - reference) * kLog2e);
          if constexpr (NB == 1) p = live[i] ? p : 0.0f;
          page_sum += p;
          weight[i] = kByte ? p * page_vs[i >> 2][i & 3] : p;
        }
        row_sum[nb] = fmaf(row_sum[nb], rescale, page_sum);
        row_max[nb] = next_max;
#pragma unroll
        for (uint32_t p = 0; p < 4; ++p) {
          if constexpr (kFp8) {
            const f16x2 pair = {_Float16(weight[2 * p]), _Float16(weight[2 * p + 1])};
            pb[nb][p] = __builtin_bit_cast(uint32_t, pair);
          } else if constexpr (kInt8) {
            // Rounded to bf16 as the reference tile does, then carried as fp16.
            const f32x2 wide = {weight[2 * p], weight[2 * p + 1]};
            const uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_convertvector(wide, bf16x2));
            const f16x2 pair = {_Float16(__uint_as_float(bits << 16)),
                                _Float16(__uint_as_float(bits & 0xffff0000u))};
            pb[nb][p] = __builtin_bit_cast(uint32_t, pair);
          } else {
            const f32x2 pair = {weight[2 * p], weight[2 * p + 1]};
            pb[nb][p] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
          }
        }
        if (__builtin_amdgcn_ballot_w64(rescale != 1.0f)) {
#pragma unroll
          for (uint32_t mb = 0; mb < 16; ++mb) {
            // Two blocks of accumulators (one wave per SIMD) live in the second register
            // file.  Named there on the way in, the moves out of it that a multiply needs
            // stay inside this branch; left to itself the compiler moves every accumulator
            // out on every page.
            if constexpr (NB == 2) asm volatile("" : "+a"(acc[nb][mb]));
            acc[nb][mb] *= rescale;
          }
        }
      }
      // ---- p.v ----
#pragma unroll
      for (uint32_t mb = 0; mb < 16; ++mb) {
        const u32x4 v = value_operand<FMT>(r.values, mb);
#pragma unroll
        for (uint32_t nb = 0; nb < NB; ++nb) acc[nb][mb] = mfma<FMT>(v, pb[nb], acc[nb][mb]);
      }
  };

  // Steady state: every refill is unconditional, so the loop body is straight-line
  // code and each wait counts exactly the loads issued after the ones it needs.
  uint32_t page = begin;
  for (; page + 2 * kSets <= end; page += kSets) {
#pragma unroll
    for (uint32_t d = 0; d < kSets; ++d) {
      // upcoming[d] is the entry of slot page + d + kSets - begin, this set's refill
      attend_page(set[d], page + d, [&] { fetch_keys(set[d], upcoming[d]); });
      fetch_values(set[d], upcoming[d]);
      upcoming[d] = scalar_entry(entries, min(page + d + 2 * kSets - begin, last_slot));
    }
  }
  // Tail: at most 2 kSets - 1 pages are left, the first kSets of them loaded.
#pragma unroll
  for (uint32_t k = 0; k < 2 * kSets - 1; ++k) {
    const uint32_t d = k % kSets;
    if (page + k < end) {
      attend_page(set[d], page + k, [] {});
      if (k + kSets < 2 * kSets - 1 && page + k + kSets < end) {
        fetch_keys(set[d], upcoming[d]);  // slot page + k + kSets - begin, and d = k here
        fetch_values(set[d], upcoming[d]);
        upcoming[d] = scalar_entry(entries, min(page + k + 2 * kSets - begin, last_slot));
      }
    }
  }

#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    // Lanes of one column hold disjoint tokens: combine their sums.
    float sum = row_sum[nb];
    sum += __shfl_xor(sum, 16);
    sum += __shfl_xor(sum, 32);
    uint16_t *out_head = output + l.q_offset + uint64_t(head) * a.row_stride * G * kD;
    if (written == 1 && !a.all_partials) {
      // One split: the merge's weights are exp(0) = 1, so the row is acc / sum.
      // Rows of the tile past the live ones read as zeros.
      if (in_tile[nb]) {
        const float denominator = live_row[nb] ? sum : 0.0f;
#pragma unroll
        for (uint32_t mb = 0; mb < 16; ++mb) {
          u32x2 packed;
#pragma unroll
          for (uint32_t i = 0; i < 2; ++i) {
            const float lo = acc[nb][mb][2 * i] * kUnscale, hi = acc[nb][mb][2 * i + 1] * kUnscale;
            const float qlo = denominator > 0.0f ? __fdiv_rn(lo, denominator) : 0.0f;
            const float qhi = denominator > 0.0f ? __fdiv_rn(hi, denominator) : 0.0f;
            packed[i] = uint32_t(f32_to_bf16(qlo)) | (uint32_t(f32_to_bf16(qhi)) << 16);
          }
          *reinterpret_cast<u32x2 *>(out_head + uint64_t(m[nb]) * kD + 16 * mb + 4 * g) = packed;
        }
      }
      continue;
    }
    if (live_row[nb]) {
      const uint64_t row =
          l.row_base + uint64_t(head) * l.split_count * M + uint64_t(split) * M + m[nb];
      float *out = partials + row * kD;
#pragma unroll
      for (uint32_t mb = 0; mb < 16; ++mb)
        *reinterpret_cast<f32x4 *>(out + 16 * mb + 4 * g) = acc[nb][mb] * kUnscale;
      if (g == 0) {
        statistics[row * 2] = row_max[nb];
        statistics[row * 2 + 1] = sum;
      }
    }
  }
}


// ---- pages shared by the waves of a workgroup: the tiles of a chunked prefill, verify ----
//
// A chunk's tiles walk the same pages, and with one wave per 32 fused rows every wave
// fetches every page for itself: a 2048-row chunk over 16 K tokens pulls 27 GB out of the L2
// for 0.9 TFLOP of arithmetic.  Here four waves form a workgroup per (lane of up to 32 query
// rows, split, KV head): each fetches a quarter of the page and writes it into LDS as
// finished MFMA operands (byte formats expanded on the way, once instead of four times),
// and all four multiply their own fused rows with the shared copy.  Two pairs of copies
// alternate: while two pages are multiplied the next two are staged, one barrier per two
// pages; each wave keeps its quarter of one page in flight.  An operand read from LDS must
// feed two row blocks: four waves reading one block's worth each would ask the LDS for
// twice what it delivers.
// The same with two waves per workgroup, each fetching half a page, serves verify batches of
// 33 to 96 fused rows per lane (a chain of 8 rows or a tree of 16 nodes for a group of 6):
// the one-wave kernels give such a lane two or three waves that each read every page, and
// on these formats the reading is what they wait for.
constexpr uint32_t kGroupWaves = 4;

// The workgroup's barrier between pairs of pages: a wave's LDS writes are done (the LDS
// counter at zero) before it arrives, and that is all; __syncthreads() would also wait for
// the global loads in flight, which are the next page to stage.
__device__ __forceinline__ void group_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

struct GroupOperands {
  u32x4 keys[2][8][64];  // [token block][dims block][lane]
  u32x4 values[16][64];  // [dims block][lane]
};
template <uint32_t FMT, uint32_t W>
struct GroupShare {  // wave w's share of a page as loaded, W waves: dims blocks (8 / W) w .. of the
                     // keys, dims blocks (16 / W) w .. of the values
  static constexpr uint32_t kKeyBlocks = 8 / W, kValueBlocks = 16 / W;
  uint32_t k[2][kKeyBlocks][Wide<FMT>::kDwords];  // [token block][dims block of the share]
  uint32_t v[kValueBlocks][Wide<FMT>::kDwords];
};

template <uint32_t FMT, uint32_t W, bool REUSED>
__device__ __forceinline__ void fetch_share(GroupShare<FMT, W> &r, const PagePlace &p, uint32_t wave,
                                            uint32_t t, uint32_t g) {
  constexpr uint32_t B = Wide<FMT>::kBytes;
  constexpr uint32_t KB = GroupShare<FMT, W>::kKeyBlocks, VB = GroupShare<FMT, W>::kValueBlocks;
#pragma unroll
  for (uint32_t tb = 0; tb < 2; ++tb) {
    const uint8_t *row = p.keys + (8 * (t >> 2) + 4 * tb + (t & 3)) * kD * B;
    if constexpr (Wide<FMT>::kByte) {
#pragma unroll
      for (uint32_t c = 0; c < KB; c += 2) {  // one 16-byte load holds two dims blocks
        const u32x4 x = load_streaming<u32x4, REUSED>(row + key_dims<FMT>(KB * wave + c, g));
        r.k[tb][c][0] = x[0], r.k[tb][c][1] = x[1], r.k[tb][c + 1][0] = x[2], r.k[tb][c + 1][1] = x[3];
      }
    } else {
#pragma unroll
      for (uint32_t c = 0; c < KB; ++c) {
        const u32x4 x = load_streaming<u32x4, REUSED>(row + key_dims<FMT>(KB * wave + c, g) * B);
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) r.k[tb][c][i] = x[i];
      }
    }
  }
#pragma unroll
  for (uint32_t i = 0; i < VB; ++i) {
    const uint8_t *at = p.values + ((16 * (VB * wave + i) + t) * kPage + 8 * g) * B;
    if constexpr (Wide<FMT>::kByte) {
      const u32x2 x = load_streaming<u32x2, REUSED>(at);
      r.v[i][0] = x[0], r.v[i][1] = x[1];
    } else {
      const u32x4 x = load_streaming<u32x4, REUSED>(at);
#pragma unroll
      for (uint32_t e = 0; e < 4; ++e) r.v[i][e] = x[e];
    }
  }
}
template <uint32_t FMT>
__device__ __forceinline__ u32x4 share_operand(const uint32_t (&raw)[Wide<FMT>::kDwords]) {
  if constexpr (Wide<FMT>::kFp8) return fp8_operand(raw[0], raw[1]);
  else if constexpr (Wide<FMT>::kInt8) return int8_operand(raw[0], raw[1]);
  else return u32x4{raw[0], raw[1], raw[2], raw[3]};
}
template <uint32_t FMT, uint32_t W>
__device__ __forceinline__ void stage_share(GroupOperands &page, const GroupShare<FMT, W> &r, uint32_t wave,
                                            uint32_t lane) {
  constexpr uint32_t KB = GroupShare<FMT, W>::kKeyBlocks, VB = GroupShare<FMT, W>::kValueBlocks;
#pragma unroll
  for (uint32_t tb = 0; tb < 2; ++tb)
#pragma unroll
    for (uint32_t c = 0; c < KB; ++c) page.keys[tb][KB * wave + c][lane] = share_operand<FMT>(r.k[tb][c]);
#pragma unroll
  for (uint32_t i = 0; i < VB; ++i) page.values[VB * wave + i][lane] = share_operand<FMT>(r.v[i]);
}

// NB blocks of 16 fused rows per wave; the lane's fused rows are dealt to the W waves in
// equal runs of ceil(M / W) (at most 16 NB).  SETS register sets hold a wave's share of
// the pages on their way: one, whose loads have a page time to arrive, for pages that come
// out of the caches (prefill) and for bf16, whose share is 32 to 64 registers; two, with
// two page times, for the byte formats' verify lanes, whose pages come from HBM.
// COPIES staged pages in LDS: four (128 KiB, a barrier every second page) where the
// workgroup's four waves fill the CU anyway; two (64 KiB, a barrier per page) for workgroups
// of two waves, so that two of them fit a CU and no SIMD stays empty.
template <uint32_t FMT, uint32_t NB, uint32_t W, bool REUSED, uint32_t SETS = 1, uint32_t COPIES = 4>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(1, 1))) void
group_wide_kernel(const uint16_t *__restrict__ queries, uint16_t *__restrict__ output,
                  float *__restrict__ partials, float *__restrict__ statistics, DecodeArgs a) {
  constexpr bool kFp8 = Wide<FMT>::kFp8, kInt8 = Wide<FMT>::kInt8, kByte = Wide<FMT>::kByte;
  static_assert(COPIES == 4 || (COPIES == 2 && SETS == 1), "two copies: one set of page registers");
  __shared__ GroupOperands shared_page[COPIES];
  const uint32_t item = blockIdx.x, head = blockIdx.y;
  uint32_t li;
  const DecodeLane l = lane_of_item(a, item, li);
  const uint32_t split = item - l.first_item;
  // Every wave of the workgroup takes the same way out: the barriers below are reached by
  // all of them or by none.
  if (split >= l.split_count) return;
  const uint32_t visible = l.committed + l.active_rows;
  const uint32_t pages = (visible + kPage - 1) / kPage;
  const uint32_t per = (pages + l.split_count - 1) / l.split_count;
  const uint32_t written = (pages + per - 1) / per;
  const uint32_t begin = split * per;
  if (begin >= pages) return;
  const uint32_t end = min(pages, begin + per);

  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63u, t = lane & 15, g = lane >> 4;
  const uint32_t H = a.kv_heads, G = a.group, M = a.fused_rows;
  const uint32_t db = Wide<FMT>::kSlab * H, sb = kByte ? kPage * H * 4 : 0;
  const RegionOffsets ro = region_offsets(a.kv.extent_pages, db, sb);
  const float score_scale = default_score_scale(kD, l.score_scale);

  const uint32_t run = (M + W - 1) / W;  // fused rows per wave
  uint32_t m[NB];
  bool in_tile[NB], live_row[NB];
  Sight sight[NB];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    m[nb] = run * wave + 16 * nb + t;
    const uint32_t query_row = m[nb] / G;
    in_tile[nb] = 16 * nb + t < run && m[nb] < M;
    live_row[nb] = in_tile[nb] && query_row < l.active_rows;
    sight[nb].committed = l.committed;
    sight[nb].visible = visible;
    sight[nb].limit =
        live_row[nb] ? min(visible, l.committed + min(query_row, l.active_rows - 1) + 1) : visible;
    sight[nb].tree = live_row[nb] && l.masks != nullptr;
    sight[nb].mask = sight[nb].tree ? l.masks[query_row] : 0u;
  }
  // A wave none of whose rows is in the lane still fetches and stages its quarter.
  const bool computes = run * wave < M;

  const uint16_t *q_head = queries + l.q_offset + uint64_t(head) * a.row_stride * G * kD;
  u32x4 q_reg[NB][8];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    const uint16_t *q_row = q_head + uint64_t(live_row[nb] ? m[nb] : 0) * kD;
#pragma unroll
    for (uint32_t kb = 0; kb < 8; ++kb) {
      u32x4 q = load_global<u32x4>(q_row + key_dims<FMT>(kb, g));
      if constexpr (kByte) {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
          const f16x2 pair = {_Float16(__uint_as_float(q[i] << 16)),
                              _Float16(__uint_as_float(q[i] & 0xffff0000u))};
          q[i] = __builtin_bit_cast(uint32_t, pair);
        }
      }
      if (!live_row[nb]) q = u32x4{0u, 0u, 0u, 0u};
      q_reg[nb][kb] = q;
    }
  }

  const uint64_t *const entries = l.table + begin;
  const uint32_t count = end - begin, last_slot = count - 1;
  static_assert(SETS == 1 || (SETS == 2 && Wide<FMT>::kByte), "two sets of page registers: byte formats only");
  GroupShare<FMT, W> raw[SETS];  // this wave's share of the pages on their way
  // bf16 pages: a page's entry is read a turn before the loads that need it, since one wave
  // per SIMD has nothing else to run while a scalar load is on its way.  With the byte
  // formats' conversions to fill that time the early read measured 10 % slower, and they
  // read the entry where they use it.
  uint64_t entry_ahead = kByte ? 0 : scalar_entry(entries, 0);
  auto next_entry = [&](uint32_t following) {
    if constexpr (kByte) return scalar_entry(entries, min(following - 1, last_slot));
    const uint64_t entry = entry_ahead;
    entry_ahead = scalar_entry(entries, min(following, last_slot));
    return entry;
  };
  auto fetch = [&](GroupShare<FMT, W> &set, uint64_t entry) {
    const PagePlace p = place_page<FMT>(entry, head, H, a.kv.offset, ro);
    asm volatile("");
    fetch_share<FMT, W, REUSED>(set, p, wave, t, g);
    asm volatile("");
  };
  // The scales of a byte format's page, by every wave for its own lanes: they are few, and
  // what a lane needs of them depends on its place in the wave alone.
  f32x4 ks_even[2], vs_even[2], ks_odd[2], vs_odd[2];
  auto fetch_scales = [&](f32x4 (&ks)[2], f32x4 (&vs)[2], uint64_t entry) {
    if constexpr (kByte) {
      const PagePlace p = place_page<FMT>(entry, head, H, a.kv.offset, ro);
      ks[0] = load_global<f32x4>(p.key_scales + 8 * g);
      ks[1] = load_global<f32x4>(p.key_scales + 8 * g + 4);
      vs[0] = load_global<f32x4>(p.value_scales + 8 * g);
      vs[1] = load_global<f32x4>(p.value_scales + 8 * g + 4);
    }
  };
  // bf16 pages need no conversion on their way: in the two-copy form the wave's share of a
  // page goes from global memory into the staged copy directly (16 bytes per lane and
  // instruction, the lanes of an instruction one operand block), with no registers in between
  // and no LDS writes to issue.  The copy must be free when the loads are sent, since they
  // land whenever they arrive; the wave waits for them before the barrier that hands the copy
  // over.  (bf16 chain verify of a batch of 32: 413 -> 396 us.  The four-copy form was slower
  // with it, a 2048-row prefill chunk 1.19 -> 1.27 ms, and stages through registers.)
  constexpr bool kDirect = !kByte && COPIES == 2;
  auto direct = [&](GroupOperands &copy, uint64_t entry) {
    constexpr uint32_t B = Wide<FMT>::kBytes;
    constexpr uint32_t KB = GroupShare<FMT, W>::kKeyBlocks, VB = GroupShare<FMT, W>::kValueBlocks;
    constexpr uint32_t kPolicy = REUSED ? 0u : 2u;  // 2: non-temporal, for pages read once
    typedef __attribute__((address_space(1))) const void GlobalBytes;
    typedef __attribute__((address_space(3))) void SharedBytes;
    const PagePlace p = place_page<FMT>(entry, head, H, a.kv.offset, ro);
#pragma unroll
    for (uint32_t tb = 0; tb < 2; ++tb) {
      const uint8_t *row = p.keys + (8 * (t >> 2) + 4 * tb + (t & 3)) * kD * B;
#pragma unroll
      for (uint32_t c = 0; c < KB; ++c)
        __builtin_amdgcn_global_load_lds(
            (GlobalBytes *)(reinterpret_cast<uintptr_t>(row + key_dims<FMT>(KB * wave + c, g) * B)),
            (SharedBytes *)(&copy.keys[tb][KB * wave + c][0]), 16, 0, kPolicy);
    }
#pragma unroll
    for (uint32_t i = 0; i < VB; ++i)
      __builtin_amdgcn_global_load_lds(
          (GlobalBytes *)(reinterpret_cast<uintptr_t>(p.values + ((16 * (VB * wave + i) + t) * kPage + 8 * g) * B)),
          (SharedBytes *)(&copy.values[VB * wave + i][0]), 16, 0, kPolicy);
  };
  // The barrier of the direct form: the wave's loads into the copies have landed.
  auto landed_barrier = [&] { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  const uint64_t entry0 = next_entry(1), entry1 = next_entry(2);
  if constexpr (!kDirect) {
    fetch(raw[0], entry0);
    if constexpr (SETS == 2) fetch(raw[1], entry1);
  }
  fetch_scales(ks_even, vs_even, entry0);
  fetch_scales(ks_odd, vs_odd, entry1);

  f32x4 acc[NB][16];  // [block][dim block]: dims 16*mb + 4g + r of column t
  float row_max[NB], row_sum[NB];
#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
#pragma unroll
    for (uint32_t mb = 0; mb < 16; ++mb) acc[nb][mb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    row_max[nb] = -INFINITY;
    row_sum[nb] = 0.0f;
  }

  // One staged page against the wave's rows.  check_tokens: whether the page can hold
  // tokens some row does not see (a page wholly inside the committed tokens cannot; one
  // copy of the page code serves both, the test itself is skipped).
  auto attend_page = [&](const GroupOperands &now, uint32_t page, const f32x4 (&page_ks)[2],
                         const f32x4 (&page_vs)[2], bool check_tokens) __attribute__((always_inline)) {
    f32x4 s[NB][2];
#pragma unroll
    for (uint32_t nb = 0; nb < NB; ++nb) s[nb][0] = s[nb][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // Operands come out of LDS kAhead reads before the MFMAs that take them: the four waves
    // of the workgroup read at the same time, and a read comes back later than the MFMAs of
    // two operands last.  The order is pinned, or the compiler pulls the reads back together.
    constexpr uint32_t kAhead = kInt8 ? 3 : 4;  // int8 with four reloads spilled registers inside the page loop
    u32x4 operand[kAhead];
#pragma unroll
    for (uint32_t i = 0; i < kAhead; ++i) operand[i] = now.keys[i & 1][i >> 1][lane];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i) {
      const uint32_t tb = i & 1, kb = i >> 1;
#pragma unroll
      for (uint32_t nb = 0; nb < NB; ++nb) s[nb][tb] = mfma<FMT>(operand[i % kAhead], q_reg[nb][kb], s[nb][tb]);
      if (i + kAhead < 16) operand[i % kAhead] = now.keys[(i + kAhead) & 1][(i + kAhead) >> 1][lane];
      __builtin_amdgcn_sched_barrier(0);
    }
    // The first value operands are on their way while the softmax runs.
#pragma unroll
    for (uint32_t i = 0; i < kAhead; ++i) operand[i] = now.values[i][lane];
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t first_token = page * kPage;
    u32x4 pb[NB];
#pragma unroll
    for (uint32_t nb = 0; nb < NB; ++nb) {
      float score[8], local_max = -INFINITY;
#pragma unroll
      for (uint32_t i = 0; i < 8; ++i) {
        const uint32_t tb = i >> 2, rr = i & 3;
        float v = s[nb][tb][rr];
        if constexpr (kByte) v *= page_ks[tb][rr];
        score[i] = v * score_scale;
      }
      // A token the row does not see scores -inf, and its weight below comes out as
      // exp(-inf) = 0 by itself.
      if (check_tokens) {
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i)
          if (!sight[nb].sees(first_token + 8 * g + 4 * (i >> 2) + (i & 3))) score[i] = -INFINITY;
      }
#pragma unroll
      for (uint32_t i = 0; i < 8; ++i) local_max = fmaxf(local_max, score[i]);
      local_max = fmaxf(local_max, __shfl_xor(local_max, 16));
      local_max = fmaxf(local_max, __shfl_xor(local_max, 32));
      const float next_max = fmaxf(row_max[nb], local_max);
      // A row that has seen nothing yet keeps -inf; its rescale is 1, not exp(nan).
      const float rescale = next_max == row_max[nb]
                                ? 1.0f
                                : __builtin_amdgcn_exp2f((row_max[nb] - next_max) * kLog2e);
      // A row that still has seen nothing measures from 0: -inf - -inf is no number.
      const float reference = next_max == -INFINITY ? 0.0f : next_max;
      float weight[8], page_sum = 0.0f;
#pragma unroll
      for (uint32_t i = 0; i < 8; ++i) {
        // The difference first, so the page's maximum gets exactly 1.
        const float p = __builtin_amdgcn_exp2f((score[i] - reference) * kLog2e);
        page_sum += p;
        weight[i] = kByte ? p * page_vs[i >> 2][i & 3] : p;
      }
      row_sum[nb] = fmaf(row_sum[nb], rescale, page_sum);
      row_max[nb] = next_max;
#pragma unroll
      for (uint32_t p = 0; p < 4; ++p) {
        if constexpr (kFp8) {
          const f16x2 pair = {_Float16(weight[2 * p]), _Float16(weight[2 * p + 1])};
          pb[nb][p] = __builtin_bit_cast(uint32_t, pair);
        } else if constexpr (kInt8) {
          // Rounded to bf16 as the reference tile does, then carried as fp16.
          const f32x2 wide = {weight[2 * p], weight[2 * p + 1]};
          const uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_convertvector(wide, bf16x2));
          const f16x2 pair = {_Float16(__uint_as_float(bits << 16)),
                              _Float16(__uint_as_float(bits & 0xffff0000u))};
          pb[nb][p] = __builtin_bit_cast(uint32_t, pair);
        } else {
          const f32x2 pair = {weight[2 * p], weight[2 * p + 1]};
          pb[nb][p] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
        }
      }
      if (__builtin_amdgcn_ballot_w64(rescale != 1.0f)) {
        // The accumulators live in the second register file and are named there on the way
        // in, so that the moves out of it that a multiply needs stay inside this branch:
        // left to itself the compiler moves all of them out on every page.
#pragma unroll
        for (uint32_t mb = 0; mb < 16; ++mb) {
          asm volatile("" : "+a"(acc[nb][mb]));
          acc[nb][mb] *= rescale;
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (uint32_t mb = 0; mb < 16; ++mb) {
#pragma unroll
      for (uint32_t nb = 0; nb < NB; ++nb) acc[nb][mb] = mfma<FMT>(operand[mb % kAhead], pb[nb], acc[nb][mb]);
      if (mb + kAhead < 16) operand[mb % kAhead] = now.values[mb + kAhead][lane];
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const uint32_t first_masked = l.committed / kPage;
  if constexpr (kDirect) {
    // Two copies, loaded directly: while slot i is multiplied out of one, slot i + 1 lands in
    // the other; a barrier per page.
    direct(shared_page[0], entry0);
    landed_barrier();
    auto turn = [&](const GroupOperands &now, GroupOperands &next, uint32_t slot) __attribute__((always_inline)) {
      direct(next, slot == 0 ? entry1 : next_entry(slot + 2));  // of slot + 1
      if (computes && slot < count) attend_page(now, begin + slot, ks_even, vs_even, begin + slot >= first_masked);
      landed_barrier();
    };
    for (uint32_t slot = 0; slot < count; slot += 2) {
      turn(shared_page[0], shared_page[1], slot);
      turn(shared_page[1], shared_page[0], slot + 1);
    }
  } else if constexpr (COPIES == 2) {
    // Two copies: while slot i is multiplied out of one, slot i + 1 goes from the raw
    // registers into the other and the registers are sent for slot i + 2; a barrier per page.
    stage_share<FMT, W>(shared_page[0], raw[0], wave, lane);
    fetch(raw[0], entry1);
    group_barrier();
    auto turn = [&](const GroupOperands &now, GroupOperands &next, uint32_t slot, f32x4 (&ks)[2],
                    f32x4 (&vs)[2]) __attribute__((always_inline)) {
      stage_share<FMT, W>(next, raw[0], wave, lane);  // slot + 1
      const uint64_t entry = next_entry(slot + 3);  // of slot + 2
      fetch(raw[0], entry);
      if (computes && slot < count) attend_page(now, begin + slot, ks, vs, begin + slot >= first_masked);
      fetch_scales(ks, vs, entry);
      group_barrier();
    };
    for (uint32_t slot = 0; slot < count; slot += 2) {
      turn(shared_page[0], shared_page[1], slot, ks_even, vs_even);
      turn(shared_page[1], shared_page[0], slot + 1, ks_odd, vs_odd);
    }
  } else {
    // The first two pages into the first two copies; the entries of the pages whose operands are on their way (slots + 2 and + 3 of a pair):
    // their scales are asked for a page time later.
    uint64_t held_even, held_odd = 0;
    stage_share<FMT, W>(shared_page[0], raw[0], wave, lane);
    if constexpr (SETS == 1) {
      fetch(raw[0], entry1);
      stage_share<FMT, W>(shared_page[1], raw[0], wave, lane);
      held_even = next_entry(3);
      fetch(raw[0], held_even);
    } else {
      held_even = next_entry(3);
      fetch(raw[0], held_even);
      stage_share<FMT, W>(shared_page[1], raw[1], wave, lane);
      held_odd = next_entry(4);
      fetch(raw[1], held_odd);
    }
    group_barrier();
    // Four copies, two pages between barriers: while slots i and i + 1 are multiplied out of
    // one pair of copies, slots i + 2 and i + 3 go from the raw registers into the other pair,
    // each one page time (two with two sets) after its loads were sent (past the end: the last
    // page again, staged into copies nobody reads).  A barrier per page cost 5 % more: the
    // waves leave it together and read their operands at the same time.  Four slots per turn
    // of the loop and no branch around the loads, so every wait names exactly the loads it
    // needs.
    auto pair = [&](const GroupOperands &now0, const GroupOperands &now1, GroupOperands &next0,
                    GroupOperands &next1, uint32_t slot) __attribute__((always_inline)) {
      stage_share<FMT, W>(next0, raw[0], wave, lane);  // slot + 2
      const uint64_t entry_a = next_entry(slot + 3 + SETS);  // of slot + 2 + SETS
      fetch(raw[0], entry_a);
      if (computes && slot < count)
        attend_page(now0, begin + slot, ks_even, vs_even, begin + slot >= first_masked);
      fetch_scales(ks_even, vs_even, held_even);  // of slot + 2
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      stage_share<FMT, W>(next1, raw[SETS - 1], wave, lane);  // slot + 3
      const uint64_t entry_b = next_entry(slot + 4 + SETS);  // of slot + 3 + SETS
      fetch(raw[SETS - 1], entry_b);
      if (computes && slot + 1 < count)
        attend_page(now1, begin + slot + 1, ks_odd, vs_odd, begin + slot + 1 >= first_masked);
      fetch_scales(ks_odd, vs_odd, SETS == 1 ? entry_a : held_odd);  // of slot + 3
      held_even = SETS == 1 ? entry_b : entry_a;
      held_odd = entry_b;
      group_barrier();
    };
    for (uint32_t slot = 0; slot < count; slot += 4) {
      pair(shared_page[0], shared_page[1], shared_page[2], shared_page[3], slot);
      pair(shared_page[2], shared_page[3], shared_page[0], shared_page[1], slot + 2);
    }
  }
  if (!computes) return;

#pragma unroll
  for (uint32_t nb = 0; nb < NB; ++nb) {
    // Lanes of one column hold disjoint tokens: combine their sums.
    float sum = row_sum[nb];
    sum += __shfl_xor(sum, 16);
    sum += __shfl_xor(sum, 32);
    uint16_t *out_head = output + l.q_offset + uint64_t(head) * a.row_stride * G * kD;
    if (written == 1 && !a.all_partials) {
      // One split: the merge's weights are exp(0) = 1, so the row is acc / sum.
      // Rows of the tile past the live ones read as zeros.
      if (in_tile[nb]) {
        const float denominator = live_row[nb] ? sum : 0.0f;
#pragma unroll
        for (uint32_t mb = 0; mb < 16; ++mb) {
          u32x2 packed;
#pragma unroll
          for (uint32_t i = 0; i < 2; ++i) {
            const float lo = acc[nb][mb][2 * i], hi = acc[nb][mb][2 * i + 1];
            const float qlo = denominator > 0.0f ? __fdiv_rn(lo, denominator) : 0.0f;
            const float qhi = denominator > 0.0f ? __fdiv_rn(hi, denominator) : 0.0f;
            packed[i] = uint32_t(f32_to_bf16(qlo)) | (uint32_t(f32_to_bf16(qhi)) << 16);
          }
          *reinterpret_cast<u32x2 *>(out_head + uint64_t(m[nb]) * kD + 16 * mb + 4 * g) = packed;
        }
      }
      continue;
    }
    if (live_row[nb]) {
      const uint64_t row =
          l.row_base + uint64_t(head) * l.split_count * M + uint64_t(split) * M + m[nb];
      float *out = partials + row * kD;
#pragma unroll
      for (uint32_t mb = 0; mb < 16; ++mb) *reinterpret_cast<f32x4 *>(out + 16 * mb + 4 * g) = acc[nb][mb];
      if (g == 0) {
        statistics[row * 2] = row_max[nb];
        statistics[row * 2 + 1] = sum;
      }
    }
  }
}

}  // namespace
}  // namespace kvx

using namespace kvx;

// Runs paged attention for bf16 or fp8 pages of head dimension 256 on the
// matrix cores; returns 1 (declined) for shapes it does not cover, 0 when
// enqueued, or a negative status.  Arguments as kvx_attend_int4_launch.
int kvx_attend_wide_launch(const kvx_storage *s, kvx_kv_layer kv, uint32_t query_heads,
                           const void *queries, void *output, const uint64_t *const *page_tables,
                           const kvx_verify_params *lanes, uint32_t n_lanes,
                           const uint32_t *row_masks, uint32_t row_stride, uint64_t lane_stride,
                           void *workspace, uint64_t workspace_bytes, int many_tiles,
                           hipStream_t stream, Tiles tile_rows, const Epilogue *epilogue) {
  const uint32_t format = s->layout.format;
  if ((format != KVX_FMT_BF16 && format != KVX_FMT_FP8E4M3 && format != KVX_FMT_INT8) ||
      !matrix_attention_covers(s, query_heads, lanes, n_lanes))
    return 1;
  const uint32_t M = lanes[0].row_capacity * (query_heads / s->layout.kv_heads);
#define KVX_WIDE(FMT, NB, WAVES, REUSED)                                                         \
  launch_matrix_attention(attend_wide_kernel<FMT, NB, WAVES, REUSED>, "attend_wide_kernel", 16 * NB, 64, s, \
                          kv, query_heads, queries, output, page_tables, lanes, n_lanes, row_masks, \
                          row_stride, lane_stride, workspace, workspace_bytes, stream,              \
                          nullptr, tile_rows, epilogue)
  // Two blocks of 16 fused rows per wave share every key and value operand; a
  // third would not fit the register file next to a page of bf16 keys and values.
  // One-byte formats run two waves per SIMD with one block (decode, the 8-row
  // tiles of a prefill with several splits); with two blocks the accumulators
  // leave too little room for that (the compiler spills inside the page loop:
  // int8 prefill 2.9 -> 4.5 ms), so those keep the SIMD to themselves.
  // The regular tiles of a chunked prefill (tile_rows > 0) walk the same pages
  // over and over: their loads may stay in the caches.
  const bool reused = tile_rows > 0;
#define KVX_GROUP(FMT, NB, W, REUSED, ...)                                                        \
  launch_matrix_attention(group_wide_kernel<FMT, NB, W, REUSED, ##__VA_ARGS__>, "group_wide_kernel", 16 * NB * W, 64 * W, \
                          s, kv, query_heads, queries, output, page_tables, lanes, n_lanes, row_masks, \
                          row_stride, lane_stride, workspace, workspace_bytes, stream, nullptr,     \
                          tile_rows, epilogue)
#define KVX_GROUP_FORMATS(NB, W, REUSED)                                                          \
  (format == KVX_FMT_BF16   ? KVX_GROUP(KVX_FMT_BF16, NB, W, REUSED)                                \
   : format == KVX_FMT_INT8 ? KVX_GROUP(KVX_FMT_INT8, NB, W, REUSED)                                \
                            : KVX_GROUP(KVX_FMT_FP8E4M3, NB, W, REUSED))
  // many_tiles == 2: lanes of several prefill tiles each, for a workgroup of four waves
  // that shares every page through LDS, two or three row blocks per wave: up to 192 fused rows.
  if (many_tiles == 2) {
    if (!tile_rows || M > 48u * kGroupWaves) return 1;
    if (M > 32u * kGroupWaves) return KVX_GROUP_FORMATS(3, 4, true);
    return KVX_GROUP_FORMATS(2, 4, true);
  }
  // Verify lanes of more than 32 fused rows: the waves that the lane needs anyway share its
  // pages.  33 .. 64 rows (a chain of 8 for a group of 6): two waves that fetch half a page
  // each, with two LDS copies so that two such workgroups fit a CU (batch of 32: bf16 706 ->
  // 400 us, int8 435 -> 387 us, fp8 405 -> 343 us; with four copies, one workgroup per CU and
  // half of the SIMDs empty, the byte formats took 550 - 650 us).  65 .. 128 rows (a tree of 16
  // nodes): four waves over four copies, the byte formats with two sets of page registers
  // (batch 4 x 65 536 tokens: int8 436 -> 282 us); bf16 up to 96 rows as two waves of 48, which
  // its direct loads leave the registers for (456 -> 212 us; four waves of 24: 238 us; the
  // byte formats spill in that form).
  // A verify lane holds 128 fused rows at most.
  if (!tile_rows && !many_tiles && M > 32 && M <= 32u * kGroupWaves) {
    if (format == KVX_FMT_BF16)
      return M > 96   ? KVX_GROUP(KVX_FMT_BF16, 2, 4, false)
             : M > 64 ? KVX_GROUP(KVX_FMT_BF16, 3, 2, false, 1, 2)
                      : KVX_GROUP(KVX_FMT_BF16, 2, 2, false, 1, 2);
    if (format == KVX_FMT_INT8) return M > 64 ? KVX_GROUP(KVX_FMT_INT8, 2, 4, false, 2) : KVX_GROUP(KVX_FMT_INT8, 2, 2, false, 1, 2);
    return M > 64 ? KVX_GROUP(KVX_FMT_FP8E4M3, 2, 4, false, 2) : KVX_GROUP(KVX_FMT_FP8E4M3, 2, 2, false, 1, 2);
  }
#undef KVX_GROUP_FORMATS
#undef KVX_GROUP
  if (format == KVX_FMT_BF16) {
    if (M > 16) return reused ? KVX_WIDE(KVX_FMT_BF16, 2, 1, true) : KVX_WIDE(KVX_FMT_BF16, 2, 1, false);
    return reused ? KVX_WIDE(KVX_FMT_BF16, 1, 1, true) : KVX_WIDE(KVX_FMT_BF16, 1, 1, false);
  }
  const bool two_blocks = M > 16 && !many_tiles;
  if (format == KVX_FMT_INT8) {
    if (two_blocks) return reused ? KVX_WIDE(KVX_FMT_INT8, 2, 1, true) : KVX_WIDE(KVX_FMT_INT8, 2, 1, false);
    return reused ? KVX_WIDE(KVX_FMT_INT8, 1, 2, true) : KVX_WIDE(KVX_FMT_INT8, 1, 2, false);
  }
  if (two_blocks) return reused ? KVX_WIDE(KVX_FMT_FP8E4M3, 2, 1, true) : KVX_WIDE(KVX_FMT_FP8E4M3, 2, 1, false);
  return reused ? KVX_WIDE(KVX_FMT_FP8E4M3, 1, 2, true) : KVX_WIDE(KVX_FMT_FP8E4M3, 1, 2, false);
#undef KVX_WIDE
}
