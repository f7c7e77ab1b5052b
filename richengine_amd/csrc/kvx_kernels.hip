// Kernels of the paged-KV path that are bandwidth-trivial or format-generic:
// quantize-on-append, the format-generic attention tile with its fixed-order
// merge, tree-path compaction and whole-page copy, with their launchers.
// The arithmetic of every kernel here keeps the operation order of the
// reference kernels it replaces (cited per kernel), with products and sums
// left unfused so the fp32 results do not depend on contraction.
#include <atomic>
#include <algorithm>
#include <vector>

#include "kvx_device.h"
#include "kvx_debug.h"

namespace kvx {

constexpr uint32_t kPage = KVX_PAGE_TOKENS;
constexpr uint32_t kLanes = KVX_LANES_PER_LAUNCH;

// ============================================================== append ====
struct AppendLane {
  const uint64_t *table;
  uint32_t committed, tokens, stride, entries;
  uint32_t group_base;  // first workgroup of this lane
  uint32_t pad;
};
struct AppendArgs {
  AppendLane lane[kLanes];
  uint32_t n_lanes;
  uint32_t kv_heads, head_dim;
  uint32_t verify_max_rows;
  uint32_t uniform_groups;  // workgroups per lane when every lane stores the same rows, else 0
  kvx_kv_layer kv;
  uint64_t lane_stride;
};

// The kernel-side contract of a store lane (reference:
// common/paged_store_row.h:14-29; verify adds rows <= bound and stride == 32,
// decode/paged_attention_store.metal:22-27).  A lane that fails writes nothing.
__device__ inline bool append_contract(const AppendLane &l, const AppendArgs &a) {
  const uint64_t required = (uint64_t(l.committed) + l.tokens + kPage - 1) / kPage;
  bool ok = l.committed <= KVX_MAX_PHYSICAL_TOKENS && l.tokens > 0 &&
            l.tokens <= KVX_PREFILL_TOKEN_BUDGET &&
            uint64_t(l.committed) + l.tokens <= KVX_MAX_PHYSICAL_TOKENS &&
            l.stride >= l.tokens && l.stride <= KVX_PREFILL_TOKEN_BUDGET &&
            l.stride % kPage == 0 && l.entries >= required && a.kv.extent_pages > 0;
  if (a.verify_max_rows)
    ok = ok && l.tokens <= a.verify_max_rows && l.stride == KVX_VERIFY_CHUNK_STRIDE;
  return ok;
}

// One thread's share of storing a row (one tensor, one head, one token): the
// row's maximum over the workgroup's D threads, its scale, this dimension's code
// (reference: common/paged_store_row.h:47-147, paged_store_row_fp8.h:28-78).
// Every thread of the workgroup calls it; `wave_max` is four floats of LDS.
template <uint32_t FMT>
__device__ __forceinline__ void store_row_element(uint16_t source, bool value_tensor, const Slab &s,
                                                  uint32_t slot, uint32_t d, uint32_t D,
                                                  float *wave_max) {
  uint8_t *data = value_tensor ? s.values : s.keys;
  // Element index inside the head's slab: keys token-major, values
  // dimension-major (packed int4: both token-major).
  const uint32_t element = (value_tensor && FMT != KVX_FMT_INT4) ? d * kPage + slot : slot * D + d;

  if constexpr (FMT == KVX_FMT_BF16) {
    reinterpret_cast<uint16_t *>(data)[element] = source;
    return;
  } else {
    const float v = bf16_to_f32(source);
    float m = fabsf(v);
    for (int offset = 32; offset; offset >>= 1) m = fmaxf(m, __shfl_xor(m, offset));
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    float maximum = wave_max[0];
    for (uint32_t w = 1; w < (D + 63) / 64; ++w) maximum = fmaxf(maximum, wave_max[w]);
    constexpr float qmax = FMT == KVX_FMT_INT4 ? 7.0f : FMT == KVX_FMT_INT8 ? 127.0f : 448.0f;
    const float scale = maximum == 0.0f ? 0.0f : __fdiv_rn(maximum, qmax);
    if (d == 0) (value_tensor ? s.value_scales : s.key_scales)[slot] = scale;
    const float scaled = maximum == 0.0f ? 0.0f : __fdiv_rn(__fmul_rn(v, qmax), maximum);
    if constexpr (FMT == KVX_FMT_FP8E4M3) {
      data[element] = maximum == 0.0f ? uint8_t(0) : uint8_t(f32_to_e4m3(scaled));
    } else {
      constexpr int limit = FMT == KVX_FMT_INT4 ? 7 : 127;
      int code = int(rintf(scaled));
      code = code < -limit ? -limit : code > limit ? limit : code;
      if (maximum == 0.0f) code = 0;
      if constexpr (FMT == KVX_FMT_INT8) {
        reinterpret_cast<int8_t *>(data)[element] = int8_t(code);
      } else {
        // Even dimension in the low nibble; the even thread writes the byte.
        const uint32_t nibble = uint32_t(code) & 0xfu;
        const uint32_t partner = __shfl_xor(nibble, 1);
        if ((d & 1) == 0) data[element >> 1] = uint8_t(nibble | (partner << 4));
      }
    }
  }
}

// One workgroup stores one row (one tensor, one head, one token) of one lane:
// head_dim threads, one per dimension (reference:
// common/paged_store_row.h:47-147, paged_store_row_fp8.h:28-78).
template <uint32_t FMT>
__global__ __launch_bounds__(256) void append_kernel(const uint16_t *__restrict__ chunk_keys,
                                                     const uint16_t *__restrict__ chunk_values,
                                                     AppendArgs a) {
  __shared__ float wave_max[4];
  const uint32_t group = blockIdx.x;
  uint32_t li = 0;
  if (a.uniform_groups) {
    li = group / a.uniform_groups;
  } else {
    for (uint32_t i = 1; i < a.n_lanes; ++i)
      if (group >= a.lane[i].group_base) li = i;
  }
  const AppendLane &l = a.lane[li];
  if (!append_contract(l, a)) return;
  const uint32_t D = a.head_dim, H = a.kv_heads;
  const uint32_t local = group - l.group_base;
  const uint32_t rows = l.tokens * H;
  if (local >= 2 * rows) return;
  const bool value_tensor = local >= rows;
  const uint32_t row = value_tensor ? local - rows : local;
  const uint32_t token = row % l.tokens, head = row / l.tokens;
  const uint32_t d = threadIdx.x;
  const uint32_t logical = l.committed + token;
  // The row's source does not depend on the page entry: both loads are in flight together.
  const uint16_t source =
      value_tensor ? chunk_values[li * a.lane_stride + (uint64_t(head) * D + d) * l.stride + token]
                   : chunk_keys[li * a.lane_stride + (uint64_t(head) * l.stride + token) * D + d];
  const Slab s = slab_of(FMT, H, D, a.kv, head, l.table[logical / kPage]);
  store_row_element<FMT>(source, value_tensor, s, logical % kPage, d, D, wave_max);
}

// QKV prepare fused with the store: per-head RMS norm, partial rotary embedding
// and the layout change from packed projection rows to attention queries
// (reference: common/attention_qkv_prepare.h:12-83, common/rms_inverse.h:14-31),
// with the key and value rows quantized straight into their page slots instead
// of a bf16 chunk that the store kernel reads back.  One workgroup per (row,
// head) task, query tasks first, head_dim threads.  The sums keep one fixed
// order (32-lane xor butterflies, then the groups in order) and every product,
// sum and quotient is rounded on its own, so results do not depend on the
// launch.
struct PrepareArgs {
  AppendArgs append;  // lanes: table, committed tokens, live rows
  const uint16_t *packed;
  const void *q_norm, *k_norm;
  const float *rope_cos, *rope_sin;
  uint16_t *queries;
  uint32_t query_heads, rotary_pairs, query_gate, norm_f32;
  uint32_t rows;        // rows per lane in packed / rope_cos / rope_sin
  uint32_t row_stride;  // rows between KV heads in the queries
  float eps;
  uint32_t group_magic;  // ceil(2^32 / group) for group > 1: head / group = mulhi(head, group_magic) for head < 2^16
};

template <uint32_t FMT>
__global__ __launch_bounds__(256) void prepare_append_kernel(PrepareArgs p) {
  // Every product and sum below is rounded on its own: no fused multiply-add may
  // be formed from them (the rounding intrinsics of the HIP headers are plain
  // operators, which the default contraction mode would still fuse).
#pragma clang fp contract(off)
  __shared__ float reductions[8];
  __shared__ float key_max[4], value_max[4];
  __shared__ uint16_t normalized[256], rotated[256];
  const AppendArgs &a = p.append;
  const uint32_t group = blockIdx.x;
  uint32_t li = 0;
  for (uint32_t i = 1; i < a.n_lanes; ++i)
    if (group >= a.lane[i].group_base) li = i;
  const AppendLane &l = a.lane[li];
  if (!append_contract(l, a)) return;
  const uint32_t D = a.head_dim, H = a.kv_heads, QH = p.query_heads, G = QH / H;
  const uint32_t local = group - l.group_base;
  if (local >= l.tokens * (QH + H)) return;
  const bool query = local < l.tokens * QH;
  const uint32_t local_task = query ? local : local - l.tokens * QH;
  const uint32_t heads = query ? QH : H;
  const uint32_t row = local_task / heads, head = local_task % heads;
  const uint32_t d = threadIdx.x;
  const uint32_t q_stride = p.query_gate ? 2 * D : D;
  const uint64_t packed_stride = uint64_t(QH) * q_stride + 2ull * H * D;
  const uint16_t *source = p.packed + (uint64_t(li) * p.rows + row) * packed_stride +
                           (query ? uint64_t(head) * q_stride : uint64_t(QH) * q_stride + uint64_t(head) * D);
  const uint16_t raw = source[d];
  const uint16_t raw_value = query ? uint16_t(0) : source[uint64_t(H) * D + d];
  const float element = bf16_to_f32(raw);
  float inverse = 1.0f, scale = 1.0f;
  if (p.q_norm) {
    float sum = element * element;
    for (int offset = 16; offset; offset >>= 1) sum = sum + __shfl_xor(sum, offset);
    if ((d & 31u) == 0) reductions[d >> 5] = sum;
    __syncthreads();
    float total = 0.0f;
    for (uint32_t i = 0; i < D / 32; ++i) total = total + reductions[i];
    // sqrtf and the quotients are correctly rounded (__fsqrt_rn is the hardware's
    // approximate root)
    const float mean = total / float(D);
    inverse = 1.0f / sqrtf(mean + p.eps);
    const void *weight = query ? p.q_norm : p.k_norm;
    scale = p.norm_f32 ? static_cast<const float *>(weight)[d]
                       : bf16_to_f32(static_cast<const uint16_t *>(weight)[d]);
  }
  const float unit = element * inverse;
  normalized[d] = f32_to_bf16(unit * scale);
  __syncthreads();
  const uint32_t RP = p.rotary_pairs;
  if (d < RP) {
    const float first = bf16_to_f32(normalized[d]), second = bf16_to_f32(normalized[d + RP]);
    const uint64_t at = (uint64_t(li) * p.rows + row) * RP + d;
    const float cosine = p.rope_cos[at], sine = p.rope_sin[at];
    const float fc = first * cosine, ss = second * sine, sc = second * cosine, fs = first * sine;
    rotated[d] = f32_to_bf16(fc - ss);
    rotated[d + RP] = f32_to_bf16(sc + fs);
  } else if (d >= 2 * RP) {
    rotated[d] = normalized[d];
  }
  __syncthreads();
  const uint16_t prepared = rotated[d];
  if (query) {
    const uint32_t kv_head = head / G, local_head = head % G;
    p.queries[uint64_t(li) * H * p.row_stride * G * D +
              ((uint64_t(kv_head) * p.row_stride + row) * G + local_head) * D + d] = prepared;
    return;
  }
  const uint32_t logical = l.committed + row;
  const Slab s = slab_of(FMT, H, D, a.kv, head, l.table[logical / kPage]);
  store_row_element<FMT>(prepared, false, s, logical % kPage, d, D, key_max);
  store_row_element<FMT>(raw_value, true, s, logical % kPage, d, D, value_max);
}

// E consecutive bf16 values (E x 2 bytes, aligned to that) as one load / store.
template <uint32_t E>
__device__ __forceinline__ void load_bf16s(const uint16_t *from, uint16_t (&out)[E]) {
  if constexpr (E == 4) {
    const uint2 v = *reinterpret_cast<const uint2 *>(from);
    out[0] = uint16_t(v.x), out[1] = uint16_t(v.x >> 16), out[2] = uint16_t(v.y), out[3] = uint16_t(v.y >> 16);
  } else if constexpr (E == 2) {
    const uint32_t v = *reinterpret_cast<const uint32_t *>(from);
    out[0] = uint16_t(v), out[1] = uint16_t(v >> 16);
  } else {
    out[0] = *from;
  }
}
template <uint32_t E>
__device__ __forceinline__ void store_bf16s(uint16_t *to, const uint16_t (&v)[E]) {
  if constexpr (E == 4) {
    *reinterpret_cast<uint2 *>(to) = uint2{uint32_t(v[0]) | (uint32_t(v[1]) << 16), uint32_t(v[2]) | (uint32_t(v[3]) << 16)};
  } else if constexpr (E == 2) {
    *reinterpret_cast<uint32_t *>(to) = uint32_t(v[0]) | (uint32_t(v[1]) << 16);
  } else {
    *to = v[0];
  }
}
template <uint32_t E>
__device__ __forceinline__ void load_floats(const float *from, float (&out)[E]) {
  if constexpr (E == 4) {
    const float4 v = *reinterpret_cast<const float4 *>(from);
    out[0] = v.x, out[1] = v.y, out[2] = v.z, out[3] = v.w;
  } else if constexpr (E == 2) {
    const float2 v = *reinterpret_cast<const float2 *>(from);
    out[0] = v.x, out[1] = v.y;
  } else {
    out[0] = *from;
  }
}

// The same work with one wave per (row, head) task for head dimensions 64, 128
// and 256: each lane owns E = D / 64 consecutive dimensions, the sums and the
// row maxima travel by lane exchange, and nothing goes through LDS.  The sum of
// squares keeps the order of the kernel above: within each 32 dimensions the
// xor butterfly over dimension offsets 16, 8, 4, 2, 1 (offsets of E and more are
// lane exchanges, smaller ones pair a lane's own elements), then the groups in
// order; the results are the same bits.  Needs rotary_pairs / E to be a power
// of two, so that a pair's two dimensions sit rotary_pairs / E lanes apart.
// x of the lane `offset` lanes away (offset a power of two below 32) through the LDS
// crossbar's fixed patterns: no address register and no address arithmetic.
template <uint32_t OFFSET>
__device__ __forceinline__ float lane_xor(float x) {
  static_assert(OFFSET && OFFSET < 32 && !(OFFSET & (OFFSET - 1)), "a power of two below 32");
  return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(x), int((OFFSET << 10) | 0x1f)));
}
// bf16 (round to nearest even) of a finite value in one instruction; a NaN stays a NaN.
__device__ __forceinline__ uint16_t f32_to_bf16_hw(float f) {
  typedef float f32x2v __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
  const f32x2v pair = {f, 0.0f};
  return uint16_t(__builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2v)));
}

template <uint32_t FMT, uint32_t E>
__device__ __forceinline__ void store_row_wave(const uint16_t (&source)[E], bool value_tensor,
                                               const Slab &s, uint32_t slot, uint32_t lane,
                                               uint32_t D) {
  uint8_t *data = value_tensor ? s.values : s.keys;
  const uint32_t d0 = E * lane;
  const bool token_major = !value_tensor || FMT == KVX_FMT_INT4;
  if constexpr (FMT == KVX_FMT_BF16) {
    uint16_t *out = reinterpret_cast<uint16_t *>(data);
    if (token_major) {
      store_bf16s<E>(out + slot * D + d0, source);
    } else {
#pragma unroll
      for (uint32_t e = 0; e < E; ++e) out[(d0 + e) * kPage + slot] = source[e];
    }
    return;
  } else {
    float v[E];
    float m = 0.0f;
#pragma unroll
    for (uint32_t e = 0; e < E; ++e) {
      v[e] = bf16_to_f32(source[e]);
      m = fmaxf(m, fabsf(v[e]));
    }
    m = fmaxf(m, __shfl_xor(m, 32));
    m = fmaxf(m, lane_xor<16>(m));
    m = fmaxf(m, lane_xor<8>(m));
    m = fmaxf(m, lane_xor<4>(m));
    m = fmaxf(m, lane_xor<2>(m));
    m = fmaxf(m, lane_xor<1>(m));
    const float maximum = m;
    constexpr float qmax = FMT == KVX_FMT_INT4 ? 7.0f : FMT == KVX_FMT_INT8 ? 127.0f : 448.0f;
    const float scale = maximum == 0.0f ? 0.0f : __fdiv_rn(maximum, qmax);
    if (lane == 0) (value_tensor ? s.value_scales : s.key_scales)[slot] = scale;
    uint32_t code[E];
#pragma unroll
    for (uint32_t e = 0; e < E; ++e) {
      const float scaled = maximum == 0.0f ? 0.0f : __fdiv_rn(__fmul_rn(v[e], qmax), maximum);
      if constexpr (FMT == KVX_FMT_FP8E4M3) {
        code[e] = maximum == 0.0f ? 0u : uint32_t(f32_to_e4m3(scaled));
      } else {
        constexpr int limit = FMT == KVX_FMT_INT4 ? 7 : 127;
        int c = int(rintf(scaled));
        c = c < -limit ? -limit : c > limit ? limit : c;
        if (maximum == 0.0f) c = 0;
        code[e] = uint32_t(c) & (FMT == KVX_FMT_INT4 ? 0xfu : 0xffu);
      }
    }
    if constexpr (FMT == KVX_FMT_INT4) {
      // Even dimension in the low nibble; both tensors token-major.
      uint8_t *out = data + (slot * D + d0) / 2;
      if constexpr (E == 1) {
        const uint32_t partner = __shfl_xor(code[0], 1);
        if ((lane & 1) == 0) *out = uint8_t(code[0] | (partner << 4));
      } else if constexpr (E == 2) {
        *out = uint8_t(code[0] | (code[1] << 4));
      } else {
        *reinterpret_cast<uint16_t *>(out) =
            uint16_t(code[0] | (code[1] << 4) | (code[2] << 8) | (code[3] << 12));
      }
    } else if (token_major) {
      uint8_t *out = data + slot * D + d0;
      if constexpr (E == 4) {
        *reinterpret_cast<uint32_t *>(out) = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
      } else if constexpr (E == 2) {
        *reinterpret_cast<uint16_t *>(out) = uint16_t(code[0] | (code[1] << 8));
      } else {
        *out = uint8_t(code[0]);
      }
    } else {
#pragma unroll
      for (uint32_t e = 0; e < E; ++e) data[(d0 + e) * kPage + slot] = uint8_t(code[e]);
    }
  }
}

// grid (blocks of four head tasks, group of R rows, lane): a wave is one head task of R
// consecutive rows, and which one it is comes from the block's coordinates without a division
// or a walk over the lane records.  Head tasks 0 .. QH - 1 are the query heads, QH .. QH + H - 1
// the KV heads.  R = 4 for chunks: a row is 512 bytes of work behind four trips to memory, and
// with the loads of four rows in flight at once a wave's wait is shared by them (2048 rows of
// 28 head tasks: 37.5 us as one row per wave).
template <uint32_t FMT, uint32_t E, uint32_t R>
__global__ __launch_bounds__(256) void prepare_append_wave_kernel(PrepareArgs p) {
#pragma clang fp contract(off)
  constexpr uint32_t D = 64 * E;
  const AppendArgs &a = p.append;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t task = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t first_row = blockIdx.y * R, li = blockIdx.z;
  const AppendLane &l = a.lane[li];
  if (!append_contract(l, a)) return;
  const uint32_t H = a.kv_heads, QH = p.query_heads, G = QH / H;
  if (first_row >= l.tokens || task >= QH + H) return;
  const bool query = task < QH;
  const uint32_t head = query ? task : task - QH;
  const uint32_t d0 = E * lane;
  const uint32_t q_stride = p.query_gate ? 2 * D : D;
  const uint64_t packed_stride = uint64_t(QH) * q_stride + 2ull * H * D;
  const uint64_t head_offset = query ? uint64_t(head) * q_stride : uint64_t(QH) * q_stride + uint64_t(head) * D;
  // Everything the task reads is requested before anything waits: the rows, the
  // value rows (a query task reads its own row twice), the norm weights (any
  // readable address when there are none), the rotation of the lane's
  // dimensions (entry 0 for dimensions past the rotated ones) and the page entries.
  // Rows past the lane's last read the last again; nothing is stored for them.
  const bool norms = p.q_norm != nullptr;
  const uint32_t RP = p.rotary_pairs, pair_lanes = RP / E;
  const bool rotated = d0 < 2 * RP, is_first = d0 < RP;
  uint16_t raw[R][E], raw_value[R][E], weight_bf16[E];
  float weight_f32[E], cosine[R][E], sine[R][E];
  uint64_t entry[R];
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) {
    const uint32_t row = min(first_row + r, l.tokens - 1);
    const uint16_t *source = p.packed + (uint64_t(li) * p.rows + row) * packed_stride + head_offset;
    load_bf16s<E>(source + d0, raw[r]);
    load_bf16s<E>(source + (query ? 0u : H * D) + d0, raw_value[r]);
    const uint64_t rope_at = (uint64_t(li) * p.rows + row) * RP + (rotated ? (is_first ? d0 : d0 - RP) : 0u);
    load_floats<E>(p.rope_cos + rope_at, cosine[r]);
    load_floats<E>(p.rope_sin + rope_at, sine[r]);
    entry[r] = l.table[(l.committed + row) / kPage];
  }
  const void *weight = norms ? (query ? p.q_norm : p.k_norm) : static_cast<const void *>(p.packed);
  if (p.norm_f32) load_floats<E>(static_cast<const float *>(weight) + d0, weight_f32);
  else load_bf16s<E>(static_cast<const uint16_t *>(weight) + d0, weight_bf16);

  float scale[E];
#pragma unroll
  for (uint32_t e = 0; e < E; ++e)
    scale[e] = !norms ? 1.0f : p.norm_f32 ? weight_f32[e] : bf16_to_f32(weight_bf16[e]);
#pragma unroll
  for (uint32_t r = 0; r < R; ++r) {
    const uint32_t row = first_row + r;
    if (row >= l.tokens) break;
    float element[E];
    float inverse = 1.0f;
#pragma unroll
    for (uint32_t e = 0; e < E; ++e) element[e] = bf16_to_f32(raw[r][e]);
    if (norms) {
      float sum[E];
#pragma unroll
      for (uint32_t e = 0; e < E; ++e) sum[e] = element[e] * element[e];
      // dimension offsets 16 .. E: the partner sits offset / E lanes away
#pragma unroll
      for (uint32_t e = 0; e < E; ++e) {
        sum[e] = sum[e] + lane_xor<16 / E>(sum[e]);
        if constexpr (8 >= E) sum[e] = sum[e] + lane_xor<(8 >= E ? 8 / E : 1)>(sum[e]);
        if constexpr (4 >= E) sum[e] = sum[e] + lane_xor<(4 >= E ? 4 / E : 1)>(sum[e]);
        if constexpr (2 >= E) sum[e] = sum[e] + lane_xor<(2 >= E ? 2 / E : 1)>(sum[e]);
        if constexpr (1 >= E) sum[e] = sum[e] + lane_xor<1>(sum[e]);
      }
      // dimension offsets below E pair the lane's own elements
      float group_sum;
      if constexpr (E == 4) {
        const float a02 = sum[0] + sum[2], a13 = sum[1] + sum[3];
        group_sum = a02 + a13;
      } else if constexpr (E == 2) {
        group_sum = sum[0] + sum[1];
      } else {
        group_sum = sum[0];
      }
      // the groups of 32 dimensions in order; a group spans 32 / E lanes
      float total = 0.0f;
#pragma unroll
      for (uint32_t g = 0; g < D / 32; ++g)
        total = total + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(group_sum), int(g * (32 / E))));
      const float mean = total / float(D);
      inverse = 1.0f / sqrtf(mean + p.eps);
    }
    uint16_t prepared[E];
#pragma unroll
    for (uint32_t e = 0; e < E; ++e) {
      const float unit = element[e] * inverse;
      const uint16_t normal = f32_to_bf16_hw(unit * scale[e]);
      const float mine = bf16_to_f32(normal);
      const float other = __shfl_xor(mine, int(pair_lanes));
      const float mc = mine * cosine[r][e], os = other * sine[r][e];
      prepared[e] = rotated ? f32_to_bf16_hw(is_first ? mc - os : mc + os) : normal;
    }
    if (query) {
      // A group of one query head has no reciprocal that fits 32 bits (2^32): the head is
      // its own KV head then.
      const uint32_t kv_head = G == 1 ? head : __umulhi(head, p.group_magic);
      const uint32_t local_head = head - kv_head * G;
      store_bf16s<E>(p.queries + uint64_t(li) * H * p.row_stride * G * D +
                         ((uint64_t(kv_head) * p.row_stride + row) * G + local_head) * D + d0,
                     prepared);
      continue;
    }
    const uint32_t logical = l.committed + row;
    const Slab s = slab_of(FMT, H, D, a.kv, head, entry[r]);
    store_row_wave<FMT, E>(prepared, false, s, logical % kPage, lane, D);
    store_row_wave<FMT, E>(raw_value[r], true, s, logical % kPage, lane, D);
  }
}

// The same store for chunks of many tokens: one workgroup per (lane, logical page
// the chunk touches, head, tensor) stages the page's share of the chunk in LDS,
// so that the value rows, which the chunk holds dimension-major, are read as
// runs of consecutive tokens instead of one element per 2 x stride bytes, and so
// that dimension-major value pages are written as runs too.  Each wave then
// quantizes whole token rows; the arithmetic and the bytes are those of
// append_kernel.
constexpr uint32_t kAppendMaxD = 256;
template <uint32_t FMT>
__global__ __launch_bounds__(256) void append_page_kernel(const uint16_t *__restrict__ chunk_keys,
                                                          const uint16_t *__restrict__ chunk_values,
                                                          AppendArgs a) {
  __shared__ uint16_t tile[kPage][kAppendMaxD + 2];
  __shared__ uint8_t codes[kPage][kAppendMaxD + 4];
  const uint32_t group = blockIdx.x;
  uint32_t li = 0;
  for (uint32_t i = 1; i < a.n_lanes; ++i)
    if (group >= a.lane[i].group_base) li = i;
  const AppendLane &l = a.lane[li];
  if (!append_contract(l, a)) return;
  const uint32_t D = a.head_dim, H = a.kv_heads;
  const uint32_t first_page = l.committed / kPage;
  const uint32_t touched = (l.committed + l.tokens - 1) / kPage - first_page + 1;
  const uint32_t local = group - l.group_base;
  if (local >= touched * 2 * H) return;
  const uint32_t page = first_page + local / (2 * H);
  const bool value_tensor = local % (2 * H) >= H;
  const uint32_t head = local % H;
  // Chunk tokens [begin, begin + n) live in this page, from slot0 on.
  const uint32_t begin = max(l.committed, page * kPage) - l.committed;
  const uint32_t n = min(l.committed + l.tokens, (page + 1) * kPage) - l.committed - begin;
  const uint32_t slot0 = (l.committed + begin) % kPage;
  const Slab s = slab_of(FMT, H, D, a.kv, head, l.table[page]);
  const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
  if (!value_tensor) {
    const uint16_t *rows = chunk_keys + li * a.lane_stride + (uint64_t(head) * l.stride + begin) * D;
    for (uint32_t i = tid; i < n * D; i += 256) tile[i / D][i % D] = rows[i];
  } else {
    const uint16_t *columns = chunk_values + li * a.lane_stride + uint64_t(head) * D * l.stride + begin;
    for (uint32_t i = tid; i < D * kPage; i += 256) {
      const uint32_t d = i / kPage, t = i % kPage;
      if (t < n) tile[t][d] = columns[uint64_t(d) * l.stride + t];
    }
  }
  __syncthreads();
  // Element index inside the head's slab: keys token-major, values
  // dimension-major (packed int4: both token-major).
  const bool dimension_major = value_tensor && FMT != KVX_FMT_INT4;
  uint8_t *data = value_tensor ? s.values : s.keys;
  if constexpr (FMT == KVX_FMT_BF16) {
    uint16_t *out = reinterpret_cast<uint16_t *>(data);
    if (!dimension_major) {
      for (uint32_t i = tid; i < n * D; i += 256) out[(slot0 + i / D) * D + i % D] = tile[i / D][i % D];
    } else {
      for (uint32_t i = tid; i < D * kPage; i += 256) {
        const uint32_t d = i / kPage, t = i % kPage;
        if (t < n) out[d * kPage + slot0 + t] = tile[t][d];
      }
    }
    return;
  } else {
    constexpr float qmax = FMT == KVX_FMT_INT4 ? 7.0f : FMT == KVX_FMT_INT8 ? 127.0f : 448.0f;
    for (uint32_t t = wave; t < n; t += 4) {
      const uint32_t slot = slot0 + t;
      float v[kAppendMaxD / 64], maximum = 0.0f;
#pragma unroll
      for (uint32_t k = 0; k < kAppendMaxD / 64; ++k) {
        const uint32_t d = lane + 64 * k;
        v[k] = d < D ? bf16_to_f32(tile[t][d]) : 0.0f;
        maximum = fmaxf(maximum, fabsf(v[k]));
      }
      for (int offset = 32; offset; offset >>= 1) maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
      const float scale = maximum == 0.0f ? 0.0f : __fdiv_rn(maximum, qmax);
      if (lane == 0) (value_tensor ? s.value_scales : s.key_scales)[slot] = scale;
#pragma unroll
      for (uint32_t k = 0; k < kAppendMaxD / 64; ++k) {
        const uint32_t d = lane + 64 * k;
        const float scaled = maximum == 0.0f ? 0.0f : __fdiv_rn(__fmul_rn(v[k], qmax), maximum);
        uint32_t byte;
        if constexpr (FMT == KVX_FMT_FP8E4M3) {
          byte = maximum == 0.0f ? 0u : f32_to_e4m3(scaled);
        } else {
          constexpr int limit = FMT == KVX_FMT_INT4 ? 7 : 127;
          int code = int(rintf(scaled));
          code = code < -limit ? -limit : code > limit ? limit : code;
          if (maximum == 0.0f) code = 0;
          byte = uint32_t(code) & (FMT == KVX_FMT_INT4 ? 0xfu : 0xffu);
        }
        if constexpr (FMT == KVX_FMT_INT4) {
          // Even dimension in the low nibble; the even lane writes the byte.
          const uint32_t partner = __shfl_xor(byte, 1);
          if (d < D && (d & 1) == 0) data[(slot * D + d) >> 1] = uint8_t(byte | (partner << 4));
        } else if (d < D) {
          if (dimension_major) codes[t][d] = uint8_t(byte);
          else data[slot * D + d] = uint8_t(byte);
        }
      }
    }
    if (dimension_major) {
      __syncthreads();
      for (uint32_t i = tid; i < D * kPage; i += 256) {
        const uint32_t d = i / kPage, t = i % kPage;
        if (t < n) data[d * kPage + slot0 + t] = codes[t][d];
      }
    }
  }
}

// ===================================================== generic attention ====
// One tile = row_capacity query rows x `group` query heads of one KV head
// (M fused rows) over the pages of one split.
struct AttendLane {
  const uint64_t *table;
  uint32_t committed, entries, split_count, active_rows;
  uint64_t row_base;   // first fused row of this lane's slots in the workspace
  uint64_t q_offset;   // element offset of the lane's queries / output
  uint32_t mask_offset;
  float score_scale;
};
struct AttendArgs {
  AttendLane lane[kLanes];
  uint32_t n_lanes;
  uint32_t kv_heads, group, head_dim;
  uint32_t row_capacity;
  uint32_t row_stride;  // rows between KV heads in queries / output
  kvx_kv_layer kv;
  // The merge's second output (see Epilogue), from the launch's first lane on.
  uint16_t *hidden;
  const uint16_t *packed_qkv;
};
struct PrefillArgs {
  const uint64_t *table;
  uint32_t committed, rows, stride, entries, splits;
  uint32_t kv_heads, group, head_dim;
  float score_scale;
  kvx_kv_layer kv;
};

__device__ inline bool attend_contract(const AttendLane &l, const AttendArgs &a) {
  return l.active_rows > 0 && l.active_rows <= a.row_capacity &&
         l.entries >= (uint64_t(l.committed) + l.active_rows + kPage - 1) / kPage &&
         a.kv.extent_pages > 0 &&
         uint64_t(l.committed) + l.active_rows <= uint64_t(KVX_MAX_PHYSICAL_TOKENS) &&
         l.split_count > 0 &&
         l.split_count <= (a.row_capacity == 1 ? KVX_DECODE_MAX_SPLITS : KVX_VERIFY_MAX_SPLITS);
}
__device__ inline bool prefill_contract(const PrefillArgs &p) {
  return p.rows > 0 && p.rows <= KVX_PREFILL_TOKEN_BUDGET && p.stride >= p.rows &&
         p.stride <= KVX_PREFILL_TOKEN_BUDGET && p.stride % kPage == 0 &&
         p.entries >= (uint64_t(p.committed) + p.rows + kPage - 1) / kPage &&
         p.kv.extent_pages > 0 && p.splits > 0 && p.splits <= KVX_PREFILL_MAX_SPLITS &&
         uint64_t(p.committed) + p.rows <= uint64_t(KVX_MAX_PHYSICAL_TOKENS);
}

constexpr uint32_t kTileThreads = 256;
constexpr uint32_t kMaxD = 256;
constexpr uint32_t kKeyPitch = kMaxD + 2;  // bf16 elements; odd word pitch avoids bank conflicts

// The page loop of one tile over one split (reference:
// common/paged_attention_tile.h:85-349; fp8: paged_attention_fp8_tile.h:34-265).
// MAXM bounds the fused rows a thread accumulates in registers.
// K and V codes are staged in LDS as bf16, which holds every int4 / int8 /
// e4m3 / bf16 code exactly.
template <uint32_t FMT, uint32_t MAXM>
__device__ __forceinline__ void attention_tile(const uint16_t *__restrict__ tile_queries,
                               const uint64_t *__restrict__ table, kvx_kv_layer kv,
                               uint32_t H, uint32_t G, uint32_t D, uint32_t row_capacity,
                               uint32_t head, uint32_t committed, uint32_t active_rows,
                               uint32_t splits, uint32_t split, float *__restrict__ partials,
                               float *__restrict__ statistics, uint64_t slot_row,
                               const uint32_t *__restrict__ row_masks, float score_scale_in) {
  __shared__ uint16_t k_lds[kPage * kKeyPitch];
  __shared__ uint16_t v_lds[kPage * kMaxD];
  __shared__ float w_lds[MAXM * (kPage + 1)];
  __shared__ float rescale_lds[MAXM];
  __shared__ uint32_t admit_lds[MAXM];

  const uint32_t tid = threadIdx.x;
  const uint32_t M = row_capacity * G;
  const uint32_t visible = committed + active_rows;
  const uint32_t pages = (visible + kPage - 1) / kPage;
  const uint32_t per = (pages + splits - 1) / splits;
  const uint32_t begin = split * per;
  if (begin >= pages) return;
  const uint32_t end = min(pages, begin + per);
  constexpr bool kFp8 = FMT == KVX_FMT_FP8E4M3;
  constexpr bool kQuant = FMT != KVX_FMT_BF16;
  const float score_scale = default_score_scale(D, score_scale_in);

  float acc[MAXM];
#pragma unroll
  for (uint32_t r = 0; r < MAXM; ++r) acc[r] = 0.0f;
  // Thread r (< M) owns the running statistics of fused row r.
  float row_max = -INFINITY, row_sum = 0.0f;
  const uint32_t my_query_row = tid / G;
  const bool owns_row = tid < M && my_query_row < active_rows;
  uint32_t my_limit = 0, my_mask = 0;
  if (owns_row) {
    const uint32_t causal_end = committed + min(my_query_row, active_rows - 1) + 1;
    my_limit = min(visible, causal_end);
    my_mask = row_masks ? row_masks[my_query_row] : 0u;
  }

  for (uint32_t page = begin; page < end; ++page) {
    const Slab s = slab_of(FMT, H, D, kv, head, table[page]);
    const uint32_t token_start = page * kPage;
    __syncthreads();  // the previous page's PV is done with the staging
    for (uint32_t e = tid; e < kPage * D; e += kTileThreads) {
      const uint32_t j = e / D, d = e % D;
      k_lds[j * kKeyPitch + d] = f32_to_bf16(load_key_code<FMT>(s.keys, D, j, d));
      v_lds[j * kMaxD + d] = f32_to_bf16(load_value_code<FMT>(s.values, D, j, d));
    }
    if (tid < M) {
      uint32_t admit = 0;
      if (owns_row) {
        for (uint32_t j = 0; j < kPage; ++j) {
          const uint32_t t = token_start + j;
          const bool in = !row_masks ? t < my_limit
                                     : (t < committed) ||
                                           (t < visible && ((my_mask >> (t - committed)) & 1u));
          admit |= uint32_t(in) << j;
        }
      }
      admit_lds[tid] = admit;
    }
    __syncthreads();

    // Scores: thread (token j, row group) walks the fused rows r = rg, rg+8, ...
    {
      const uint32_t j = tid & 31, rg = tid >> 5;
      const float key_scale = kQuant ? s.key_scales[j] : 1.0f;
      for (uint32_t r = rg; r < M; r += 8) {
        float score = -INFINITY;
        if ((admit_lds[r] >> j) & 1u) {
          const uint16_t *q = tile_queries + uint64_t(r) * D;
          float dot = 0.0f;
          for (uint32_t d = 0; d < D; ++d) {
            float qv = bf16_to_f32(q[d]);
            if constexpr (kFp8) qv = round_f16(qv);  // the fp8 tile stages queries as fp16
            dot = __fadd_rn(dot, __fmul_rn(qv, bf16_to_f32(k_lds[j * kKeyPitch + d])));
          }
          if constexpr (kQuant) dot = __fmul_rn(dot, key_scale);
          score = __fmul_rn(dot, score_scale);
        }
        w_lds[r * (kPage + 1) + j] = score;
      }
    }
    __syncthreads();

    // Online softmax of one page, one thread per fused row, in the reference's
    // order: four groups of eight tokens summed, then paired.
    if (tid < M) {
      float rescale = 1.0f;
      if (owns_row) {
        const uint32_t admit = admit_lds[tid];
        float *w = w_lds + tid * (kPage + 1);
        float local_max = -INFINITY;
        for (uint32_t j = 0; j < kPage; ++j) local_max = fmaxf(local_max, w[j]);
        const float next_max = fmaxf(row_max, local_max);
        float lane_sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t j = 0; j < kPage; ++j) {
          const bool in = (admit >> j) & 1u;
          const float p = in ? expf(__fsub_rn(w[j], next_max)) : 0.0f;
          lane_sum[j >> 3] = __fadd_rn(lane_sum[j >> 3], p);
          float weight = 0.0f;
          if (in && w[j] > -INFINITY)
            weight = kQuant ? __fmul_rn(p, s.value_scales[j]) : p;
          w[j] = kFp8 ? round_f16(weight) : round_bf16(weight);
        }
        const float local_sum =
            __fadd_rn(__fadd_rn(lane_sum[0], lane_sum[1]), __fadd_rn(lane_sum[2], lane_sum[3]));
        rescale = (next_max == -INFINITY || next_max == row_max)
                      ? 1.0f
                      : expf(__fsub_rn(row_max, next_max));
        row_sum = __fadd_rn(__fmul_rn(row_sum, rescale), local_sum);
        row_max = next_max;
      }
      rescale_lds[tid] = rescale;
    }
    __syncthreads();

    // PV: thread d accumulates dimension d of every fused row.
    if (tid < D) {
#pragma unroll
      for (uint32_t r = 0; r < MAXM; ++r) {
        if (r < M) {
          const uint32_t admit = admit_lds[r];
          if (r / G < active_rows) {
            float sum = 0.0f;
            for (uint32_t j = 0; j < kPage; ++j)
              if ((admit >> j) & 1u)
                sum = __fadd_rn(sum, __fmul_rn(w_lds[r * (kPage + 1) + j],
                                               bf16_to_f32(v_lds[j * kMaxD + tid])));
            const float scale = rescale_lds[r];
            acc[r] = __fadd_rn(scale != 1.0f ? __fmul_rn(acc[r], scale) : acc[r], sum);
          }
        }
      }
    }
  }

  if (tid < D) {
#pragma unroll
    for (uint32_t r = 0; r < MAXM; ++r)
      if (r < M && r / G < active_rows) partials[(slot_row + r) * D + tid] = acc[r];
  }
  if (owns_row) {
    statistics[(slot_row + tid) * 2] = row_max;
    statistics[(slot_row + tid) * 2 + 1] = row_sum;
  }
}

template <uint32_t FMT, uint32_t MAXM>
__global__ __launch_bounds__(kTileThreads) void attend_split_kernel(
    const uint16_t *__restrict__ queries, float *__restrict__ partials,
    float *__restrict__ statistics, const uint32_t *__restrict__ row_masks, AttendArgs a) {
  const uint32_t split = blockIdx.x, head = blockIdx.y, li = blockIdx.z;
  const AttendLane &l = a.lane[li];
  if (!attend_contract(l, a) || split >= l.split_count) return;
  const uint32_t M = a.row_capacity * a.group;
  const uint16_t *tile_q =
      queries + l.q_offset + uint64_t(head) * a.row_stride * a.group * a.head_dim;
  const uint64_t slot_row = l.row_base + (uint64_t(head) * l.split_count + split) * M;
  attention_tile<FMT, MAXM>(tile_q, l.table, a.kv, a.kv_heads, a.group, a.head_dim,
                            a.row_capacity, head, l.committed, l.active_rows, l.split_count,
                            split, partials, statistics, slot_row,
                            row_masks ? row_masks + l.mask_offset : nullptr, l.score_scale);
}

// Prefill: KV heads, query tiles of eight rows, history splits (reference:
// prefill/paged_attention.metal:7-67); slots are [tile][head][split].
template <uint32_t FMT, uint32_t MAXM>
__global__ __launch_bounds__(kTileThreads) void prefill_split_kernel(
    const uint16_t *__restrict__ queries, float *__restrict__ partials,
    float *__restrict__ statistics, PrefillArgs p) {
  const uint32_t split = blockIdx.x, head = blockIdx.y, tile = blockIdx.z;
  const uint32_t tile_start = tile * KVX_PREFILL_TILE_ROWS;
  if (!prefill_contract(p) || tile_start >= p.rows) return;
  const uint32_t active = min(KVX_PREFILL_TILE_ROWS, p.rows - tile_start);
  const uint32_t M = KVX_PREFILL_TILE_ROWS * p.group;
  const uint64_t tile_offset = (uint64_t(head) * p.stride + tile_start) * p.group * p.head_dim;
  const uint64_t slot_row = ((uint64_t(tile) * p.kv_heads + head) * p.splits + split) * M;
  attention_tile<FMT, MAXM>(queries + tile_offset, p.table, p.kv, p.kv_heads, p.group, p.head_dim,
                            KVX_PREFILL_TILE_ROWS, head, p.committed + tile_start, active, p.splits,
                            split, partials, statistics, slot_row, nullptr, p.score_scale);
}

// ---- head dimensions 64 and 128 on the matrix cores -------------------------
// The same tile for the reference's narrower heads (its _hd128, _hd64, _k8q5d64 and
// _k8q4d128 layouts, runtime/ops/PagedAttention.cpp:66-115), every format: the workgroup
// stages a page's key and value codes in LDS as bf16 (fp16 on fp8 pages: the fp8 tile
// multiplies fp16), which holds every code exactly, and each of its four waves multiplies
// the blocks of 16 fused rows it owns (blocks w and w + 4) out of that copy with
// v_mfma_f32_16x16x32: q.k as keys (16 tokens x 32 dims) x queries, p.v as values
// (16 dims x 32 tokens) x probabilities.  A lane of q.k's result holds tokens 4g + j and
// 16 + 4g + j of its row; the value operand is read from the staged copy in that token
// order, so the rounded probabilities are the B operand of p.v as they stand.  Partial rows
// and statistics go where attention_tile puts them, for the same reduce kernels.
typedef float small_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t small_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t small_u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 small_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 small_bf16x2 __attribute__((ext_vector_type(2)));
typedef float small_f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 small_f16x8 __attribute__((ext_vector_type(8)));

template <bool F16>
__device__ __forceinline__ small_f32x4 small_mfma(small_u32x4 a, small_u32x4 b, small_f32x4 c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(small_f16x8, a),
                                                  __builtin_bit_cast(small_f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(small_bf16x8, a),
                                                   __builtin_bit_cast(small_bf16x8, b), c, 0, 0, 0);
}
// The 16 bits of x in the tile's operand format (x is exact in it, or is rounded to it).
template <bool F16>
__device__ __forceinline__ uint16_t operand_bits(float x) {
  if constexpr (F16) return __builtin_bit_cast(uint16_t, _Float16(x));
  else return f32_to_bf16(x);
}

// exp of a difference of scores: expf, as the oracle takes it.  With the same exponentials the
// rounded weights are the oracle's, and most rows of these tiles come out as its bits; one
// v_exp_f32 of the difference in units of log 2 (the head-dimension-256 kernels' form, up to
// 3.5e-6 from expf) was 6 to 16 per cent faster, but turned enough roundings that a row of 64
// elements could land 2.2e-3 from the oracle with seven of them rounded the other way.
__device__ __forceinline__ float small_exp(float difference) { return expf(difference); }

constexpr uint32_t kSmallBlocks = 2;  // at most: blocks of 16 fused rows per wave, 128 rows per tile

// Sixteen bytes of a page as they lie (32 int4 codes, 16 int8 or e4m3 codes, 8 bf16 values)
// to that many 16-bit operand elements, in order: int4 and int8 codes as the bf16 numbers
// they are (a small integer's float, cut to its upper half, is exact), e4m3 as fp16 (one
// v_cvt_scalef32_pk_f16_fp8 per pair, exact), bf16 as it is.
template <uint32_t FMT>
struct SmallChunk {
  static constexpr uint32_t kElements = FMT == KVX_FMT_INT4 ? 32 : FMT == KVX_FMT_BF16 ? 8 : 16;
  uint32_t pair[kElements / 2];  // elements 2i (low half) and 2i + 1
  __device__ __forceinline__ explicit SmallChunk(small_u32x4 raw) {
    if constexpr (FMT == KVX_FMT_BF16) {
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) pair[i] = raw[i];
    } else if constexpr (FMT == KVX_FMT_FP8E4M3) {
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        pair[2 * i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[i], 1.0f, false));
        pair[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[i], 1.0f, true));
      }
    } else if constexpr (FMT == KVX_FMT_INT8) {
#pragma unroll
      for (uint32_t i = 0; i < 8; ++i) {
        const int lo = __builtin_amdgcn_sbfe(int(raw[i / 2]), 16 * (i & 1), 8);
        const int hi = __builtin_amdgcn_sbfe(int(raw[i / 2]), 16 * (i & 1) + 8, 8);
        pair[i] = (__float_as_uint(float(lo)) >> 16) | (__float_as_uint(float(hi)) & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (uint32_t i = 0; i < 16; ++i) {
        const int lo = __builtin_amdgcn_sbfe(int(raw[i / 4]), 8 * (i & 3), 4);
        const int hi = __builtin_amdgcn_sbfe(int(raw[i / 4]), 8 * (i & 3) + 4, 4);
        pair[i] = (__float_as_uint(float(lo)) >> 16) | (__float_as_uint(float(hi)) & 0xffff0000u);
      }
    }
  }
};

// Eight key elements of one token as they lie in the page (16 bytes of bf16, 8 of int8 or
// e4m3, 4 of int4), which is a lane's share of q.k's key operand: a wave whose tile is its
// own reads its keys straight from the page and keeps no staged copy of them.
template <uint32_t FMT>
struct SmallKeyPiece {
  static constexpr uint32_t kWords = FMT == KVX_FMT_BF16 ? 4 : FMT == KVX_FMT_INT4 ? 1 : 2;
  uint32_t raw[kWords];
  __device__ __forceinline__ void load(const uint8_t *from) {
    if constexpr (kWords == 4) {
      const small_u32x4 v = *reinterpret_cast<const small_u32x4 *>(from);
      raw[0] = v[0]; raw[1] = v[1]; raw[2] = v[2]; raw[3] = v[3];
    } else if constexpr (kWords == 2) {
      const small_u32x2 v = *reinterpret_cast<const small_u32x2 *>(from);
      raw[0] = v[0]; raw[1] = v[1];
    } else {
      raw[0] = *reinterpret_cast<const uint32_t *>(from);
    }
  }
  // The eight elements as 16-bit operand elements, as SmallChunk makes them.
  __device__ __forceinline__ small_u32x4 operand() const {
    small_u32x4 out;
    if constexpr (FMT == KVX_FMT_BF16) {
      out = small_u32x4{raw[0], raw[1], raw[2], raw[3]};
    } else if constexpr (FMT == KVX_FMT_FP8E4M3) {
#pragma unroll
      for (uint32_t i = 0; i < 2; ++i) {
        out[2 * i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[i], 1.0f, false));
        out[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[i], 1.0f, true));
      }
    } else {
      constexpr uint32_t kBits = FMT == KVX_FMT_INT8 ? 8 : 4;
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t word = raw[(2 * i * kBits) / 32];
        const int lo = __builtin_amdgcn_sbfe(int(word), (2 * i * kBits) % 32, kBits);
        const int hi = __builtin_amdgcn_sbfe(int(word), (2 * i * kBits) % 32 + kBits, kBits);
        out[i] = (__float_as_uint(float(lo)) >> 16) | (__float_as_uint(float(hi)) & 0xffff0000u);
      }
    }
    return out;
  }
};

// PRIVATE = 0: the four waves of the workgroup share the tile (row blocks by wave, the page
// staged by all 256 threads, a barrier on either side of the staging).  PRIVATE = n: the
// workgroup is n independent waves, each with a tile of at most 16 fused rows (one-row decode,
// short chains of small groups) and a staged copy of its own: a wave's LDS operations complete
// in the order it issues them, so it needs no barrier, and every wave of a CU multiplies
// instead of one in four.  Such a wave stages the values only: a lane's share of the key
// operand is eight consecutive elements of one token, which it reads from the page itself,
// and half the staged bytes leave room for twice the waves.
// Several consecutive prefill tiles of one (KV head, split) on one staged page: tile k of the
// group lies `row_capacity` rows further on in the chunk (its history, its queries) and
// `slot_stride` rows further on in the workspace.  The caller sees to it that every tile of a
// group has the same pages under the same split (a history that ends on a page boundary and
// groups that do not straddle one).  The blocks of 16 fused rows of all tiles are dealt to the
// four waves in turn.  {1, 4 * BLOCKS, .., 0} is a single tile.
struct SmallGroup {
  uint32_t tiles;        // tiles of the group that have rows
  uint32_t blocks;       // blocks of 16 fused rows to a tile
  uint32_t rows_left;    // chunk rows from the group's first tile on
  uint64_t slot_stride;  // workspace rows from a tile's slot to the next tile's
};

template <uint32_t FMT, uint32_t D, uint32_t BLOCKS, uint32_t PRIVATE = 0>
__device__ __forceinline__ void attention_tile_small(const uint16_t *__restrict__ tile_queries,
                                     const uint64_t *__restrict__ table, kvx_kv_layer kv,
                                     uint32_t H, uint32_t G, uint32_t row_capacity, uint32_t head,
                                     uint32_t committed, uint32_t active_rows, uint32_t splits,
                                     uint32_t split, float *__restrict__ partials,
                                     float *__restrict__ statistics, uint64_t slot_row,
                                     const uint32_t *__restrict__ row_masks, float score_scale_in,
                                     SmallGroup group = SmallGroup{1u, 4u * BLOCKS, 0u, 0u}) {
  constexpr bool kFp8 = FMT == KVX_FMT_FP8E4M3;
  constexpr bool kQuant = FMT != KVX_FMT_BF16;
  constexpr uint32_t kKeyRow = D + 8;        // staged halves per token: 16 bytes past a power of two
  constexpr uint32_t kValueRow = kPage + 4;  // staged halves per dimension
  // Where dimension d's staged values begin.  int4 values lie token-major in the page, and a
  // thread that holds 32 dimensions of a token writes them two bytes at a time, the threads of
  // a wave 32 dimensions apart: a multiple of 32 rows is a multiple of 32 banks whatever the
  // row length, so every group of 32 rows starts 16 halves (8 banks) further on.
  constexpr uint32_t kValueSkew = FMT == KVX_FMT_INT4 ? 16u : 0u;
  const auto value_row = [](uint32_t d) { return d * kValueRow + (d >> 5) * kValueSkew; };
  constexpr uint32_t kSteps = D / 32, kTiles = D / 16;
  static_assert(!PRIVATE || BLOCKS == 1, "a private tile is one block of 16 fused rows");
  constexpr uint32_t kCopies = PRIVATE ? PRIVATE : 1, kThreads = PRIVATE ? 64u : kTileThreads;
  constexpr bool kDirectKeys = PRIVATE != 0;
  __shared__ __align__(16) uint16_t k_lds_all[kCopies][kDirectKeys ? 8 : kPage * kKeyRow];
  __shared__ __align__(16) uint16_t v_lds_all[kCopies][D * kValueRow + (D / 32) * 16];
  __shared__ float key_scale_all[kCopies][kPage], value_scale_all[kCopies][kPage];
  const uint32_t copy = PRIVATE ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0u;
  uint16_t *const k_lds = k_lds_all[copy], *const v_lds = v_lds_all[copy];
  float *const key_scale_lds = key_scale_all[copy], *const value_scale_lds = value_scale_all[copy];
  const auto tile_barrier = [] {
    if constexpr (PRIVATE) __builtin_amdgcn_wave_barrier();
    else __syncthreads();
  };

  const uint32_t lane = threadIdx.x & 63u, t = lane & 15u, g = lane >> 4;
  const uint32_t tid = PRIVATE ? lane : threadIdx.x, wave = PRIVATE ? 0u : threadIdx.x >> 6;
  const uint32_t M = row_capacity * G;
  const uint32_t visible = committed + active_rows;
  const uint32_t pages = (visible + kPage - 1) / kPage;
  const uint32_t per = (pages + splits - 1) / splits;
  const uint32_t begin = split * per;
  if (begin >= pages) return;
  const uint32_t end = min(pages, begin + per);
  const float score_scale = default_score_scale(D, score_scale_in);
  const bool tree = row_masks != nullptr;

  small_u32x4 q[BLOCKS][kSteps];
  small_f32x4 acc[BLOCKS][kTiles];
  float row_max[BLOCKS], row_sum[BLOCKS];
  uint32_t limit[BLOCKS], mask[BLOCKS], fused[BLOCKS];
  uint64_t out_row[BLOCKS];
  bool live[BLOCKS], used[BLOCKS];
#pragma unroll
  for (uint32_t b = 0; b < BLOCKS; ++b) {
    // the wave's b-th block: block `block` of tile `k` of the group
    const uint32_t dealt = wave + 4 * b, k = dealt / group.blocks, block = dealt % group.blocks;
    const uint32_t tile_committed = committed + k * row_capacity;
    const uint32_t tile_rows =
        group.tiles == 1 ? active_rows
                         : min(row_capacity, group.rows_left - min(group.rows_left, k * row_capacity));
    fused[b] = 16 * block + t;
    used[b] = k < group.tiles && 16 * block < M && tile_rows > 0;  // the same in every lane of the wave
    const uint32_t query_row = fused[b] / G;
    live[b] = used[b] && fused[b] < M && query_row < tile_rows;
    limit[b] = live[b] ? min(tile_committed + tile_rows, tile_committed + min(query_row, tile_rows - 1) + 1) : 0u;
    mask[b] = (live[b] && tree) ? row_masks[query_row] : 0u;
    out_row[b] = slot_row + k * group.slot_stride + fused[b];
    const uint16_t *block_queries = tile_queries + uint64_t(k) * row_capacity * G * D;
    row_max[b] = -INFINITY;
    row_sum[b] = 0.0f;
#pragma unroll
    for (uint32_t i = 0; i < kTiles; ++i) acc[b][i] = small_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t kb = 0; kb < kSteps; ++kb) {
      small_u32x4 raw = {0u, 0u, 0u, 0u};
      if (live[b])
        raw = *reinterpret_cast<const small_u32x4 *>(block_queries + uint64_t(fused[b]) * D + 32 * kb + 8 * g);
      if constexpr (kFp8) {  // the fp8 tile stages its queries as fp16
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i)
          raw[i] = uint32_t(operand_bits<true>(bf16_to_f32(uint16_t(raw[i])))) |
                   uint32_t(operand_bits<true>(bf16_to_f32(uint16_t(raw[i] >> 16)))) << 16;
      }
      q[b][kb] = raw;
    }
  }

  // A page's keys and values come in as whole 16-byte pieces, a piece (or two) per thread,
  // one page ahead of the page being multiplied, and go to the staged copy as operand
  // elements: keys [token][dim], values [dim][token].
  using Chunk = SmallChunk<FMT>;
  constexpr uint32_t kPieces = kPage * D / Chunk::kElements;         // per tensor
  constexpr uint32_t kPerThread = (kPieces + kThreads - 1) / kThreads;
  small_u32x4 raw_keys[kDirectKeys ? 1 : kPerThread], raw_values[kPerThread];
  SmallKeyPiece<FMT> key_piece[2][kDirectKeys ? kSteps : 1];  // tokens 16 tb + t, dims 32 kb + 8 g ..
  constexpr uint32_t kKeyRowBytes = D * 16 / Chunk::kElements;
  float raw_scale = 1.0f;
  const auto fetch_keys = [&](uint64_t entry) {
    const Slab s = slab_of(FMT, H, D, kv, head, entry);
#pragma unroll
    for (uint32_t tb = 0; tb < 2; ++tb)
#pragma unroll
      for (uint32_t kb = 0; kb < kSteps; ++kb)
        key_piece[tb][kb].load(s.keys + (16 * tb + t) * kKeyRowBytes + (32 * kb + 8 * g) * 16 / Chunk::kElements);
  };
  const auto fetch = [&](uint64_t entry) {
    const Slab s = slab_of(FMT, H, D, kv, head, entry);
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; ++i) {
      const uint32_t piece = tid + i * kThreads;
      if (kPieces % kThreads == 0 || piece < kPieces) {
        if constexpr (!kDirectKeys) raw_keys[i] = *reinterpret_cast<const small_u32x4 *>(s.keys + 16 * piece);
        raw_values[i] = *reinterpret_cast<const small_u32x4 *>(s.values + 16 * piece);
      }
    }
    if constexpr (kQuant)
      if (tid < 2 * kPage) raw_scale = tid < kPage ? s.key_scales[tid] : s.value_scales[tid - kPage];
  };
  const auto stage = [&]() {
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; ++i) {
      const uint32_t piece = tid + i * kThreads;
      if (kPieces % kThreads != 0 && piece >= kPieces) continue;
      const uint32_t first = piece * Chunk::kElements;
      if constexpr (!kDirectKeys) {  // keys are token-major in every format
        const Chunk c(raw_keys[i]);
        uint32_t *to = reinterpret_cast<uint32_t *>(&k_lds[(first / D) * kKeyRow + first % D]);
#pragma unroll
        for (uint32_t w = 0; w < Chunk::kElements / 2; w += 4)
          *reinterpret_cast<small_u32x4 *>(to + w) =
              small_u32x4{c.pair[w], c.pair[w + 1], c.pair[w + 2], c.pair[w + 3]};
      }
      const Chunk c(raw_values[i]);
      if constexpr (FMT == KVX_FMT_INT4) {  // token-major values: one element per staged row
        const uint32_t token = first / D, d0 = first % D;
#pragma unroll
        for (uint32_t w = 0; w < Chunk::kElements / 2; ++w) {
          v_lds[value_row(d0 + 2 * w) + token] = uint16_t(c.pair[w]);
          v_lds[value_row(d0 + 2 * w + 1) + token] = uint16_t(c.pair[w] >> 16);
        }
      } else {  // dimension-major values: a run of tokens of one dimension
        uint32_t *to = reinterpret_cast<uint32_t *>(&v_lds[value_row(first / kPage) + first % kPage]);
#pragma unroll
        for (uint32_t w = 0; w < Chunk::kElements / 2; w += 2)
          *reinterpret_cast<small_u32x2 *>(to + w) = small_u32x2{c.pair[w], c.pair[w + 1]};
      }
    }
    if (tid < kPage) key_scale_lds[tid] = raw_scale;
    else if (tid < 2 * kPage) value_scale_lds[tid - kPage] = raw_scale;
  };

  // A page's table entry is read one page before its bytes are asked for, so that a fetch
  // is one trip to memory and not two in a row.
  uint64_t entry_ahead = table[min(begin + 1, end - 1)];
  fetch(table[begin]);
  if constexpr (kDirectKeys) fetch_keys(table[begin]);
  for (uint32_t page = begin; page < end; ++page) {
    const uint32_t token_start = page * kPage;
    tile_barrier();  // the previous page's products are done with the staged copy
    stage();
    const uint64_t entry = entry_ahead;
    if (page + 1 < end) {
      entry_ahead = table[min(page + 2, end - 1)];
      fetch(entry);
    }
    tile_barrier();

#pragma unroll
    for (uint32_t b = 0; b < BLOCKS; ++b) {
      if (!used[b]) continue;
      small_f32x4 scores[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
      for (uint32_t tb = 0; tb < 2; ++tb)
#pragma unroll
        for (uint32_t kb = 0; kb < kSteps; ++kb) {
          small_u32x4 keys;
          if constexpr (kDirectKeys) keys = key_piece[tb][kb].operand();
          else keys = *reinterpret_cast<const small_u32x4 *>(&k_lds[(16 * tb + t) * kKeyRow + 32 * kb + 8 * g]);
          scores[tb] = small_mfma<kFp8>(keys, q[b][kb], scores[tb]);
        }
      // the next page's keys, now that this page's are multiplied (a private tile is one block)
      if constexpr (kDirectKeys)
        if (page + 1 < end) fetch_keys(entry);
      // page softmax of the lane's eight tokens of its row (reference:
      // common/paged_attention_tile.h:129-188).  A page that lies wholly in the committed
      // history is seen by every row, so its tokens skip the tests (rows past the live ones
      // then hold numbers instead of nothing, and are not written either way).
      float rescale;
      small_u32x4 weights;
      const auto page_softmax = [&](auto whole_page) {
        constexpr bool kWhole = decltype(whole_page)::value;
        float score[8], local_max = -INFINITY;
        bool in[8];
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) {
          const uint32_t token = 16 * (i >> 2) + 4 * g + (i & 3), at = token_start + token;
          in[i] = kWhole || (live[b] && (tree ? (at < committed || (at < visible && ((mask[b] >> ((at - committed) & 31u)) & 1u)))
                                              : at < limit[b]));
          float v = scores[i >> 2][i & 3];
          if constexpr (kQuant) v = __fmul_rn(v, key_scale_lds[token]);
          v = __fmul_rn(v, score_scale);
          score[i] = in[i] ? v : -INFINITY;
          local_max = fmaxf(local_max, score[i]);
        }
        local_max = fmaxf(local_max, __shfl_xor(local_max, 16));
        local_max = fmaxf(local_max, __shfl_xor(local_max, 32));
        const float next_max = fmaxf(row_max[b], local_max);
        rescale = (next_max == -INFINITY || next_max == row_max[b])
                      ? 1.0f
                      : small_exp(__fsub_rn(row_max[b], next_max));
        float page_sum = 0.0f, weight[8];
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) {
          const uint32_t token = 16 * (i >> 2) + 4 * g + (i & 3);
          const float p = in[i] ? small_exp(__fsub_rn(score[i], next_max)) : 0.0f;
          page_sum = __fadd_rn(page_sum, p);
          weight[i] = 0.0f;
          if (kWhole || (in[i] && score[i] > -INFINITY))
            weight[i] = kQuant ? __fmul_rn(p, value_scale_lds[token]) : p;
        }
        row_sum[b] = __fadd_rn(__fmul_rn(row_sum[b], rescale), page_sum);
        row_max[b] = next_max;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
          // two weights to their 16-bit operand elements, round to nearest even, in one
          // instruction where the operand is bf16
          if constexpr (kFp8)
            weights[i] = uint32_t(operand_bits<true>(weight[2 * i])) | uint32_t(operand_bits<true>(weight[2 * i + 1])) << 16;
          else
            weights[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(small_f32x2{weight[2 * i], weight[2 * i + 1]}, small_bf16x2));
        }
      };
      if (token_start + kPage <= committed) page_softmax(std::true_type{});
      else page_softmax(std::false_type{});
      if (__builtin_amdgcn_ballot_w64(rescale != 1.0f)) {
#pragma unroll
        for (uint32_t i = 0; i < kTiles; ++i) acc[b][i] *= rescale;
      }
#pragma unroll
      for (uint32_t i = 0; i < kTiles; ++i) {
        const uint16_t *row = &v_lds[value_row(16 * i + t) + 4 * g];
        const small_u32x2 lo = *reinterpret_cast<const small_u32x2 *>(row);
        const small_u32x2 hi = *reinterpret_cast<const small_u32x2 *>(row + 16);
        acc[b][i] = small_mfma<kFp8>(small_u32x4{lo[0], lo[1], hi[0], hi[1]}, weights, acc[b][i]);
      }
    }
  }

#pragma unroll
  for (uint32_t b = 0; b < BLOCKS; ++b) {
    if (!used[b]) continue;
    // the lanes of a row hold disjoint tokens
    float sum = row_sum[b];
    sum = __fadd_rn(sum, __shfl_xor(sum, 16));
    sum = __fadd_rn(sum, __shfl_xor(sum, 32));
    if (!live[b]) continue;
    float *out = partials + out_row[b] * D + 4 * g;
#pragma unroll
    for (uint32_t i = 0; i < kTiles; ++i) *reinterpret_cast<small_f32x4 *>(out + 16 * i) = acc[b][i];
    if (g == 0) {
      statistics[out_row[b] * 2] = row_max[b];
      statistics[out_row[b] * 2 + 1] = sum;
    }
  }
}

// BLOCKS = 1 (tiles of up to 64 fused rows) leaves registers for four waves per SIMD.
template <uint32_t FMT, uint32_t D, uint32_t BLOCKS>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(BLOCKS == 1 ? 4 : 2, BLOCKS == 1 ? 4 : 2))) void attend_split_small_kernel(
    const uint16_t *__restrict__ queries, float *__restrict__ partials,
    float *__restrict__ statistics, const uint32_t *__restrict__ row_masks, AttendArgs a) {
  const uint32_t split = blockIdx.x, head = blockIdx.y, li = blockIdx.z;
  const AttendLane &l = a.lane[li];
  if (!attend_contract(l, a) || split >= l.split_count) return;
  const uint32_t M = a.row_capacity * a.group;
  const uint16_t *tile_q = queries + l.q_offset + uint64_t(head) * a.row_stride * a.group * D;
  const uint64_t slot_row = l.row_base + (uint64_t(head) * l.split_count + split) * M;
  attention_tile_small<FMT, D, BLOCKS>(tile_q, l.table, a.kv, a.kv_heads, a.group, a.row_capacity, head,
                               l.committed, l.active_rows, l.split_count, split, partials,
                               statistics, slot_row,
                               row_masks ? row_masks + l.mask_offset : nullptr, l.score_scale);
}

// Tiles of at most 16 fused rows: a wave per (split, KV head, lane), PRIVATE of them to a
// workgroup (the staged values take 9.3 KiB a wave at head dimension 128).
template <uint32_t D>
constexpr uint32_t kSmallPrivateWaves = D == 128 ? 2 : 4;
// Four waves to a SIMD where the page's raw bytes leave the registers for it: at head dimension
// 128, bf16 pages keep 64 registers of them in flight, and int8 and e4m3 pages would spill a few.
template <uint32_t FMT, uint32_t D>
constexpr uint32_t kSmallPrivatePerSimd = D != 128 || FMT == KVX_FMT_INT4 ? 4 : FMT == KVX_FMT_BF16 ? 2 : 3;
template <uint32_t FMT, uint32_t D>
__global__ __launch_bounds__(64 * kSmallPrivateWaves<D>)
__attribute__((amdgpu_waves_per_eu(kSmallPrivatePerSimd<FMT, D>, kSmallPrivatePerSimd<FMT, D>))) void attend_split_small_wave_kernel(
    const uint16_t *__restrict__ queries, float *__restrict__ partials,
    float *__restrict__ statistics, const uint32_t *__restrict__ row_masks, AttendArgs a) {
  constexpr uint32_t kWaves = kSmallPrivateWaves<D>;
  const uint32_t split = kWaves * blockIdx.x + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t head = blockIdx.y, li = blockIdx.z;
  const AttendLane &l = a.lane[li];
  if (!attend_contract(l, a) || split >= l.split_count) return;
  const uint32_t M = a.row_capacity * a.group;
  const uint16_t *tile_q = queries + l.q_offset + uint64_t(head) * a.row_stride * a.group * D;
  const uint64_t slot_row = l.row_base + (uint64_t(head) * l.split_count + split) * M;
  attention_tile_small<FMT, D, 1, kWaves>(tile_q, l.table, a.kv, a.kv_heads, a.group, a.row_capacity, head,
                                          l.committed, l.active_rows, l.split_count, split, partials,
                                          statistics, slot_row,
                                          row_masks ? row_masks + l.mask_offset : nullptr, l.score_scale);
}

template <uint32_t FMT, uint32_t D, uint32_t BLOCKS>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(BLOCKS == 1 ? 4 : 2, BLOCKS == 1 ? 4 : 2))) void prefill_split_small_kernel(
    const uint16_t *__restrict__ queries, float *__restrict__ partials,
    float *__restrict__ statistics, PrefillArgs p) {
  const uint32_t split = blockIdx.x, head = blockIdx.y, tile = blockIdx.z;
  const uint32_t tile_start = tile * KVX_PREFILL_TILE_ROWS;
  if (!prefill_contract(p) || tile_start >= p.rows) return;
  const uint32_t active = min(KVX_PREFILL_TILE_ROWS, p.rows - tile_start);
  const uint32_t M = KVX_PREFILL_TILE_ROWS * p.group;
  const uint64_t tile_offset = (uint64_t(head) * p.stride + tile_start) * p.group * D;
  const uint64_t slot_row = ((uint64_t(tile) * p.kv_heads + head) * p.splits + split) * M;
  attention_tile_small<FMT, D, BLOCKS>(queries + tile_offset, p.table, p.kv, p.kv_heads, p.group,
                               KVX_PREFILL_TILE_ROWS, head, p.committed + tile_start, active,
                               p.splits, split, partials, statistics, slot_row, nullptr,
                               p.score_scale);
}

// The same for `tiles_per_group` consecutive tiles of a chunk at once, on a history that ends
// on a page boundary: the page is staged once for all of them, and every wave multiplies one
// or two blocks of 16 fused rows a page where a single tile of a small group of query heads
// leaves it one, or none.  Slots and results are those of the tile-by-tile launch.
template <uint32_t FMT, uint32_t D, uint32_t BLOCKS>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void prefill_group_small_kernel(
    const uint16_t *__restrict__ queries, float *__restrict__ partials,
    float *__restrict__ statistics, PrefillArgs p, uint32_t tiles_per_group) {
  const uint32_t split = blockIdx.x, head = blockIdx.y, tile = blockIdx.z * tiles_per_group;
  const uint32_t tile_start = tile * KVX_PREFILL_TILE_ROWS;
  if (!prefill_contract(p) || tile_start >= p.rows) return;
  const uint32_t rows_left = p.rows - tile_start;
  const uint32_t M = KVX_PREFILL_TILE_ROWS * p.group;
  const uint64_t tile_offset = (uint64_t(head) * p.stride + tile_start) * p.group * D;
  const uint64_t slot_row = ((uint64_t(tile) * p.kv_heads + head) * p.splits + split) * M;
  const SmallGroup group = {min(tiles_per_group, (rows_left + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS),
                            (M + 15) / 16, rows_left, uint64_t(p.kv_heads) * p.splits * M};
  attention_tile_small<FMT, D, BLOCKS>(queries + tile_offset, p.table, p.kv, p.kv_heads, p.group,
                               KVX_PREFILL_TILE_ROWS, head, p.committed + tile_start,
                               min(KVX_PREFILL_TILE_ROWS, rows_left), p.splits, split, partials,
                               statistics, slot_row, nullptr, p.score_scale, group);
}

// Fixed-order merge of one fused row's splits (reference:
// common/paged_attention_tile.h:362-417).  One thread per dimension, in whole waves;
// returns the thread's bf16 element, zero for rows past the live ones.
template <uint32_t kAhead>
__device__ __forceinline__ uint16_t reduce_row(const float *__restrict__ partials,
                               const float *__restrict__ statistics, uint32_t G, uint32_t D,
                               uint32_t M, uint32_t committed, uint32_t active_rows,
                               uint32_t splits, uint64_t head_row, uint32_t fused_row) {
  // Workgroups of whole waves: thread d sums dimension d (threads past D only lend their
  // lanes).  Lane i of every wave holds the statistics of split base + i, 64 splits at a
  // time, and hands weight and term round with shuffles; the partial values of kAhead splits
  // (32; 8 for launches of at most 8 splits) are asked for together and then added in split order.
  const uint32_t d = threadIdx.x, lane = threadIdx.x & 63u;
  if (fused_row / G >= active_rows) return 0;
  const uint32_t pages = (committed + active_rows + kPage - 1) / kPage;
  const uint32_t per = (pages + splits - 1) / splits;
  const uint32_t written = (pages + per - 1) / per;
  const auto statistic = [&](uint32_t s) { return statistics + (head_row + uint64_t(s) * M + fused_row) * 2; };
  const auto partial = [&](uint32_t s) {
    return d < D ? partials[(head_row + uint64_t(s) * M + fused_row) * D + d] : 0.0f;
  };
  // The statistics of the first 64 splits and the partial values of the first kAhead are asked
  // for together, before anything waits.
  float first_max = -INFINITY, first_sum = 0.0f;
  if (lane < written) {
    first_max = statistic(lane)[0];
    first_sum = statistic(lane)[1];
  }
  float early[kAhead];
#pragma unroll
  for (uint32_t u = 0; u < kAhead; ++u) early[u] = partial(min(u, written - 1));
  float maximum = first_max;
  for (uint32_t base = 64; base < written; base += 64)
    if (base + lane < written) maximum = fmaxf(maximum, statistic(base + lane)[0]);
  for (int offset = 32; offset; offset >>= 1) maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
  float numerator = 0.0f, denominator = 0.0f;
  for (uint32_t base = 0; base < written; base += 64) {
    const uint32_t count = min(64u, written - base);
    float my_max = first_max, my_sum = first_sum;
    if (base && lane < count) {
      my_max = statistic(base + lane)[0];
      my_sum = statistic(base + lane)[1];
    }
    float my_weight = 0.0f, my_term = 0.0f;
    if (lane < count) {
      my_weight = expf(__fsub_rn(my_max, maximum));
      my_term = __fmul_rn(my_weight, my_sum);
    }
    for (uint32_t i = 0; i < count; i += kAhead) {
      float part[kAhead];
#pragma unroll
      for (uint32_t u = 0; u < kAhead; ++u)
        part[u] = (base == 0 && i == 0) ? early[u] : partial(base + min(i + u, count - 1));
#pragma unroll
      for (uint32_t u = 0; u < kAhead; ++u) {
        if (i + u < count) {  // split order is part of the contract
          numerator = __fadd_rn(numerator, __fmul_rn(__shfl(my_weight, i + u), part[u]));
          denominator = __fadd_rn(denominator, __shfl(my_term, i + u));
        }
      }
    }
  }
  return f32_to_bf16(denominator > 0.0f ? __fdiv_rn(numerator, denominator) : 0.0f);
}

template <uint32_t AHEAD>
__global__ __launch_bounds__(256) void attend_reduce_kernel(const float *__restrict__ partials,
                                                            const float *__restrict__ statistics,
                                                            uint16_t *__restrict__ output,
                                                            AttendArgs a) {
  // blockDim.y rows to a workgroup, each on waves of its own (no row waits for another)
  const uint32_t fused_row = blockIdx.x * blockDim.y + threadIdx.y, head = blockIdx.y, li = blockIdx.z;
  const AttendLane &l = a.lane[li];
  if (!attend_contract(l, a)) return;
  const uint32_t M = a.row_capacity * a.group, D = a.head_dim, d = threadIdx.x;
  if (fused_row >= M) return;
  const uint16_t value =
      reduce_row<AHEAD>(partials, statistics, a.group, D, M, l.committed, l.active_rows, l.split_count,
                 l.row_base + uint64_t(head) * l.split_count * M, fused_row);
  if (d >= D) return;
  if (output)
    output[l.q_offset + uint64_t(head) * a.row_stride * a.group * D + uint64_t(fused_row) * D + d] =
        value;
  if (!a.hidden) return;
  // The out-projection's operand, [lane][row][query head][D], scaled by the
  // sigmoid of the element's gate where packed rows are given (reference:
  // decode/paged_attention.metal:302-308, 389-393).
  const uint64_t hidden_row = uint64_t(li) * a.row_capacity + fused_row / a.group;
  const uint32_t query_heads = a.kv_heads * a.group;
  const uint32_t query_head = head * a.group + fused_row % a.group;
  uint16_t hidden = value;
  if (a.packed_qkv) {
    const uint16_t gate = a.packed_qkv[hidden_row * (2ull * query_heads + 2ull * a.kv_heads) * D +
                                       uint64_t(query_head) * 2 * D + D + d];
    hidden = f32_to_bf16(__fmul_rn(bf16_to_f32(value), sigmoid(bf16_to_f32(gate))));
  }
  a.hidden[(hidden_row * query_heads + query_head) * D + d] = hidden;
}

template <uint32_t AHEAD>
__global__ __launch_bounds__(256) void prefill_reduce_kernel(const float *__restrict__ partials,
                                                             const float *__restrict__ statistics,
                                                             uint16_t *__restrict__ output,
                                                             PrefillArgs p) {
  const uint32_t fused_row = blockIdx.x * blockDim.y + threadIdx.y, head = blockIdx.y, tile = blockIdx.z;
  const uint32_t tile_start = tile * KVX_PREFILL_TILE_ROWS;
  if (!prefill_contract(p) || tile_start >= p.rows) return;
  const uint32_t active = min(KVX_PREFILL_TILE_ROWS, p.rows - tile_start);
  const uint32_t M = KVX_PREFILL_TILE_ROWS * p.group, D = p.head_dim;
  if (fused_row >= M) return;
  const uint64_t tile_offset = (uint64_t(head) * p.stride + tile_start) * p.group * D;
  const uint16_t value =
      reduce_row<AHEAD>(partials, statistics, p.group, D, M, p.committed + tile_start, active, p.splits,
                 (uint64_t(tile) * p.kv_heads + head) * p.splits * M, fused_row);
  if (threadIdx.x < D) output[tile_offset + uint64_t(fused_row) * D + threadIdx.x] = value;
}

// =========================================================== compaction ====
struct CompactLane {
  const uint64_t *table;
  uint32_t committed, tokens, entries, pad;
};
struct CompactArgs {
  CompactLane lane[kLanes];
  uint32_t n_lanes, kv_heads, head_dim, format;
  uint32_t first_layer, path_stride;
  uint32_t extent_pages, data_bytes, scale_bytes;
};

// Forward-order copy of the retained path's rows to their path slots, one
// workgroup per (head, lane, layer) (reference:
// decode/paged_attention_store.metal:198-278).  All loads of a row complete
// before its stores.  A lane whose path is not a strictly increasing list of
// stored rows, or whose slots fall outside its table, moves nothing.
__global__ __launch_bounds__(256) void compact_kernel(const uint32_t *__restrict__ retained_path,
                                                      const uint32_t *__restrict__ retained_count,
                                                      uint32_t lane_first, CompactArgs a) {
  const uint32_t head = blockIdx.x, li = blockIdx.y, layer = a.first_layer + blockIdx.z;
  const CompactLane &l = a.lane[li];
  const uint32_t lane = lane_first + li;
  const uint32_t count = retained_count[lane];
  const uint32_t *path = retained_path + uint64_t(lane) * a.path_stride;
  if (count == 0 || count > a.path_stride || count > l.tokens) return;
  if (l.entries < (uint64_t(l.committed) + l.tokens + kPage - 1) / kPage) return;
  for (uint32_t i = 0; i < count; ++i)
    if (path[i] >= l.tokens || path[i] < i || (i && path[i] <= path[i - 1])) return;
  const uint32_t D = a.head_dim, H = a.kv_heads, F = a.format;
  kvx_kv_layer kv;
  kv.extent_pages = a.extent_pages;
  kv.offset = uint32_t(uint64_t(layer) * a.extent_pages * 2 * (uint64_t(a.data_bytes) + a.scale_bytes));
  const uint32_t d = threadIdx.x;
  const uint32_t element_bytes = F == KVX_FMT_BF16 ? 2 : 1;
  const uint32_t row_units = F == KVX_FMT_INT4 ? D / 2 : D;  // elements (bytes for int4) per row
  for (uint32_t i = 0; i < count; ++i) {
    const uint32_t src_row = path[i];
    if (src_row == i) continue;
    const uint32_t src_token = l.committed + src_row, dst_token = l.committed + i;
    const Slab src = slab_of(F, H, D, kv, head, l.table[src_token / kPage]);
    const Slab dst = slab_of(F, H, D, kv, head, l.table[dst_token / kPage]);
    const uint32_t so = src_token % kPage, dof = dst_token % kPage;
    uint16_t key = 0, value = 0;
    float key_scale = 0.0f, value_scale = 0.0f;
    const bool active = d < row_units;
    if (active) {
      const uint32_t ks = so * row_units + d;
      const uint32_t vs = F == KVX_FMT_INT4 ? ks : d * kPage + so;
      if (element_bytes == 2) {
        key = reinterpret_cast<const uint16_t *>(src.keys)[ks];
        value = reinterpret_cast<const uint16_t *>(src.values)[vs];
      } else {
        key = src.keys[ks];
        value = src.values[vs];
      }
    }
    if (d == 0 && F != KVX_FMT_BF16) {
      key_scale = src.key_scales[so];
      value_scale = src.value_scales[so];
    }
    __syncthreads();
    if (active) {
      const uint32_t kd = dof * row_units + d;
      const uint32_t vd = F == KVX_FMT_INT4 ? kd : d * kPage + dof;
      if (element_bytes == 2) {
        reinterpret_cast<uint16_t *>(dst.keys)[kd] = key;
        reinterpret_cast<uint16_t *>(dst.values)[vd] = value;
      } else {
        dst.keys[kd] = uint8_t(key);
        dst.values[vd] = uint8_t(value);
      }
    }
    if (d == 0 && F != KVX_FMT_BF16) {
      dst.key_scales[dof] = key_scale;
      dst.value_scales[dof] = value_scale;
    }
    __threadfence_block();
    __syncthreads();
  }
}

// ============================================================ page copy ====
constexpr uint32_t kCopiesPerLaunch = 128;
constexpr uint32_t kCopyChunk = 16384;
struct CopyArgs {
  uint64_t from[kCopiesPerLaunch];
  uint64_t to[kCopiesPerLaunch];
  uint32_t extent_pages, data_bytes, scale_bytes, layers;
};

// Every tensor of every layer of each page, 16 bytes per thread per step
// (reference: runtime/ops/PageStorage.mm:95-167 copies the same spans on the
// host).  blockIdx = (chunk of the span, layer * 4 + tensor, copy).
__global__ __launch_bounds__(256) void page_copy_kernel(CopyArgs a) {
  const uint32_t tensor = blockIdx.y & 3, layer = blockIdx.y >> 2;
  const uint32_t bytes = (tensor & 1) ? a.scale_bytes : a.data_bytes;
  const uint32_t begin = blockIdx.x * kCopyChunk;
  if (begin >= bytes) return;
  const uint32_t end = min(bytes, begin + kCopyChunk);
  const uint64_t from = a.from[blockIdx.z], to = a.to[blockIdx.z];
  const uint32_t fi = uint32_t(from) & KVX_PAGE_INDEX_MASK, ti = uint32_t(to) & KVX_PAGE_INDEX_MASK;
  const RegionOffsets r = region_offsets(a.extent_pages, a.data_bytes, a.scale_bytes);
  const uint64_t region = uint64_t(layer) * a.extent_pages * 2 * (uint64_t(a.data_bytes) + a.scale_bytes);
  const uint64_t start = tensor == 0 ? 0 : tensor == 1 ? r.key_scales : tensor == 2 ? r.values : r.value_scales;
  const uint8_t *src = reinterpret_cast<const uint8_t *>(from - fi) + region + start + uint64_t(fi) * bytes;
  uint8_t *dst = reinterpret_cast<uint8_t *>(to - ti) + region + start + uint64_t(ti) * bytes;
  // A chunk is four steps of the workgroup: all four loads go out before the
  // first store, so a thread has 64 bytes in flight instead of 16.
  static_assert(kCopyChunk == 4 * 256 * 16, "a chunk is four 16-byte steps of 256 threads");
  const uint32_t o = begin + threadIdx.x * 16;
  typedef uint32_t word4 __attribute__((ext_vector_type(4)));
  word4 v[4];
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i)
    if (o + i * 4096 < end)
      v[i] = __builtin_nontemporal_load(reinterpret_cast<const word4 *>(src + o + i * 4096));
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i)
    if (o + i * 4096 < end)
      __builtin_nontemporal_store(v[i], reinterpret_cast<word4 *>(dst + o + i * 4096));
}

// Pages to and from their wire form: a page's spans in the order the reference's
// storage hands them to its disk tier (PageStorage::spans,
// runtime/ops/PageStorage.mm:143-167: layer by layer, keys, key scales, values,
// value scales), bytes_per_page per page, page after page in one linear buffer.
// Same grid as page_copy_kernel: blockIdx = (chunk of the span, layer * 4 +
// tensor, page of the launch).
struct WireArgs {
  uint64_t page[kCopiesPerLaunch];  // page entries (extent address | index)
  uint8_t *buffer;                  // wire bytes of the launch's first page
  uint32_t extent_pages, data_bytes, scale_bytes, layers;
};
template <bool EXPORT>
__global__ __launch_bounds__(256) void page_wire_kernel(WireArgs a) {
  const uint32_t tensor = blockIdx.y & 3, layer = blockIdx.y >> 2;
  const uint32_t bytes = (tensor & 1) ? a.scale_bytes : a.data_bytes;
  const uint32_t begin = blockIdx.x * kCopyChunk;
  if (begin >= bytes) return;
  const uint32_t end = min(bytes, begin + kCopyChunk);
  const uint64_t entry = a.page[blockIdx.z];
  const uint32_t index = uint32_t(entry) & KVX_PAGE_INDEX_MASK;
  const RegionOffsets r = region_offsets(a.extent_pages, a.data_bytes, a.scale_bytes);
  const uint64_t layer_bytes = 2 * (uint64_t(a.data_bytes) + a.scale_bytes);
  const uint64_t start = tensor == 0 ? 0 : tensor == 1 ? r.key_scales : tensor == 2 ? r.values : r.value_scales;
  uint8_t *paged = reinterpret_cast<uint8_t *>(entry - index) + uint64_t(layer) * a.extent_pages * layer_bytes +
                   start + uint64_t(index) * bytes;
  const uint64_t wire_start = tensor == 0   ? 0
                              : tensor == 1 ? a.data_bytes
                              : tensor == 2 ? uint64_t(a.data_bytes) + a.scale_bytes
                                            : 2 * uint64_t(a.data_bytes) + a.scale_bytes;
  uint8_t *wire = a.buffer + (uint64_t(blockIdx.z) * a.layers + layer) * layer_bytes + wire_start;
  const uint8_t *src = EXPORT ? paged : wire;
  uint8_t *dst = EXPORT ? wire : paged;
  typedef uint32_t word4 __attribute__((ext_vector_type(4)));
  const uint32_t o = begin + threadIdx.x * 16;
  word4 v[4];
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i)
    if (o + i * 4096 < end) v[i] = *reinterpret_cast<const word4 *>(src + o + i * 4096);
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i)
    if (o + i * 4096 < end) *reinterpret_cast<word4 *>(dst + o + i * 4096) = v[i];
}

// ============================================ attention over a shared prefix ====
// Sequences whose page tables begin with the same pages: the prefix is attended
// once, the sequences' one-row queries stacked as the rows of one lane, and each
// sequence's own pages as a decode lane of its own; this merge then combines, per
// sequence, KV head and query head, the partial rows of the prefix's splits and of
// the sequence's splits: the maximum over all of them, then the weighted sums in
// a fixed order (prefix splits in split order, then the sequence's), as
// reduce_row does for one list.
constexpr uint32_t kSharedLanes = KVX_TREE_NODES;
constexpr uint32_t kSharedD = 256;  // the matrix-core kernels' head dimension
typedef float vec4f __attribute__((ext_vector_type(4)));
typedef uint32_t vec2u __attribute__((ext_vector_type(2)));
struct SharedLane {
  uint64_t base;     // first fused row of the sequence's own slots
  uint32_t splits;   // its split count (the slot stride) and how many of them own a page
  uint32_t written;
};
struct SharedArgs {
  SharedLane lane[kSharedLanes];
  const float *prefix_partials, *prefix_statistics;
  const float *own_partials, *own_statistics;
  uint32_t prefix_splits, prefix_written, prefix_rows;  // rows: fused rows of the prefix lane
  uint32_t kv_heads, group, row_stride;
};

// Stacks the sequences' query rows as the rows of one lane, [kv head][sequence][g][D],
// and clears the row masks of that lane (a row sees the committed prefix only).
__global__ __launch_bounds__(256) void shared_stage_kernel(const uint16_t *__restrict__ queries,
                                                           uint16_t *__restrict__ staged,
                                                           uint32_t *__restrict__ masks, uint32_t lanes,
                                                           uint32_t kv_heads, uint32_t group,
                                                           uint32_t row_stride) {
  const uint32_t lane = blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  if (head == 0 && d == 0) masks[lane] = 0;
  const uint64_t from = (uint64_t(lane) * kv_heads + head) * row_stride * group * kSharedD;
  const uint64_t to = (uint64_t(head) * lanes + lane) * group * kSharedD;
  for (uint32_t g = 0; g < group; ++g) staged[to + g * kSharedD + d] = queries[from + g * kSharedD + d];
}

// grid (query head in group, KV head, sequence), four waves, each lane four dimensions.
// The two lists are walked as one: entry t is prefix split t, or the sequence's own
// split t - prefix_written.  The entries are cut into four consecutive ranges, one per
// wave; a wave fetches its statistics 64 entries at a time, one per lane, and its
// partial rows eight at a time, so that the loads of a batch are in flight together,
// and sums its range in entry order; the ranges are then added in range order, which
// keeps the result a function of the inputs and the split counts alone.
constexpr uint32_t kSharedWaves = 4;
__global__ __launch_bounds__(64 * kSharedWaves) void shared_merge_kernel(uint16_t *__restrict__ output,
                                                                         SharedArgs a) {
  const uint32_t g = blockIdx.x, head = blockIdx.y, li = blockIdx.z;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const SharedLane l = a.lane[li];
  const uint32_t G = a.group;
  const uint64_t prefix_row = uint64_t(head) * a.prefix_splits * a.prefix_rows + li * G + g;
  const uint64_t own_row = l.base + uint64_t(head) * l.splits * G + g;
  const uint32_t entries = a.prefix_written + l.written;
  const auto statistics_of = [&](uint32_t t) {
    return t < a.prefix_written
               ? a.prefix_statistics + (prefix_row + uint64_t(t) * a.prefix_rows) * 2
               : a.own_statistics + (own_row + uint64_t(t - a.prefix_written) * G) * 2;
  };
  const auto partials_of = [&](uint32_t t) {
    return t < a.prefix_written
               ? a.prefix_partials + (prefix_row + uint64_t(t) * a.prefix_rows) * kSharedD
               : a.own_partials + (own_row + uint64_t(t - a.prefix_written) * G) * kSharedD;
  };
  const uint32_t share = (entries + kSharedWaves - 1) / kSharedWaves;
  const uint32_t first = min(entries, wave * share), last = min(entries, first + share);
  // The statistics of all entries (for the maximum) and the wave's first sixteen partial
  // rows are requested before anything waits; loads return in order, so the wait for
  // the statistics leaves the rows in flight.
  constexpr uint32_t kEarly = 16;
  float early_max[2];
#pragma unroll
  for (uint32_t b = 0; b < 2; ++b)
    early_max[b] = 64 * b + lane < entries ? statistics_of(64 * b + lane)[0] : -INFINITY;
  vec4f early[kEarly];
#pragma unroll
  for (uint32_t u = 0; u < kEarly; ++u)
    early[u] = *reinterpret_cast<const vec4f *>(partials_of(min(first + u, entries - 1)) + 4 * lane);
  float maximum = fmaxf(early_max[0], early_max[1]);  // over all entries, by every wave
  for (uint32_t base = 128; base < entries; base += 64)
    maximum = fmaxf(maximum, base + lane < entries ? statistics_of(base + lane)[0] : -INFINITY);
  for (int offset = 32; offset; offset >>= 1) maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
  vec4f numerator = {0.0f, 0.0f, 0.0f, 0.0f};
  float denominator = 0.0f;
  for (uint32_t base = first; base < last; base += 64) {
    const uint32_t mine = base + lane, count = min(64u, last - base);
    float my_max = -INFINITY, my_sum = 0.0f;
    if (mine < last) {
      const float *stat = statistics_of(mine);
      my_max = stat[0];
      my_sum = stat[1];
    }
    const float my_weight = expf(__fsub_rn(my_max, maximum));
    const float my_term = __fmul_rn(my_weight, my_sum);
    for (uint32_t i = 0; i < count; i += kEarly) {
      vec4f part[kEarly];
#pragma unroll
      for (uint32_t u = 0; u < kEarly; ++u) {
        if (base == first && i == 0)
          part[u] = early[u];
        else
          part[u] = *reinterpret_cast<const vec4f *>(partials_of(base + min(i + u, count - 1)) + 4 * lane);
      }
#pragma unroll
      for (uint32_t u = 0; u < kEarly; ++u) {
        if (i + u < count) {
          const float weight = __shfl(my_weight, int(i + u));
#pragma unroll
          for (uint32_t c = 0; c < 4; ++c)
            numerator[c] = __fadd_rn(numerator[c], __fmul_rn(weight, part[u][c]));
          denominator = __fadd_rn(denominator, __shfl(my_term, int(i + u)));
        }
      }
    }
  }
  __shared__ vec4f numerators[kSharedWaves][64];
  __shared__ float denominators[kSharedWaves][64];
  numerators[wave][lane] = numerator;
  denominators[wave][lane] = denominator;
  __syncthreads();
  if (wave) return;
#pragma unroll
  for (uint32_t w = 1; w < kSharedWaves; ++w) {
    const vec4f other = numerators[w][lane];
#pragma unroll
    for (uint32_t c = 0; c < 4; ++c) numerator[c] = __fadd_rn(numerator[c], other[c]);
    denominator = __fadd_rn(denominator, denominators[w][lane]);
  }
  vec2u packed;
#pragma unroll
  for (uint32_t i = 0; i < 2; ++i) {
    const float lo = denominator > 0.0f ? __fdiv_rn(numerator[2 * i], denominator) : 0.0f;
    const float hi = denominator > 0.0f ? __fdiv_rn(numerator[2 * i + 1], denominator) : 0.0f;
    packed[i] = uint32_t(f32_to_bf16(lo)) | (uint32_t(f32_to_bf16(hi)) << 16);
  }
  *reinterpret_cast<vec2u *>(output + (uint64_t(li) * a.kv_heads + head) * a.row_stride * G * kSharedD +
                             uint64_t(g) * kSharedD + 4 * lane) = packed;
}

// ============================================================= launchers ====
namespace {

template <class F>
int dispatch_format(uint32_t format, F &&f) {
  switch (format) {
  case KVX_FMT_INT8: return f(std::integral_constant<uint32_t, KVX_FMT_INT8>{});
  case KVX_FMT_BF16: return f(std::integral_constant<uint32_t, KVX_FMT_BF16>{});
  case KVX_FMT_INT4: return f(std::integral_constant<uint32_t, KVX_FMT_INT4>{});
  case KVX_FMT_FP8E4M3: return f(std::integral_constant<uint32_t, KVX_FMT_FP8E4M3>{});
  }
  return fail(KVX_EINVAL, "invalid KV format");
}

template <class F>
int dispatch_rows(uint32_t M, F &&f) {
  if (M <= 8) return f(std::integral_constant<uint32_t, 8>{});
  if (M <= 48) return f(std::integral_constant<uint32_t, 48>{});
  if (M <= 64) return f(std::integral_constant<uint32_t, 64>{});
  if (M <= 96) return f(std::integral_constant<uint32_t, 96>{});
  if (M <= 128) return f(std::integral_constant<uint32_t, 128>{});
  return fail(KVX_EINVAL, "tile holds more than 128 fused rows");
}

int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? KVX_OK : hip_fail(e, what);
}

}  // namespace
}  // namespace kvx

using namespace kvx;

// Implemented by the int4 MFMA kernels: enqueues the whole attention and
// returns 0, or declines (returns 1) shapes it does not cover.  With
// append_keys / append_values (bf16 chunk rows, one token per lane at
// committed_tokens) the kernel also stores that token before it attends;
// declined unless the lanes are one-row decode lanes.
int kvx_attend_int4_launch(const kvx_storage *storage, kvx_kv_layer kv, uint32_t query_heads,
                           const void *queries, void *output, const uint64_t *const *page_tables,
                           const kvx_verify_params *lanes, uint32_t n_lanes,
                           const uint32_t *row_masks, uint32_t row_stride, uint64_t lane_stride,
                           void *workspace, uint64_t workspace_bytes, int many_tiles,
                           hipStream_t stream, const void *append_keys = nullptr,
                           const void *append_values = nullptr, uint64_t append_lane_stride = 0,
                           uint32_t append_stride = 0, Tiles tile_rows = 0,
                           const Epilogue *epilogue = nullptr);

int kvx_attend_wide_launch(const kvx_storage *storage, kvx_kv_layer kv, uint32_t query_heads,
                           const void *queries, void *output, const uint64_t *const *page_tables,
                           const kvx_verify_params *lanes, uint32_t n_lanes,
                           const uint32_t *row_masks, uint32_t row_stride, uint64_t lane_stride,
                           void *workspace, uint64_t workspace_bytes, int many_tiles,
                           hipStream_t stream, Tiles tile_rows = 0,
                           const Epilogue *epilogue = nullptr);

// int4 pages go to their own kernels, bf16, fp8 and int8 pages to the wide-element
// ones; 1 = neither covers the shape.
static int attend_matrix(const kvx_storage *s, kvx_kv_layer kv, uint32_t query_heads,
                         const void *queries, void *output, const uint64_t *const *page_tables,
                         const kvx_verify_params *lanes, uint32_t n_lanes,
                         const uint32_t *row_masks, uint32_t row_stride, uint64_t lane_stride,
                         void *workspace, uint64_t workspace_bytes, int many_tiles,
                         hipStream_t stream, Tiles tile_rows = 0,
                         const Epilogue *epilogue = nullptr) {
  // tile_rows > 0: the lanes are regular (lane i = lane 0 moved on by i x tile_rows
  // rows and tokens over one table, all full but perhaps the last), which lets
  // any number of them share a launch.
  const int fast = kvx_attend_int4_launch(s, kv, query_heads, queries, output, page_tables, lanes,
                                          n_lanes, row_masks, row_stride, lane_stride, workspace,
                                          workspace_bytes, many_tiles, stream, nullptr, nullptr, 0, 0,
                                          tile_rows, epilogue);
  if (fast <= 0) return fast;
  return kvx_attend_wide_launch(s, kv, query_heads, queries, output, page_tables, lanes, n_lanes,
                                row_masks, row_stride, lane_stride, workspace, workspace_bytes,
                                many_tiles, stream, tile_rows, epilogue);
}

namespace {
std::atomic<uint64_t> g_generic_attends{0}, g_matrix_attends{0};  // callers may be on several threads
int took(int fast) {  // counts which kernels an attend call went to
  if (fast == 0) g_matrix_attends.fetch_add(1, std::memory_order_relaxed);
  if (fast > 0) g_generic_attends.fetch_add(1, std::memory_order_relaxed);
  return fast;
}
}  // namespace

extern "C" {

uint32_t kvx_debug_prefill_tiles_together(const kvx_layout *layout, uint32_t query_heads,
                                          uint32_t committed_tokens, uint32_t rows, uint32_t splits) {
  if (!kvx_layout_valid(layout) || !query_heads || query_heads % layout->kv_heads) return 0;
  return kvx::small_prefill_tiles_together(layout->head_dim, layout->kv_heads, query_heads / layout->kv_heads,
                                      committed_tokens, rows, splits);
}

void kvx_debug_attend_paths(uint64_t *generic_calls, uint64_t *matrix_core_calls) {
  if (generic_calls) *generic_calls = g_generic_attends.load(std::memory_order_relaxed);
  if (matrix_core_calls) *matrix_core_calls = g_matrix_attends.load(std::memory_order_relaxed);
}

int kv_append(const kvx_storage *s, uint32_t layer, const void *chunk_keys,
              const void *chunk_values, const uint64_t *const *page_tables,
              const kvx_chunk_params *lanes, uint32_t n_lanes, uint64_t lane_stride,
              uint32_t verify_max_rows, void *stream) {
  if (!s || !chunk_keys || !chunk_values || !page_tables || !lanes || !n_lanes)
    return fail(KVX_EINVAL, "kv_append: null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  if (verify_max_rows > KVX_TREE_NODES)
    return fail(KVX_EINVAL, "verify stores hold at most 16 rows per lane");
  for (uint32_t i = 0; i < n_lanes; ++i) {
    static const char *const names[] = {"", "chunk_tokens_out_of_range", "context_out_of_range",
                                        "chunk_stride_invalid", "page_table_too_short"};
    if (const int e = kvx_chunk_validation(&lanes[i])) return fail(KVX_EINVAL, names[e]);
    if (verify_max_rows && (lanes[i].chunk_tokens > verify_max_rows ||
                            lanes[i].chunk_stride != KVX_VERIFY_CHUNK_STRIDE))
      return fail(KVX_EINVAL, "verify store rows or stride are out of range");
    if (!page_tables[i]) return fail(KVX_EINVAL, "kv_append: null page table");
  }
  const uint32_t H = s->layout.kv_heads, D = s->layout.head_dim;
  for (uint32_t first = 0; first < n_lanes; first += kLanes) {
    AppendArgs a{};
    a.n_lanes = std::min(kLanes, n_lanes - first);
    a.kv_heads = H;
    a.head_dim = D;
    a.verify_max_rows = verify_max_rows;
    a.kv = kv;
    a.lane_stride = lane_stride;
    uint32_t groups = 0;
    for (uint32_t i = 0; i < a.n_lanes; ++i) {
      const kvx_chunk_params &p = lanes[first + i];
      a.lane[i] = {page_tables[first + i], p.committed_tokens, p.chunk_tokens, p.chunk_stride,
                   p.page_table_entries, groups, 0};
      groups += 2 * p.chunk_tokens * H;
    }
    a.uniform_groups = 2 * lanes[first].chunk_tokens * H;
    for (uint32_t i = 0; i < a.n_lanes; ++i)
      if (lanes[first + i].chunk_tokens != lanes[first].chunk_tokens) a.uniform_groups = 0;
    const auto *keys = static_cast<const uint16_t *>(chunk_keys) + uint64_t(first) * lane_stride;
    const auto *values = static_cast<const uint16_t *>(chunk_values) + uint64_t(first) * lane_stride;
    // Chunks of many tokens go page by page through LDS; a few rows per lane
    // (decode, verify) keep one workgroup per row, which has the shorter latency.
    bool by_page = !verify_max_rows && D <= kAppendMaxD;
    uint32_t most = 0;
    for (uint32_t i = 0; i < a.n_lanes; ++i) most = std::max(most, lanes[first + i].chunk_tokens);
    by_page = by_page && most > KVX_TREE_NODES;
    if (by_page) {
      groups = 0;
      for (uint32_t i = 0; i < a.n_lanes; ++i) {
        const kvx_chunk_params &p = lanes[first + i];
        a.lane[i].group_base = groups;
        groups += ((p.committed_tokens + p.chunk_tokens - 1) / kPage - p.committed_tokens / kPage + 1) * 2 * H;
      }
      a.uniform_groups = 0;
    }
    const int rc = dispatch_format(s->layout.format, [&](auto fmt) {
      if (by_page) {
        hipLaunchKernelGGL((append_page_kernel<decltype(fmt)::value>), dim3(groups), dim3(256), 0,
                           static_cast<hipStream_t>(stream), keys, values, a);
        return check_launch("append_page_kernel");
      }
      hipLaunchKernelGGL((append_kernel<decltype(fmt)::value>), dim3(groups), dim3(D), 0,
                         static_cast<hipStream_t>(stream), keys, values, a);
      return check_launch("append_kernel");
    });
    if (rc) return rc;
  }
  return KVX_OK;
}

int kv_prepare_append(const kvx_storage *s, uint32_t layer, const kvx_qkv_shape *shape,
                      const void *packed_qkv, const void *q_norm, const void *k_norm,
                      const float *rope_cos, const float *rope_sin, void *queries,
                      uint32_t row_stride, const uint64_t *const *page_tables,
                      const kvx_chunk_params *lanes, uint32_t n_lanes, uint32_t rows,
                      uint32_t verify_max_rows, void *stream) {
  if (!s || !shape || !packed_qkv || !rope_cos || !rope_sin || !queries || !page_tables || !lanes ||
      !n_lanes)
    return fail(KVX_EINVAL, "kv_prepare_append: null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  const uint32_t H = s->layout.kv_heads, D = s->layout.head_dim;
  if (!shape->query_heads || shape->query_heads % H)
    return fail(KVX_EINVAL, "query heads are not a multiple of the KV heads");
  if (D % 32 || D > 256) return fail(KVX_EINVAL, "QKV prepare covers head dimensions 32..256 in steps of 32");
  if (!shape->rotary_pairs || 2 * shape->rotary_pairs > D)
    return fail(KVX_EINVAL, "rotary pairs do not fit the head dimension");
  if (shape->norm_type > 2 || (shape->norm_type && (!q_norm || !k_norm)))
    return fail(KVX_EINVAL, "norm weights are missing or of an unknown type");
  if (packed_qkv == queries) return fail(KVX_EINVAL, "packed rows and queries must not alias");
  for (const void *buffer : {packed_qkv, q_norm, k_norm, static_cast<const void *>(rope_cos),
                             static_cast<const void *>(rope_sin), static_cast<const void *>(queries)})
    if (reinterpret_cast<uintptr_t>(buffer) % 16)
      return fail(KVX_EINVAL, "kv_prepare_append: buffers must be 16-byte aligned");
  if (verify_max_rows > KVX_TREE_NODES)
    return fail(KVX_EINVAL, "verify stores hold at most 16 rows per lane");
  for (uint32_t i = 0; i < n_lanes; ++i) {
    static const char *const names[] = {"", "chunk_tokens_out_of_range", "context_out_of_range",
                                        "chunk_stride_invalid", "page_table_too_short"};
    if (const int e = kvx_chunk_validation(&lanes[i])) return fail(KVX_EINVAL, names[e]);
    if (lanes[i].chunk_tokens > rows || rows > row_stride)
      return fail(KVX_EINVAL, "a lane's rows exceed the packed rows or the row stride");
    if (verify_max_rows && lanes[i].chunk_tokens > verify_max_rows)
      return fail(KVX_EINVAL, "verify store rows are out of range");
    if (!page_tables[i]) return fail(KVX_EINVAL, "kv_prepare_append: null page table");
  }
  const uint32_t QH = shape->query_heads;
  const uint64_t packed_lane = uint64_t(rows) * (uint64_t(QH) * (shape->query_gate ? 2 : 1) + 2ull * H) * D;
  for (uint32_t first = 0; first < n_lanes; first += kLanes) {
    PrepareArgs p{};
    AppendArgs &a = p.append;
    a.n_lanes = std::min(kLanes, n_lanes - first);
    a.kv_heads = H;
    a.head_dim = D;
    a.verify_max_rows = 0;  // the rows bound was checked above; there is no chunk stride here
    a.kv = kv;
    uint32_t groups = 0;
    for (uint32_t i = 0; i < a.n_lanes; ++i) {
      const kvx_chunk_params &c = lanes[first + i];
      a.lane[i] = {page_tables[first + i], c.committed_tokens, c.chunk_tokens, c.chunk_stride,
                   c.page_table_entries, groups, 0};
      groups += c.chunk_tokens * (QH + H);
    }
    a.uniform_groups = lanes[first].chunk_tokens * (QH + H);
    for (uint32_t i = 0; i < a.n_lanes; ++i)
      if (lanes[first + i].chunk_tokens != lanes[first].chunk_tokens) a.uniform_groups = 0;
    p.packed = static_cast<const uint16_t *>(packed_qkv) + uint64_t(first) * packed_lane;
    p.q_norm = shape->norm_type ? q_norm : nullptr;
    p.k_norm = shape->norm_type ? k_norm : nullptr;
    p.rope_cos = rope_cos + uint64_t(first) * rows * shape->rotary_pairs;
    p.rope_sin = rope_sin + uint64_t(first) * rows * shape->rotary_pairs;
    p.queries = static_cast<uint16_t *>(queries) + uint64_t(first) * H * row_stride * (QH / H) * D;
    p.query_heads = QH;
    p.rotary_pairs = shape->rotary_pairs;
    p.query_gate = shape->query_gate ? 1 : 0;
    p.norm_f32 = shape->norm_type == 2;
    p.rows = rows;
    p.row_stride = row_stride;
    p.eps = shape->eps != 0.0f ? shape->eps : 1e-6f;
    p.group_magic = QH / H > 1 ? uint32_t((0x100000000ull + QH / H - 1) / (QH / H)) : 0u;
    // One wave per task where the head dimension is 64, 128 or 256 and a rotary pair's
    // dimensions are a power-of-two number of lanes apart; else one workgroup per task.
    const uint32_t E = D / 64, pair_lanes = E ? shape->rotary_pairs / E : 0;
    const bool by_wave = (D == 64 || D == 128 || D == 256) && shape->rotary_pairs % E == 0 &&
                         pair_lanes && !(pair_lanes & (pair_lanes - 1));
    const int rc = dispatch_format(s->layout.format, [&](auto fmt) {
      constexpr uint32_t F = decltype(fmt)::value;
      const hipStream_t st = static_cast<hipStream_t>(stream);
      if (by_wave) {
        uint32_t most_rows = 0;
        for (uint32_t i = 0; i < a.n_lanes; ++i) most_rows = std::max(most_rows, lanes[first + i].chunk_tokens);
        // chunks: four rows per wave; a decode or verify step's few rows one each
        const auto launch = [&](auto rows_per_wave) {
          constexpr uint32_t R = decltype(rows_per_wave)::value;
          const dim3 grid((QH + H + 3) / 4, (most_rows + R - 1) / R, a.n_lanes), block(256);
          if (E == 4) hipLaunchKernelGGL((prepare_append_wave_kernel<F, 4, R>), grid, block, 0, st, p);
          else if (E == 2) hipLaunchKernelGGL((prepare_append_wave_kernel<F, 2, R>), grid, block, 0, st, p);
          else hipLaunchKernelGGL((prepare_append_wave_kernel<F, 1, R>), grid, block, 0, st, p);
        };
        if (most_rows >= 64) launch(std::integral_constant<uint32_t, 4>{});
        else launch(std::integral_constant<uint32_t, 1>{});
        return check_launch("prepare_append_wave_kernel");
      }
      hipLaunchKernelGGL((prepare_append_kernel<F>), dim3(groups), dim3(D), 0, st, p);
      return check_launch("prepare_append_kernel");
    });
    if (rc) return rc;
  }
  return KVX_OK;
}

// page_tables may be null where no pages are read (the merge alone).
static int validate_attend(const kvx_storage *s, uint32_t query_heads,
                           const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                           const uint64_t *const *page_tables, uint64_t workspace_bytes) {
  const kvx_layout &l = s->layout;
  if (!query_heads || query_heads % l.kv_heads)
    return fail(KVX_EINVAL, "query heads are not a multiple of the KV heads");
  const uint32_t capacity = lanes[0].row_capacity;
  const uint32_t max_splits = capacity == 1 ? KVX_DECODE_MAX_SPLITS : KVX_VERIFY_MAX_SPLITS;
  for (uint32_t i = 0; i < n_lanes; ++i) {
    const kvx_verify_params &p = lanes[i];
    if (p.row_capacity != capacity || !capacity || capacity > row_stride)
      return fail(KVX_EINVAL, "verify lanes must share one row capacity within the row stride");
    if (!p.active_rows || p.active_rows > capacity)
      return fail(KVX_EINVAL, "verify active rows are out of range");
    if (uint64_t(p.committed_tokens) + p.active_rows > KVX_MAX_PHYSICAL_TOKENS)
      return fail(KVX_EINVAL, "verify attention history exceeds physical context");
    // (a call that reads no pages, the merge alone, brings no tables and need not size them)
    if (page_tables && p.page_table_entries < (uint64_t(p.committed_tokens) + p.active_rows + 31) / 32)
      return fail(KVX_EINVAL, "page_table_too_short");
    if (!p.split_count || p.split_count > max_splits)
      return fail(KVX_EINVAL, "verify split count is out of range");
    // The reference strides a lane's slots by slot_splits and requires
    // split_count <= slot_splits <= the maximum (common/paged_attention_tile.h:57-58).
    // Slots are packed by split_count here, so the field only has to be consistent;
    // 0 stands for "the split count".
    if (p.slot_splits && (p.slot_splits < p.split_count || p.slot_splits > max_splits))
      return fail(KVX_EINVAL, "verify slot splits are out of range");
    if (page_tables && !page_tables[i]) return fail(KVX_EINVAL, "null page table");
  }
  if (capacity * (query_heads / l.kv_heads) > 128)
    return fail(KVX_EINVAL, "tile holds more than 128 fused rows");
  if (workspace_bytes < kvx_attend_workspace_bytes(lanes, n_lanes, query_heads, &l))
    return fail(KVX_EINVAL, "verify attention scratch is smaller than its bound");
  return KVX_OK;
}

static int attend_generic(const kvx_storage *s, kvx_kv_layer kv, uint32_t query_heads,
                          const void *queries, void *output, const uint64_t *const *page_tables,
                          const kvx_verify_params *lanes, uint32_t n_lanes,
                          const uint32_t *row_masks, uint32_t row_stride, void *workspace,
                          hipStream_t stream, const Epilogue *epilogue = nullptr) {
  // The generic split kernel always writes partial rows; the phases are its two launches.
  const uint32_t phases = (epilogue && epilogue->merge_only ? 0u : 1u) |
                          (epilogue && epilogue->partials_only ? 0u : 2u);
  const kvx_layout &l = s->layout;
  const uint32_t H = l.kv_heads, G = query_heads / H, D = l.head_dim;
  const uint32_t capacity = lanes[0].row_capacity, M = capacity * G;
  uint64_t total_rows = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) total_rows += uint64_t(lanes[i].split_count) * H * M;
  float *partials = static_cast<float *>(workspace);
  float *statistics = reinterpret_cast<float *>(
      static_cast<uint8_t *>(workspace) + (total_rows * D * sizeof(float) + 255) / 256 * 256);
  uint64_t row_base = 0;
  for (uint32_t first = 0; first < n_lanes; first += kLanes) {
    AttendArgs a{};
    a.n_lanes = std::min(kLanes, n_lanes - first);
    a.kv_heads = H;
    a.group = G;
    a.head_dim = D;
    a.row_capacity = capacity;
    a.row_stride = row_stride;
    a.kv = kv;
    if (epilogue && epilogue->hidden) {
      a.hidden = epilogue->hidden + uint64_t(first) * capacity * query_heads * D;
      a.packed_qkv = epilogue->packed_qkv
                         ? epilogue->packed_qkv +
                               uint64_t(first) * capacity * (2ull * query_heads + 2ull * H) * D
                         : nullptr;
    }
    uint32_t max_splits = 0;
    for (uint32_t i = 0; i < a.n_lanes; ++i) {
      const kvx_verify_params &p = lanes[first + i];
      AttendLane &al = a.lane[i];
      al.table = page_tables ? page_tables[first + i] : nullptr;
      al.committed = p.committed_tokens;
      al.entries = p.page_table_entries;
      al.split_count = p.split_count;
      al.active_rows = p.active_rows;
      al.row_base = row_base;
      al.q_offset = uint64_t(first + i) * H * row_stride * G * D;
      al.mask_offset = (first + i) * capacity;
      al.score_scale = p.score_scale != 0.0f ? p.score_scale : l.score_scale;
      row_base += uint64_t(p.split_count) * H * M;
      max_splits = std::max(max_splits, p.split_count);
    }
    int rc = KVX_OK;
    if ((phases & 1u) && (D == 64 || D == 128) && M <= 64 * kSmallBlocks)
      rc = dispatch_format(l.format, [&](auto fmt) {
        // head dimensions 64 and 128: the tile on the matrix cores
        const auto launch = [&](auto kernel) {
          hipLaunchKernelGGL(kernel, dim3(max_splits, H, a.n_lanes), dim3(kTileThreads), 0, stream,
                             static_cast<const uint16_t *>(queries), partials, statistics, row_masks, a);
        };
        constexpr uint32_t F = decltype(fmt)::value;
        if (M <= 16) {  // one wave per tile
          const auto wave_launch = [&](auto kernel, uint32_t waves) {
            hipLaunchKernelGGL(kernel, dim3((max_splits + waves - 1) / waves, H, a.n_lanes), dim3(64 * waves), 0,
                               stream, static_cast<const uint16_t *>(queries), partials, statistics, row_masks, a);
          };
          if (D == 64) wave_launch(attend_split_small_wave_kernel<F, 64>, kSmallPrivateWaves<64>);
          else wave_launch(attend_split_small_wave_kernel<F, 128>, kSmallPrivateWaves<128>);
          return check_launch("attend_split_small_wave_kernel");
        }
        if (D == 64 && M <= 64) launch(attend_split_small_kernel<F, 64, 1>);
        else if (D == 64) launch(attend_split_small_kernel<F, 64, 2>);
        else if (M <= 64) launch(attend_split_small_kernel<F, 128, 1>);
        else launch(attend_split_small_kernel<F, 128, 2>);
        return check_launch("attend_split_small_kernel");
      });
    else if (phases & 1u)
      rc = dispatch_format(l.format, [&](auto fmt) {
        return dispatch_rows(M, [&](auto maxm) {
          hipLaunchKernelGGL((attend_split_kernel<decltype(fmt)::value, decltype(maxm)::value>),
                             dim3(max_splits, H, a.n_lanes), dim3(kTileThreads), 0, stream,
                             static_cast<const uint16_t *>(queries), partials, statistics,
                             row_masks, a);
          return check_launch("attend_split_kernel");
        });
      });
    if (rc) return rc;
    if (phases & 2u) {
      const uint32_t row_threads = (D + 63) / 64 * 64, together = 256 / row_threads;  // rows to a workgroup
      hipLaunchKernelGGL(max_splits <= 8 ? attend_reduce_kernel<8> : attend_reduce_kernel<32>,
                         dim3((M + together - 1) / together, H, a.n_lanes),
                         dim3(row_threads, together), 0, stream, partials,
                         statistics, static_cast<uint16_t *>(output), a);
      if ((rc = check_launch("attend_reduce_kernel"))) return rc;
    }
  }
  return KVX_OK;
}

static int attend_verify(const char *entry, const kvx_storage *s, uint32_t layer,
                         uint32_t query_heads, const void *queries, void *output,
                         const uint64_t *const *page_tables, const kvx_verify_params *lanes,
                         uint32_t n_lanes, const uint32_t *row_masks, uint32_t row_stride,
                         void *workspace, uint64_t workspace_bytes, const Epilogue *epilogue,
                         void *stream) {
  const bool merges = !(epilogue && epilogue->partials_only);
  const bool splits = !(epilogue && epilogue->merge_only);
  if (!s || !lanes || !n_lanes || !workspace || (splits && (!queries || !page_tables)) ||
      (merges && !output && !(epilogue && epilogue->hidden)))
    return fail(KVX_EINVAL, std::string(entry) + ": null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  if (queries && queries == output) return fail(KVX_EINVAL, "queries and output must not alias");
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  if (row_masks && s->layout.format == KVX_FMT_FP8E4M3)
    return fail(KVX_EINVAL, "tree verify has no fp8 kernels");
  if (int rc = validate_attend(s, query_heads, lanes, n_lanes, row_stride, page_tables,
                               workspace_bytes))
    return rc;
  const uint32_t group = query_heads / s->layout.kv_heads;
  const int fast = took(attend_matrix(
      s, kv, query_heads, queries, output, page_tables, lanes, n_lanes, row_masks, row_stride,
      uint64_t(s->layout.kv_heads) * row_stride * group * s->layout.head_dim, workspace,
      workspace_bytes, 0, static_cast<hipStream_t>(stream), 0, epilogue));
  if (fast <= 0) return fast;
  return attend_generic(s, kv, query_heads, queries, output, page_tables, lanes, n_lanes, row_masks,
                        row_stride, workspace, static_cast<hipStream_t>(stream), epilogue);
}

int kv_attend_split(const kvx_storage *s, uint32_t layer, uint32_t query_heads, const void *queries,
                    const uint64_t *const *page_tables, const kvx_verify_params *lanes,
                    uint32_t n_lanes, const uint32_t *row_masks, uint32_t row_stride,
                    void *workspace, uint64_t workspace_bytes, void *stream) {
  Epilogue epilogue{nullptr, nullptr};
  epilogue.partials_only = true;
  return attend_verify("kv_attend_split", s, layer, query_heads, queries, nullptr, page_tables,
                       lanes, n_lanes, row_masks, row_stride, workspace, workspace_bytes, &epilogue,
                       stream);
}

int kv_attend_merge(const kvx_storage *s, uint32_t query_heads, void *output,
                    const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                    void *workspace, uint64_t workspace_bytes, void *stream) {
  Epilogue epilogue{nullptr, nullptr};
  epilogue.merge_only = true;
  return attend_verify("kv_attend_merge", s, 0, query_heads, nullptr, output, nullptr, lanes,
                       n_lanes, nullptr, row_stride, workspace, workspace_bytes, &epilogue, stream);
}

int kv_attend_verify(const kvx_storage *s, uint32_t layer, uint32_t query_heads,
                     const void *queries, void *output, const uint64_t *const *page_tables,
                     const kvx_verify_params *lanes, uint32_t n_lanes, const uint32_t *row_masks,
                     uint32_t row_stride, void *workspace, uint64_t workspace_bytes, void *stream) {
  return attend_verify("kv_attend_verify", s, layer, query_heads, queries, output, page_tables,
                       lanes, n_lanes, row_masks, row_stride, workspace, workspace_bytes, nullptr,
                       stream);
}

int kv_attend_verify_hidden(const kvx_storage *s, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes,
                            const uint32_t *row_masks, uint32_t row_stride, void *workspace,
                            uint64_t workspace_bytes, const void *packed_qkv, void *hidden,
                            void *stream) {
  if (!hidden) return fail(KVX_EINVAL, "kv_attend_verify_hidden: null hidden rows");
  if (hidden == queries || hidden == output || hidden == packed_qkv)
    return fail(KVX_EINVAL, "hidden rows must not alias another argument");
  const Epilogue epilogue{static_cast<const uint16_t *>(packed_qkv), static_cast<uint16_t *>(hidden)};
  return attend_verify("kv_attend_verify_hidden", s, layer, query_heads, queries, output,
                       page_tables, lanes, n_lanes, row_masks, row_stride, workspace,
                       workspace_bytes, &epilogue, stream);
}

namespace {
uint64_t align256(uint64_t bytes) { return (bytes + 255) / 256 * 256; }
// Bytes of one attend call's partials and statistics over `rows` slot rows.
uint64_t slot_bytes(uint64_t rows, uint32_t head_dim) {
  return align256(rows * head_dim * sizeof(float)) + rows * 2 * sizeof(float);
}
}  // namespace

uint64_t kvx_attend_shared_workspace_bytes(const kvx_verify_params *lanes, uint32_t n_lanes,
                                           uint32_t prefix_splits, uint32_t query_heads,
                                           const kvx_layout *layout) {
  if (!lanes || !layout || !n_lanes) return 0;
  const uint64_t staged = align256(uint64_t(n_lanes) * query_heads * layout->head_dim * 2);
  const uint64_t masks = 256;
  const uint64_t prefix = align256(slot_bytes(uint64_t(prefix_splits) * n_lanes * query_heads, layout->head_dim));
  uint64_t own_rows = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) own_rows += uint64_t(lanes[i].split_count) * query_heads;
  return staged + masks + prefix + slot_bytes(own_rows, layout->head_dim);
}

int kv_attend_decode_shared(const kvx_storage *s, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t shared_pages,
                            uint32_t prefix_splits, uint32_t row_stride, void *workspace,
                            uint64_t workspace_bytes, void *stream) {
  if (!s || !queries || !output || !page_tables || !lanes || !n_lanes || !workspace)
    return fail(KVX_EINVAL, "kv_attend_decode_shared: null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  if (queries == output) return fail(KVX_EINVAL, "queries and output must not alias");
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  const kvx_layout &l = s->layout;
  const uint32_t H = l.kv_heads, D = l.head_dim;
  if (!query_heads || query_heads % H)
    return fail(KVX_EINVAL, "query heads are not a multiple of the KV heads");
  const uint32_t G = query_heads / H;
  if (D != 256 || G > 16 || l.format == KVX_FMT_FP8E4M3)
    return fail(KVX_EINVAL, "shared-prefix attention covers head dimension 256, groups of at most "
                            "16 query heads and int4, int8 or bf16 pages");
  if (n_lanes > kSharedLanes || n_lanes * G > 128)
    return fail(KVX_EINVAL, "too many sequences share the prefix for one call (16, and 128 fused rows)");
  if (!shared_pages || !prefix_splits || prefix_splits > KVX_VERIFY_MAX_SPLITS || !row_stride)
    return fail(KVX_EINVAL, "shared pages, prefix splits or row stride are out of range");
  const uint64_t shared_tokens = uint64_t(shared_pages) * kPage;
  std::vector<kvx_verify_params> own(n_lanes);
  std::vector<const uint64_t *> own_tables(n_lanes);
  for (uint32_t i = 0; i < n_lanes; ++i) {
    const kvx_verify_params &p = lanes[i];
    if (p.active_rows != 1 || p.row_capacity != 1)
      return fail(KVX_EINVAL, "decode attends exactly one row per lane");
    if (!page_tables[i]) return fail(KVX_EINVAL, "null page table");
    if (p.committed_tokens < shared_tokens)
      return fail(KVX_EINVAL, "a sequence's row lies inside the shared pages");
    if (uint64_t(p.committed_tokens) + 1 > KVX_MAX_PHYSICAL_TOKENS)
      return fail(KVX_EINVAL, "verify attention history exceeds physical context");
    if (p.page_table_entries < (uint64_t(p.committed_tokens) + 1 + kPage - 1) / kPage)
      return fail(KVX_EINVAL, "page_table_too_short");
    if (!p.split_count || p.split_count > KVX_DECODE_MAX_SPLITS)
      return fail(KVX_EINVAL, "verify split count is out of range");
    if (p.score_scale != lanes[0].score_scale)
      return fail(KVX_EINVAL, "sequences that share a prefix share the score scale");
    own[i] = p;
    own[i].committed_tokens = uint32_t(p.committed_tokens - shared_tokens);
    own[i].page_table_entries = p.page_table_entries - shared_pages;
    own_tables[i] = page_tables[i] + shared_pages;
  }
  if (workspace_bytes < kvx_attend_shared_workspace_bytes(lanes, n_lanes, prefix_splits, query_heads, &l))
    return fail(KVX_EINVAL, "verify attention scratch is smaller than its bound");
  // The prefix as one lane of n rows over the first sequence's table; its rows see
  // the committed prefix only (masks of zero), so the one page past it, which the
  // row slots would occupy, is read but never attended.
  kvx_verify_params prefix{};
  prefix.committed_tokens = uint32_t(shared_tokens);
  prefix.page_table_entries = lanes[0].page_table_entries;
  prefix.split_count = prefix.slot_splits = prefix_splits;
  prefix.active_rows = prefix.row_capacity = n_lanes;
  prefix.score_scale = lanes[0].score_scale;
  uint8_t *base = static_cast<uint8_t *>(workspace);
  uint16_t *staged = reinterpret_cast<uint16_t *>(base);
  base += align256(uint64_t(n_lanes) * query_heads * D * 2);
  uint32_t *masks = reinterpret_cast<uint32_t *>(base);
  base += 256;
  void *prefix_space = base;
  const uint64_t prefix_rows_total = uint64_t(prefix_splits) * H * n_lanes * G;
  const uint64_t prefix_bytes = align256(slot_bytes(prefix_rows_total, D));
  base += prefix_bytes;
  void *own_space = base;
  uint64_t own_rows_total = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) own_rows_total += uint64_t(own[i].split_count) * H * G;
  const uint64_t own_bytes = slot_bytes(own_rows_total, D);

  const hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(shared_stage_kernel, dim3(n_lanes, H), dim3(D), 0, st,
                     static_cast<const uint16_t *>(queries), staged, masks, n_lanes, H, G, row_stride);
  if (int rc = check_launch("shared_stage_kernel")) return rc;
  Epilogue partials{nullptr, nullptr, true};
  const uint64_t *prefix_table[1] = {page_tables[0]};
  int rc = took(attend_matrix(s, kv, query_heads, staged, nullptr, prefix_table, &prefix, 1, masks,
                              n_lanes, uint64_t(H) * n_lanes * G * D, prefix_space, prefix_bytes, 0, st, 0,
                              &partials));
  if (rc) return rc < 0 ? rc : fail(KVX_EINVAL, "no matrix-core kernel covers the shared prefix");
  rc = took(attend_matrix(s, kv, query_heads, queries, nullptr, own_tables.data(), own.data(), n_lanes,
                          nullptr, row_stride, uint64_t(H) * row_stride * G * D, own_space, own_bytes, 0,
                          st, 0, &partials));
  if (rc) return rc < 0 ? rc : fail(KVX_EINVAL, "no matrix-core kernel covers the sequences' own pages");

  SharedArgs a{};
  a.prefix_partials = static_cast<const float *>(prefix_space);
  a.prefix_statistics = reinterpret_cast<const float *>(static_cast<uint8_t *>(prefix_space) +
                                                        align256(prefix_rows_total * D * sizeof(float)));
  a.own_partials = static_cast<const float *>(own_space);
  a.own_statistics = reinterpret_cast<const float *>(static_cast<uint8_t *>(own_space) +
                                                     align256(own_rows_total * D * sizeof(float)));
  const auto written_of = [](uint64_t tokens, uint32_t splits) {
    const uint32_t pages = uint32_t((tokens + kPage - 1) / kPage);
    const uint32_t per = (pages + splits - 1) / splits;
    return (pages + per - 1) / per;
  };
  a.prefix_splits = prefix_splits;
  a.prefix_written = written_of(shared_tokens + n_lanes, prefix_splits);
  a.prefix_rows = n_lanes * G;
  a.kv_heads = H;
  a.group = G;
  a.row_stride = row_stride;
  uint64_t row_base = 0;
  for (uint32_t i = 0; i < n_lanes; ++i) {
    a.lane[i] = {row_base, own[i].split_count,
                 written_of(uint64_t(own[i].committed_tokens) + 1, own[i].split_count)};
    row_base += uint64_t(own[i].split_count) * H * G;
  }
  hipLaunchKernelGGL(shared_merge_kernel, dim3(G, H, n_lanes), dim3(64 * kSharedWaves), 0, st,
                     static_cast<uint16_t *>(output), a);
  return check_launch("shared_merge_kernel");
}

int kv_attend_decode(const kvx_storage *s, uint32_t layer, uint32_t query_heads,
                     const void *queries, void *output, const uint64_t *const *page_tables,
                     const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                     void *workspace, uint64_t workspace_bytes, void *stream) {
  if (!s || !queries || !output || !page_tables || !lanes || !n_lanes || !workspace)
    return fail(KVX_EINVAL, "kv_attend_decode: null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  if (queries == output) return fail(KVX_EINVAL, "queries and output must not alias");
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  for (uint32_t i = 0; i < n_lanes; ++i)
    if (lanes[i].active_rows != 1 || lanes[i].row_capacity != 1)
      return fail(KVX_EINVAL, "decode attends exactly one row per lane");
  if (int rc = validate_attend(s, query_heads, lanes, n_lanes, row_stride, page_tables,
                               workspace_bytes))
    return rc;
  const uint32_t group = query_heads / s->layout.kv_heads;
  const int fast = took(attend_matrix(
      s, kv, query_heads, queries, output, page_tables, lanes, n_lanes, nullptr, row_stride,
      uint64_t(s->layout.kv_heads) * row_stride * group * s->layout.head_dim, workspace,
      workspace_bytes, 0, static_cast<hipStream_t>(stream)));
  if (fast <= 0) return fast;
  return attend_generic(s, kv, query_heads, queries, output, page_tables, lanes, n_lanes, nullptr,
                        row_stride, workspace, static_cast<hipStream_t>(stream));
}

// ---- decode attention without a caller's workspace ------------------------------
// The split kernels' partial rows and statistics live in this array instead: device
// memory of the library's code object, one copy per GPU, held until the process ends.
// In host code the array's name is only a stand-in for the symbol; its address on a
// device comes from hipGetSymbolAddress, asked once per device with that device current,
// and that pointer is what every launch is given.
constexpr uint64_t kStaticScratchBytes = KVX_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char kvx_static_scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
// The array's address on each device, once known.  Written once per device (any thread
// that asks gets the same answer from the runtime), read by every launch.
std::atomic<void *> g_static_scratch[kMaxDevices];
}  // namespace

// Asks the runtime for the array's address on `device`, which must be the current one.
// Creating a storage does this for its device, so that no launch has to: asking is a
// call of the runtime that is no stream operation and may load the library's code
// object, neither of which belongs into a stream capture.
extern "C++" {
int kvx::prime_static_workspace(int device) {
  if (device < 0 || device >= kMaxDevices) return fail(KVX_EDEVICE, "device index out of range");
  if (g_static_scratch[device].load(std::memory_order_acquire)) return KVX_OK;
  void *address = nullptr;
  KVX_HIP(hipGetSymbolAddress(&address, HIP_SYMBOL(kvx_static_scratch)));
  if (!address) return fail(KVX_EDEVICE, "the static workspace has no address on this device");
  g_static_scratch[device].store(address, std::memory_order_release);
  return KVX_OK;
}
}  // extern "C++"

namespace {
// The address of the scratch array on the current device, which must be the storage's.
int static_scratch(const kvx_storage *s, hipStream_t stream, void **out) {
  int device = -1;
  KVX_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return fail(KVX_EDEVICE, "device index out of range");
  if (device != s->device)
    return fail(KVX_ESTATE, "the storage's device is not the current device");
  if (!g_static_scratch[device].load(std::memory_order_acquire)) {
    // Not asked yet on this device (the storage was created while another was current).
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing != hipStreamCaptureStatusNone)
      return fail(KVX_ESTATE, "the static workspace's address is not known on this device yet: "
                              "call kvx_static_workspace_prime before the capture");
    if (const int rc = kvx::prime_static_workspace(device)) return rc;
  }
  *out = g_static_scratch[device].load(std::memory_order_acquire);
  return KVX_OK;
}
}  // namespace

int kvx_static_workspace_prime(const kvx_storage *s) {
  if (!s) return fail(KVX_EINVAL, "kvx_static_workspace_prime: null storage");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  int device = -1;
  KVX_HIP(hipGetDevice(&device));
  if (device != s->device)
    return fail(KVX_ESTATE, "the storage's device is not the current device");
  return kvx::prime_static_workspace(device);
}

int kv_attend_decode_static(const kvx_storage *s, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                            void *stream) {
  if (!s || !lanes || !n_lanes) return fail(KVX_EINVAL, "kv_attend_decode_static: null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  const uint64_t needed = kvx_attend_workspace_bytes(lanes, n_lanes, query_heads, &s->layout);
  if (needed > kStaticScratchBytes)
    return fail(KVX_EINVAL, "kv_attend_decode_static: the lanes' partial rows need " +
                                std::to_string(needed) + " bytes, the static workspace holds " +
                                std::to_string(kStaticScratchBytes) +
                                "; use kv_attend_decode with a workspace of the caller's");
  void *scratch = nullptr;
  if (const int rc = static_scratch(s, static_cast<hipStream_t>(stream), &scratch)) return rc;
  // Every partial row and statistic a merge reads is written by the split kernel of the
  // same call first, so nothing of the previous call's contents has to be cleared.
  return kv_attend_decode(s, layer, query_heads, queries, output, page_tables, lanes, n_lanes,
                          row_stride, scratch, kStaticScratchBytes, stream);
}

namespace {
// kv_append_attend_decode and its form whose merge also writes the hidden rows (epilogue
// given; `output` may then be null).
int append_attend_decode(const kvx_storage *s, uint32_t layer, const void *chunk_keys,
                         const void *chunk_values, uint64_t chunk_lane_stride, uint32_t chunk_stride,
                         uint32_t query_heads, const void *queries, void *output,
                         const uint64_t *const *page_tables, const kvx_verify_params *lanes,
                         uint32_t n_lanes, uint32_t row_stride, void *workspace,
                         uint64_t workspace_bytes, const Epilogue *epilogue, void *stream) {
  if (!s || !chunk_keys || !chunk_values || !queries || (!output && !epilogue) || !page_tables ||
      !lanes || !n_lanes || !workspace)
    return fail(KVX_EINVAL, "kv_append_attend_decode: null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  if (queries == output) return fail(KVX_EINVAL, "queries and output must not alias");
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  for (uint32_t i = 0; i < n_lanes; ++i) {
    if (lanes[i].active_rows != 1 || lanes[i].row_capacity != 1)
      return fail(KVX_EINVAL, "decode attends exactly one row per lane");
    if (!page_tables[i]) return fail(KVX_EINVAL, "kv_append_attend_decode: null page table");
    const kvx_chunk_params chunk{lanes[i].committed_tokens, 1, chunk_stride,
                                 lanes[i].page_table_entries, {}};
    static const char *const names[] = {"", "chunk_tokens_out_of_range", "context_out_of_range",
                                        "chunk_stride_invalid", "page_table_too_short"};
    if (const int e = kvx_chunk_validation(&chunk)) return fail(KVX_EINVAL, names[e]);
  }
  if (int rc = validate_attend(s, query_heads, lanes, n_lanes, row_stride, page_tables,
                               workspace_bytes))
    return rc;
  const uint32_t group = query_heads / s->layout.kv_heads;
  const uint64_t lane_stride = uint64_t(s->layout.kv_heads) * row_stride * group * s->layout.head_dim;
  // int4 pages: the wave that owns a sequence's last page stores the token itself.
  const int fused = kvx_attend_int4_launch(s, kv, query_heads, queries, output, page_tables, lanes,
                                           n_lanes, nullptr, row_stride, lane_stride, workspace,
                                           workspace_bytes, 0, static_cast<hipStream_t>(stream),
                                           chunk_keys, chunk_values, chunk_lane_stride, chunk_stride, 0,
                                           epilogue);
  if (fused <= 0) return took(fused);
  // Every other shape: the two entries one after the other.
  std::vector<kvx_chunk_params> chunks(n_lanes);
  for (uint32_t i = 0; i < n_lanes; ++i)
    chunks[i] = {lanes[i].committed_tokens, 1, chunk_stride, lanes[i].page_table_entries, {}};
  if (int rc = kv_append(s, layer, chunk_keys, chunk_values, page_tables, chunks.data(), n_lanes,
                         chunk_lane_stride, 0, stream))
    return rc;
  if (epilogue)
    return kv_attend_verify_hidden(s, layer, query_heads, queries, output, page_tables, lanes, n_lanes,
                                   nullptr, row_stride, workspace, workspace_bytes, epilogue->packed_qkv,
                                   epilogue->hidden, stream);
  return kv_attend_decode(s, layer, query_heads, queries, output, page_tables, lanes, n_lanes,
                          row_stride, workspace, workspace_bytes, stream);
}
}  // namespace

int kv_append_attend_decode(const kvx_storage *s, uint32_t layer, const void *chunk_keys,
                            const void *chunk_values, uint64_t chunk_lane_stride,
                            uint32_t chunk_stride, uint32_t query_heads, const void *queries,
                            void *output, const uint64_t *const *page_tables,
                            const kvx_verify_params *lanes, uint32_t n_lanes, uint32_t row_stride,
                            void *workspace, uint64_t workspace_bytes, void *stream) {
  if (!output) return fail(KVX_EINVAL, "kv_append_attend_decode: null argument or no lanes");
  return append_attend_decode(s, layer, chunk_keys, chunk_values, chunk_lane_stride, chunk_stride,
                              query_heads, queries, output, page_tables, lanes, n_lanes, row_stride,
                              workspace, workspace_bytes, nullptr, stream);
}

int kv_append_attend_decode_hidden(const kvx_storage *s, uint32_t layer, const void *chunk_keys,
                                   const void *chunk_values, uint64_t chunk_lane_stride,
                                   uint32_t chunk_stride, uint32_t query_heads, const void *queries,
                                   void *output, const uint64_t *const *page_tables,
                                   const kvx_verify_params *lanes, uint32_t n_lanes,
                                   uint32_t row_stride, void *workspace, uint64_t workspace_bytes,
                                   const void *packed_qkv, void *hidden, void *stream) {
  if (!hidden) return fail(KVX_EINVAL, "kv_append_attend_decode_hidden: null hidden rows");
  if (hidden == queries || hidden == output || hidden == packed_qkv || hidden == chunk_keys ||
      hidden == chunk_values)
    return fail(KVX_EINVAL, "hidden rows must not alias another argument");
  const Epilogue epilogue{static_cast<const uint16_t *>(packed_qkv), static_cast<uint16_t *>(hidden)};
  return append_attend_decode(s, layer, chunk_keys, chunk_values, chunk_lane_stride, chunk_stride,
                              query_heads, queries, output, page_tables, lanes, n_lanes, row_stride,
                              workspace, workspace_bytes, &epilogue, stream);
}

namespace {
// How the tiles of a chunk go to the matrix-core kernels.
// With a single split every tile walks its pages from the first, so two
// neighbouring tiles can share one walk as a lane of 16 rows: a row's softmax
// runs over the same pages in the same order (the page the second tile may
// add is invisible to the first tile's rows and changes nothing), and every
// key and value is fetched and expanded once for 16 rows instead of 8.
// With several splits the two tiles must also cut their pages into the same
// splits, which they do when they see the same number of pages
// (prefill_tiles_pair: true for every pair of the chunk, or for none), and pay
// only where the paired launch fills the GPU (prefill_pairs_with_splits).
// bf16, fp8 and int8 pages: lanes of four (or two) tiles for a workgroup that shares
// every page through LDS (prefill_group_width); with several splits only where a
// lane's tiles cut their pages alike.
struct TileShape {
  uint32_t width;  // tiles per lane
  int lane_kind;   // attend_matrix's many_tiles
  bool operator==(const TileShape &o) const { return width == o.width && lane_kind == o.lane_kind; }
};
TileShape tile_shape(const kvx_layout &l, uint32_t query_heads, const kvx_prefill_params &p) {
  const uint32_t H = l.kv_heads, G = query_heads / H;
  const uint32_t tiles = (p.rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  TileShape shape;
  shape.width = (tiles >= 2 && (p.split_count == 1 ||
                                prefill_pairs_with_splits(l.format, p.committed_tokens, tiles,
                                                          p.split_count, H, G)))
                    ? 2
                    : 1;
  shape.lane_kind = shape.width == 1 ? 1 : 0;
  const uint32_t grouped = prefill_group_width(l.format, l.head_dim, p.rows, G);
  if (grouped && tiles >= grouped &&
      (p.split_count == 1 || prefill_group_splits_alike(grouped, p.committed_tokens))) {
    shape.width = grouped;
    shape.lane_kind = 2;
  }
  return shape;
}

int validate_prefill(const kvx_layout &l, uint32_t query_heads, const kvx_prefill_params &p) {
  const kvx_chunk_params chunk{p.committed_tokens, p.rows, p.chunk_stride, p.page_table_entries, {}};
  static const char *const names[] = {"", "chunk_tokens_out_of_range", "context_out_of_range",
                                      "chunk_stride_invalid", "page_table_too_short"};
  if (const int e = kvx_chunk_validation(&chunk)) return fail(KVX_EINVAL, names[e]);
  if (!p.split_count || p.split_count > KVX_PREFILL_MAX_SPLITS)
    return fail(KVX_EINVAL, "prefill split count is out of range");
  if (KVX_PREFILL_TILE_ROWS * (query_heads / l.kv_heads) > 128)
    return fail(KVX_EINVAL, "tile holds more than 128 fused rows");
  return KVX_OK;
}
uint64_t prefill_rows(const kvx_layout &l, uint32_t query_heads, const kvx_prefill_params &p) {
  const uint32_t tiles = (p.rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  return uint64_t(tiles) * l.kv_heads * p.split_count * KVX_PREFILL_TILE_ROWS * (query_heads / l.kv_heads);
}

// The chunks of `sequences` sequences (equal rows, stride, split count and tile shape; one
// sequence is the plain call) on the matrix-core kernels, every sequence's tiles in the same
// launch: 0 when enqueued, 1 when the kernels decline the shape, or a negative status.
int prefill_matrix(const kvx_storage *s, kvx_kv_layer kv, uint32_t query_heads, const void *queries,
                   void *output, const uint64_t *const *page_tables, const kvx_prefill_params *params,
                   uint32_t sequences, uint64_t sequence_stride, void *workspace,
                   uint64_t workspace_bytes, hipStream_t st) {
  const kvx_layout &l = s->layout;
  const uint32_t H = l.kv_heads, G = query_heads / H, D = l.head_dim;
  const uint32_t T = KVX_PREFILL_TILE_ROWS;
  const uint32_t tiles = (params[0].rows + T - 1) / T;
  // The matrix-core kernels take the tiles as lanes: tile t attends rows 8t..8t+7
  // over committed + 8t tokens, its queries 8 rows further on in the chunk.
  const TileShape shape = tile_shape(l, query_heads, params[0]);
  const uint32_t width = shape.width;
  const uint32_t wide_lanes = tiles / width, rest = tiles - wide_lanes * width;
  // every sequence's wide lanes, then every sequence's odd last tile
  std::vector<kvx_verify_params> tile_lanes(size_t(sequences) * (wide_lanes + rest));
  std::vector<const uint64_t *> tile_tables(tile_lanes.size());
  for (uint32_t q = 0; q < sequences; ++q) {
    const kvx_prefill_params &p = params[q];
    for (uint32_t t = 0; t < wide_lanes + rest; ++t) {
      const bool wide = t < wide_lanes;
      const uint32_t first_row = wide ? T * width * t : T * (wide_lanes * width + (t - wide_lanes));
      const uint32_t capacity = wide ? T * width : T;
      // the odd last tiles tile by tile, so that each launch of them has one lane per sequence
      const size_t at = wide ? size_t(q) * wide_lanes + t
                             : size_t(sequences) * wide_lanes + size_t(t - wide_lanes) * sequences + q;
      tile_lanes[at] = {p.committed_tokens + first_row, p.page_table_entries, {}, p.split_count,
                        p.split_count, std::min(capacity, p.rows - first_row), capacity,
                        p.score_scale};
      tile_tables[at] = page_tables[q];
    }
  }
  int fast = 1;
  if (wide_lanes)
    fast = took(attend_matrix(s, kv, query_heads, queries, output, tile_tables.data(),
                              tile_lanes.data(), sequences * wide_lanes, nullptr,
                              params[0].chunk_stride, uint64_t(T) * width * G * D, workspace,
                              workspace_bytes, shape.lane_kind, st,
                              Tiles(T * width, sequences, sequence_stride)));
  if (!wide_lanes) fast = 0;
  // The odd last tiles on their own, as ordinary lanes; lanes of one launch share a row
  // capacity.  One sequence: its last tiles in one launch, a tile apart.  Several: the
  // sequences' k-th last tiles in one launch, a sequence apart.
  const uint32_t rest_launches = sequences > 1 ? rest : (rest ? 1u : 0u);
  for (uint32_t k = 0; k < rest_launches && fast == 0; ++k) {
    const uint64_t skip = uint64_t(T) * (uint64_t(width) * wide_lanes + k) * G * D;
    const size_t at = size_t(sequences) * wide_lanes + size_t(k) * sequences;
    fast = attend_matrix(s, kv, query_heads, static_cast<const uint16_t *>(queries) + skip,
                         static_cast<uint16_t *>(output) + skip, tile_tables.data() + at,
                         tile_lanes.data() + at, sequences > 1 ? sequences : rest, nullptr,
                         params[0].chunk_stride, sequences > 1 ? sequence_stride : uint64_t(T) * G * D,
                         workspace, workspace_bytes, 1, st);
    if (fast > 0 && (wide_lanes || k))
      return fail(KVX_ESTATE, "the last prefill tile was declined after the others ran");
  }
  return fast;
}
}  // namespace

int kv_attend_prefill(const kvx_storage *s, uint32_t layer, uint32_t query_heads,
                      const void *queries, void *output, const uint64_t *page_table,
                      const kvx_prefill_params *params, void *workspace, uint64_t workspace_bytes,
                      void *stream) {
  if (!s || !queries || !output || !page_table || !params || !workspace)
    return fail(KVX_EINVAL, "kv_attend_prefill: null argument");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  if (queries == output) return fail(KVX_EINVAL, "queries and output must not alias");
  const kvx_layout &l = s->layout;
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  if (!query_heads || query_heads % l.kv_heads)
    return fail(KVX_EINVAL, "query heads are not a multiple of the KV heads");
  if (int rc = validate_prefill(l, query_heads, *params)) return rc;
  const uint32_t H = l.kv_heads, G = query_heads / H, D = l.head_dim;
  const uint32_t tiles = (params->rows + KVX_PREFILL_TILE_ROWS - 1) / KVX_PREFILL_TILE_ROWS;
  const uint32_t M = KVX_PREFILL_TILE_ROWS * G;
  const uint64_t rows = prefill_rows(l, query_heads, *params);
  const uint64_t partial_bytes = rows * D * sizeof(float);
  if (workspace_bytes < partial_bytes + rows * 2 * sizeof(float))
    return fail(KVX_EINVAL, "prefill attention scratch is smaller than its bound");
  auto st = static_cast<hipStream_t>(stream);
  {
    const int fast = prefill_matrix(s, kv, query_heads, queries, output, &page_table, params, 1, 0,
                                    workspace, workspace_bytes, st);
    if (fast <= 0) return fast;
  }
  float *partials = static_cast<float *>(workspace);
  float *statistics = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + partial_bytes);
  PrefillArgs p{page_table, params->committed_tokens, params->rows, params->chunk_stride,
                params->page_table_entries, params->split_count, H, G, D,
                params->score_scale != 0.0f ? params->score_scale : l.score_scale, kv};
  int rc = KVX_OK;
  if ((D == 64 || D == 128) && M <= 64 * kSmallBlocks)
    rc = dispatch_format(l.format, [&](auto fmt) {
      const auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(params->split_count, H, tiles), dim3(kTileThreads), 0, st,
                           static_cast<const uint16_t *>(queries), partials, statistics, p);
      };
      constexpr uint32_t F = decltype(fmt)::value;
      const uint32_t blocks = (M + 15) / 16;
      const uint32_t together = kvx::small_prefill_tiles_together(D, H, G, params->committed_tokens,
                                                             params->rows, params->split_count);
      if (together > 1) {
        const uint32_t per_wave = (blocks * together + 3) / 4;  // 1 or 2
        const auto group_launch = [&](auto kernel) {
          hipLaunchKernelGGL(kernel, dim3(params->split_count, H, (tiles + together - 1) / together),
                             dim3(kTileThreads), 0, st, static_cast<const uint16_t *>(queries), partials,
                             statistics, p, together);
        };
        if (D == 128) group_launch(prefill_group_small_kernel<F, 128, 1>);
        else if (per_wave <= 1) group_launch(prefill_group_small_kernel<F, 64, 1>);
        else group_launch(prefill_group_small_kernel<F, 64, 2>);
        return check_launch("prefill_group_small_kernel");
      }
      if (D == 64 && M <= 64) launch(prefill_split_small_kernel<F, 64, 1>);
      else if (D == 64) launch(prefill_split_small_kernel<F, 64, 2>);
      else if (M <= 64) launch(prefill_split_small_kernel<F, 128, 1>);
      else launch(prefill_split_small_kernel<F, 128, 2>);
      return check_launch("prefill_split_small_kernel");
    });
  else rc = dispatch_format(l.format, [&](auto fmt) {
    return dispatch_rows(M, [&](auto maxm) {
      hipLaunchKernelGGL((prefill_split_kernel<decltype(fmt)::value, decltype(maxm)::value>),
                         dim3(params->split_count, H, tiles), dim3(kTileThreads), 0, st,
                         static_cast<const uint16_t *>(queries), partials, statistics, p);
      return check_launch("prefill_split_kernel");
    });
  });
  if (rc) return rc;
  const uint32_t row_threads = (D + 63) / 64 * 64, together = 256 / row_threads;  // rows to a workgroup
  hipLaunchKernelGGL(params->split_count <= 8 ? prefill_reduce_kernel<8> : prefill_reduce_kernel<32>,
                     dim3((M + together - 1) / together, H, tiles),
                     dim3(row_threads, together), 0, st, partials, statistics,
                     static_cast<uint16_t *>(output), p);
  return check_launch("prefill_reduce_kernel");
}

int kv_attend_prefill_batch(const kvx_storage *s, uint32_t layer, uint32_t query_heads,
                            const void *queries, void *output, const uint64_t *const *page_tables,
                            const kvx_prefill_params *params, uint32_t n_sequences,
                            uint64_t sequence_stride, void *workspace, uint64_t workspace_bytes,
                            void *stream) {
  if (!s || !queries || !output || !page_tables || !params || !workspace || !n_sequences)
    return fail(KVX_EINVAL, "kv_attend_prefill_batch: null argument or no sequences");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  if (queries == output) return fail(KVX_EINVAL, "queries and output must not alias");
  const kvx_layout &l = s->layout;
  kvx_kv_layer kv;
  if (int rc = kvx_storage_layer(s, layer, &kv)) return rc;
  if (!query_heads || query_heads % l.kv_heads)
    return fail(KVX_EINVAL, "query heads are not a multiple of the KV heads");
  // Nothing is enqueued unless every sequence is valid.
  const uint32_t G = query_heads / l.kv_heads;
  uint64_t rows = 0;
  bool alike = true;
  for (uint32_t q = 0; q < n_sequences; ++q) {
    if (!page_tables[q]) return fail(KVX_EINVAL, "null page table");
    if (int rc = validate_prefill(l, query_heads, params[q])) return rc;
    if (n_sequences > 1 &&
        sequence_stride < uint64_t(l.kv_heads) * params[q].chunk_stride * G * l.head_dim)
      return fail(KVX_EINVAL, "sequence stride is smaller than a sequence's chunk");
    rows += prefill_rows(l, query_heads, params[q]);
    alike = alike && params[q].rows == params[0].rows &&
            params[q].chunk_stride == params[0].chunk_stride &&
            params[q].split_count == params[0].split_count &&
            tile_shape(l, query_heads, params[q]) == tile_shape(l, query_heads, params[0]);
  }
  if (workspace_bytes < rows * l.head_dim * sizeof(float) + 256 + rows * 2 * sizeof(float))
    return fail(KVX_EINVAL, "prefill attention scratch is smaller than its bound");
  auto st = static_cast<hipStream_t>(stream);
  // Equal chunks (what a scheduler that cuts chunks of its token budget produces) share
  // their launches, 32 sequences at a time; anything else runs sequence by sequence.
  if (alike && n_sequences > 1) {
    int fast = 0;
    for (uint32_t first = 0; first < n_sequences && fast == 0; first += KVX_LANES_PER_LAUNCH) {
      const uint32_t count = std::min<uint32_t>(KVX_LANES_PER_LAUNCH, n_sequences - first);
      fast = prefill_matrix(s, kv, query_heads,
                            static_cast<const uint16_t *>(queries) + first * sequence_stride,
                            static_cast<uint16_t *>(output) + first * sequence_stride,
                            page_tables + first, params + first, count, sequence_stride, workspace,
                            workspace_bytes, st);
      if (fast > 0 && first) return fail(KVX_ESTATE, "a later part of the batch was declined");
    }
    if (fast <= 0) return fast;
  }
  for (uint32_t q = 0; q < n_sequences; ++q)
    if (int rc = kv_attend_prefill(s, layer, query_heads,
                                   static_cast<const uint16_t *>(queries) + q * sequence_stride,
                                   static_cast<uint16_t *>(output) + q * sequence_stride,
                                   page_tables[q], &params[q], workspace, workspace_bytes, stream))
      return rc;
  return KVX_OK;
}

int kv_compact_path(const kvx_storage *s, uint32_t layer, const uint64_t *const *page_tables,
                    const kvx_chunk_params *lanes, uint32_t n_lanes,
                    const uint32_t *retained_path, const uint32_t *retained_count,
                    uint32_t path_stride, void *stream) {
  if (!s || !page_tables || !lanes || !n_lanes || !retained_path || !retained_count)
    return fail(KVX_EINVAL, "kv_compact_path: null argument or no lanes");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  const kvx_layout &l = s->layout;
  if (layer != UINT32_MAX && layer >= l.layers)
    return fail(KVX_ERANGE, "KV layer is outside the layout");
  if (!path_stride || path_stride > KVX_TREE_NODES)
    return fail(KVX_EINVAL, "retained path stride is out of range");
  for (uint32_t i = 0; i < n_lanes; ++i) {
    static const char *const names[] = {"", "chunk_tokens_out_of_range", "context_out_of_range",
                                        "chunk_stride_invalid", "page_table_too_short"};
    if (const int e = kvx_chunk_validation(&lanes[i])) return fail(KVX_EINVAL, names[e]);
    if (lanes[i].chunk_tokens > KVX_TREE_NODES)
      return fail(KVX_EINVAL, "a tree lane holds at most 16 rows");
    if (!page_tables[i]) return fail(KVX_EINVAL, "null page table");
  }
  for (uint32_t first = 0; first < n_lanes; first += kLanes) {
    CompactArgs a{};
    a.n_lanes = std::min(kLanes, n_lanes - first);
    a.kv_heads = l.kv_heads;
    a.head_dim = l.head_dim;
    a.format = l.format;
    a.first_layer = layer == UINT32_MAX ? 0 : layer;
    a.path_stride = path_stride;
    a.extent_pages = s->extent_pages;
    a.data_bytes = s->data_bytes;
    a.scale_bytes = s->scale_bytes;
    for (uint32_t i = 0; i < a.n_lanes; ++i) {
      const kvx_chunk_params &p = lanes[first + i];
      a.lane[i] = {page_tables[first + i], p.committed_tokens, p.chunk_tokens,
                   p.page_table_entries, 0};
    }
    const uint32_t layers = layer == UINT32_MAX ? l.layers : 1;
    hipLaunchKernelGGL(compact_kernel, dim3(l.kv_heads, a.n_lanes, layers), dim3(l.head_dim), 0,
                       static_cast<hipStream_t>(stream), retained_path, retained_count, first, a);
    if (int rc = check_launch("compact_kernel")) return rc;
  }
  return KVX_OK;
}

int kv_page_copy(kvx_storage *s, const kvx_page_copy *copies, uint32_t n, void *stream) {
  if (!s || (n && !copies)) return fail(KVX_EINVAL, "kv_page_copy: null argument");
  // All-or-nothing: validate every page before any copy is enqueued.
  for (uint32_t i = 0; i < n; ++i) {
    if (copies[i].from >= s->page_count || copies[i].to >= s->page_count)
      return fail(KVX_ERANGE, "invalid KV page id");
    if (!s->extents[copies[i].from / s->extent_pages] || !s->extents[copies[i].to / s->extent_pages])
      return fail(KVX_ESTATE, "cannot copy a KV page of an extent that is not allocated");
  }
  {
    std::vector<uint32_t> sources(n);
    for (uint32_t i = 0; i < n; ++i) sources[i] = copies[i].from;
    std::sort(sources.begin(), sources.end());
    std::vector<uint32_t> targets(n);
    for (uint32_t i = 0; i < n; ++i) targets[i] = copies[i].to;
    std::sort(targets.begin(), targets.end());
    for (uint32_t i = 0; i < n; ++i) {
      if (std::binary_search(sources.begin(), sources.end(), copies[i].to))
        return fail(KVX_EINVAL, "a page copy destination is also a source of the batch");
      if (i && targets[i] == targets[i - 1])
        return fail(KVX_EINVAL, "two page copies share a destination");
    }
  }
  if (s->accounting) return KVX_OK;  // nothing behind the pages: the bookkeeping is the copy
  const uint32_t span = std::max(s->data_bytes, s->scale_bytes);
  const uint32_t chunks = (span + kCopyChunk - 1) / kCopyChunk;
  for (uint32_t first = 0; first < n; first += kCopiesPerLaunch) {
    CopyArgs a{};
    const uint32_t count = std::min(kCopiesPerLaunch, n - first);
    a.extent_pages = s->extent_pages;
    a.data_bytes = s->data_bytes;
    a.scale_bytes = s->scale_bytes;
    a.layers = s->layout.layers;
    for (uint32_t i = 0; i < count; ++i) {
      const kvx_page_copy &c = copies[first + i];
      a.from[i] = reinterpret_cast<uint64_t>(s->extents[c.from / s->extent_pages]) |
                  (c.from % s->extent_pages);
      a.to[i] = reinterpret_cast<uint64_t>(s->extents[c.to / s->extent_pages]) |
                (c.to % s->extent_pages);
    }
    hipLaunchKernelGGL(page_copy_kernel, dim3(chunks, s->layout.layers * 4, count), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a);
    if (int rc = check_launch("page_copy_kernel")) return rc;
  }
  return KVX_OK;
}


static int page_wire(const kvx_storage *s, const uint32_t *pages, uint32_t n, void *buffer,
                     bool to_wire, void *stream) {
  if (!s || (n && (!pages || !buffer))) return fail(KVX_EINVAL, "page export / import: null argument");
  if (s->accounting) return fail(KVX_ESTATE, "accounting-only storage has no memory to run on");
  // All-or-nothing: validate every page before anything is enqueued.
  for (uint32_t i = 0; i < n; ++i) {
    if (pages[i] >= s->page_count) return fail(KVX_ERANGE, "invalid KV page id");
    if (!s->extents[pages[i] / s->extent_pages])
      return fail(KVX_ESTATE, "KV page of an extent that is not allocated");
  }
  if (!to_wire) {
    std::vector<uint32_t> sorted(pages, pages + n);
    std::sort(sorted.begin(), sorted.end());
    if (std::adjacent_find(sorted.begin(), sorted.end()) != sorted.end())
      return fail(KVX_EINVAL, "two imported pages share a destination");
  }
  const uint32_t span = std::max(s->data_bytes, s->scale_bytes);
  const uint32_t chunks = (span + kCopyChunk - 1) / kCopyChunk;
  const uint64_t page_bytes = kvx_storage_bytes_per_page(s);
  for (uint32_t first = 0; first < n; first += kCopiesPerLaunch) {
    WireArgs a{};
    const uint32_t count = std::min(kCopiesPerLaunch, n - first);
    a.buffer = static_cast<uint8_t *>(buffer) + uint64_t(first) * page_bytes;
    a.extent_pages = s->extent_pages;
    a.data_bytes = s->data_bytes;
    a.scale_bytes = s->scale_bytes;
    a.layers = s->layout.layers;
    for (uint32_t i = 0; i < count; ++i) {
      const uint32_t page = pages[first + i];
      a.page[i] = reinterpret_cast<uint64_t>(s->extents[page / s->extent_pages]) | (page % s->extent_pages);
    }
    const dim3 grid(chunks, s->layout.layers * 4, count);
    if (to_wire)
      hipLaunchKernelGGL(page_wire_kernel<true>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a);
    else
      hipLaunchKernelGGL(page_wire_kernel<false>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a);
    if (int rc = check_launch("page_wire_kernel")) return rc;
  }
  return KVX_OK;
}

int kv_page_export(const kvx_storage *s, const uint32_t *pages, uint32_t n, void *buffer,
                   void *stream) {
  return page_wire(s, pages, n, buffer, true, stream);
}
int kv_page_import(kvx_storage *s, const uint32_t *pages, uint32_t n, const void *buffer,
                   void *stream) {
  return page_wire(s, pages, n, const_cast<void *>(buffer), false, stream);
}

}  // extern "C"
