// Device-side helpers shared by the kernels: codecs and exact (unfused) fp32
// arithmetic.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "kvx_internal.h"

namespace kvx {

__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
  return __uint_as_float(uint32_t(b) << 16);
}

// Round to nearest even; NaN payloads that live only in the low half keep a
// mantissa bit so the result stays a NaN.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  const uint32_t bits = __float_as_uint(f);
  if ((bits & 0x7f800000u) == 0x7f800000u) {
    uint32_t upper = bits >> 16;
    if ((bits & 0x007fffffu) && !(upper & 0x7fu)) upper |= 1u;
    return uint16_t(upper);
  }
  return uint16_t((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }
// The logistic sigmoid as the reference's kernels take it, 1 / (1 + 2^(-x log2 e))
// (reference: common/activation.h:14-16).
__device__ __forceinline__ float sigmoid(float x) {
  return __fdiv_rn(1.0f, __fadd_rn(1.0f, exp2f(__fmul_rn(-1.44269504089f, x))));
}
__device__ __forceinline__ float round_f16(float f) { return float(_Float16(f)); }

// OCP e4m3 (bias 7, no infinities, 0x7f NaN): round to nearest even, saturate
// at 448, subnormal step 2^-9.  Integer/exact-scaling arithmetic only, so the
// code equals the CPU encoder's for every input.
__device__ __forceinline__ uint32_t f32_to_e4m3(float v) {
  const uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
  const float a = fabsf(v);
  if (!(a <= 3.4028234663852886e38f)) return sign | 0x7fu;  // inf or NaN
  if (a >= 512.0f) return sign | 0x7eu;
  if (a < 0.015625f) {
    const int m = int(rintf(a * 512.0f));
    return sign | uint32_t(m < 8 ? m : 8);
  }
  int e = int((__float_as_uint(a) >> 23) & 0xffu) - 127;
  int m = int(rintf(ldexpf(a, 3 - e)));  // 8..16
  if (m == 16) {
    ++e;
    m = 8;
  }
  if (e > 8 || (e == 8 && m > 14)) return sign | 0x7eu;
  return sign | uint32_t((e + 7) << 3) | uint32_t(m - 8);
}

__device__ __forceinline__ float e4m3_to_f32(uint32_t c) {
  const int e = int(c >> 3) & 0xf, m = int(c) & 7;
  float mag;
  if (e == 0) mag = ldexpf(float(m), -9);
  else if (e == 15 && m == 7) mag = __uint_as_float(0x7fc00000u);
  else mag = ldexpf(1.0f + float(m) * 0.125f, e - 7);
  return (c & 0x80u) ? -mag : mag;
}

__device__ __forceinline__ int nibble_code(uint32_t byte, uint32_t hi) {
  const int code = int(byte >> (hi * 4)) & 0xf;
  return code - ((code & 8) << 1);
}

// A key / value element of a head's slab as the float its code stands for
// (before the per-token scale).  Keys are token-major; values dimension-major
// except for packed int4, whose values are token-major like the keys.
template <uint32_t FMT>
__device__ __forceinline__ float load_key_code(const uint8_t *keys, uint32_t head_dim,
                                               uint32_t token, uint32_t d) {
  const uint32_t e = token * head_dim + d;
  if constexpr (FMT == KVX_FMT_INT8) return float(reinterpret_cast<const int8_t *>(keys)[e]);
  else if constexpr (FMT == KVX_FMT_INT4) return float(nibble_code(keys[e >> 1], e & 1));
  else if constexpr (FMT == KVX_FMT_FP8E4M3) return e4m3_to_f32(keys[e]);
  else return bf16_to_f32(reinterpret_cast<const uint16_t *>(keys)[e]);
}
template <uint32_t FMT>
__device__ __forceinline__ float load_value_code(const uint8_t *values, uint32_t head_dim,
                                                 uint32_t token, uint32_t d) {
  if constexpr (FMT == KVX_FMT_INT4) {
    const uint32_t e = token * head_dim + d;
    return float(nibble_code(values[e >> 1], e & 1));
  } else {
    const uint32_t e = d * KVX_PAGE_TOKENS + token;
    if constexpr (FMT == KVX_FMT_INT8) return float(reinterpret_cast<const int8_t *>(values)[e]);
    else if constexpr (FMT == KVX_FMT_FP8E4M3) return e4m3_to_f32(values[e]);
    else return bf16_to_f32(reinterpret_cast<const uint16_t *>(values)[e]);
  }
}

__device__ __forceinline__ float default_score_scale(uint32_t head_dim, float requested) {
  if (requested != 0.0f) return requested;
  return head_dim == 64 ? 0.125f : head_dim == 128 ? 0.08838834764831845f : 0.0625f;
}

}  // namespace kvx
