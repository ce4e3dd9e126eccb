// FP8 (OCP E4M3FN: 1 sign, 4 exponent bits with bias 7, 3 mantissa bits; largest finite value
// 448, no infinities, S.1111.111 is NaN) storage of K/V rows with one fp32 scale per kv head:
//     stored code = e4m3(clamp(x / scale, -448, 448))   round to nearest even
//     value used  = decode(code) * scale
// gfx950 converts both ways in hardware. Decoding to fp16 is exact (every E4M3 value, subnormals
// included, is an fp16 number), so attention over an fp8 pool is fp16 attention over the decoded
// values: the K scale folds into the softmax scale and the V scale into the final normalisation.
#pragma once

#include "common.h"

namespace litekv {

typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr float kFp8Max = 448.0f;

// Eight codes (byte i of the pair = element i) -> eight fp16 values, exact.
__device__ __forceinline__ half8_t fp8x8_to_half(uint2_t codes) {
  const half2_t a = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)codes[0], 1.0f, false);
  const half2_t b = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)codes[0], 1.0f, true);
  const half2_t c = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)codes[1], 1.0f, false);
  const half2_t d = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)codes[1], 1.0f, true);
  return half8_t{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

__device__ __forceinline__ float clamp_fp8(float x) {
  return __builtin_fminf(__builtin_fmaxf(x, -kFp8Max), kFp8Max);  // NaN stays out: inputs are finite
}

// Eight fp16 values times `inv_scale` -> eight codes.
__device__ __forceinline__ uint2_t half8_to_fp8(half8_t x, float inv_scale) {
  float f[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = clamp_fp8((float)x[i] * inv_scale);
  int lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
  int hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
  return uint2_t{(uint32_t)lo, (uint32_t)hi};
}

// ---- int8 storage -----------------------------------------------------------------------------
// The same pools and scales with signed 8-bit codes:
//     stored code = clamp(round_to_nearest_even(x / scale), -127, 127)
//     value used  = code * scale
// Every code is an fp16 number, so attention over an int8 pool is fp16 attention over the codes
// with the scales folded in where the fp8 pool folds them.

// Eight codes -> eight fp16 values, exact: byte c ^ 0x80 = c + 128 under the exponent byte of
// 1024.0 is the fp16 number 1024 + 128 + c, and 1152 is subtracted from pairs.
__device__ __forceinline__ half8_t int8x8_to_half(uint2_t codes) {
  const half2_t bias = half2_t{(_Float16)1152.0f, (_Float16)1152.0f};
  half2_t h[4];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const uint32_t x = codes[w] ^ 0x80808080u;
    h[2 * w] = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u)) - bias;
    h[2 * w + 1] = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u)) - bias;
  }
  return half8_t{h[0][0], h[0][1], h[1][0], h[1][1], h[2][0], h[2][1], h[3][0], h[3][1]};
}

// Eight fp16 values times `inv_scale` -> eight codes.
__device__ __forceinline__ uint2_t half8_to_int8(half8_t x, float inv_scale) {
  uint32_t w[2] = {0u, 0u};
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float f = __builtin_rintf((float)x[i] * inv_scale);  // v_rndne_f32: halves go to the even integer
    f = __builtin_fminf(__builtin_fmaxf(f, -127.0f), 127.0f);
    w[i >> 2] |= ((uint32_t)(int)f & 0xffu) << (8 * (i & 3));
  }
  return uint2_t{w[0], w[1]};
}

// The storage formats of a pool, as template arguments of the kernels that read or write one.
constexpr int kKvF16 = 0, kKvFp8 = 1, kKvInt8 = 2;

template <int KV>
__device__ __forceinline__ half8_t codes_to_half(uint2_t codes) {
  static_assert(KV == kKvFp8 || KV == kKvInt8, "an 8-bit format");
  if constexpr (KV == kKvInt8) {
    return int8x8_to_half(codes);
  } else {
    return fp8x8_to_half(codes);
  }
}
template <int KV>
__device__ __forceinline__ uint2_t half_to_codes(half8_t x, float inv_scale) {
  static_assert(KV == kKvFp8 || KV == kKvInt8, "an 8-bit format");
  if constexpr (KV == kKvInt8) {
    return half8_to_int8(x, inv_scale);
  } else {
    return half8_to_fp8(x, inv_scale);
  }
}

}  // namespace litekv
