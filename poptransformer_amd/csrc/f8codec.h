// Scalar codecs of the Graphcore FP8 formats (F143 / F152 bytes with a power-of-two scale), shared by the
// cast kernels, the FP8 KV cache and the epilogues that leave their result on the FP8 grid.
//
// Reference: custom_ops/cast_to_uint8.cpp:107-127 (CastToUint8), custom_ops/matmul_fp8.cpp:904-930 and
// custom_ops/kv_cache.cpp:56-74 (the cast back).
#pragma once
#include "common.h"

// ------------------------------------------------------------------------------------------
// scalar FP8 codecs (F143 / F152 bytes, see fp8.hip)
// ------------------------------------------------------------------------------------------
template <int FMT>  // 0 = F143, 1 = F152
struct F8 {
  static constexpr int MB = FMT == 0 ? 3 : 2;
  static constexpr int BIAS = FMT == 0 ? 8 : 16;
  static constexpr int EMAX = FMT == 0 ? 15 : 31;
  static __device__ __forceinline__ float max_value() { return FMT == 0 ? 240.0f : 57344.0f; }

  static __device__ __forceinline__ float decode(uint8_t c) {
    if (c == 0x80) return __builtin_nanf("");
    const int e = (c & 0x7F) >> MB, m = c & ((1 << MB) - 1);
    const float mag = e == 0 ? ldexpf((float)m, 1 - BIAS - MB) : ldexpf((float)((1 << MB) + m), e - BIAS - MB);
    return (c & 0x80) ? -mag : mag;
  }

  // round to nearest even on the format's grid, saturating; v is the already descaled value
  static __device__ __forceinline__ uint8_t encode(float v) {
    if (v != v) return 0x80;
    const float mag = fabsf(v);
    if (mag == 0.0f) return 0;             // no negative zero in these formats
    if (mag >= max_value()) return (v < 0 ? 0x80 : 0) | 0x7F;
    int e;
    (void)frexpf(mag, &e);                 // mag = f * 2^e, f in [0.5, 1)
    int ef = e - 1 + BIAS;                 // biased exponent of the format
    if (ef < 1) ef = 1;                    // subnormal range shares the grid of exponent 1
    const float q = ldexpf(mag, MB - (ef - BIAS));   // value in units of the grid step
    float r = rintf(q);                    // ties to even
    int code;
    if (ef == 1 && r < (float)(1 << MB)) code = (int)r;                    // subnormal (or zero)
    else {
      if (r >= (float)(2 << MB)) { r *= 0.5f; ef += 1; }                   // rounded up to the next binade
      code = (ef << MB) | ((int)r - (1 << MB));
      if (code > 0x7F) code = 0x7F;
    }
    return (uint8_t)((v < 0 && code != 0) ? (code | 0x80) : code);
  }
};

// decode(encode(v)) without going through the byte: round |v| to the format's grid (MB mantissa bits,
// nearest, ties to even, directly on the fp32 bits; below the smallest normal the grid is uniform),
// saturate at the largest value, NaN stays NaN, and a result of zero is +0 (the formats have no -0).
template <int FMT>
__device__ __forceinline__ float f8_grid_round(float v) {
  constexpr int MB = F8<FMT>::MB, BIAS = F8<FMT>::BIAS;
  const float a = fabsf(v);
  float r;
  if (a >= __builtin_ldexpf(1.0f, 1 - BIAS)) {
    uint32_t b = __builtin_bit_cast(uint32_t, a);
    b += ((1u << (22 - MB)) - 1u) + ((b >> (23 - MB)) & 1u);
    b &= ~((1u << (23 - MB)) - 1u);
    r = __builtin_bit_cast(float, b);
  } else {
    r = rintf(a * __builtin_ldexpf(1.0f, BIAS - 1 + MB)) * __builtin_ldexpf(1.0f, 1 - BIAS - MB);
  }
  r = fminf(r, F8<FMT>::max_value());
  if (v != v) return v;
  return r == 0.0f ? 0.0f : copysignf(r, v);
}

// fp16 value of x on the grid of format `fmt` at exponent `scale`, WITHOUT the scale:
// decode(encode(x * 2^-scale)) - what half_to_uint8 followed by fp8_matmul makes of an activation
// (utils/param_handler/precision_strategy.py:62-66) before the power of two is applied.
__device__ __forceinline__ f16 f8_grid_value(f16 x, int scale, int fmt) {
  const float v = ldexpf((float)x, -scale);
  return fmt == PTA_F143 ? (f16)f8_grid_round<0>(v) : (f16)f8_grid_round<1>(v);
}
