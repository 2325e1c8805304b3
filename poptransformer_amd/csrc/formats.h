// Weight formats of the small-M GEMM core (gemm_core.h): how a tile is laid out and how its
// bytes become the fp16 A operand of the MFMA.
#pragma once
#include "gemm_core.h"

// ------------------------------------------------------------------------------------------
// Fused W4A16 GEMV/GEMM.
// ------------------------------------------------------------------------------------------

// The four dwords of a lane -> the 8 fp16 weights of MFMA step m (features m*32 + (l/16)*8 + 0..7
// of channel l%16), each fp16(q * s) with a single rounding (the product of an integer in [-8, 7]
// held exactly in fp16 and the fp16 scale), which is what the reference's `half(nibble) * scale`
// computes.  Dword d holds features 2d (low half) and 2d + 1 (high half) of every step, step m in
// nibble m of each half, stored offset-binary (q + 8).
// (a & mask) | orv in one VALU instruction.  The mask travels in an SGPR and the OR value in a
// VGPR: a VOP3 encoding on this target takes no literal and at most one scalar operand.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t orv) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(orv));
  return r;
}

__device__ __forceinline__ f16x8 dequant_step(u32x4 w, int m, f16x2 s2) {
  const uint32_t MAGIC = 0x64006400u;  // fp16 1024.0 in both halves
  const f16x2 c1032 = {(f16)1032.0f, (f16)1032.0f};
  const f16x2 c16th = {(f16)0.0625f, (f16)0.0625f};
  const f16x2 c72 = {(f16)-72.0f, (f16)-72.0f};
  f16x8 r;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const uint32_t wd = m >= 2 ? w[d] >> 8 : w[d];
    f16x2 p;
    if (m & 1) {
      p = bitcast<f16x2>(and_or(wd, 0x00f000f0u, MAGIC));       // 1024 + 16 u
      p = __builtin_elementwise_fma(p, c16th, c72) * s2;        // (1024 + 16u)/16 - 72 = u - 8, exact; one rounding
    } else {
      p = bitcast<f16x2>(and_or(wd, 0x000f000fu, MAGIC));       // 1024 + u
      p = (p - c1032) * s2;                                     // exact integer, then one rounding
    }
    r[2 * d] = p[0];
    r[2 * d + 1] = p[1];
  }
  return r;
}


struct FmtW4 {
  static constexpr int kVec = 1;
  typedef f16x2 Scale;
  static __device__ __forceinline__ Scale load_scale(const void* scale, const int32_t*, int row, int N) {
    const f16 v = reinterpret_cast<const f16*>(scale)[row < N ? row : N - 1];      // (a load without a branch round it)
    const f16 s = row < N ? v : (f16)0.0f;
    return f16x2{s, s};
  }
  static __device__ __forceinline__ f16x8 a_operand(const u32x4 (&raw)[1], int j, Scale s) {
    return dequant_step(raw[0], j, s);
  }
  static __device__ __forceinline__ float finish(float acc, Scale) { return acc; }
};


// Tile = 16 output channels x 128 input features = 4 vectors of 1 KiB; in vector j lane l holds
// the 8 consecutive features  kt*128 + j*32 + (l/16)*8 + 0..7  of channel l%16, which is the
// A operand of one 16x16x32 MFMA as it stands.
struct FmtF16 {
  static constexpr int kVec = 4;
  struct Scale {};
  static __device__ __forceinline__ Scale load_scale(const void*, const int32_t*, int, int) { return Scale{}; }
  static __device__ __forceinline__ f16x8 a_operand(const u32x4 (&raw)[4], int j, Scale) {
    return bitcast<f16x8>(raw[j]);
  }
  static __device__ __forceinline__ float finish(float acc, Scale) { return acc; }
};


// ------------------------------------------------------------------------------------------
// in-register decode of 4 bytes to 4 fp16 values carrying decode(byte) * 2^-7 (F143) or
// decode(byte) * 2^-1 ... see the constants below; the missing power of two joins the scale.
// ------------------------------------------------------------------------------------------
// F143: moving the 7 magnitude bits to fp16 bits 13..7 yields exponent field e and the mantissa in
// the top three mantissa bits: the fp16 value is decode * 2^(8-15) for normals and subnormals
// alike (an F143 subnormal becomes an fp16 subnormal).  One fp16 multiply by 2^7 (exact) brings
// it to decode(byte) and leaves no subnormal operand for the matrix unit.
__device__ __forceinline__ f16x2 f143_pair(uint32_t t /* byte a in bits 15..8, byte b in bits 31..24 */) {
  uint32_t mag;
  const uint32_t sign = t & 0x80008000u;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(mag) : "v"(t >> 1), "s"(0x3F803F80u), "v"(sign));
  const f16x2 k = {(f16)128.0f, (f16)128.0f};
  return bitcast<f16x2>(mag) * k;
}

__device__ __forceinline__ f16x8 f143_decode8(uint32_t lo, uint32_t hi) {
  f16x2 p0 = f143_pair(__builtin_amdgcn_perm(0, lo, 0x010C000Cu));
  f16x2 p1 = f143_pair(__builtin_amdgcn_perm(0, lo, 0x030C020Cu));
  f16x2 p2 = f143_pair(__builtin_amdgcn_perm(0, hi, 0x010C000Cu));
  f16x2 p3 = f143_pair(__builtin_amdgcn_perm(0, hi, 0x030C020Cu));
  f16x8 r;
  r[0] = p0[0]; r[1] = p0[1]; r[2] = p1[0]; r[3] = p1[1];
  r[4] = p2[0]; r[5] = p2[1]; r[6] = p3[0]; r[7] = p3[1];
  return r;
}

// F152 goes through arithmetic on the fields (exponent 31 is a finite binade here, so the byte
// cannot simply be widened): values are produced as decode(byte) exactly.
__device__ __forceinline__ f16 f152_one(uint32_t c) {
  const uint32_t e = (c >> 2) & 31u, m = c & 3u;
  // decode = 2^(e-16) (1 + m/4), e >= 1; 2^-15 m/4, e == 0.  As fp16 (bias 15): exponent field
  // e - 1 with mantissa m << 8 when e >= 2; subnormal patterns below that.
  uint32_t bits;
  if (e >= 2) bits = ((e - 1) << 10) | (m << 8);
  else if (e == 1) bits = 0x200u | (m << 7);      // 2^-15 (1 + m/4) = 2^-14 * (512 + 128 m)/1024
  else bits = m << 7;                              // 2^-15 m/4      = 2^-14 * (128 m)/1024
  bits |= (c & 0x80u) << 8;
  return bitcast<f16>((uint16_t)bits);
}

__device__ __forceinline__ f16x8 f152_decode8(uint32_t lo, uint32_t hi) {
  f16x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) { r[i] = f152_one((lo >> (8 * i)) & 0xFF); r[4 + i] = f152_one((hi >> (8 * i)) & 0xFF); }
  return r;
}

struct F8Scale { float mul; };

template <int FMT>
struct FmtF8 {
  static constexpr int kVec = 2;
  typedef F8Scale Scale;
  static __device__ __forceinline__ Scale load_scale(const void* scale, const int32_t* x_scale, int, int) {
    const int e = reinterpret_cast<const int32_t*>(scale)[0] + (x_scale ? x_scale[0] : 0);
    return Scale{ldexpf(1.0f, e)};
  }
  static __device__ __forceinline__ f16x8 a_operand(const u32x4 (&raw)[2], int j, Scale) {
    const uint32_t lo = raw[j >> 1][(j & 1) * 2], hi = raw[j >> 1][(j & 1) * 2 + 1];
    return FMT == 0 ? f143_decode8(lo, hi) : f152_decode8(lo, hi);
  }
  static __device__ __forceinline__ float finish(float acc, Scale s) { return acc * s.mul; }
};

