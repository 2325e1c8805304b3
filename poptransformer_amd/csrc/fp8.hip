// FP8 path: Graphcore F143 / F152 bytes with a power-of-two QuarterMetadata scale.
//
// Reference: poptransformer/ops/customized.py:127-148 (half_to_uint8, fp8_matmul),
// custom_ops/cast_to_uint8.cpp:107-127, custom_ops/matmul_fp8.cpp:177-250,885-1003,
// poptransformer/utils/param_handler/precision_strategy.py:44-51,62-81.
//
// Formats: F143 = 1-4-3, bias 8, NaN 0x80, max 240; F152 = 1-5-2, bias 16, NaN 0x80, max 57344
// (the fnuz encodings); real value = decode(byte) * 2^scale.  Every decoded value is exactly
// representable in fp16, so a product of two FP8 operands is computed exactly by decoding both
// to fp16 and using the fp16 MFMA with fp32 accumulation; the two scales are applied to the
// fp32 sum as one power of two.  The OCP e4m3/e5m2 encodings that the fp8 MFMA of this target
// reads give twice the value of the same F143/F152 byte but turn 0x7F/0xFF (+-240, the
// saturation code) into NaN, so the fp16 route is the one that is exact for every byte.
#include "common.h"
#include "gemm_core.h"

// ------------------------------------------------------------------------------------------
// scalar codecs
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

template <int FMT>
__global__ __launch_bounds__(256) void f8_encode_kernel(const f16* __restrict__ x, uint8_t* __restrict__ out,
                                                        const int32_t* __restrict__ scale, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  out[i] = F8<FMT>::encode(ldexpf((float)x[i], -scale[0]));
}

template <int FMT>
__global__ __launch_bounds__(256) void f8_decode_kernel(const uint8_t* __restrict__ in, f16* __restrict__ out,
                                                        const int32_t* __restrict__ scale, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  out[i] = (f16)ldexpf(F8<FMT>::decode(in[i]), scale[0]);
}

static int parse_format(int fmt, const char* name) {
  // "Unsupport fp8 meata data ..., it must be F143 or F152" (custom_ops/cast_to_uint8.cpp:86-93)
  PTA_REQUIRE(fmt == PTA_F143 || fmt == PTA_F152, "%s: unsupported fp8 format %d, it must be F143 or F152", name, fmt);
  return PTA_OK;
}

extern "C" int pta_half_to_fp8(const pta_half* x, uint8_t* out, const int32_t* scale, size_t n, int format,
                               pta_stream_t stream) {
  int rc = parse_format(format, "pta_half_to_fp8");
  if (rc) return rc;
  PTA_REQUIRE(x && out && scale, "pta_half_to_fp8: null pointer");
  if (n == 0) return PTA_OK;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (format == PTA_F143)
    hipLaunchKernelGGL(f8_encode_kernel<0>, grid, dim3(256), 0, (hipStream_t)stream, (const f16*)x, out, scale, n);
  else
    hipLaunchKernelGGL(f8_encode_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, (const f16*)x, out, scale, n);
  PTA_CHECK_LAUNCH("pta_half_to_fp8");
  return PTA_OK;
}

extern "C" int pta_fp8_to_half(const uint8_t* in, pta_half* out, const int32_t* scale, size_t n, int format,
                               pta_stream_t stream) {
  int rc = parse_format(format, "pta_fp8_to_half");
  if (rc) return rc;
  PTA_REQUIRE(in && out && scale, "pta_fp8_to_half: null pointer");
  if (n == 0) return PTA_OK;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (format == PTA_F143)
    hipLaunchKernelGGL(f8_decode_kernel<0>, grid, dim3(256), 0, (hipStream_t)stream, in, (f16*)out, scale, n);
  else
    hipLaunchKernelGGL(f8_decode_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, in, (f16*)out, scale, n);
  PTA_CHECK_LAUNCH("pta_fp8_to_half");
  return PTA_OK;
}

// ------------------------------------------------------------------------------------------
// tiling: 16 output channels x 128 input features = 2 vectors of 1 KiB; in vector v lane l holds
// 16 bytes: features kt*128 + j*32 + (l/16)*8 + 0..7 of channel l%16 for j = 2v (bytes 0..7)
// and j = 2v+1 (bytes 8..15).
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void f8_tile_kernel(const uint8_t* __restrict__ w, u32x4* __restrict__ tiled, int N,
                                                      int K, int KT, int w_is_kn, size_t total_vec) {
  const size_t vi = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (vi >= total_vec) return;
  const int lane = (int)(vi & 63);
  const int v = (int)((vi >> 6) & 1);
  const size_t tile = vi >> 7;
  const int kt = (int)(tile % KT);
  const int nb = (int)(tile / KT);
  const int row = nb * 16 + (lane & 15);
  uint8_t b[16];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int k0 = kt * 128 + (2 * v + h) * 32 + (lane >> 4) * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + i;
      uint8_t c = 0;
      if (row < N && k < K) c = w_is_kn ? w[(size_t)k * N + row] : w[(size_t)row * K + k];
      b[h * 8 + i] = c;
    }
  }
  u32x4 o;
#pragma unroll
  for (int d = 0; d < 4; ++d)
    o[d] = (uint32_t)b[4 * d] | ((uint32_t)b[4 * d + 1] << 8) | ((uint32_t)b[4 * d + 2] << 16) | ((uint32_t)b[4 * d + 3] << 24);
  tiled[vi] = o;
}

extern "C" size_t pta_fp8_tiled_bytes(int N, int K) { return gemv_tiled_bytes(N, K, 2); }

extern "C" int pta_fp8_tile(const uint8_t* w, void* tiled, int N, int K, int w_is_kn, pta_stream_t stream) {
  PTA_REQUIRE(w && tiled, "pta_fp8_tile: null pointer");
  PTA_REQUIRE(N > 0 && K > 0, "pta_fp8_tile: need N > 0 and K > 0, got N=%d K=%d", N, K);
  PTA_REQUIRE(pta_aligned(tiled, 16), "pta_fp8_tile: tiled buffer must be 16-byte aligned");
  const int KT = (K + 127) / 128;
  const size_t total = pta_fp8_tiled_bytes(N, K) / 16;
  hipLaunchKernelGGL(f8_tile_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, w,
                     (u32x4*)tiled, N, K, KT, w_is_kn, total);
  PTA_CHECK_LAUNCH("pta_fp8_tile");
  return PTA_OK;
}

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
  static __device__ __forceinline__ Scale load_scale(const void* scale, int, int) {
    // scale points at {int32 exponent of the weight, int32 exponent of the activations (0 for fp16)}
    const int32_t* s = reinterpret_cast<const int32_t*>(scale);
    return Scale{ldexpf(1.0f, s[0] + s[1])};
  }
  static __device__ __forceinline__ f16x8 a_operand(const u32x4 (&raw)[2], int j, Scale) {
    const uint32_t lo = raw[j >> 1][(j & 1) * 2], hi = raw[j >> 1][(j & 1) * 2 + 1];
    return FMT == 0 ? f143_decode8(lo, hi) : f152_decode8(lo, hi);
  }
  static __device__ __forceinline__ float finish(float acc, Scale s) { return acc * s.mul; }
};

// 0x80 decodes to NaN in both formats; the in-register decoders above map it to -0, so tensors are
// screened for it when they are tiled (weights) or produced (activations never hold it: the
// encoder emits 0x80 only for a NaN input).

// Scales live in device memory (they are graph tensors in the reference); a tiny kernel gathers
// the two exponents next to each other for the GEMM to read.
__global__ void f8_scale_pair_kernel(const int32_t* w_scale, const int32_t* x_scale, int32_t* pair) {
  pair[0] = w_scale[0];
  pair[1] = x_scale ? x_scale[0] : 0;
}

// lhs fp8 -> fp16 (unscaled decode) into a caller-provided buffer, for the fp8 x fp8 form.
template <int FMT>
__global__ __launch_bounds__(256) void f8_decode_unscaled_kernel(const uint8_t* __restrict__ in, f16* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  out[i] = (f16)F8<FMT>::decode(in[i]);
}

extern "C" size_t pta_fp8_gemm_workspace_bytes(int M, int K) {
  if (M <= 0 || K <= 0) return 0;
  return 16 + (size_t)M * K * 2;     // scale pair + decoded left-hand side
}

extern "C" int pta_fp8_gemm(const void* lhs, int lhs_is_fp8, const void* tiled_rhs, pta_half* Y, int M, int K, int N,
                            int format_lhs, int format_rhs, const int32_t* scale_lhs, const int32_t* scale_rhs,
                            void* workspace, const pta_fusion* fuse, pta_stream_t stream) {
  int rc = parse_format(format_rhs, "pta_fp8_gemm");
  if (rc) return rc;
  if (lhs_is_fp8) { rc = parse_format(format_lhs, "pta_fp8_gemm"); if (rc) return rc; }
  PTA_REQUIRE(lhs && tiled_rhs && Y && scale_rhs && workspace, "pta_fp8_gemm: null pointer");
  PTA_REQUIRE(!lhs_is_fp8 || scale_lhs, "pta_fp8_gemm: an fp8 left-hand side needs its scale");
  PTA_REQUIRE(pta_aligned(workspace, 16) && pta_aligned(tiled_rhs, 16), "pta_fp8_gemm: workspace and weights must be 16-byte aligned");
  PTA_REQUIRE(N > 0, "pta_fp8_gemm: N = %d", N);
  hipStream_t s = (hipStream_t)stream;
  int32_t* pair = reinterpret_cast<int32_t*>(workspace);
  const f16* X = (const f16*)lhs;
  hipLaunchKernelGGL(f8_scale_pair_kernel, dim3(1), dim3(1), 0, s, scale_rhs, lhs_is_fp8 ? scale_lhs : nullptr, pair);
  if (lhs_is_fp8) {
    f16* xd = reinterpret_cast<f16*>(reinterpret_cast<char*>(workspace) + 16);
    const size_t n = (size_t)M * K;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (format_lhs == PTA_F143)
      hipLaunchKernelGGL(f8_decode_unscaled_kernel<0>, grid, dim3(256), 0, s, (const uint8_t*)lhs, xd, n);
    else
      hipLaunchKernelGGL(f8_decode_unscaled_kernel<1>, grid, dim3(256), 0, s, (const uint8_t*)lhs, xd, n);
    X = xd;
  }
  rc = check_gemv_common("pta_fp8_gemm", X, M, K);
  if (rc) return rc;
  GemmArgs a{};
  a.count = 1; a.X = X; a.M = M; a.K = K; a.KT = (K + 127) / 128;
  a.mat[0] = GemmMat{tiled_rhs, pair, (f16*)Y, N, 0};
  rc = make_epilogue(fuse, &a.epi, "pta_fp8_gemm");
  if (rc) return rc;
  if (format_rhs == PTA_F143) return dispatch_gemv<FmtF8<0>, false>(a, (N + 15) / 16, s, "pta_fp8_gemm");
  return dispatch_gemv<FmtF8<1>, false>(a, (N + 15) / 16, s, "pta_fp8_gemm");
}
