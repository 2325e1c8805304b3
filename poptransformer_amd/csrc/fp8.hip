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
#include "formats.h"

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

// One flag byte per tile behind the tiles: nonzero when the tile holds one of the three codes whose F143 value is not
// half of the OCP e4m3 value of the same bits (0x7F, 0xFF: +-240 against NaN; 0x80: NaN against -0).  The kernels that
// feed the bytes to the FP8 matrix instruction multiply such a tile the exact way instead (gemm_f8n.h).
__global__ __launch_bounds__(64) void f8_tile_flags_kernel(const u32x4* __restrict__ tiled, uint8_t* __restrict__ flags,
                                                           size_t tiles) {
  const size_t tile = blockIdx.x;
  if (tile >= tiles) return;
  bool special = false;
#pragma unroll
  for (int v = 0; v < 2; ++v) {
    const u32x4 w = tiled[(tile * 2 + v) * 64 + threadIdx.x];
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t b = (w[d] >> (8 * i)) & 0xFFu;
        special = special || b == 0x7Fu || b == 0xFFu || b == 0x80u;
      }
  }
  const bool any = __any(special);
  if (threadIdx.x == 0) flags[tile] = any ? 1 : 0;
}

extern "C" size_t pta_fp8_tiled_bytes(int N, int K) {
  const size_t tiles = gemv_tiled_bytes(N, K, 2);
  if (tiles == 0) return 0;
  return tiles + ((tiles / 2048 + 15) & ~(size_t)15);
}

extern "C" int pta_fp8_tile(const uint8_t* w, void* tiled, int N, int K, int w_is_kn, pta_stream_t stream) {
  PTA_REQUIRE(w && tiled, "pta_fp8_tile: null pointer");
  PTA_REQUIRE(N > 0 && K > 0, "pta_fp8_tile: need N > 0 and K > 0, got N=%d K=%d", N, K);
  PTA_REQUIRE(pta_aligned(tiled, 16), "pta_fp8_tile: tiled buffer must be 16-byte aligned");
  const int KT = (K + 127) / 128;
  const size_t tile_bytes = gemv_tiled_bytes(N, K, 2);
  const size_t total = tile_bytes / 16;
  hipLaunchKernelGGL(f8_tile_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, w,
                     (u32x4*)tiled, N, K, KT, w_is_kn, total);
  hipLaunchKernelGGL(f8_tile_flags_kernel, dim3((unsigned)(tile_bytes / 2048)), dim3(64), 0, (hipStream_t)stream,
                     (const u32x4*)tiled, (uint8_t*)tiled + tile_bytes, tile_bytes / 2048);
  PTA_CHECK_LAUNCH("pta_fp8_tile");
  return PTA_OK;
}

// ------------------------------------------------------------------------------------------
// fp16 values on the FP8 grid (decode without the scale): what an FP8 operand contributes to a
// product before the power-of-two scale is applied.
// ------------------------------------------------------------------------------------------
template <int FMT>
__global__ __launch_bounds__(256) void f8_decode_unscaled_kernel(const uint8_t* __restrict__ in, f16* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  out[i] = (f16)F8<FMT>::decode(in[i]);
}

template <int FMT>
__global__ __launch_bounds__(256) void f8_grid_kernel(const f16* __restrict__ x, f16* __restrict__ out,
                                                      const int32_t* __restrict__ scale, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  out[i] = (f16)F8<FMT>::decode(F8<FMT>::encode(ldexpf((float)x[i], -scale[0])));
}

int f8_decode_unscaled_launch(const uint8_t* in, f16* out, size_t n, int format, hipStream_t s) {
  const dim3 grid((unsigned)((n + 255) / 256));
  if (format == PTA_F143) hipLaunchKernelGGL(f8_decode_unscaled_kernel<0>, grid, dim3(256), 0, s, in, out, n);
  else hipLaunchKernelGGL(f8_decode_unscaled_kernel<1>, grid, dim3(256), 0, s, in, out, n);
  return PTA_OK;
}

extern "C" int pta_half_to_fp8_grid(const pta_half* x, pta_half* out, const int32_t* scale, size_t n, int format,
                                    pta_stream_t stream) {
  int rc = parse_format(format, "pta_half_to_fp8_grid");
  if (rc) return rc;
  PTA_REQUIRE(x && out && scale, "pta_half_to_fp8_grid: null pointer");
  if (n == 0) return PTA_OK;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (format == PTA_F143)
    hipLaunchKernelGGL(f8_grid_kernel<0>, grid, dim3(256), 0, (hipStream_t)stream, (const f16*)x, (f16*)out, scale, n);
  else
    hipLaunchKernelGGL(f8_grid_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, (const f16*)x, (f16*)out, scale, n);
  PTA_CHECK_LAUNCH("pta_half_to_fp8_grid");
  return PTA_OK;
}
