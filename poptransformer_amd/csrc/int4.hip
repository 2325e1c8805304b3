// INT4 weight path: exact Int4ToHalf, load-time tiling, and the fused
// dequantise-in-register W4A16 GEMV/GEMM built on the gfx950 16x16x32 fp16 MFMA.
//
// Reference semantics: custom_ops/int4_to_half_codelets.cpp:18-74 (nibble extraction),
// custom_ops/int4_to_half_custom_op.cpp:139-149 (the 256x2 truth table), :362-378 (layout of
// the axis=1 result and the fp16 multiply by the per-channel scale),
// poptransformer/utils/param_handler/precision_strategy.py:56-60,74-75 (unpack then MatMul).
#include "common.h"
#include "formats.h"

// ------------------------------------------------------------------------------------------
// Int4ToHalf, standalone and bit-exact.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ int nib_hi(int8_t b) { return ((int)b) >> 4; }
__device__ __forceinline__ int nib_lo(int8_t b) { return ((int)(int8_t)((uint8_t)b << 4)) >> 4; }

// axis == 1: out[2j + h, r] = nib_h(P[r, j]) * scale[r]; out is [2m, n].
// A 64x64-byte tile of P goes through LDS so that both the reads of P (along j) and the
// writes of out (along r) are coalesced.
__global__ __launch_bounds__(256) void int4_to_half_axis1_kernel(const int8_t* __restrict__ P,
                                                                 const f16* __restrict__ scale,
                                                                 f16* __restrict__ out, int n, int m) {
  __shared__ int8_t tile[64][65];
  const int r0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int rr = ty; rr < 64; rr += 4) {
    int r = r0 + rr, j = j0 + tx;
    tile[rr][tx] = (r < n && j < m) ? P[(size_t)r * m + j] : (int8_t)0;
  }
  __syncthreads();
  const int r = r0 + tx;
  if (r >= n) return;
  const f16 s = scale[r];
  for (int jj = ty; jj < 64; jj += 4) {
    int j = j0 + jj;
    if (j >= m) break;
    int8_t b = tile[tx][jj];
    out[(size_t)(2 * j) * n + r] = (f16)nib_hi(b) * s;
    out[(size_t)(2 * j + 1) * n + r] = (f16)nib_lo(b) * s;
  }
}

// axis == 0: out[2i + h, c] = nib_h(P[i, c]) * scale[c]; out is [2n, m].
__global__ __launch_bounds__(256) void int4_to_half_axis0_kernel(const int8_t* __restrict__ P,
                                                                 const f16* __restrict__ scale,
                                                                 f16* __restrict__ out, int n, int m) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)n * m) return;
  const int i = (int)(idx / m), c = (int)(idx % m);
  const int8_t b = P[idx];
  const f16 s = scale[c];
  out[(size_t)(2 * i) * m + c] = (f16)nib_hi(b) * s;
  out[(size_t)(2 * i + 1) * m + c] = (f16)nib_lo(b) * s;
}

extern "C" int pta_int4_to_half(const int8_t* packed, const pta_half* scale, pta_half* out, int n,
                                int m, int axis, pta_stream_t stream) {
  // Guards of Int4ToHalfOp::setup (int4_to_half_custom_op.cpp:65-98): rank/shape agreement is
  // the caller's to state through n and m; the axis must be 0 or 1.
  PTA_REQUIRE(axis == 0 || axis == 1, "[Int4ToHalf] 'axis' should be 0 or 1. But now it is %d.", axis);
  PTA_REQUIRE(packed && scale && out, "[Int4ToHalf] null pointer");
  PTA_REQUIRE(n > 0 && m > 0, "[Int4ToHalf] empty input [%d,%d]", n, m);
  hipStream_t s = (hipStream_t)stream;
  if (axis == 1) {
    dim3 grid((m + 63) / 64, (n + 63) / 64);
    hipLaunchKernelGGL(int4_to_half_axis1_kernel, grid, dim3(256), 0, s, packed, (const f16*)scale,
                       (f16*)out, n, m);
  } else {
    size_t total = (size_t)n * m;
    hipLaunchKernelGGL(int4_to_half_axis0_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       packed, (const f16*)scale, (f16*)out, n, m);
  }
  PTA_CHECK_LAUNCH("pta_int4_to_half");
  return PTA_OK;
}

// ------------------------------------------------------------------------------------------
// Load-time tiling.
//
// A tile covers 16 output channels x 128 input features and is 1 KiB, stored so that lane l
// of a wave finds its 16 bytes at byte offset 16*l.  The A operand of MFMA step m (0..3) of a
// tile is, for lane l, the 8 weights of channel (l % 16) for features
// kt*128 + m*32 + (l/16)*8 + 0..7.  Dword d (0..3) of the lane holds features 2d (in its low
// half) and 2d + 1 (in its high half) of all four steps, step m in nibble m of each half,
// stored offset-binary (q + 8): one AND|OR per dword and step yields an fp16 pair of
// consecutive features, and all weights of one step sit at the same bit position of their
// half.  Tiles of one 16-channel block are contiguous over kt, so a block streams one
// contiguous range.  Padding rows / features hold the code of zero.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void w4_tile_kernel(const int8_t* __restrict__ P,
                                                      uint32_t* __restrict__ tiled, int N, int K,
                                                      int KT, size_t total_dwords) {
  const size_t d = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (d >= total_dwords) return;
  const int dw = (int)(d & 3);
  const int lane = (int)((d >> 2) & 63);
  const size_t tile = d >> 8;
  const int kt = (int)(tile % KT);
  const int nb = (int)(tile / KT);
  const int row = nb * 16 + (lane & 15);
  uint32_t w = 0;
#pragma unroll
  for (int m = 0; m < 4; ++m) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int k = kt * 128 + m * 32 + (lane >> 4) * 8 + 2 * dw + h;
      uint32_t u = 8;  // q = 0
      if (row < N && k < K) {
        const int8_t b = P[(size_t)row * (K / 2) + (k >> 1)];
        const int q = (k & 1) ? nib_lo(b) : nib_hi(b);
        u = (uint32_t)(q + 8);
      }
      w |= u << (16 * h + 4 * m);
    }
  }
  tiled[d] = w;
}

extern "C" size_t pta_w4_tiled_bytes(int N, int K) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)((N + 15) / 16) * (size_t)((K + 127) / 128) * 1024;
}

extern "C" int pta_w4_tile(const int8_t* packed, void* tiled, int N, int K, pta_stream_t stream) {
  PTA_REQUIRE(packed && tiled, "pta_w4_tile: null pointer");
  PTA_REQUIRE(N > 0 && K > 0 && (K % 2) == 0, "pta_w4_tile: need N > 0 and even K > 0, got N=%d K=%d", N, K);
  PTA_REQUIRE(pta_aligned(tiled, 16), "pta_w4_tile: tiled buffer must be 16-byte aligned");
  const int KT = (K + 127) / 128;
  const size_t total = pta_w4_tiled_bytes(N, K) / 4;
  hipLaunchKernelGGL(w4_tile_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, packed, (uint32_t*)tiled, N, K, KT, total);
  PTA_CHECK_LAUNCH("pta_w4_tile");
  return PTA_OK;
}

