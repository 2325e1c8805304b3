// FP8 x FP8 products on the FP8 matrix instruction: the reference multiplies its QUARTER operands directly
// (custom_ops/matmul_fp8.cpp:915-924,995-1003: both sides F143 bytes with a power-of-two metadata scale,
// fp32 partials, HALF output); this is the same for gfx950, whose matrix unit takes OCP e4m3 bytes.
//
// A Graphcore F143 byte and the OCP e4m3 byte of the same bits differ by the exponent bias only (8 against 7):
// OCP(b) = 2 * F143(b) for every b except three codes - 0x80 (F143: NaN, OCP: -0) and 0x7F / 0xFF (F143: +-240,
// OCP: NaN).  So the bytes go to the instruction as they are, a product sum comes out four times too large
// (2 per operand; the factor 1/4 is exact and joins the fp32 sum), and a 32-feature step in which either operand
// holds one of the three codes is multiplied the other way instead: both operands decoded exactly to fp16 (every
// F143 value is an fp16 value) into the fp16 instruction, with a second accumulator.  Which weight tiles hold such
// a code is recorded once, when the weights are tiled (one flag byte per tile behind the tiles); the activations
// are checked as they are loaded.  Activations of +-240 are what a saturating cast leaves, so they can be frequent;
// they stay on the FP8 instruction: 240 = 224 + 16, both F143 values with OCP bytes, so the step is multiplied twice,
// once with 224 and once with 16 in the places of the 240s (zero elsewhere), which is exact.  Only a NaN activation
// sends a step the slow way.
//
// Activations arrive either as F143 bytes [M, K] (an uint8 left-hand side, as the reference's FP8MatMul takes it)
// or as fp16 values on the F143 grid without their scale (what pta_half_to_fp8_grid and the producers' output
// casts leave); the latter are turned into bytes in registers, exactly (a grid value has one byte).
//
// Shape: the decode step - up to 16 rows, one X shared by all matrices of the launch - with the workgroup layout of
// gemv_wide_kernel (16 waves; NB channel blocks per workgroup share the activation fragments of a feature tile).
#pragma once
#include "gemm_core.h"
#include "formats.h"

// flag bytes of a tiled FP8 weight: one per tile, nonzero when the tile holds 0x7F, 0xFF or 0x80
__host__ __device__ inline size_t f8_tile_flags_offset(int N, int K) {
  return (size_t)((N + 15) / 16) * (size_t)((K + 127) / 128) * 2048;
}

// 8 fp16 values on the F143 grid (|v| <= 240 or NaN) -> their 8 F143 bytes (+-240 -> 0x7F / 0xFF), and whether any of
// them is beyond 240 (NaN).  v * 2^-7 is exact (an F143 subnormal becomes an fp16 subnormal) and carries the byte's exponent and
// mantissa in bits 13..7 of each half.
__device__ __forceinline__ u32x2 f143_bytes_of_grid(f16x8 v, bool& special) {
  const u32x4 d = bitcast<u32x4>(v);
  const f16x2 k = {(f16)0.0078125f, (f16)0.0078125f};
  uint32_t p[4], big = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t mag = d[i] & 0x7FFF7FFFu;
    const uint32_t lo16 = mag & 0xFFFFu, hi16 = mag >> 16;
    big = big > lo16 ? big : lo16;
    big = big > hi16 ? big : hi16;
    const uint32_t t = bitcast<uint32_t>(bitcast<f16x2>(d[i]) * k);
    const uint32_t sign = (t & 0x80008000u) >> 8;
    uint32_t b;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(b) : "v"(t >> 7), "s"(0x007F007Fu), "v"(sign));
    p[i] = b;      // byte of the low half in bits 7..0, of the high half in bits 23..16
  }
  special = big > 0x5B80u;       // above fp16 240.0: NaN (a grid value is never larger)
  u32x2 r;
  r[0] = __builtin_amdgcn_perm(p[1], p[0], 0x06040200u);
  r[1] = __builtin_amdgcn_perm(p[3], p[2], 0x06040200u);
  return r;
}

// whether any of the 8 bytes is 0x80 (NaN)
__device__ __forceinline__ bool f143_has_nan(u32x2 q) {
  bool s = false;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t nonzero = ((q[i] & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) & 0x80808080u;      // low seven bits not all zero
    s = s || (q[i] & ~nonzero & 0x80808080u) != 0;
  }
  return s;
}

// Splits the bytes 0x7F / 0xFF (+-240) of q into +-224 (0x7E / 0xFE, left in q) and +-16 (0x60 / 0xE0, returned; zero
// bytes elsewhere).  Returns whether there was any.
__device__ __forceinline__ bool f143_split_240(u32x2& q, u32x2& extra) {
  bool any = false;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t is7f = ((q[i] & 0x7F7F7F7Fu) + 0x01010101u) & 0x80808080u;         // 0x80 where the low seven bits are all ones
    const uint32_t one = is7f >> 7;
    extra[i] = one * 0x60u | (q[i] & is7f);
    q[i] -= one;
    any = any || is7f != 0;
  }
  return any;
}

// exact decode of 8 bytes, NaN for 0x80 (the slow path takes no shortcuts; kept out of line: it is rare)
__device__ __noinline__ f16x8 f143_decode8_exact(uint32_t lo, uint32_t hi) {
  f16x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[i] = (f16)F8<0>::decode((uint8_t)(lo >> (8 * i)));
    r[4 + i] = (f16)F8<0>::decode((uint8_t)(hi >> (8 * i)));
  }
  return r;
}

template <int NB, bool PAIR, bool XBYTES>
__global__ __launch_bounds__(WIDE_WAVES * 64) void gemv_f8n_kernel(GemmArgs a, int total_nb) {
  constexpr int NACC = PAIR ? 2 : 1;
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);          // [WIDE_WAVES][NB][NACC][256]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int G = gridDim.x;
  const int K = a.K, KT = a.KT;

  int mi[NB], nb[NB];
  float mul[NB][NACC];
  const u32x4* wp[NB][NACC];
  const uint8_t* flags[NB][NACC];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    int blk = blockIdx.x + b * G;
    blk = blk < total_nb ? blk : total_nb - 1;          // a duplicate whose results are not stored
    int m_ = 0;
    if (!PAIR) {
#pragma unroll
      for (int i = 1; i < 4; ++i)
        if (i < a.count && blk >= a.mat[i].nb_begin) m_ = i;
    }
    mi[b] = m_;
    nb[b] = blk - a.mat[m_].nb_begin;
#pragma unroll
    for (int g = 0; g < NACC; ++g) {
      const GemmMat& m = a.mat[PAIR ? g : m_];
      mul[b][g] = ldexpf(1.0f, reinterpret_cast<const int32_t*>(m.scale)[0] + a.x_scale[0]);
      wp[b][g] = reinterpret_cast<const u32x4*>(m.tiled) + (size_t)nb[b] * KT * 128 + lane;
      flags[b][g] = reinterpret_cast<const uint8_t*>(m.tiled) + f8_tile_flags_offset(m.N, K) + (size_t)nb[b] * KT;
    }
  }
  int mrow = lane & 15;
  mrow = mrow < a.M ? mrow : a.M - 1;                   // padding rows compute values that are never stored
  const size_t xoff = (size_t)mrow * K + (lane >> 4) * 8;
  const f16* xh = a.X + xoff;
  const uint8_t* xq8 = reinterpret_cast<const uint8_t*>(a.X) + xoff;

  f32x4 acc[NB][NACC], accx[NB][NACC];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int g = 0; g < NACC; ++g) acc[b][g] = accx[b][g] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kt = wave; kt < KT; kt += WIDE_WAVES) {
    u32x4 w[NB][NACC][2];
    uint32_t fl[NB][NACC];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int g = 0; g < NACC; ++g) {
#pragma unroll
        for (int v = 0; v < 2; ++v) w[b][g][v] = __builtin_nontemporal_load(wp[b][g] + ((size_t)kt * 2 + v) * 64);
        fl[b][g] = flags[b][g][kt];
      }
    u32x2 xq[4], xe[4];
    unsigned xnan = 0, xsplit = 0;   // bit j: step j holds a NaN activation / activations of +-240 (same in every lane)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = kt * 128 + j * 32;
      const bool in = k + (lane >> 4) * 8 < K;
      bool nan = false;
      if constexpr (XBYTES) {
        xq[j] = in ? *reinterpret_cast<const u32x2*>(xq8 + k) : u32x2{0, 0};
        nan = f143_has_nan(xq[j]);
      } else {
        const f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        xq[j] = f143_bytes_of_grid(in ? *reinterpret_cast<const f16x8*>(xh + k) : z, nan);
      }
      if (__any(nan)) xnan |= 1u << j;
      if (__any(f143_split_240(xq[j], xe[j]))) xsplit |= 1u << j;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long xb = bitcast<long>(xq[j]), xb2 = bitcast<long>(xe[j]);
      const bool split = (xsplit >> j) & 1u;
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g = 0; g < NACC; ++g) {
          const uint32_t lo = w[b][g][j >> 1][(j & 1) * 2], hi = w[b][g][j >> 1][(j & 1) * 2 + 1];
          const bool slow = __builtin_amdgcn_readfirstlane(fl[b][g]) != 0 || ((xnan >> j) & 1u);
          if (!slow) {
            const long wb = bitcast<long>(u32x2{lo, hi});
            acc[b][g] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(wb, xb, acc[b][g], 0, 0, 0);
            if (split) acc[b][g] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(wb, xb2, acc[b][g], 0, 0, 0);
          } else {
            // both operands decoded exactly; the activation bytes are put together again first (224 + 16 -> 240)
            const u32x2 whole = {xq[j][0] + ((xe[j][0] >> 6) & 0x01010101u), xq[j][1] + ((xe[j][1] >> 6) & 0x01010101u)};
            f16x8 xv;
            if constexpr (XBYTES) xv = f143_decode8_exact(whole[0], whole[1]);
            else {
              const int k = kt * 128 + j * 32;
              const f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
              xv = k + (lane >> 4) * 8 < K ? *reinterpret_cast<const f16x8*>(xh + k) : z;
            }
            accx[b][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f143_decode8_exact(lo, hi), xv, accx[b][g], 0, 0, 0);
          }
        }
    }
  }

  // The accumulator of lane l holds channels (l/16)*4 + r, r = 0..3, for activation row l%16.
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int g = 0; g < NACC; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        red[(((wave * NB + b) * NACC + g) * 4 + r) * 64 + lane] = acc[b][g][r] * 0.25f + accx[b][g][r];
  __syncthreads();
  const int quarter = threadIdx.x >> 8;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if ((b & 3) != quarter) continue;
    const int nn = threadIdx.x & 15, m = (threadIdx.x >> 4) & 15;
    const GemmMat& mat = a.mat[PAIR ? 0 : mi[b]];
    const int N = mat.N, n = nb[b] * 16 + nn;
    if ((int)blockIdx.x + b * G >= total_nb || m >= a.M || n >= N) continue;
    const int r = nn & 3, ln = (nn >> 2) * 16 + m;
    float sum[NACC];
#pragma unroll
    for (int g = 0; g < NACC; ++g) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < WIDE_WAVES; ++w) t += red[(((w * NB + b) * NACC + g) * 4 + r) * 64 + ln];
      sum[g] = t * mul[b][g];
    }
    if (PAIR) {
      mat.Y[(size_t)m * N + n] = swiglu_out(a.epi, (f16)sum[0], (f16)sum[1]);
    } else {
      f16 y0 = (f16)sum[0];
      if (mat.bias) y0 = y0 + mat.bias[n];
      y0 = apply_act(mat.act, y0);
      mat.Y[(size_t)m * N + n] = apply_epilogue(a.epi, y0, m, n, N);
    }
  }
}

template <int NB, bool PAIR, bool XBYTES>
static int launch_gemv_f8n(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  static bool ready = false;
  const size_t smem = (size_t)WIDE_WAVES * NB * (PAIR ? 2 : 1) * 256 * sizeof(float);
  if (!ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)gemv_f8n_kernel<NB, PAIR, XBYTES>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem) == hipSuccess,
                "%s: cannot reserve %zu bytes of LDS", name, smem);
    ready = true;
  }
  hipLaunchKernelGGL((gemv_f8n_kernel<NB, PAIR, XBYTES>), dim3((total_nb + NB - 1) / NB), dim3(WIDE_WAVES * 64), smem, s, a,
                     total_nb);
  return PTA_OK;
}

// the shapes the kernel takes: up to 16 rows, one shared X, enough feature tiles for the 16 waves, no fused norm
static inline bool f8n_fits(const GemmArgs& a) {
  if (a.M > 16 || a.KT < 8 || a.epi.norm != PTA_NORM_NONE || !a.x_scale) return false;
  for (int i = 0; i < a.count; ++i)
    if (a.mat[i].X) return false;
  return true;
}

template <bool PAIR, bool XBYTES>
static int dispatch_gemv_f8n(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  const int per_cu = (total_nb + device_compute_units() - 1) / device_compute_units();
  int rc;
  if (per_cu <= 1) rc = launch_gemv_f8n<1, PAIR, XBYTES>(a, total_nb, s, name);
  else if (per_cu == 2 || PAIR) rc = launch_gemv_f8n<2, PAIR, XBYTES>(a, total_nb, s, name);
  else rc = launch_gemv_f8n<3, PAIR, XBYTES>(a, total_nb, s, name);
  if (rc) return rc;
  PTA_CHECK_LAUNCH(name);
  return PTA_OK;
}
