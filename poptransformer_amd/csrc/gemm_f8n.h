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

// ------------------------------------------------------------------------------------------
// More than 16 rows (prompt passes): the workgroup tile of gemm_panel_kernel - every wave holds the weight tiles of
// its own NST channel blocks in registers and multiplies all RG row groups of the workgroup, which go through LDS -
// on the 16x16x128 FP8 instruction: one instruction takes a whole 128-feature tile of a channel block and a row
// group, at twice the fp16 instruction's rate, and the weight bytes are its A operand as they lie in memory (lane l:
// channel l % 16, the 32 bytes of features j * 32 + (l / 16) * 8 + 0..7, j = 0..3; a sum over features does not mind
// their order as long as the B operand follows it).  The activations arrive as fp16 values on the F143 grid; the
// wave that fetches a piece of a row turns it into bytes on its way to LDS (once per workgroup, not once per wave),
// where a row takes 128 bytes in the B operand's order, 16 more between rows so that the sixteen rows of an operand
// read fall into different banks.
// The codes on which F143 and OCP e4m3 differ go through a second operand: an activation of +-240 leaves 224 in the
// first operand and 16 in the second, a NaN leaves 0 and the OCP NaN byte, and a tile's row group with any of them
// (one flag per four rows, in LDS) is multiplied with both.  The same holds for a weight tile whose flag byte says
// so (+-240, or the NaN code 0x80, which as an OCP byte is -0 and contributes nothing to the first product): its two
// operands are made in registers when the tile is met.  Sums come out four times too large (two per operand).
// ------------------------------------------------------------------------------------------
constexpr int F8P_ROW = 144;          // bytes from one row to the next in LDS

typedef int i32x8 __attribute__((ext_vector_type(8)));

// 8 weight bytes -> first operand (q: 224 for +-240) and second (16 there; the OCP NaN byte where q holds 0x80)
__device__ __forceinline__ void f143_weight_operands(u32x2& q, u32x2& extra) {
  u32x2 nan;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t nonzero = ((q[i] & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) & 0x80808080u;
    nan[i] = ((q[i] & ~nonzero & 0x80808080u) >> 7) * 0x7Fu;
  }
  f143_split_240(q, extra);
  extra[0] |= nan[0];
  extra[1] |= nan[1];
}

// 8 fp16 values on the F143 grid -> their 8 bytes as f143_bytes_of_grid makes them; `big` gathers the largest magnitude
// seen (fp16 bits, in either half), from which the caller tells +-240 (0x5B80) and NaN (anything above) at little cost
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x2 f143_bytes_of_grid_fast(f16x8 v, uint32_t& big) {
  const u32x4 d = bitcast<u32x4>(v);
  const f16x2 k = {(f16)0.0078125f, (f16)0.0078125f};
  uint32_t p[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    big = bitcast<uint32_t>(__builtin_elementwise_max(bitcast<u16x2>(big), bitcast<u16x2>(d[i] & 0x7FFF7FFFu)));
    const uint32_t t = bitcast<uint32_t>(bitcast<f16x2>(d[i]) * k);
    const uint32_t sign = (t & 0x80008000u) >> 8;
    uint32_t b;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(b) : "v"(t >> 7), "s"(0x007F007Fu), "v"(sign));
    p[i] = b;
  }
  u32x2 r;
  r[0] = __builtin_amdgcn_perm(p[1], p[0], 0x06040200u);
  r[1] = __builtin_amdgcn_perm(p[3], p[2], 0x06040200u);
  return r;
}

// The second operand of 8 activations whose bytes are q (made from the grid values v): 16 where q holds +-240 (224
// stays in q), the OCP NaN byte where v is beyond 240 (NaN; q gets 0 there).
__device__ __forceinline__ void f143_activation_second(f16x8 v, u32x2& q, u32x2& e) {
  f143_split_240(q, e);
  const u32x4 d = bitcast<u32x4>(v);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t lo = (d[i] & 0x7FFFu) > 0x5B80u ? 0xFFu : 0u, hi = ((d[i] >> 16) & 0x7FFFu) > 0x5B80u ? 0xFF00u : 0u;
    const uint32_t nan = (lo | hi) << ((i & 1) * 16);
    q[i >> 1] &= ~nan;
    e[i >> 1] = (e[i >> 1] & ~nan) | (nan & 0x7F7F7F7Fu);
  }
}

__device__ __forceinline__ i32x8 f8p_operand(const u32x4& lo, const u32x4& hi) {
  return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}
__device__ __forceinline__ f32x4 f8p_mfma(const i32x8& a, const i32x8& b, const f32x4& c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);     // e4m3 x e4m3, no scales
}

// NST, RG, KH, PAIR, the launch's arguments and the workgroup's place in the tile list as in gemm_panel_kernel.
template <int NST, int RG, int KH, bool PAIR>
__global__ __launch_bounds__(PANEL_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_f8n_panel_kernel(GemmArgs a, int groups, int row_blocks, int unit0, int units) {
  typedef FmtF8<0> Fmt;
  constexpr int CW = PANEL_WAVES / KH;            // channel units (waves side by side) per workgroup
  constexpr int ROWS = RG * 16;
  constexpr int XPART = ROWS * F8P_ROW;           // bytes of one feature tile of the workgroup's rows
  constexpr int XSTAGE = KH * XPART;              // one stage: a tile per part
  constexpr int QALL = KH * RG * 4;               // row loads (4 rows each) of a stage
  constexpr int QN = (QALL + PANEL_WAVES - 1) / PANEL_WAVES;     // ... per wave
  static_assert(!PAIR || NST % 2 == 0, "gate and up blocks in equal numbers");
  static_assert(KH == 1 || KH == 2, "parts of K");
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* xmain = smem;                                          // [2][KH][ROWS][F8P_ROW]: first operands
  unsigned char* xextra = smem + 2 * XSTAGE;                            // the same for the second operands (where flagged)
  uint32_t* xflags = reinterpret_cast<uint32_t*>(smem + 4 * XSTAGE);    // [2][KH][RG] words: a byte per four rows
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int cw = wave % CW, kh = wave / CW;
  const int K = a.K, M = a.M;
  const int per = (int)gridDim.x / 8;
  const int tile = ((int)blockIdx.x % 8) * per + (int)blockIdx.x / 8;
  if (tile >= groups * row_blocks) return;
  const int row_block = tile % row_blocks, group = tile / row_blocks;
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  const int per_slice = (a.KT + nsl - 1) / nsl;
  const int kt_first = (int)blockIdx.y * per_slice;
  const int kt_end = kt_first + per_slice < a.KT ? kt_first + per_slice : a.KT;
  const int steps = kt_end > kt_first ? (kt_end - kt_first + KH - 1) / KH : 0;

  const int wu = unit0 + group * CW + cw;
  const bool active = wu < units;
  const int gb = (active ? wu : 0) * (PAIR ? NST / 2 : NST);
  int mi = 0;
  if (!PAIR) {
#pragma unroll
    for (int i = 1; i < 4; ++i)
      if (i < a.count && gb >= a.mat[i].nb_begin) mi = i;
  }
  const int blk0 = PAIR ? gb : gb - a.mat[mi].nb_begin;
  constexpr int NBW = PAIR ? NST / 2 : NST;
  const uint32_t blk_bytes = (uint32_t)a.KT * 2048;
  const GemmMat& m0 = a.mat[PAIR ? 0 : mi];
  const GemmMat& m1 = a.mat[PAIR ? 1 : mi];
  const unsigned char* w0 = reinterpret_cast<const unsigned char*>(m0.tiled) + (size_t)blk0 * blk_bytes;
  const unsigned char* w1 = reinterpret_cast<const unsigned char*>(m1.tiled) + (size_t)blk0 * blk_bytes;
  const __amdgpu_buffer_rsrc_t wr0 = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(w0), 0, (int)(NBW * blk_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t wr1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(w1), 0, (int)(NBW * blk_bytes), 0x00020000);
  // the tiles' flag bytes: one per tile, block by block, behind the tiles of a matrix
  const uint8_t* f0 = reinterpret_cast<const uint8_t*>(m0.tiled) + f8_tile_flags_offset(m0.N, K) + (size_t)blk0 * a.KT;
  const uint8_t* f1 = reinterpret_cast<const uint8_t*>(m1.tiled) + f8_tile_flags_offset(m1.N, K) + (size_t)blk0 * a.KT;
  const int wlane = lane * 16;
  const int row0 = row_block * ROWS;
  const int rows_here = M - row0 < ROWS ? M - row0 : ROWS;
  const __amdgpu_buffer_rsrc_t xr0 = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<f16*>(a.X + (size_t)row0 * K), 0, (int)((size_t)rows_here * K * 2), 0x00020000);

  // this wave's weight tiles of step i and their flags (past the end of the range: an offset beyond the descriptor,
  // which reads as zeros; every load is issued, so that the count of loads in flight is a constant of the program)
  auto fetch_w = [&](int i, u32x4 (&wv)[NST][2], uint32_t (&fl)[NST]) {
    const int kt = kt_first + i * KH + kh;
    const int at = kt < kt_end ? wlane : -1;
    const int ktc = kt < kt_end ? kt : kt_first;
#pragma unroll
    for (int st = 0; st < NST; ++st) {
      const bool second = PAIR && st >= NST / 2;
      const int b = PAIR ? st % (NST / 2) : st;
#pragma unroll
      for (int v = 0; v < 2; ++v)
        wv[st][v] = __builtin_amdgcn_raw_buffer_load_b128(second ? wr1 : wr0, at, (int)(b * blk_bytes + (uint32_t)(ktc * 2 + v) * 1024), 0);
      fl[st] = (second ? f1 : f0)[(size_t)b * a.KT + ktc];
    }
  };
  // Row load q = 8 j + w (w: the wave) of a stage brings rows 4 (q % (4 RG)) .. + 3 of the tile of part q / (4 RG):
  // lane l the eight values of piece l % 16 of row l / 16 (rows past M and features past K read as zero) ...
  auto fetch_x = [&](int i, u32x4 (&xr)[QN]) {
#pragma unroll
    for (int j = 0; j < QN; ++j) {
      const int q = j * PANEL_WAVES + wave;
      const int part = q / (4 * RG), rb = q % (4 * RG);
      const int row = rb * 4 + (lane >> 4), piece = lane & 15;
      const int kt = kt_first + i * KH + part;
      const bool in_k = q < QALL && kt < kt_end && kt * 128 + piece * 8 < K;
      xr[j] = __builtin_amdgcn_raw_buffer_load_b128(xr0, in_k ? row * K * 2 + piece * 16 : -1, kt * 256, 0);
    }
  };
  // ... which go to LDS as the operands' bytes: piece p = 4 j + g holds the features of 32-feature step j that lane
  // group g of the instruction takes, so its bytes lie at g * 32 + j * 8 of the row
  auto stage_x = [&](const u32x4 (&xr)[QN], int stage) {
#pragma unroll
    for (int j = 0; j < QN; ++j) {
      const int q = j * PANEL_WAVES + wave;
      if (q >= QALL) continue;
      const int part = q / (4 * RG), rb = q % (4 * RG);
      const int row = rb * 4 + (lane >> 4), piece = lane & 15;
      uint32_t big = 0;
      u32x2 b = f143_bytes_of_grid_fast(bitcast<f16x8>(xr[j]), big), e;
      const uint32_t largest = (big & 0xFFFFu) > (big >> 16) ? (big & 0xFFFFu) : (big >> 16);
      const bool second = __any(largest >= 0x5B80u);            // +-240 or NaN somewhere in these four rows
      const int at = stage * XSTAGE + part * XPART + row * F8P_ROW + (piece & 3) * 32 + (piece >> 2) * 8;
      e = u32x2{0, 0};
      if (second) f143_activation_second(bitcast<f16x8>(xr[j]), b, e);
      *reinterpret_cast<u32x2*>(xmain + at) = b;
      *reinterpret_cast<u32x2*>(xextra + at) = e;
      if (lane == 0) reinterpret_cast<uint8_t*>(xflags)[((stage * KH + part) * RG) * 4 + rb] = second ? 1 : 0;
    }
  };

  f32x4 acc[RG][NST];
#pragma unroll
  for (int rg = 0; rg < RG; ++rg)
#pragma unroll
    for (int st = 0; st < NST; ++st) acc[rg][st] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 wa[NST][2], wb[NST][2], xr[QN];
  uint32_t fa[NST], fb[NST];
  if (steps > 0) {
    fetch_x(0, xr);
    if (active) fetch_w(0, wa, fa);
    stage_x(xr, 0);
  }
  __syncthreads();

  auto feature_tile = [&](int i, u32x4 (&wc)[NST][2], const uint32_t (&fc)[NST], u32x4 (&wn)[NST][2], uint32_t (&fn)[NST]) {
    const bool more = i + 1 < steps;
    if (more) {
      fetch_x(i + 1, xr);                     // rows first: the wait for them leaves the weights in flight
      if (active) fetch_w(i + 1, wn, fn);
    }
    if (active) {
      const int base = (i & 1) * XSTAGE + kh * XPART + (lane & 15) * F8P_ROW + (lane >> 4) * 32;
      const uint32_t* flags = xflags + ((i & 1) * KH + kh) * RG;
      auto b_operand = [&](const unsigned char* plane, int rg) {
        const unsigned char* at = plane + base + rg * 16 * F8P_ROW;
        return f8p_operand(*reinterpret_cast<const u32x4*>(at), *reinterpret_cast<const u32x4*>(at + 16));
      };
      uint32_t wany = 0, xany = 0;
#pragma unroll
      for (int st = 0; st < NST; ++st) wany |= fc[st];
#pragma unroll
      for (int rg = 0; rg < RG; ++rg) xany |= flags[rg];
      wany = __builtin_amdgcn_readfirstlane(wany);
      xany = __builtin_amdgcn_readfirstlane(xany);
      // A weight tile with codes of its own (few per matrix): its first operand replaces the bytes, and the products
      // of its second operand with both operands of the rows are added here.
      if (wany != 0) {
#pragma unroll
        for (int st = 0; st < NST; ++st) {
          if (__builtin_amdgcn_readfirstlane(fc[st]) == 0) continue;
          u32x4 e[2];
#pragma unroll
          for (int v = 0; v < 2; ++v)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              u32x2 q = {wc[st][v][2 * h], wc[st][v][2 * h + 1]}, x;
              f143_weight_operands(q, x);
              wc[st][v][2 * h] = q[0]; wc[st][v][2 * h + 1] = q[1];
              e[v][2 * h] = x[0]; e[v][2 * h + 1] = x[1];
            }
          const i32x8 ae = f8p_operand(e[0], e[1]);
#pragma unroll
          for (int rg = 0; rg < RG; ++rg) {
            acc[rg][st] = f8p_mfma(ae, b_operand(xmain, rg), acc[rg][st]);
            acc[rg][st] = f8p_mfma(ae, b_operand(xextra, rg), acc[rg][st]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      // the first operands of both sides (the scheduling barriers keep the compiler from fetching all row groups'
      // operands ahead of the first product, which the registers do not hold)
      {
        i32x8 b = b_operand(xmain, 0);
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
          i32x8 bn = b;
          if (rg + 1 < RG) bn = b_operand(xmain, rg + 1);
#pragma unroll
          for (int st = 0; st < NST; ++st) acc[rg][st] = f8p_mfma(f8p_operand(wc[st][0], wc[st][1]), b, acc[rg][st]);
          b = bn;
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // row groups whose activations have second operands
      if (xany != 0) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
          if (__builtin_amdgcn_readfirstlane(flags[rg]) == 0) continue;
          const i32x8 be = b_operand(xextra, rg);
#pragma unroll
          for (int st = 0; st < NST; ++st) acc[rg][st] = f8p_mfma(f8p_operand(wc[st][0], wc[st][1]), be, acc[rg][st]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (more) stage_x(xr, (i + 1) & 1);
    __syncthreads();
  };
  for (int i = 0; i < steps; i += 2) {
    feature_tile(i, wa, fa, wb, fb);
    if (i + 1 < steps) feature_tile(i + 1, wb, fb, wa, fa);
  }
  // (the last barrier has passed: what follows reuses the row buffers)
#pragma unroll
  for (int rg = 0; rg < RG; ++rg)
#pragma unroll
    for (int st = 0; st < NST; ++st) acc[rg][st] = acc[rg][st] * 0.25f;
  if constexpr (KH > 1) {
    // the sums of part 1 go to part 0's wave of the same channel unit, half of the row groups at a time
    f32x4* ex = reinterpret_cast<f32x4*>(smem);                   // [CW][RG / 2 * NST][64]
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      if (kh > 0 && active) {
#pragma unroll
        for (int rg = 0; rg < RG / 2; ++rg)
#pragma unroll
          for (int st = 0; st < NST; ++st) ex[(cw * (RG / 2 * NST) + rg * NST + st) * 64 + lane] = acc[half * (RG / 2) + rg][st];
      }
      __syncthreads();
      if (kh == 0 && active) {
#pragma unroll
        for (int rg = 0; rg < RG / 2; ++rg)
#pragma unroll
          for (int st = 0; st < NST; ++st) {
            const f32x4 other = ex[(cw * (RG / 2 * NST) + rg * NST + st) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[half * (RG / 2) + rg][st][r] += other[r];
          }
      }
      __syncthreads();
    }
    if (kh > 0) return;
  }
  if (!active) return;
  const Fmt::Scale s0 = Fmt::load_scale(m0.scale, a.x_scale, 0, 1), s1 = Fmt::load_scale(m1.scale, a.x_scale, 0, 1);
  panel_store<Fmt, NST, RG, PAIR>(a, acc, smem, cw, mi, blk0, row0, nsl, s0, s1);
}

// LDS of gemm_f8n_panel_kernel: two stages of both operands and their flags; the parts' meeting; the epilogue strips
template <int NST, int RG, int KH>
constexpr size_t f8n_panel_lds() {
  constexpr size_t stages = (size_t)4 * KH * RG * 16 * F8P_ROW + (size_t)2 * KH * RG * 4;
  constexpr size_t meet = KH > 1 ? (size_t)(PANEL_WAVES / KH) * (RG / 2 * NST) * 1024 : 0;
  constexpr size_t strips = (size_t)(PANEL_WAVES / KH) * 16 * (NST * 16 + 4) * 4;
  return stages > meet ? (stages > strips ? stages : strips) : (meet > strips ? meet : strips);
}

// units [unit0, unit1) of the launch's matrices, as launch_gemm_panel
template <int NST, int RG, int KH, bool PAIR>
static int launch_gemm_f8n_panel(const GemmArgs& a, int unit0, int unit1, hipStream_t s, const char* name) {
  static bool ready = false;
  constexpr int CW = PANEL_WAVES / KH;
  constexpr size_t smem = f8n_panel_lds<NST, RG, KH>();
  static_assert(smem <= 160 * 1024, "LDS");
  if (!ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)gemm_f8n_panel_kernel<NST, RG, KH, PAIR>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem) == hipSuccess,
                "%s: cannot reserve %zu bytes of LDS", name, smem);
    ready = true;
  }
  const int groups = (unit1 - unit0 + CW - 1) / CW;
  const int row_blocks = (a.M + RG * 16 - 1) / (RG * 16);
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  const int per = (groups * row_blocks + 7) / 8;
  hipLaunchKernelGGL((gemm_f8n_panel_kernel<NST, RG, KH, PAIR>), dim3(per * 8, nsl), dim3(PANEL_WAVES * 64), smem, s, a, groups, row_blocks, unit0, unit1);
  if (nsl > 1) {
    const size_t total = (size_t)a.M * a.mat[0].N;
    hipLaunchKernelGGL((splitk_finish_kernel<FmtF8<0>>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a);
  }
  return PTA_OK;
}

// The shapes gemm_f8n_panel_kernel takes: more than 16 rows of one shared X (fp16 values on the F143 grid, whole
// 16-byte pieces per row), every matrix a whole number of wave tiles of four channel blocks, no fused norm.
static inline bool f8n_panel_fits(const GemmArgs& a, bool pair) {
  return a.M > 16 && a.x_scale && a.K % 8 == 0 && a.X && panel_fits(a, 4, pair);
}

// Row blocks of 128, 64 or 32 rows, and for the smaller two also K in halves inside the workgroup (tiles of half the
// channels): the one that the model below makes fastest.  A workgroup takes steps x t, t the measured time of one step
// of that kind (gate / up pair, q | kv, o and down of the ChatGLM2-6B shape at 128 .. 2048 rows: 2.7 us for 128 rows,
// 1.85 for 64, 1.45 for 32, a step of two half tiles 2.5 and 1.8), and the launch as many rounds of them as its tiles
// need on the compute units.  (128 rows with K in halves keeps 8 row loads per lane in flight beside the weights and
// spills: measured three times slower than the others, not offered.)
template <bool PAIR>
static int dispatch_f8n_panel(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  const int cus = device_compute_units();
  const int units = PAIR ? total_nb / 2 : total_nb / 4;
  struct Kind { int rows, kh; float t; };
  static const Kind kinds[5] = {{128, 1, 2.7f}, {64, 1, 1.85f}, {64, 2, 2.5f}, {32, 1, 1.45f}, {32, 2, 1.8f}};
  int best = 0;
  float best_t = 0.f;
  for (int k = 0; k < 5; ++k) {
    const Kind& c = kinds[k];
    if (c.kh == 2 && a.KT < 16) continue;
    const int per = c.kh == 2 ? 4 : 8;
    const long tiles = (long)((units + per - 1) / per) * ((a.M + c.rows - 1) / c.rows);
    const float t = (float)((tiles + cus - 1) / cus) * (float)((a.KT + c.kh - 1) / c.kh) * c.t;
    if (k == 0 || t < best_t) { best = k; best_t = t; }
  }
  int rc;
  switch (best) {
    case 0: rc = launch_gemm_f8n_panel<4, 8, 1, PAIR>(a, 0, units, s, name); break;
    case 1: rc = launch_gemm_f8n_panel<4, 4, 1, PAIR>(a, 0, units, s, name); break;
    case 2: rc = launch_gemm_f8n_panel<4, 4, 2, PAIR>(a, 0, units, s, name); break;
    case 3: rc = launch_gemm_f8n_panel<4, 2, 1, PAIR>(a, 0, units, s, name); break;
    default: rc = launch_gemm_f8n_panel<4, 2, 2, PAIR>(a, 0, units, s, name); break;
  }
  if (rc) return rc;
  PTA_CHECK_LAUNCH(name);
  return PTA_OK;
}
