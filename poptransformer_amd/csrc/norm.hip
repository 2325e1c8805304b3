// Row normalisations of the decode step: RMSNorm and the NormCE LayerNorm.
//
// RMSNorm follows poptransformer/layers/rms_layer_norm.py:26-36 (fp32 statistics, the inverse
// RMS rounded to fp16, then two fp16 multiplies).  LayerNorm follows the NormCE custom op:
// custom_ops/NormCE.cpp:122-200 + NormCECodelets.cpp:65-112 when there is a single row, and
// the assembly kernel custom_ops/NormCE.S:243-423 (C form NormCECodelets.cpp:181-211) when
// there are several.  One workgroup normalises one row in a single pass over registers.
#include "common.h"
#include "f8codec.h"

constexpr int NORM_THREADS = 256;
constexpr int NORM_MAX_VEC = 4;  // 8-element vectors per thread: rows up to 8192 columns

__device__ __forceinline__ float block_sum(float v, float* sh) {
  v = wave_total_dpp(v);      // (every thread of the workgroup calls this)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < NORM_THREADS / 64; ++w) t += sh[w];
  return t;
}

// The RWKV token shift behind a LayerNorm (models/rwkv/attention.py:59-72, models/rwkv/ffn.py:44-51): the
// normalised row h feeds out[i] = h * w[i] + (1 - w[i]) * prev for up to three mixing vectors, then prev <- h.
struct NormMix {
  f16* prev;          // [rows, cols], or null: no shift
  const f16* w[3];    // [cols] each; null entries are skipped
  f16* out[3];
};

// mode 0: RMSNorm.  mode 1: NormCE with one row.  mode 2: NormCE with several rows.
template <int MODE, bool MIX = false>
__global__ __launch_bounds__(NORM_THREADS) void norm_kernel(const f16* __restrict__ x, const f16* __restrict__ gamma,
                                                            const f16* __restrict__ beta, f16* __restrict__ y,
                                                            int cols, float eps, const int32_t* __restrict__ grid_scale,
                                                            int grid_format, NormMix mix = NormMix{}) {
  __shared__ float sh[NORM_THREADS / 64];
  const size_t base = (size_t)blockIdx.x * cols;
  const int nvec = cols >> 3;
  f16x8 v[NORM_MAX_VEC], gv[NORM_MAX_VEC], bv[NORM_MAX_VEC], pv[MIX ? NORM_MAX_VEC : 1];
  float s = 0.f, sq = 0.f;
  // (the weights are requested with the row: one round trip to memory before the sums instead of one on either side)
#pragma unroll
  for (int i = 0; i < NORM_MAX_VEC; ++i) {
    const int c = threadIdx.x + i * NORM_THREADS;
    if (c < nvec) {
      v[i] = *reinterpret_cast<const f16x8*>(x + base + (size_t)c * 8);
      gv[i] = *reinterpret_cast<const f16x8*>(gamma + (size_t)c * 8);
      if (MODE != 0) bv[i] = *reinterpret_cast<const f16x8*>(beta + (size_t)c * 8);
      if (MIX) pv[i] = *reinterpret_cast<const f16x8*>(mix.prev + base + (size_t)c * 8);
    }
  }
#pragma unroll
  for (int i = 0; i < NORM_MAX_VEC; ++i) {
    const int c = threadIdx.x + i * NORM_THREADS;
    if (c < nvec) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = (float)v[i][e];
        s += f;
        sq = __builtin_fmaf(f, f, sq);
      }
    }
  }
  const float inv_n = 1.0f / (float)cols;
  f16 mean16 = (f16)0.0f, r16;
  if (MODE == 0) {
    const float ms = block_sum(sq, sh) * inv_n;
    r16 = (f16)(1.0f / sqrtf(ms + eps));
  } else {
    const float sum = block_sum(s, sh);
    const float sqs = block_sum(sq, sh);
    const float mean = sum * inv_n;
    mean16 = (f16)mean;
    float var;
    if (MODE == 1) {
      var = sqs * inv_n - mean * mean + eps;  // fp32 mean, no clamp
    } else {
      const float m = (float)mean16;          // the rounded mean is what gets squared
      var = fmaxf(sqs * inv_n - m * m, 0.0f) + eps;
    }
    r16 = (f16)(1.0f / sqrtf(var));
  }
#pragma unroll
  for (int i = 0; i < NORM_MAX_VEC; ++i) {
    const int c = threadIdx.x + i * NORM_THREADS;
    if (c < nvec) {
      const f16x8 g = gv[i];
      f16x8 o;
      if (MODE == 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (v[i][e] * r16) * g[e];
      } else {
        const f16x8 b = bv[i];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = ((v[i][e] - mean16) * r16) * g[e] + b[e];
      }
      if (grid_scale) {           // the cast of the FP8 Linear that consumes these rows
        const int gs = grid_scale[0];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = f8_grid_value(o[e], gs, grid_format);
      }
      if (!MIX || y) *reinterpret_cast<f16x8*>(y + base + (size_t)c * 8) = o;
      if (MIX) {
        // each step an fp16 operation, in the order of the separate kernel: h * w + (1 - w) * prev
        const f16 one = (f16)1.0f;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          if (!mix.w[j]) continue;
          const f16x8 wv = *reinterpret_cast<const f16x8*>(mix.w[j] + (size_t)c * 8);
          f16x8 m;
#pragma unroll
          for (int e = 0; e < 8; ++e) m[e] = o[e] * wv[e] + (one - wv[e]) * pv[i][e];
          *reinterpret_cast<f16x8*>(mix.out[j] + base + (size_t)c * 8) = m;
        }
        *reinterpret_cast<f16x8*>(mix.prev + base + (size_t)c * 8) = o;
      }
    }
  }
}

static int check_norm(const char* name, const void* x, const void* g, const void* y, int rows, int cols) {
  PTA_REQUIRE(x && g && y, "%s: null pointer", name);
  PTA_REQUIRE(rows > 0, "%s: rows = %d", name, rows);
  PTA_REQUIRE(cols > 0 && (cols % 8) == 0 && cols <= 8 * NORM_THREADS * NORM_MAX_VEC,
              "%s: the normalised size must be a multiple of 8 and at most %d, got %d", name,
              8 * NORM_THREADS * NORM_MAX_VEC, cols);
  PTA_REQUIRE(pta_aligned(x, 16) && pta_aligned(g, 16) && pta_aligned(y, 16), "%s: pointers must be 16-byte aligned", name);
  return PTA_OK;
}

extern "C" int pta_rmsnorm(const pta_half* x, const pta_half* weight, pta_half* y, int rows, int cols,
                           float eps, pta_stream_t stream) {
  int rc = check_norm("pta_rmsnorm", x, weight, y, rows, cols);
  if (rc) return rc;
  hipLaunchKernelGGL(norm_kernel<0>, dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (const f16*)x,
                     (const f16*)weight, (const f16*)nullptr, (f16*)y, cols, eps, (const int32_t*)nullptr, 0);
  PTA_CHECK_LAUNCH("pta_rmsnorm");
  return PTA_OK;
}

extern "C" int pta_rmsnorm_fp8_grid(const pta_half* x, const pta_half* weight, pta_half* y, const int32_t* scale,
                                    int format, int rows, int cols, float eps, pta_stream_t stream) {
  int rc = check_norm("pta_rmsnorm_fp8_grid", x, weight, y, rows, cols);
  if (rc) return rc;
  PTA_REQUIRE(scale, "pta_rmsnorm_fp8_grid: null scale");
  PTA_REQUIRE(format == PTA_F143 || format == PTA_F152, "pta_rmsnorm_fp8_grid: unsupported fp8 format %d, it must be F143 or F152", format);
  hipLaunchKernelGGL(norm_kernel<0>, dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (const f16*)x,
                     (const f16*)weight, (const f16*)nullptr, (f16*)y, cols, eps, scale, format);
  PTA_CHECK_LAUNCH("pta_rmsnorm_fp8_grid");
  return PTA_OK;
}

extern "C" int pta_layer_norm_ce(const pta_half* x, const pta_half* gamma, const pta_half* beta, pta_half* y,
                                 int rows, int cols, float eps, pta_stream_t stream) {
  int rc = check_norm("pta_layer_norm_ce", x, gamma, y, rows, cols);
  if (rc) return rc;
  // Guards of NormCEOutplaceOpx::grow (custom_ops/NormCE.cpp:541-577) and of the Python wrapper
  // (poptransformer/ops/customized.py:81-82): fp16 only, size < 8192.
  PTA_REQUIRE(beta && pta_aligned(beta, 16), "pta_layer_norm_ce: beta must be a 16-byte aligned pointer");
  PTA_REQUIRE(cols < 8192, "pta_layer_norm_ce: the normalised size must be below 8192, got %d", cols);
  if (rows == 1)
    hipLaunchKernelGGL(norm_kernel<1>, dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (const f16*)x,
                       (const f16*)gamma, (const f16*)beta, (f16*)y, cols, eps, (const int32_t*)nullptr, 0);
  else
    hipLaunchKernelGGL(norm_kernel<2>, dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (const f16*)x,
                       (const f16*)gamma, (const f16*)beta, (f16*)y, cols, eps, (const int32_t*)nullptr, 0);
  PTA_CHECK_LAUNCH("pta_layer_norm_ce");
  return PTA_OK;
}

extern "C" int pta_layer_norm_ce_mix(const pta_half* x, const pta_half* gamma, const pta_half* beta, pta_half* y,
                                     pta_half* prev, const pta_half* w0, const pta_half* w1, const pta_half* w2,
                                     pta_half* o0, pta_half* o1, pta_half* o2, int rows, int cols, float eps,
                                     pta_stream_t stream) {
  int rc = check_norm("pta_layer_norm_ce_mix", x, gamma, prev, rows, cols);
  if (rc) return rc;
  PTA_REQUIRE(beta && pta_aligned(beta, 16), "pta_layer_norm_ce_mix: beta must be a 16-byte aligned pointer");
  PTA_REQUIRE(cols < 8192, "pta_layer_norm_ce_mix: the normalised size must be below 8192, got %d", cols);
  PTA_REQUIRE(w0 && o0, "pta_layer_norm_ce_mix: null pointer");
  PTA_REQUIRE((!w1 || o1) && (!w2 || o2), "pta_layer_norm_ce_mix: a mixing vector needs its output");
  const void* ptrs[7] = {y, w0, w1, w2, o0, o1, o2};
  for (const void* q : ptrs) PTA_REQUIRE(!q || pta_aligned(q, 16), "pta_layer_norm_ce_mix: pointers must be 16-byte aligned");
  const NormMix mix{(f16*)prev, {(const f16*)w0, (const f16*)w1, (const f16*)w2}, {(f16*)o0, (f16*)o1, (f16*)o2}};
  if (rows == 1)
    hipLaunchKernelGGL((norm_kernel<1, true>), dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (const f16*)x,
                       (const f16*)gamma, (const f16*)beta, (f16*)y, cols, eps, (const int32_t*)nullptr, 0, mix);
  else
    hipLaunchKernelGGL((norm_kernel<2, true>), dim3(rows), dim3(NORM_THREADS), 0, (hipStream_t)stream, (const f16*)x,
                       (const f16*)gamma, (const f16*)beta, (f16*)y, cols, eps, (const int32_t*)nullptr, 0, mix);
  PTA_CHECK_LAUNCH("pta_layer_norm_ce_mix");
  return PTA_OK;
}
