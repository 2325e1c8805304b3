// Elementwise pieces of the decode step that are not fused into a GEMM epilogue.
#include "common.h"
#include "gemm_core.h"

// out = up * swish(gate): `ops.swish` then `ops.mul` (models/llama2/mlp.py:22-26,
// models/chatglm2/mlp.py:53-57), each an fp16 op.
__global__ __launch_bounds__(256) void swiglu_kernel(const f16* __restrict__ gate, const f16* __restrict__ up,
                                                     f16* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  out[i] = up[i] * swish_f16(gate[i]);
}

extern "C" int pta_swiglu(const pta_half* gate, const pta_half* up, pta_half* out, size_t n, pta_stream_t stream) {
  PTA_REQUIRE(gate && up && out, "pta_swiglu: null pointer");
  if (n == 0) return PTA_OK;
  hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const f16*)gate, (const f16*)up, (f16*)out, n);
  PTA_CHECK_LAUNCH("pta_swiglu");
  return PTA_OK;
}

// ------------------------------------------------------------------------------------------
// RWKV-4 (models/rwkv/attention.py:59-105, models/rwkv/ffn.py:40-59)
// ------------------------------------------------------------------------------------------

// Token-shift mixes: out_i = x * w_i + (1 - w_i) * prev for up to three mixing vectors, each step an
// fp16 op as in `gate` (attention.py:59-64): y1 = x*w; y2 = (1 - w); y2 = y2*prev; y = y1 + y2.
// Then prev <- x (attention.py:72 / ffn.py:51).
__global__ __launch_bounds__(256) void rwkv_mix_kernel(const f16* __restrict__ x, f16* __restrict__ prev,
                                                       const f16* __restrict__ w0, const f16* __restrict__ w1,
                                                       const f16* __restrict__ w2, f16* __restrict__ o0,
                                                       f16* __restrict__ o1, f16* __restrict__ o2, int rows, int cols) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * cols) return;
  const int c = i % cols;
  const f16 xv = x[i], pv = prev[i];
  const f16 one = (f16)1.0f;
  o0[i] = xv * w0[c] + (one - w0[c]) * pv;
  if (w1) o1[i] = xv * w1[c] + (one - w1[c]) * pv;
  if (w2) o2[i] = xv * w2[c] + (one - w2[c]) * pv;
  prev[i] = xv;
}

extern "C" int pta_rwkv_mix(const pta_half* x, pta_half* prev, const pta_half* w0, const pta_half* w1,
                            const pta_half* w2, pta_half* o0, pta_half* o1, pta_half* o2, int rows, int cols,
                            pta_stream_t stream) {
  PTA_REQUIRE(x && prev && w0 && o0, "pta_rwkv_mix: null pointer");
  PTA_REQUIRE((!w1 || o1) && (!w2 || o2), "pta_rwkv_mix: a mixing vector needs its output");
  PTA_REQUIRE(rows > 0 && cols > 0, "pta_rwkv_mix: empty shape");
  hipLaunchKernelGGL(rwkv_mix_kernel, dim3((rows * cols + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                     (const f16*)x, (f16*)prev, (const f16*)w0, (const f16*)w1, (const f16*)w2, (f16*)o0, (f16*)o1,
                     (f16*)o2, rows, cols);
  PTA_CHECK_LAUNCH("pta_rwkv_mix");
  return PTA_OK;
}

// WKV recurrence in fp32 (attention.py:84-100), one element per thread:
//   t = k + u; M = max(p, t); e1 = exp(p - M); e2 = exp(t - M); out = (e1 a + e2 v) / (e1 b + e2)
//   p2 = p - exp(w); M2 = max(p2, k); e1 = exp(p2 - M2); e2 = exp(k - M2);
//   a <- e1 a + e2 v; b <- e1 b + e2; p <- M2
// then y = r * fp16(out) (attention.py:101-103), r being the sigmoid of the receptance Linear.
// `ops.maximum(x, y)` is where(x > y, x, y) (ops/popart.py:212-215).
__global__ __launch_bounds__(256) void rwkv_wkv_kernel(const f16* __restrict__ k, const f16* __restrict__ v,
                                                       const f16* __restrict__ r, const f16* __restrict__ time_decay,
                                                       const f16* __restrict__ time_first, float* __restrict__ num,
                                                       float* __restrict__ den, float* __restrict__ mx,
                                                       f16* __restrict__ y, int rows, int cols) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * cols) return;
  const int c = i % cols;
  const float kf = (float)k[i], vf = (float)v[i];
  const float u = (float)time_first[c], w = (float)time_decay[c];
  const float a = num[i], b = den[i], p = mx[i];
  const float t = kf + u;
  const float M = p > t ? p : t;
  float e1 = expf(p - M), e2 = expf(t - M);
  const float out = (e1 * a + e2 * vf) / (e1 * b + e2);
  const float p2 = p - expf(w);
  const float M2 = p2 > kf ? p2 : kf;
  e1 = expf(p2 - M2);
  e2 = expf(kf - M2);
  num[i] = e1 * a + e2 * vf;
  den[i] = e1 * b + e2;
  mx[i] = M2;
  y[i] = r[i] * (f16)out;
}

extern "C" int pta_rwkv_wkv(const pta_half* k, const pta_half* v, const pta_half* r, const pta_half* time_decay,
                            const pta_half* time_first, float* num, float* den, float* max_state, pta_half* y, int rows,
                            int cols, pta_stream_t stream) {
  PTA_REQUIRE(k && v && r && time_decay && time_first && num && den && max_state && y, "pta_rwkv_wkv: null pointer");
  PTA_REQUIRE(rows > 0 && cols > 0, "pta_rwkv_wkv: empty shape");
  hipLaunchKernelGGL(rwkv_wkv_kernel, dim3((rows * cols + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                     (const f16*)k, (const f16*)v, (const f16*)r, (const f16*)time_decay, (const f16*)time_first, num,
                     den, max_state, (f16*)y, rows, cols);
  PTA_CHECK_LAUNCH("pta_rwkv_wkv");
  return PTA_OK;
}
