// SoftmaxV3 over the last axis (poptransformer/ops/customized.py:57-65,
// custom_ops/softmax.cpp:41-83): optional max subtraction, exp in the input type, the sum and
// its reciprocal in fp32, the reciprocal rounded to the input type, one multiply.
#include "common.h"

constexpr int SM_THREADS = 256;

template <typename T>
__global__ __launch_bounds__(SM_THREADS) void softmax_kernel(const T* __restrict__ x, T* __restrict__ y, int n,
                                                             int stable) {
  __shared__ float sh[SM_THREADS / 64];
  const T* xr = x + (size_t)blockIdx.x * n;
  T* yr = y + (size_t)blockIdx.x * n;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  T mx = (T)0.0f;
  if (stable) {
    float m = -INFINITY;
    for (int i = threadIdx.x; i < n; i += SM_THREADS) m = fmaxf(m, (float)xr[i]);
    m = wave_max(m);
    if (lane == 0) sh[wave] = m;
    __syncthreads();
    m = sh[0];
#pragma unroll
    for (int w = 1; w < SM_THREADS / 64; ++w) m = fmaxf(m, sh[w]);
    mx = (T)m;
    __syncthreads();
  }
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += SM_THREADS) {
    const T d = stable ? (T)(xr[i] - mx) : xr[i];   // subtraction in the input type
    const T e = (T)expf((float)d);                   // exp rounded to the input type
    yr[i] = e;
    s += (float)e;
  }
  s = wave_sum(s);
  if (lane == 0) sh[wave] = s;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < SM_THREADS / 64; ++w) tot += sh[w];
  const T r = (T)(1.0f / tot);
  for (int i = threadIdx.x; i < n; i += SM_THREADS) yr[i] = yr[i] * r;
}

extern "C" int pta_softmax_ce(const void* x, void* y, int rows, int n, int dtype, int stable_mode,
                              pta_stream_t stream) {
  // SoftmaxOp::setup (custom_ops/softmax.hpp:71-91) requires rank >= 2 and the last axis; the
  // caller flattens the leading axes into `rows`.
  PTA_REQUIRE(x && y, "[Softmax] null pointer");
  PTA_REQUIRE(rows > 0 && n > 0, "[Softmax] empty input [%d,%d]", rows, n);
  PTA_REQUIRE(dtype == PTA_F16 || dtype == PTA_F32, "[Softmax] input type must be FLOAT16 or FLOAT");
  if (dtype == PTA_F16)
    hipLaunchKernelGGL(softmax_kernel<f16>, dim3(rows), dim3(SM_THREADS), 0, (hipStream_t)stream, (const f16*)x,
                       (f16*)y, n, stable_mode);
  else
    hipLaunchKernelGGL(softmax_kernel<float>, dim3(rows), dim3(SM_THREADS), 0, (hipStream_t)stream,
                       (const float*)x, (float*)y, n, stable_mode);
  PTA_CHECK_LAUNCH("pta_softmax_ce");
  return PTA_OK;
}
