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
