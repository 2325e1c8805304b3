// FP16-weight GEMV/GEMM for initializers on the right-hand side of ops.matmul
// (poptransformer/ops/popart.py:55-67): lm_head (layers/lm_head.py:47-57), tied embedding heads
// and every Linear of an fp16 model (layers/linear.py:42-46).  fp16 in, fp32 accumulate
// (the reference's default partials type), fp16 out.
#include "common.h"
#include "formats.h"

__global__ __launch_bounds__(256) void f16_tile_kernel(const f16* __restrict__ w, u32x4* __restrict__ tiled,
                                                       int N, int K, int KT, size_t total_vec) {
  const size_t v = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (v >= total_vec) return;
  const int lane = (int)(v & 63);
  const int j = (int)((v >> 6) & 3);
  const size_t tile = v >> 8;
  const int kt = (int)(tile % KT);
  const int nb = (int)(tile / KT);
  const int row = nb * 16 + (lane & 15);
  const int k0 = kt * 128 + j * 32 + (lane >> 4) * 8;
  f16x8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = (row < N && k0 + i < K) ? w[(size_t)row * K + k0 + i] : (f16)0.0f;
  tiled[v] = bitcast<u32x4>(r);
}

extern "C" size_t pta_f16_tiled_bytes(int N, int K) { return gemv_tiled_bytes(N, K, FmtF16::kVec); }

extern "C" int pta_f16_tile(const pta_half* w, void* tiled, int N, int K, pta_stream_t stream) {
  PTA_REQUIRE(w && tiled, "pta_f16_tile: null pointer");
  PTA_REQUIRE(N > 0 && K > 0, "pta_f16_tile: need N > 0 and K > 0, got N=%d K=%d", N, K);
  PTA_REQUIRE(pta_aligned(tiled, 16), "pta_f16_tile: tiled buffer must be 16-byte aligned");
  const int KT = (K + 127) / 128;
  const size_t total = pta_f16_tiled_bytes(N, K) / 16;
  hipLaunchKernelGGL(f16_tile_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const f16*)w, (u32x4*)tiled, N, K, KT, total);
  PTA_CHECK_LAUNCH("pta_f16_tile");
  return PTA_OK;
}

