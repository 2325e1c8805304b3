// KV cache (poptransformer/ops/customized.py:21-35).
//
// The reference op keeps a persistent tensor with the sequence axis extended to max_len and,
// every step, rebuilds it as concat(new, old[0 : max_len - step_len]) after zeroing `old` when
// step == 0 (custom_ops/kv_cache.cpp:108-132): a shift register, newest entry first, paid for
// with two full-cache copies per step.  KVCachePipeline keeps max_bps such registers and
// touches only register step % max_bps (custom_ops/kv_cache_pipeline.cpp:374-451,
// custom_ops/kv_cache_codelet.cpp:18-131).
//
// Two forms are provided:
//   * pta_kv_cache_update: the literal shift register (any step_len), for callers that want
//     the reference's tensor as it stands;
//   * pta_kv_cache_append / pta_kv_cache_read: a ring buffer in arrival order written in O(1)
//     (one row per step), plus the gather that materialises the reference's newest-first
//     tensor from it bit for bit.  The fused decode attention reads the ring directly.
// All shapes are [outer, seq, inner] with `inner` contiguous; rows are moved as raw bytes.
#include "common.h"

template <typename V>
__global__ __launch_bounds__(256) void kv_clone_kernel(const V* __restrict__ cache, V* __restrict__ clone,
                                                       const int32_t* __restrict__ step, size_t nvec) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  V z;
  __builtin_memset(&z, 0, sizeof(V));
  clone[i] = (*step != 0) ? cache[i] : z;
}

template <typename V>
__global__ __launch_bounds__(256) void kv_shift_kernel(V* __restrict__ cache, const V* __restrict__ clone,
                                                       const V* __restrict__ upd, int max_len, int step_len,
                                                       int row_vec, size_t nvec) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const int c = (int)(i % row_vec);
  const size_t t = i / row_vec;
  const int p = (int)(t % max_len);
  const size_t o = t / max_len;
  cache[i] = p < step_len ? upd[(o * step_len + p) * row_vec + c]
                          : clone[(o * max_len + (p - step_len)) * row_vec + c];
}

// Ring write: row (count % max_len) of register (step % max_bps), count = step / max_bps.
template <typename V>
__global__ __launch_bounds__(256) void kv_append_kernel(V* __restrict__ cache, const V* __restrict__ upd,
                                                        const int32_t* __restrict__ step, int outer, int max_len,
                                                        int row_vec, int max_bps) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)outer * row_vec) return;
  const int st = *step;
  const int slot = st % max_bps;
  const int pos = (st / max_bps) % max_len;
  const int c = (int)(i % row_vec);
  const size_t o = i / row_vec;
  cache[(((size_t)slot * outer + o) * max_len + pos) * row_vec + c] = upd[i];
}

// Newest-first view of register (step % max_bps): out[o][i] = ring[(count - i) mod max_len] for
// i <= count, zero above (rows the shift register has not received since step 0).
template <typename V>
__global__ __launch_bounds__(256) void kv_read_kernel(const V* __restrict__ cache, V* __restrict__ out,
                                                      const int32_t* __restrict__ step, int outer, int max_len,
                                                      int row_vec, int max_bps, size_t nvec) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const int st = *step;
  const int slot = st % max_bps;
  const int count = st / max_bps;
  const int c = (int)(i % row_vec);
  const size_t t = i / row_vec;
  const int p = (int)(t % max_len);
  const size_t o = t / max_len;
  V v;
  __builtin_memset(&v, 0, sizeof(V));
  if (p <= count) {
    const int src = ((count - p) % max_len + max_len) % max_len;
    v = cache[(((size_t)slot * outer + o) * max_len + src) * row_vec + c];
  }
  out[i] = v;
}

static int vec_bytes(size_t row_bytes, const void* a, const void* b, const void* c) {
  if (row_bytes % 16 == 0 && pta_aligned(a, 16) && pta_aligned(b, 16) && (!c || pta_aligned(c, 16))) return 16;
  if (row_bytes % 4 == 0 && pta_aligned(a, 4) && pta_aligned(b, 4) && (!c || pta_aligned(c, 4))) return 4;
  if (row_bytes % 2 == 0 && pta_aligned(a, 2) && pta_aligned(b, 2) && (!c || pta_aligned(c, 2))) return 2;
  return 1;
}

static int check_kv(const char* name, int outer, int max_len, int step_len, int inner, int elem_bytes) {
  // dtypes FLOAT16 / FLOAT (custom_ops/kv_cache.hpp:85); uint8 rows cover the fp8 storage mode.
  PTA_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, "%s: element size must be 1, 2 or 4 bytes", name);
  PTA_REQUIRE(outer > 0 && inner > 0 && max_len > 0, "%s: empty shape", name);
  PTA_REQUIRE(step_len >= 1 && step_len <= max_len, "%s: step_len %d must be in [1, max_len=%d]", name, step_len, max_len);
  return PTA_OK;
}

#define KV_DISPATCH(VB, CALL)                         \
  switch (VB) {                                       \
    case 16: { typedef u32x4 V; CALL; } break;        \
    case 4: { typedef uint32_t V; CALL; } break;      \
    case 2: { typedef uint16_t V; CALL; } break;      \
    default: { typedef uint8_t V; CALL; } break;      \
  }

extern "C" int pta_kv_cache_update(void* cache, void* clone, const void* updater, const int32_t* step, int outer,
                                   int max_len, int step_len, int inner, int elem_bytes, pta_stream_t stream) {
  int rc = check_kv("pta_kv_cache_update", outer, max_len, step_len, inner, elem_bytes);
  if (rc) return rc;
  PTA_REQUIRE(cache && clone && updater && step, "pta_kv_cache_update: null pointer");
  const size_t row_bytes = (size_t)inner * elem_bytes;
  const int vb = vec_bytes(row_bytes, cache, clone, updater);
  const int row_vec = (int)(row_bytes / vb);
  const size_t nvec = (size_t)outer * max_len * row_vec;
  const dim3 grid((unsigned)((nvec + 255) / 256));
  hipStream_t s = (hipStream_t)stream;
  KV_DISPATCH(vb, hipLaunchKernelGGL(kv_clone_kernel<V>, grid, dim3(256), 0, s, (const V*)cache, (V*)clone, step, nvec);
              hipLaunchKernelGGL(kv_shift_kernel<V>, grid, dim3(256), 0, s, (V*)cache, (const V*)clone,
                                 (const V*)updater, max_len, step_len, row_vec, nvec));
  PTA_CHECK_LAUNCH("pta_kv_cache_update");
  return PTA_OK;
}

extern "C" int pta_kv_cache_append(void* cache, const void* updater, const int32_t* step, int outer, int max_len,
                                   int inner, int elem_bytes, int max_bps, pta_stream_t stream) {
  int rc = check_kv("pta_kv_cache_append", outer, max_len, 1, inner, elem_bytes);
  if (rc) return rc;
  PTA_REQUIRE(cache && updater && step, "pta_kv_cache_append: null pointer");
  PTA_REQUIRE(max_bps >= 1, "pta_kv_cache_append: max_bps must be >= 1, got %d", max_bps);
  const size_t row_bytes = (size_t)inner * elem_bytes;
  const int vb = vec_bytes(row_bytes, cache, updater, nullptr);
  const int row_vec = (int)(row_bytes / vb);
  const size_t nvec = (size_t)outer * row_vec;
  KV_DISPATCH(vb, hipLaunchKernelGGL(kv_append_kernel<V>, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0,
                                     (hipStream_t)stream, (V*)cache, (const V*)updater, step, outer, max_len,
                                     row_vec, max_bps));
  PTA_CHECK_LAUNCH("pta_kv_cache_append");
  return PTA_OK;
}

extern "C" int pta_kv_cache_read(const void* cache, void* out, const int32_t* step, int outer, int max_len,
                                 int inner, int elem_bytes, int max_bps, pta_stream_t stream) {
  int rc = check_kv("pta_kv_cache_read", outer, max_len, 1, inner, elem_bytes);
  if (rc) return rc;
  PTA_REQUIRE(cache && out && step, "pta_kv_cache_read: null pointer");
  PTA_REQUIRE(max_bps >= 1, "pta_kv_cache_read: max_bps must be >= 1, got %d", max_bps);
  const size_t row_bytes = (size_t)inner * elem_bytes;
  const int vb = vec_bytes(row_bytes, cache, out, nullptr);
  const int row_vec = (int)(row_bytes / vb);
  const size_t nvec = (size_t)outer * max_len * row_vec;
  KV_DISPATCH(vb, hipLaunchKernelGGL(kv_read_kernel<V>, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0,
                                     (hipStream_t)stream, (const V*)cache, (V*)out, step, outer, max_len, row_vec,
                                     max_bps, nvec));
  PTA_CHECK_LAUNCH("pta_kv_cache_read");
  return PTA_OK;
}

// KVCachePipeline with transpose = 1 (custom_ops/kv_cache_pipeline.cpp:397-451, codelet
// custom_ops/kv_cache_codelet.cpp:170-212): the max_bps persistent caches keep the sequence as their LAST axis,
// [outer, inner, max_len]; register step % max_bps is shifted by one element along that axis IN PLACE (there
// is no clone), the new row goes to index 0, and the op's output is that register in the input's own layout
// [outer, max_len, inner].  All registers are zeroed when step == 0 (codelet:46-64).  step_len is 1: the op
// copies the input into output[..., 0:1] (pipeline.cpp:410).
// One workgroup owns KT_D features of one `outer` row of one register and walks the sequence in chunks from the
// end to the start: a chunk's sources (element l - 1 for element l) lie in the chunk itself or at the end of
// the next lower one, which is still untouched, and inside a chunk every load is done before the first store.
constexpr int KT_D = 32, KT_L = 64;

template <typename E>
__global__ __launch_bounds__(256) void kv_seq_last_kernel(E* __restrict__ caches, E* __restrict__ out,
                                                          const E* __restrict__ upd, const int32_t* __restrict__ step_p,
                                                          int outer, int max_len, int inner, int max_bps) {
  __shared__ E tile[KT_D][KT_L + 1];
  const int st = *step_p;
  const int reg = blockIdx.z, sel = ((st % max_bps) + max_bps) % max_bps;
  if (reg != sel && st != 0) return;             // other registers are only touched by the zeroing at step 0
  const int o = blockIdx.y, d0 = blockIdx.x * KT_D;
  E* cache = caches + ((size_t)reg * outer + o) * inner * max_len;
  const int nd = inner - d0 < KT_D ? inner - d0 : KT_D;
  const int chunks = (max_len + KT_L - 1) / KT_L;
  for (int c = chunks - 1; c >= 0; --c) {
    const int l0 = c * KT_L;
    const int nl = max_len - l0 < KT_L ? max_len - l0 : KT_L;
    // tile[d][j] = the value element l0 + j will hold
    for (int t = threadIdx.x; t < KT_D * KT_L; t += 256) {
      const int d = t / KT_L, j = t % KT_L;
      if (d < nd && j < nl) {
        const int l = l0 + j;
        E v = (E)0;
        if (reg == sel) {
          if (l == 0) v = upd[(size_t)o * inner + d0 + d];
          else if (st != 0) v = cache[(size_t)(d0 + d) * max_len + l - 1];
        }
        tile[d][j] = v;
      }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < KT_D * KT_L; t += 256) {
      const int d = t / KT_L, j = t % KT_L;
      if (d < nd && j < nl) cache[(size_t)(d0 + d) * max_len + l0 + j] = tile[d][j];
    }
    if (reg == sel) {
      for (int t = threadIdx.x; t < KT_D * KT_L; t += 256) {
        const int j = t / KT_D, d = t % KT_D;
        if (d < nd && j < nl) out[((size_t)o * max_len + l0 + j) * inner + d0 + d] = tile[d][j];
      }
    }
    __syncthreads();
  }
}

extern "C" int pta_kv_cache_pipeline_seq_last(void* caches, void* out, const void* updater, const int32_t* step, int outer,
                                              int max_len, int inner, int elem_bytes, int max_bps, pta_stream_t stream) {
  int rc = check_kv("pta_kv_cache_pipeline_seq_last", outer, max_len, 1, inner, elem_bytes);
  if (rc) return rc;
  PTA_REQUIRE(caches && out && updater && step, "pta_kv_cache_pipeline_seq_last: null pointer");
  PTA_REQUIRE(max_bps >= 1 && max_bps <= 65535 && outer <= 65535,
              "pta_kv_cache_pipeline_seq_last: max_bps and outer must lie in [1, 65535]");
  const dim3 grid((unsigned)((inner + KT_D - 1) / KT_D), (unsigned)outer, (unsigned)max_bps);
  hipStream_t s = (hipStream_t)stream;
  if (elem_bytes == 1)
    hipLaunchKernelGGL(kv_seq_last_kernel<uint8_t>, grid, dim3(256), 0, s, (uint8_t*)caches, (uint8_t*)out,
                       (const uint8_t*)updater, step, outer, max_len, inner, max_bps);
  else if (elem_bytes == 2)
    hipLaunchKernelGGL(kv_seq_last_kernel<uint16_t>, grid, dim3(256), 0, s, (uint16_t*)caches, (uint16_t*)out,
                       (const uint16_t*)updater, step, outer, max_len, inner, max_bps);
  else
    hipLaunchKernelGGL(kv_seq_last_kernel<uint32_t>, grid, dim3(256), 0, s, (uint32_t*)caches, (uint32_t*)out,
                       (const uint32_t*)updater, step, outer, max_len, inner, max_bps);
  PTA_CHECK_LAUNCH("pta_kv_cache_pipeline_seq_last");
  return PTA_OK;
}
