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
