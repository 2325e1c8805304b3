// Next-token selection and the per-step loop bookkeeping.
//
// Greedy selection: layers/lm_head.py:47-57 -> ops.topk(k=1, axis=2) (ops/popart.py:135-137)
// over fp16 logits; equal maxima resolve to the lowest index (ONNX TopK).
// Loop bookkeeping: models/base_model.py:313-355 (step_containers, step_loop_cond).
// Embedding rows: layers/embedding.py:34-36, models/gpt2/embedding.py:31-36.
#include "common.h"

constexpr int AM_THREADS = 1024;

__global__ __launch_bounds__(AM_THREADS) void argmax_kernel(const f16* __restrict__ x, int32_t* __restrict__ idx,
                                                            f16* __restrict__ val, int n) {
  __shared__ float sv[AM_THREADS / 64];
  __shared__ int si[AM_THREADS / 64];
  const f16* xr = x + (size_t)blockIdx.x * n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  // 16-byte vectors where the row allows them (a thread's loads of a row are independent: four at a time travel
  // together), single elements for a row that does not start on a 16-byte boundary and for the tail
  const int nvec = (reinterpret_cast<uintptr_t>(xr) & 15) == 0 ? n >> 3 : 0;
  for (int c = threadIdx.x; c < nvec; c += 4 * AM_THREADS) {
    f16x8 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int cu = c + u * AM_THREADS;
      v[u] = *reinterpret_cast<const f16x8*>(xr + (size_t)(cu < nvec ? cu : c) * 8);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int cu = c + u * AM_THREADS;
      if (cu < nvec) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float f = (float)v[u][e];
          const int i = cu * 8 + e;
          if (f > best || (f == best && i < bi)) { best = f; bi = i; }
        }
      }
    }
  }
  for (int i = nvec * 8 + threadIdx.x; i < n; i += AM_THREADS) {
    const float v = (float)xr[i];
    if (v > best || (v == best && i < bi)) { best = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { sv[wave] = best; si[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < AM_THREADS / 64; ++w)
      if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
    // A row without any finite-comparable value (all NaN) selects index 0.
    idx[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    if (val) val[blockIdx.x] = (f16)best;
  }
}

extern "C" int pta_argmax(const pta_half* logits, int32_t* ids, pta_half* values, int rows, int n, pta_stream_t stream) {
  PTA_REQUIRE(logits && ids, "pta_argmax: null pointer");
  PTA_REQUIRE(rows > 0 && n > 0, "pta_argmax: empty input [%d,%d]", rows, n);
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(AM_THREADS), 0, (hipStream_t)stream, (const f16*)logits, ids,
                     (f16*)values, n);
  PTA_CHECK_LAUNCH("pta_argmax");
  return PTA_OK;
}

// ops.topk(k) over the last axis (ops/popart.py:135-137; layers/lm_head.py:52-53,89 with topk > 1):
// the k largest logits of a row in descending order, equal values in ascending order of index (ONNX
// TopK).  One workgroup per row; pass j finds the largest element that comes after pick j - 1 in that
// order, so no state beyond the previous pick is kept and equal values are handled exactly.
__global__ __launch_bounds__(AM_THREADS) void topk_kernel(const f16* __restrict__ x, int32_t* __restrict__ idx,
                                                          f16* __restrict__ val, int n, int k) {
  __shared__ float sv[AM_THREADS / 64];
  __shared__ int si[AM_THREADS / 64];
  __shared__ float pv;
  __shared__ int pi;
  const f16* xr = x + (size_t)blockIdx.x * n;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // A row of up to 65536 elements that starts on a 16-byte boundary is read once: thread t keeps the 16-byte vectors
  // t, t + 1024, ... in registers (NaN - never picked - past the end) and the k passes run over those.
  constexpr int TK_VEC = 8;
  const bool kept = (reinterpret_cast<uintptr_t>(xr) & 15) == 0 && (n & 7) == 0 && n <= TK_VEC * 8 * AM_THREADS;
  f16x8 keep[TK_VEC];
  if (kept) {
    const f16 nan = bitcast<f16>((uint16_t)0x7E00u);
#pragma unroll
    for (int u = 0; u < TK_VEC; ++u) {
      const int c = threadIdx.x + u * AM_THREADS;
      keep[u] = f16x8{nan, nan, nan, nan, nan, nan, nan, nan};
      if (c * 8 < n) keep[u] = *reinterpret_cast<const f16x8*>(xr + (size_t)c * 8);
    }
  }
  // A thread's best remaining element stays its best until that element is picked (it lost to every pick so far, so
  // it comes after them in the order): only the thread whose element was picked looks through its elements again.
  float last_v = INFINITY, best = -INFINITY;
  int last_i = -1, bi = 0x7fffffff;
  bool stale = true;
  for (int j = 0; j < k; ++j) {
    if (stale) {
      best = -INFINITY;
      bi = 0x7fffffff;
      if (kept) {
#pragma unroll
        for (int u = 0; u < TK_VEC; ++u)
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float v = (float)keep[u][e];
            const int i = (threadIdx.x + u * AM_THREADS) * 8 + e;
            const bool after = v < last_v || (v == last_v && i > last_i);      // NaN compares false: never picked
            if (after && (v > best || (v == best && i < bi))) { best = v; bi = i; }
          }
      } else {
        for (int i = threadIdx.x; i < n; i += AM_THREADS) {
          const float v = (float)xr[i];
          const bool after = v < last_v || (v == last_v && i > last_i);
          if (after && (v > best || (v == best && i < bi))) { best = v; bi = i; }
        }
      }
      stale = false;
    }
    float wb = best;
    int wi = bi;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(wb, o, 64);
      const int oi = __shfl_xor(wi, o, 64);
      if (ov > wb || (ov == wb && oi < wi)) { wb = ov; wi = oi; }
    }
    if (lane == 0) { sv[wave] = wb; si[wave] = wi; }
    __syncthreads();
    if (wave == 0) {      // the sixteen waves' candidates meet in the first wave's lanes
      static_assert(AM_THREADS / 64 == 16, "one lane per wave, four exchange steps");
      wb = sv[lane & 15];
      wi = si[lane & 15];
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) {
        const float ov = __shfl_xor(wb, o, 64);
        const int oi = __shfl_xor(wi, o, 64);
        if (ov > wb || (ov == wb && oi < wi)) { wb = ov; wi = oi; }
      }
      if (lane == 0) {
        // fewer than k comparable values (NaN rows, or -inf repeated): index 0 with value -inf
        idx[(size_t)blockIdx.x * k + j] = wi == 0x7fffffff ? 0 : wi;
        if (val) val[(size_t)blockIdx.x * k + j] = (f16)wb;
        pv = wb;
        pi = wi;
      }
    }
    __syncthreads();
    last_v = pv;
    last_i = pi;
    stale = bi == last_i;          // the picked element was this thread's (or nothing is left to pick: every thread looks again, and finds nothing)
    __syncthreads();
  }
}

extern "C" int pta_topk(const pta_half* logits, int32_t* ids, pta_half* values, int rows, int n, int k, pta_stream_t stream) {
  PTA_REQUIRE(logits && ids, "pta_topk: null pointer");
  PTA_REQUIRE(rows > 0 && n > 0, "pta_topk: empty input [%d,%d]", rows, n);
  PTA_REQUIRE(k >= 1 && k <= n, "pta_topk: k must be in [1, %d], got %d", n, k);
  hipLaunchKernelGGL(topk_kernel, dim3(rows), dim3(AM_THREADS), 0, (hipStream_t)stream, (const f16*)logits, ids,
                     (f16*)values, n, k);
  PTA_CHECK_LAUNCH("pta_topk");
  return PTA_OK;
}

// ops.random_sample (ops/popart.py:25-29): next[r] = candidates[r, *pick], the same column of the top-k
// candidates for every row (the reference draws one index per step: the argmax of k normal draws).
__global__ void take_column_kernel(const int32_t* __restrict__ cand, const int32_t* __restrict__ pick,
                                   int32_t* __restrict__ out, int rows, int k) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  int c = *pick;
  c = c < 0 ? 0 : (c >= k ? k - 1 : c);
  out[r] = cand[(size_t)r * k + c];
}

extern "C" int pta_take_column(const int32_t* candidates, const int32_t* pick, int32_t* out, int rows, int k,
                               pta_stream_t stream) {
  PTA_REQUIRE(candidates && pick && out, "pta_take_column: null pointer");
  PTA_REQUIRE(rows > 0 && k > 0, "pta_take_column: empty input [%d,%d]", rows, k);
  hipLaunchKernelGGL(take_column_kernel, dim3((rows + 255) / 256), dim3(256), 0, (hipStream_t)stream, candidates, pick,
                     out, rows, k);
  PTA_CHECK_LAUNCH("pta_take_column");
  return PTA_OK;
}

// out[b, :] = table[id_b, :] (+ pos_table[*pos, :] in fp16 when pos_table is given), with
// id_b = ids[b * ids_stride + (ids_index ? *ids_index : 0)]: the column `step` of the id container
// (dynamic_slice of models/llama2/model.py:168) is read in place.
__global__ __launch_bounds__(256) void gather_rows_kernel(const f16* __restrict__ table, const int32_t* __restrict__ ids,
                                                          int ids_stride, const int32_t* __restrict__ ids_index,
                                                          const f16* __restrict__ pos_table, const int32_t* __restrict__ pos,
                                                          f16* __restrict__ out, int cols, int vocab) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= cols) return;
  int col = ids_index ? *ids_index : 0;
  col = col < 0 ? 0 : (col >= ids_stride ? ids_stride - 1 : col);
  int id = ids[(size_t)b * ids_stride + col];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  f16 v = table[(size_t)id * cols + c];
  if (pos_table) v = v + pos_table[(size_t)(*pos) * cols + c];
  out[(size_t)b * cols + c] = v;
}

extern "C" int pta_embedding(const pta_half* table, const int32_t* ids, int ids_stride, const int32_t* ids_index,
                             const pta_half* pos_table, const int32_t* pos, pta_half* out, int rows, int cols,
                             int vocab, pta_stream_t stream) {
  PTA_REQUIRE(table && ids && out, "pta_embedding: null pointer");
  PTA_REQUIRE(!pos_table || pos, "pta_embedding: a position table needs a position");
  PTA_REQUIRE(rows > 0 && cols > 0 && vocab > 0 && ids_stride > 0, "pta_embedding: empty shape");
  hipLaunchKernelGGL(gather_rows_kernel, dim3((cols + 255) / 256, rows), dim3(256), 0, (hipStream_t)stream,
                     (const f16*)table, ids, ids_stride, ids_index, (const f16*)pos_table, pos, (f16*)out, cols, vocab);
  PTA_CHECK_LAUNCH("pta_embedding");
  return PTA_OK;
}

// One loop iteration of the generation bookkeeping, for all sequences:
//   next_step = step + 1; mask[:, next_step] = 0;
//   slot = container[:, next_step]; id = (slot == pad_id) ? next_ids : slot;
//   container[:, next_step] = id; stop_mask |= (id == eos_id);
//   keep_going = early_stop ? sum(stop_mask before this update) < B : true.
// Writes at index max_len fall outside the containers and are dropped.  ids_out receives
// container[:, next_step] (the input of the next iteration); *step is advanced last.
__global__ void step_update_kernel(int32_t* container, f16* mask, int32_t* stop_mask, int32_t* step,
                                   const int32_t* next_ids, int32_t* ids_out, int32_t* keep_going, int B,
                                   int max_len, int pad_id, int eos_id, int early_stop) {
  __shared__ int stopped_before;
  // Once the loop condition has gone false the reference's Loop stops iterating: a further
  // call must leave every container as it is.
  if (keep_going && *keep_going == 0) return;
  if (threadIdx.x == 0) stopped_before = 0;
  __syncthreads();
  const int st = *step;
  const int ns = st + 1;
  for (int b = threadIdx.x; b < B; b += blockDim.x) {
    if (stop_mask[b]) atomicAdd(&stopped_before, 1);
    int id = next_ids[b];
    if (ns < max_len) {
      if (mask) mask[(size_t)b * max_len + ns] = (f16)0.0f;
      const int slot = container[(size_t)b * max_len + ns];
      id = slot == pad_id ? id : slot;
      container[(size_t)b * max_len + ns] = id;
    }
    stop_mask[b] |= (id == eos_id) ? 1 : 0;
    if (ids_out) ids_out[b] = id;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    if (keep_going) *keep_going = early_stop ? (stopped_before < B ? 1 : 0) : 1;
    *step = ns;
  }
}

extern "C" int pta_step_update(int32_t* container, pta_half* mask, int32_t* stop_mask, int32_t* step,
                               const int32_t* next_ids, int32_t* ids_out, int32_t* keep_going, int B, int max_len,
                               int pad_id, int eos_id, int early_stop, pta_stream_t stream) {
  PTA_REQUIRE(container && stop_mask && step && next_ids, "pta_step_update: null pointer");
  PTA_REQUIRE(B > 0 && max_len > 0, "pta_step_update: empty shape");
  hipLaunchKernelGGL(step_update_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, container, (f16*)mask, stop_mask,
                     step, next_ids, ids_out, keep_going, B, max_len, pad_id, eos_id, early_stop);
  PTA_CHECK_LAUNCH("pta_step_update");
  return PTA_OK;
}
