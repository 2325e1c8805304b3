// One step of beam search: the BeamSearch custom op (custom_ops/beam_search_custom_op.cpp:333-478).
//
// The reference composes the step from poplibs calls - a top-k over the vocabulary per beam, an add of the
// hypotheses' running scores, a scatter of the candidate ids into a beam-by-beam expanded copy of the
// hypothesis container, a second top-k over the beam * beam candidates and two grouped gathers - and
// materialises a [batch, max_len, beam, beam] temporary on the way.  Here the step is two kernels: one
// workgroup per (sequence, beam) selects that beam's `beam` best vocabulary entries into a small workspace,
// then one workgroup per sequence selects the `beam` best of the beam * beam candidates and rewrites the
// sequence's containers in place (each container row is read whole before it is written).  Equal scores are
// taken in ascending order of index in both selections.
#include "common.h"

namespace {

constexpr int BS_THREADS = 256;
constexpr int BS_MAX_BEAM = 64;

template <class T>
__device__ __forceinline__ float to_f32(T v) { return (float)v; }

// The j-th pass of a selection over `n` values held by the workgroup's threads (thread t holds values
// t, t + BS_THREADS, ...): the largest value not yet taken, the lowest index among equals.  `last_v`, `last_i`
// are the previous pass's pick (INFINITY / -1 before the first).  Returns the pick to every thread.
template <class Load>
__device__ __forceinline__ void select_pass(int n, Load load, float last_v, int last_i, float* sv, int* si, float& out_v,
                                            int& out_i) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < n; i += BS_THREADS) {
    const float v = load(i);
    const bool after = v < last_v || (v == last_v && i > last_i);      // NaN compares false: never picked
    if (after && (v > best || (v == best && i < bi))) { best = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
  }
  if (lane == 0) { sv[wave] = best; si[wave] = bi; }
  __syncthreads();
  for (int w = 0; w < BS_THREADS / 64; ++w)
    if (w == 0 || sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
  __syncthreads();
  out_v = best;
  out_i = bi == 0x7fffffff ? 0 : bi;      // fewer comparable values than picks (NaN rows): index 0, value -inf
}

// beamBestProb / beamBestId of :347-354: row (b, i) of the logits -> its `beam` largest entries
template <class T>
__global__ __launch_bounds__(BS_THREADS) void beam_topk_kernel(const T* __restrict__ logits, T* __restrict__ vals,
                                                               int32_t* __restrict__ ids, int V, int beam) {
  __shared__ float sv[BS_THREADS / 64];
  __shared__ int si[BS_THREADS / 64];
  const T* row = logits + (size_t)blockIdx.x * V;
  float last_v = INFINITY;
  int last_i = -1;
  for (int j = 0; j < beam; ++j) {
    float v;
    int i;
    select_pass(V, [&](int k) { return to_f32(row[k]); }, last_v, last_i, sv, si, v, i);
    if (threadIdx.x == 0) {
      vals[(size_t)blockIdx.x * beam + j] = row[i];
      ids[(size_t)blockIdx.x * beam + j] = i;
    }
    last_v = v;
    last_i = i;
  }
}

template <class T>
__global__ __launch_bounds__(BS_THREADS) void beam_update_kernel(const T* __restrict__ vals, const int32_t* __restrict__ ids,
                                                                 int32_t* __restrict__ hyp, T* __restrict__ prob,
                                                                 const int32_t* __restrict__ step_p,
                                                                 int32_t* __restrict__ next_id,
                                                                 int32_t* __restrict__ global_best_id, int beam,
                                                                 int max_len) {
  __shared__ float sv[BS_THREADS / 64];
  __shared__ int si[BS_THREADS / 64];
  __shared__ float cand[BS_MAX_BEAM * BS_MAX_BEAM];
  __shared__ int pick[BS_MAX_BEAM];
  const int b = blockIdx.x, step = *step_p;
  const int nn = beam * beam;
  const T* bv = vals + (size_t)b * nn;
  const int32_t* bid = ids + (size_t)b * nn;
  int32_t* bh = hyp + (size_t)b * max_len * beam;
  T* bp = prob + (size_t)b * beam;
  if (step == 0) {      // :371-385: the candidates of beam 0 seed every beam
    for (int j = threadIdx.x; j < beam; j += BS_THREADS) {
      next_id[(size_t)b * beam + j] = bid[j];
      global_best_id[(size_t)b * beam + j] = bid[j];
      bh[j] = bid[j];
      bp[j] = bv[j];
    }
    return;
  }
  // candidate (i, j) = score j of beam i + running score of hypothesis i, added in the containers' type (:400-401)
  for (int c = threadIdx.x; c < nn; c += BS_THREADS) cand[c] = to_f32((T)(bv[c] + bp[c / beam]));
  __syncthreads();
  float last_v = INFINITY;
  int last_i = -1;
  for (int r = 0; r < beam; ++r) {
    float v;
    int i;
    select_pass(nn, [&](int k) { return cand[k]; }, last_v, last_i, sv, si, v, i);
    if (threadIdx.x == 0) pick[r] = i;
    last_v = v;
    last_i = i;
  }
  __syncthreads();
  for (int r = threadIdx.x; r < beam; r += BS_THREADS) {
    const int g = pick[r];
    global_best_id[(size_t)b * beam + r] = g;           // flat index i * beam + j (:432)
    next_id[(size_t)b * beam + r] = bid[g];             // :438-446
    bp[r] = (T)cand[g];                                 // :465-466 (cand holds values of type T exactly)
  }
  // every row of the container is re-gathered from the parent hypotheses; row `step` takes the new ids (:403-463)
  for (int l = threadIdx.x; l < max_len; l += BS_THREADS) {
    int32_t old[BS_MAX_BEAM];
    int32_t* row = bh + (size_t)l * beam;
    for (int i = 0; i < beam; ++i) old[i] = row[i];
    for (int r = 0; r < beam; ++r) {
      const int g = pick[r];
      row[r] = l == step ? bid[g] : old[g / beam];
    }
  }
}

}  // namespace

extern "C" size_t pta_beam_search_workspace_bytes(int batch, int beam) {
  if (batch <= 0 || beam <= 0 || beam > BS_MAX_BEAM) return 0;
  const size_t n = (size_t)batch * beam * beam;
  return ((n * 4 + 255) & ~(size_t)255) + n * 4;
}

extern "C" int pta_beam_search_step(const void* logits, int dtype, int32_t* hyp_container, void* prob_container,
                                    const int32_t* step, int32_t* next_id, int32_t* global_best_id, void* workspace,
                                    int batch, int beam, int vocab, int max_len, pta_stream_t stream) {
  PTA_REQUIRE(logits && hyp_container && prob_container && step && next_id && global_best_id && workspace,
              "pta_beam_search_step: null pointer");
  PTA_REQUIRE(dtype == PTA_F16 || dtype == PTA_F32, "pta_beam_search_step: dtype must be PTA_F16 or PTA_F32");
  PTA_REQUIRE(batch > 0 && vocab > 0 && max_len > 0, "pta_beam_search_step: empty shape");
  PTA_REQUIRE(beam >= 1 && beam <= vocab,
              "[Beam Search] The parameter 'beam_size'(%d) should not be greater than the vocab_size(%d).", beam, vocab);
  PTA_REQUIRE(beam <= BS_MAX_BEAM, "pta_beam_search_step: beam_size %d exceeds %d", beam, BS_MAX_BEAM);
  PTA_REQUIRE(pta_aligned(workspace, 256), "pta_beam_search_step: the workspace must be 256-byte aligned");
  const size_t n = (size_t)batch * beam * beam;
  void* vals = workspace;
  int32_t* ids = (int32_t*)((char*)workspace + ((n * 4 + 255) & ~(size_t)255));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PTA_F16) {
    hipLaunchKernelGGL(beam_topk_kernel<f16>, dim3(batch * beam), dim3(BS_THREADS), 0, s, (const f16*)logits, (f16*)vals, ids,
                       vocab, beam);
    hipLaunchKernelGGL(beam_update_kernel<f16>, dim3(batch), dim3(BS_THREADS), 0, s, (const f16*)vals, ids, hyp_container,
                       (f16*)prob_container, step, next_id, global_best_id, beam, max_len);
  } else {
    hipLaunchKernelGGL(beam_topk_kernel<float>, dim3(batch * beam), dim3(BS_THREADS), 0, s, (const float*)logits, (float*)vals,
                       ids, vocab, beam);
    hipLaunchKernelGGL(beam_update_kernel<float>, dim3(batch), dim3(BS_THREADS), 0, s, (const float*)vals, ids, hyp_container,
                       (float*)prob_container, step, next_id, global_best_id, beam, max_len);
  }
  PTA_CHECK_LAUNCH("pta_beam_search_step");
  return PTA_OK;
}
