// One decode-loop iteration of a Llama-2-shaped INT4 model as ONE persistent kernel.
//
// The loop body of the reference (models/base_model.py:271-355 around models/llama2/model.py:162-197)
// is a chain of phases each of which needs ALL results of the previous one: [RMSNorm + q/k/v] ->
// [rotary + KV append + attention] -> [o_proj + residual] -> [RMSNorm + gate/up + SwiGLU] ->
// [down + residual], once per layer, then [RMSNorm + lm_head] -> [top-1 + container update].
// Launched as separate kernels, every phase pays a launch boundary and a cold start of the weight
// stream; at batch 1 a 7B layer's 101 MB of weights stream in 13 us and the boundaries take longer
// than that.  Here one workgroup per compute unit stays resident for the whole iteration, phases
// are separated by a grid barrier, and every wave holds the weight tiles of the next phase(s) in
// registers: they are requested one phase (or more) before they are used, so HBM streams while
// the grid synchronises and the phases themselves only wait for activations.
//
// Numerics are those of the per-operator entry points (formats.h, norm.hip, attention.hip,
// select.hip), which the parity tests compare against the CPU restatement; this file only changes
// when things happen (and the order in which attention partials are merged).
//
// Memory ordering between workgroups.  Results that another workgroup reads in the same launch are
// written with agent-scope stores (they go through the writer's L2 to memory) and read with
// agent-scope loads (they do not hit stale lines); a writer only has to wait until its stores have
// completed before it signals.  A write-back or invalidation of the whole L2 per barrier, which is
// what fences at agent scope cost, measured 5-20 us here and is avoided.
//
// Grid barrier.  sync[0] holds the epoch base, sync[1] an error flag, sync[16 + g] the arrival
// word of workgroup g.  The waves that wrote results wait for their stores, the workgroup meets,
// thread 0 publishes the epoch in its arrival word, wave 0 polls all arrival words, and the
// workgroup meets again.  The poll is bounded: if an epoch has not arrived after DS_SPIN_LIMIT
// polls the (sticky) error flag is set, every workgroup passes its remaining barriers without
// waiting, and the kernel ends without advancing the loop.
//
// Loads return in order within a wave, so a wave that waits for a small activation load also waits
// for every weight tile it requested before; each phase therefore requests its activations first
// and the next weights second, and all waves request weights at the same program points, which
// lets the compiler count exactly how many requests may stay in flight at each use.
#include "common.h"
#include "formats.h"

namespace {

constexpr int DS_WAVES = 16;
constexpr int DS_THREADS = DS_WAVES * 64;
constexpr int DS_STORE_WAVES = 4;
constexpr unsigned DS_SPIN_LIMIT = 1u << 20;
constexpr int DS_MAXB = 4;
constexpr int DS_D = 128;                                   // head size
constexpr int DS_MAX_SPLIT = 16;
constexpr int DS_RED = DS_WAVES * 3 * 16 * DS_MAXB;         // floats in one reduction buffer
constexpr int DS_ATT_FLOATS = 3 * DS_D / 2 + 2 * DS_WAVES + DS_WAVES * DS_D;
constexpr int DS_TAIL_FLOATS = DS_WAVES * DS_MAXB + 64 + 4; // norm sums | selection scratch | flags
constexpr int DS_LAYER_WORDS = sizeof(pta_decode_layer) / 4;

// indices of the pointers in pta_decode_layer
enum { P_WQ, P_WK, P_WV, P_WO, P_WG, P_WU, P_WD, P_SQ, P_SK, P_SV, P_SO, P_SG, P_SU, P_SD, P_N1, P_N2, P_KV };
static_assert(sizeof(pta_decode_layer) == 17 * sizeof(void*), "layer descriptor layout");

struct DsArgs {
  const uint32_t* layers;   // [n_layer] pta_decode_layer
  int n_layer;
  const f16* embed;
  const f16* final_norm;
  const u32x4* head;     // fp16 tiled
  const f16* inv_freq;   // fp16 [D/2]
  int B, d, H, ffn, vocab, max_len;
  float eps;
  int32_t* container; f16* mask; int32_t* stop_mask; int32_t* step; int32_t* keep_going; int32_t* next_ids;
  int pad_id, eos_id, early_stop;
  f16* x; f16* qkv; f16* ctx; f16* act; f16* logits;
  float* attn_part;      // [B*H, nsplit, D + 2]
  unsigned* tickets;     // [B*H], zero between launches
  unsigned* sync;
  int nsplit;
  int region0;           // bytes of the activation / attention area at the start of LDS
  unsigned long long* trace;
};

#ifdef DS_TRACE
#define TRACE(i) do { if (li == 1 && thread_id() == 0) a.trace[g.wg * 32 + (i)] = wall_clock64(); } while (0)
#else
#define TRACE(i) do {} while (0)
#endif

struct Grid {
  unsigned* sync;
  unsigned epoch;
  int G, wg;
  bool dead;
};

// The asm statements make the thread index opaque at each use, so that what a phase derives from
// it is recomputed there (a few integer instructions) instead of being kept in registers across
// the whole layer loop.
__device__ __forceinline__ int thread_id() { int t = threadIdx.x; asm volatile("" : "+v"(t)); return t; }
__device__ __forceinline__ int lane_id() { return thread_id() & 63; }
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(thread_id() >> 6); }

__device__ __forceinline__ void wg_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Pointers rebuilt from descriptor words carry no address space; loads through them would be FLAT
// loads, which count against the LDS counter as well and stall every LDS wait behind the weight
// stream.  These casts state that the memory is global.
#define DS_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ const DS_GLOBAL T* as_global(const T* p) { return (const DS_GLOBAL T*)p; }
template <class T>
__device__ __forceinline__ DS_GLOBAL T* as_global(T* p) { return (DS_GLOBAL T*)p; }

__device__ __forceinline__ void put(f16* p, f16 v) {
  __hip_atomic_store((DS_GLOBAL uint16_t*)p, bitcast<uint16_t>(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void put(float* p, float v) {
  __hip_atomic_store((DS_GLOBAL float*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float get(const float* p) {
  return __hip_atomic_load((const DS_GLOBAL float*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f16 get(const f16* p) {
  return bitcast<f16>(__hip_atomic_load((const DS_GLOBAL uint16_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// 16 bytes at agent scope, through a buffer descriptor because only buffer loads take the scope
// bits together with a 128-bit width
__device__ __forceinline__ f16x8 get8(const f16* base, size_t bytes, int byte_offset) {
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<f16*>(base), 0, (int)bytes, 0x00020000);
  return bitcast<f16x8>(__builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, 0, 16 /* sc1 */));
}

// the agent-scope stores of this wave have completed; called before the grid barrier (or a ticket)
// by the waves that store results, i.e. the first DS_STORE_WAVES of a workgroup
__device__ __forceinline__ void release_results() {
  if (wave_id() < DS_STORE_WAVES) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

__device__ __forceinline__ void grid_barrier(Grid& g, int* lds_flag) {
  const int wave = wave_id(), lane = lane_id();
  wg_sync();
  if (!g.dead) {
    if (thread_id() == 0)
      __hip_atomic_store(g.sync + 16 + g.wg, g.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (wave == 0) {
      unsigned spins = 0;
      int bad = 0;
      for (;;) {
        // the arrival words and the error flag travel in one batch of loads: one round trip per poll
        const unsigned err = __hip_atomic_load(g.sync + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bool ok = true;
        for (int i = lane; i < g.G; i += 64) {
          const unsigned v = __hip_atomic_load(g.sync + 16 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ok = ok && ((int)(v - g.epoch) >= 0);
        }
        if (__all(ok)) break;
        if (err != 0 || ++spins > DS_SPIN_LIMIT) { bad = 1; break; }
      }
      if (bad && lane == 0) __hip_atomic_store(g.sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (lane == 0) *lds_flag = bad;
    }
  }
  wg_sync();
  if (!g.dead && *lds_flag) g.dead = true;
  g.epoch += 1;
}

// The 17 pointers of one layer as scalars: lane l reads descriptor word l from LDS (one read for
// the whole descriptor), and each pointer is two lane reads.
struct LayerPtrs {
  uint32_t w;   // word min(lane, DS_LAYER_WORDS - 1) of the descriptor
  template <class T>
  __device__ __forceinline__ T* get(int which) const {
    const uint32_t lo = __builtin_amdgcn_readlane(w, 2 * which), hi = __builtin_amdgcn_readlane(w, 2 * which + 1);
    return reinterpret_cast<T*>(((uint64_t)hi << 32) | lo);
  }
};
__device__ __forceinline__ LayerPtrs layer_ptrs(const uint32_t* lds_layers, int li) {
  const int lane = lane_id();
  return LayerPtrs{lds_layers[li * DS_LAYER_WORDS + (lane < DS_LAYER_WORDS ? lane : DS_LAYER_WORDS - 1)]};
}

// ------------------------------------------------------------------------------------------ GEMV phases
// The tiles of one unit (row-block u of NRB matrices) that one wave multiplies: K tiles wave,
// wave + 16, ..., with the scales of the unit's 16 output channels.
template <class Fmt, int NRB, int TPW>
struct Unit {
  u32x4 w[NRB][TPW][Fmt::kVec];
  typename Fmt::Scale sc[NRB];
};

struct Mat {
  const u32x4* tiled;
  const f16* scale;
};
__device__ __forceinline__ Mat layer_mat(const LayerPtrs& L, int wi, int si) {
  return Mat{L.get<const u32x4>(wi), L.get<const f16>(si)};
}

// Requests the tiles of unit u.  Every wave executes the same loads: tiles beyond KT and units
// beyond n_units are replaced by valid ones (their products are never used).
template <class Fmt, int NRB, int TPW>
__device__ __forceinline__ void load_unit(Unit<Fmt, NRB, TPW>& t, const Mat (&m)[NRB], int u, int n_units, int N, int KT) {
  constexpr int KV = Fmt::kVec;
  const int wave = wave_id(), lane = lane_id();
  u = u < n_units ? u : n_units - 1;
#pragma unroll
  for (int r = 0; r < NRB; ++r) {
    const DS_GLOBAL u32x4* p = as_global(m[r].tiled) + (size_t)u * KT * (64 * KV) + lane;
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
      int kt = wave + i * DS_WAVES;
      kt = kt < KT ? kt : KT - 1;
#pragma unroll
      for (int v = 0; v < KV; ++v) t.w[r][i][v] = __builtin_nontemporal_load(p + ((size_t)kt * KV + v) * 64);
    }
    int row = u * 16 + (lane & 15);
    row = row < N ? row : N - 1;
    if constexpr (KV == 1) {      // INT4: one fp16 scale per output channel
      const f16 sv = as_global(m[r].scale)[row];
      t.sc[r] = f16x2{sv, sv};
    } else {
      t.sc[r] = Fmt::load_scale(m[r].scale, nullptr, row, N);
    }
  }
}

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2 };

// out[r][m, n] = sum_k xs[m, k] * W_r[n, k] for unit u, whose tiles are in t.  `res` is the residual
// element of this thread (EPI_RESIDUAL), read at the start of the phase.
template <class Fmt, int NRB, int TPW, int EPI>
__device__ __forceinline__ void gemv_unit(const Unit<Fmt, NRB, TPW>& t, f16* const (&out)[NRB], int ostride, f16 res,
                                          int u, int n_units, int N, int KT, int M, const f16* xs, int xstride,
                                          float* red, int& red_buf) {
  if (u >= n_units) return;
  const int wave = wave_id(), lane = lane_id();
  int mrow = lane & 15;
  mrow = mrow < M ? mrow : M - 1;
  const f16* xl = xs + (size_t)mrow * xstride + (lane >> 4) * 8;
  f32x4 acc[NRB];
#pragma unroll
  for (int r = 0; r < NRB; ++r) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < TPW; ++i) {
    const int kt = wave + i * DS_WAVES;
    if (kt < KT) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f16x8 xb = *reinterpret_cast<const f16x8*>(xl + kt * 128 + j * 32);
#pragma unroll
        for (int r = 0; r < NRB; ++r)
          acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Fmt::a_operand(t.w[r][i], j, t.sc[r]), xb, acc[r], 0, 0, 0);
      }
    }
  }
  // the partial sums of the useful accumulator columns (activation rows m < M) meet in LDS
  float* rb = red + red_buf * DS_RED;
  if ((lane & 15) < M) {
#pragma unroll
    for (int r = 0; r < NRB; ++r)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        rb[((wave * NRB + r) * 16 + (lane >> 4) * 4 + q) * DS_MAXB + (lane & 15)] = acc[r][q];
  }
  wg_sync();
  {
    const int tid = thread_id();
    const int per = 16 * M;
    const int total = (EPI == EPI_SWIGLU ? 1 : NRB) * per;
    if (tid < total) {
      const int r = tid / per, ch = (tid % per) / M, m_ = tid % M;
      const int n = u * 16 + ch;
      if (n < N) {
        if (EPI == EPI_SWIGLU) {
          float sg = 0.f, su = 0.f;
#pragma unroll
          for (int w = 0; w < DS_WAVES; ++w) {
            sg += rb[((w * NRB + 0) * 16 + ch) * DS_MAXB + m_];
            su += rb[((w * NRB + (NRB > 1 ? 1 : 0)) * 16 + ch) * DS_MAXB + m_];
          }
          put(out[0] + (size_t)m_ * ostride + n, (f16)su * swish_f16((f16)sg));
        } else {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < DS_WAVES; ++w) s += rb[((w * NRB + r) * 16 + ch) * DS_MAXB + m_];
          f16 y = (f16)s;
          if (EPI == EPI_RESIDUAL) y = y + res;
          put(out[r] + (size_t)m_ * ostride + n, y);
        }
      }
    }
  }
  red_buf ^= 1;
}

// the residual element the epilogue thread of unit u adds (same thread mapping as gemv_unit)
__device__ __forceinline__ f16 residual_at(const f16* residual, int u, int N, int M) {
  const int tid = thread_id();
  if (tid >= 16 * M) return (f16)0.0f;
  const int n = u * 16 + tid / M;
  return n < N ? get(residual + (size_t)(tid % M) * N + n) : (f16)0.0f;
}

// Activations of a phase, first half: every thread requests its 16-byte vectors of X (fp16 [M, K]).
template <int NS>
struct Staged {
  f16x8 v[NS];
};
template <int NS>
__device__ __forceinline__ void stage_request(Staged<NS>& s, const f16* X, int M, int K, int KT) {
  const int vec_per_row = KT * 16, total = M * vec_per_row;
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const int i = thread_id() + k * DS_THREADS;
    const int m = i / vec_per_row, c = i % vec_per_row;
    s.v[k] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (i < total && c * 8 < K) s.v[k] = get8(X, (size_t)M * K * 2, (m * K + c * 8) * 2);
  }
}
// Second half: the vectors go to LDS (zero from K up to KT*128), RMS-normalised on the way when
// norm_w (in LDS) is given, as pta_rmsnorm does it (layers/rms_layer_norm.py:26-36).
template <int NS>
__device__ __forceinline__ void stage_commit(const Staged<NS>& s, int M, int K, int KT, f16* xs, int xstride,
                                             const f16* norm_w, float eps, float* scratch) {
  const int vec_per_row = KT * 16, total = M * vec_per_row;
  const int lane = lane_id(), wave = wave_id();
  if (!norm_w) {
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const int i = thread_id() + k * DS_THREADS;
      if (i < total) *reinterpret_cast<f16x8*>(xs + (size_t)(i / vec_per_row) * xstride + (i % vec_per_row) * 8) = s.v[k];
    }
    wg_sync();
    return;
  }
  float pq[DS_MAXB] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const int i = thread_id() + k * DS_THREADS;
    if (i < total) {
      const int m = i / vec_per_row;
      float s2 = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float f = (float)s.v[k][e]; s2 = __builtin_fmaf(f, f, s2); }
#pragma unroll
      for (int mm = 0; mm < DS_MAXB; ++mm) if (mm == m) pq[mm] += s2;
    }
  }
#pragma unroll
  for (int mm = 0; mm < DS_MAXB; ++mm) pq[mm] = wave_sum(pq[mm]);
  if (lane == 0) {
#pragma unroll
    for (int mm = 0; mm < DS_MAXB; ++mm) scratch[wave * DS_MAXB + mm] = pq[mm];
  }
  wg_sync();
  const float inv_n = 1.0f / (float)K;
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const int i = thread_id() + k * DS_THREADS;
    if (i < total) {
      const int m = i / vec_per_row, c = i % vec_per_row;
      f16x8 v = s.v[k];
      if (c * 8 < K) {
        float sq = 0.f;
#pragma unroll
        for (int w = 0; w < DS_WAVES; ++w) sq += scratch[w * DS_MAXB + m];
        const f16 r16 = (f16)(1.0f / sqrtf(sq * inv_n + eps));
        const f16x8 gm = *reinterpret_cast<const f16x8*>(norm_w + c * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (v[e] * r16) * gm[e];
      }
      *reinterpret_cast<f16x8*>(xs + (size_t)m * xstride + c * 8) = v;
    }
  }
  wg_sync();
}

// RMSNorm weights travel global -> register (requested a phase early) -> LDS (committed at the
// end of that phase, after the stage that used the previous weights)
__device__ __forceinline__ f16x8 normw_request(const f16* w, int d) {
  const int i = thread_id();
  return i * 8 < d ? *reinterpret_cast<const DS_GLOBAL f16x8*>(as_global(w) + i * 8) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
}
__device__ __forceinline__ void normw_commit(f16x8 v, f16* lds_w, int d) {
  const int i = thread_id();
  if (i * 8 < d) *reinterpret_cast<f16x8*>(lds_w + i * 8) = v;
}

// ------------------------------------------------------------------------------------------ attention phase
// rotate-half rotary of one element, as rope_llama in attention.hip (models/llama2/attention.py:83-97);
// cs holds fp16(cos(angle_i)) and fp16(sin(angle_i)) of this step
__device__ __forceinline__ f16 rope_at(const f16* x, int d, const f16* cs) {
  const int half = DS_D >> 1;
  const int i = d < half ? d : d - half;
  const f16 rot = d < half ? -get(x + d + half) : get(x + d - half);
  return get(x + d) * cs[i] + rot * cs[half + i];
}

// merges the online-softmax state of the lane `o` lanes away into this lane's
__device__ __forceinline__ void merge_lanes(float& m, float& l, float (&acc)[8], int o) {
  const float mo = __shfl_xor(m, o, 64), lo = __shfl_xor(l, o, 64);
  const float mn = fmaxf(m, mo);
  const float ca = m == -INFINITY ? 0.f : __expf(m - mn);
  const float cb = mo == -INFINITY ? 0.f : __expf(mo - mn);
  l = l * ca + lo * cb;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = acc[e] * ca + __shfl_xor(acc[e], o, 64) * cb;
  m = mn;
}

// One (sequence, head, split) unit: rotary of q and of the new k, append of the new K/V row to the
// ring by the split whose range holds it, online-softmax attention over this split's rows, partial
// result to global memory; the last split of a head to finish combines the partials into ctx.
__device__ __forceinline__ void attention_unit(const DsArgs& a, f16* kring_base, int unit, int step, float* lds,
                                               const f16* cs, int* lds_i) {
  constexpr int D = DS_D, LPP = D / 8, PPW = 64 / LPP;
  const int wave = wave_id(), lane = lane_id();
  const int bh = unit / a.nsplit, split = unit % a.nsplit;
  const int b = bh / a.H, h = bh % a.H;
  const int valid = step + 1 < a.max_len ? step + 1 : a.max_len;
  const int pos = step % a.max_len;
  const int chunk = ((valid + a.nsplit - 1) / a.nsplit + 63) & ~63;
  const int c0 = split * chunk;
  const int c1 = c0 + chunk < valid ? c0 + chunk : valid;
  f16* q_s = reinterpret_cast<f16*>(lds);            // [D] rotated q
  f16* k_s = q_s + D;                                 // [D] rotated new k
  f16* v_s = k_s + D;                                 // [D] new v
  float* sm_m = lds + 3 * D / 2;                      // [DS_WAVES]
  float* sm_l = sm_m + DS_WAVES;
  float* sm_acc = sm_l + DS_WAVES;                    // [DS_WAVES][D]
  const f16* qrow = a.qkv + (size_t)b * 3 * a.d + h * D;
  const f16* krow = qrow + a.d;
  const f16* vrow = qrow + 2 * a.d;
  f16* kring = kring_base + ((size_t)b * a.H + h) * a.max_len * D;
  f16* vring = kring + (size_t)a.B * a.H * a.max_len * D;
  const bool owner = pos >= c0 && pos < c0 + chunk;
  {
    const int tid = thread_id();
    if (tid < D) {
      q_s[tid] = rope_at(qrow, tid, cs);
    } else if (tid < 2 * D) {
      const int d_ = tid - D;
      const f16 kr = rope_at(krow, d_, cs);
      k_s[d_] = kr;
      if (owner) as_global(kring)[(size_t)pos * D + d_] = kr;
    } else if (tid < 3 * D) {
      const int d_ = tid - 2 * D;
      const f16 vv = get(vrow + d_);
      v_s[d_] = vv;
      if (owner) as_global(vring)[(size_t)pos * D + d_] = vv;
    }
  }
  wg_sync();
  float* part = a.attn_part + ((size_t)bh * a.nsplit + split) * (D + 2);
  if (c0 < valid) {
    const int grp = lane / LPP, sub = lane % LPP, d0 = sub * 8;
    float qf[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[e] = (float)q_s[d0 + e];
    const f16 scale = (f16)0.08838834764831845f;   // fp16(1/sqrt(128))
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    for (int p0 = c0 + wave * PPW; p0 < c1; p0 += DS_WAVES * PPW) {
      const int p = p0 + grp;
      const bool on = p < c1;
      const int pc = on ? p : c1 - 1;
      f16x8 k8, v8;
      if (pc == pos) {      // this step's row: taken from LDS, its global copy is being written
        k8 = *reinterpret_cast<const f16x8*>(k_s + d0);
        v8 = *reinterpret_cast<const f16x8*>(v_s + d0);
      } else {
        k8 = *reinterpret_cast<const DS_GLOBAL f16x8*>(as_global(kring) + (size_t)pc * D + d0);
        v8 = *reinterpret_cast<const DS_GLOBAL f16x8*>(as_global(vring) + (size_t)pc * D + d0);
      }
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s = __builtin_fmaf(qf[e], (float)k8[e], s);
#pragma unroll
      for (int o = LPP / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
      f16 s16 = (f16)s;          // fp16 output of the q.K^T MatMul
      s16 = s16 * scale;         // fp16 multiply by fp16(1/sqrt(D))
      const float x = on ? (float)s16 : -INFINITY;
      const float mn = fmaxf(m, x);
      const float corr = m == -INFINITY ? 0.f : __expf(m - mn);
      const float pe = on ? __expf(x - mn) : 0.f;
      l = l * corr + pe;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(pe, (float)v8[e], acc[e] * corr);
      m = mn;
    }
    // the four row groups of a wave merge in registers, the sixteen waves in LDS
    merge_lanes(m, l, acc, 16);
    merge_lanes(m, l, acc, 32);
    if (lane == 0) { sm_m[wave] = m; sm_l[wave] = l; }
    if (lane < LPP) {
#pragma unroll
      for (int e = 0; e < 8; ++e) sm_acc[wave * D + d0 + e] = acc[e];
    }
    wg_sync();
    if (thread_id() < D) {
      const int d_ = thread_id();
      float Mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < DS_WAVES; ++i) Mx = fmaxf(Mx, sm_m[i]);
      float Ls = 0.f, As = 0.f;
#pragma unroll
      for (int i = 0; i < DS_WAVES; ++i) {
        const float w = sm_m[i] == -INFINITY ? 0.f : __expf(sm_m[i] - Mx);
        Ls = __builtin_fmaf(sm_l[i], w, Ls);
        As = __builtin_fmaf(sm_acc[i * D + d_], w, As);
      }
      put(part + 2 + d_, As);
      if (d_ == 0) { put(part, Mx); put(part + 1, Ls); }
    }
  } else if (thread_id() == 0) {
    put(part, -INFINITY); put(part + 1, 0.f);      // an empty split contributes nothing
  }
  // ticket: the last split of this head to arrive combines all partials into ctx
  release_results();
  wg_sync();
  if (thread_id() == 0) {
    const unsigned t = __hip_atomic_fetch_add(a.tickets + bh, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = (t == (unsigned)a.nsplit - 1) ? 1 : 0;
    if (last) __hip_atomic_store(a.tickets + bh, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *lds_i = last;
  }
  wg_sync();
  if (*lds_i && thread_id() < D) {
    const int d_ = thread_id();
    const float* p = a.attn_part + (size_t)bh * a.nsplit * (D + 2);
    float pm[DS_MAX_SPLIT], pl[DS_MAX_SPLIT], pa[DS_MAX_SPLIT];
#pragma unroll
    for (int s = 0; s < DS_MAX_SPLIT; ++s) {       // all loads in one batch
      const bool on = s < a.nsplit;
      const float* ps = p + (size_t)(on ? s : 0) * (D + 2);
      pm[s] = get(ps); pl[s] = get(ps + 1); pa[s] = get(ps + 2 + d_);
      if (!on) pm[s] = -INFINITY;
    }
    float Mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < DS_MAX_SPLIT; ++s) Mx = fmaxf(Mx, pm[s]);
    float Ls = 0.f, As = 0.f;
#pragma unroll
    for (int s = 0; s < DS_MAX_SPLIT; ++s) {
      const float w = pm[s] == -INFINITY ? 0.f : __expf(pm[s] - Mx);
      Ls = __builtin_fmaf(pl[s], w, Ls);
      As = __builtin_fmaf(pm[s] == -INFINITY ? 0.f : pa[s], w, As);
    }
    put(a.ctx + (size_t)b * a.d + h * D + d_, (f16)(As / Ls));
  }
  wg_sync();
}

// ------------------------------------------------------------------------------------------ selection and bookkeeping
// Top-1 per sequence (lowest index among equals), then the container / mask / stop-mask update of
// models/base_model.py:313-355 exactly as step_update_kernel in select.hip; workgroup 0 only.
__device__ __forceinline__ void select_and_advance(const DsArgs& a, float* lds) {
  float* sv = lds;
  int* si = reinterpret_cast<int*>(lds + DS_WAVES);
  int* ids = si + DS_WAVES;
  const int lane = lane_id(), wave = wave_id();
  for (int b = 0; b < a.B; ++b) {
    const f16* xr = a.logits + (size_t)b * a.vocab;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i0 = thread_id() * 8; i0 < a.vocab; i0 += DS_THREADS * 8) {
      if (i0 + 8 <= a.vocab) {
        const f16x8 v8 = get8(xr, (size_t)a.vocab * 2, i0 * 2);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float v = (float)v8[e];
          if (v > best) { best = v; bi = i0 + e; }
        }
      } else {
        for (int i = i0; i < a.vocab; ++i) {
          const float v = (float)get(xr + i);
          if (v > best) { best = v; bi = i; }
        }
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (lane == 0) { sv[wave] = best; si[wave] = bi; }
    wg_sync();
    if (thread_id() == 0) {
      for (int w = 1; w < DS_WAVES; ++w)
        if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
      ids[b] = bi == 0x7fffffff ? 0 : bi;
    }
    wg_sync();
  }
  if (thread_id() == 0) {
    const int ns = *a.step + 1;
    int stopped_before = 0;
    for (int b = 0; b < a.B; ++b) {
      if (a.stop_mask[b]) ++stopped_before;
      int id = ids[b];
      a.next_ids[b] = id;
      if (ns < a.max_len) {
        a.mask[(size_t)b * a.max_len + ns] = (f16)0.0f;
        const int slot = a.container[(size_t)b * a.max_len + ns];
        id = slot == a.pad_id ? id : slot;
        a.container[(size_t)b * a.max_len + ns] = id;
      }
      a.stop_mask[b] |= (id == a.eos_id) ? 1 : 0;
    }
    *a.keep_going = a.early_stop ? (stopped_before < a.B ? 1 : 0) : 1;
    *a.step = ns;
  }
}

// ------------------------------------------------------------------------------------------ the kernel
// TPW_D / TPW_F: K tiles per wave for K = hidden / ffn; U_F: gate/up row-blocks per workgroup.
// hidden row-blocks (q/k/v, o_proj, down) are at most one per workgroup.
// MAXB: largest batch the instance stages (vectors per thread: NS_D for K = hidden, NS_F for K = ffn).
template <int TPW_D, int TPW_F, int U_F, int MAXB>
__global__ __launch_bounds__(DS_THREADS) void decode_step_kernel(DsArgs a) {
  constexpr int NS_D = (MAXB * TPW_D * DS_WAVES * 16 + DS_THREADS - 1) / DS_THREADS;
  constexpr int NS_F = (MAXB * TPW_F * DS_WAVES * 16 + DS_THREADS - 1) / DS_THREADS;
  extern __shared__ __align__(16) unsigned char smem[];
  // once the loop condition has gone false a further iteration leaves everything as it is
  if (*a.keep_going == 0) return;
  const int KT_D = (a.d + 127) / 128, KT_F = (a.ffn + 127) / 128;
  const int xstride = (KT_D > KT_F ? KT_D : KT_F) * 128 + 8;
  f16* xs = reinterpret_cast<f16*>(smem);
  float* att_lds = reinterpret_cast<float*>(smem);           // the attention phase reuses the activation area
  float* red = reinterpret_cast<float*>(smem + a.region0);
  float* scratch = red + 2 * DS_RED;                          // norm sums, then selection scratch, then flags
  int* lds_flag = reinterpret_cast<int*>(scratch + DS_WAVES * DS_MAXB + 64);
  f16* normw = reinterpret_cast<f16*>(scratch + DS_TAIL_FLOATS);   // [d]
  f16* cs = normw + ((a.d + 7) & ~7);                              // [D]: cos, sin of this step's angles
  uint32_t* lds_layers = reinterpret_cast<uint32_t*>(cs + DS_D);   // [n_layer] descriptors

  const int M = a.B;
  const int step = *a.step;
  const int nb_d = (a.d + 15) / 16, nb_f = (a.ffn + 15) / 16, nb_v = (a.vocab + 15) / 16;
  Grid g;
  g.sync = a.sync; g.G = gridDim.x; g.wg = blockIdx.x; g.dead = false;
  g.epoch = __hip_atomic_load(a.sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
  int red_buf = 0;

  // ---- set-up: descriptors and this step's rotary factors into LDS, embedding rows into x
  {
    const int tid = thread_id();
    for (int i = tid; i < a.n_layer * DS_LAYER_WORDS; i += DS_THREADS) lds_layers[i] = a.layers[i];
    if (tid < DS_D / 2) {
      const f16 ang = (f16)((float)(f16)(float)step * (float)a.inv_freq[tid]);
      cs[tid] = (f16)cosf((float)ang);
      cs[DS_D / 2 + tid] = (f16)sinf((float)ang);
    }
    if (tid == 0) { lds_flag[0] = 0; lds_flag[1] = 0; }
    // x[b] = embed[container[b, step]] (layers/embedding.py:34-36)
    const int col = step < a.max_len ? step : a.max_len - 1;
    for (int i = g.wg * DS_THREADS + tid; i < M * a.d; i += g.G * DS_THREADS) {
      const int b = i / a.d, c = i % a.d;
      int id = a.container[(size_t)b * a.max_len + col];
      id = id < 0 ? 0 : (id >= a.vocab ? a.vocab - 1 : id);
      put(a.x + i, a.embed[(size_t)id * a.d + c]);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // every wave stored here
  wg_sync();

  Unit<FmtW4, 3, TPW_D> t_qkv;
  Unit<FmtW4, 1, TPW_D> t_o;
  Unit<FmtW4, 2, TPW_D> t_gu[U_F];
  Unit<FmtW4, 1, TPW_F> t_d;
  {
    const LayerPtrs L0 = layer_ptrs(lds_layers, 0);
    normw_commit(normw_request(L0.get<const f16>(P_N1), a.d), normw, a.d);
    const Mat m3[3] = {layer_mat(L0, P_WQ, P_SQ), layer_mat(L0, P_WK, P_SK), layer_mat(L0, P_WV, P_SV)};
    load_unit(t_qkv, m3, g.wg, nb_d, a.d, KT_D);
  }
  grid_barrier(g, lds_flag);

  // Within a phase the order is: request the activations, wait for them, and only then request
  // weights for later phases.  A compute unit returns loads in the order it received them from all
  // of its waves, so an activation load issued behind a burst of weight requests would wait for
  // those; issued first it takes half a microsecond.  Weights requested in one phase land while it
  // computes, publishes and synchronises; the attention phase, all latency, requests none.
  for (int li = 0; li < a.n_layer && !g.dead; ++li) {
    const LayerPtrs L = layer_ptrs(lds_layers, li);
    const Mat mgu[2] = {layer_mat(L, P_WG, P_SG), layer_mat(L, P_WU, P_SU)};
    Staged<NS_D> st;
    Staged<NS_F> st_f;
    // ---- RMSNorm + q/k/v; a row of the [B, 3d] buffer holds q | k | v.
    //      Requests o_proj and the first two gate/up units.
    TRACE(0);
    stage_request(st, a.x, M, a.d, KT_D);
    stage_commit(st, M, a.d, KT_D, xs, xstride, normw, a.eps, scratch);
    {
      const Mat mo[1] = {layer_mat(L, P_WO, P_SO)};
      load_unit(t_o, mo, g.wg, nb_d, a.d, KT_D);
#pragma unroll
      for (int k = 0; k < U_F && k < 2; ++k) load_unit(t_gu[k], mgu, g.wg + k * g.G, nb_f, a.ffn, KT_D);
    }
    TRACE(1);
    {
      f16* const o3[3] = {a.qkv, a.qkv + a.d, a.qkv + 2 * a.d};
      gemv_unit<FmtW4, 3, TPW_D, EPI_STORE>(t_qkv, o3, 3 * a.d, (f16)0.0f, g.wg, nb_d, a.d, KT_D, M, xs, xstride, red,
                                            red_buf);
    }
    TRACE(2);
    release_results();
    TRACE(3);
    grid_barrier(g, lds_flag);
    TRACE(4);
    // ---- rotary + KV append + attention
    {
      f16* kring = L.get<f16>(P_KV);
      const int units = M * a.H * a.nsplit;
      for (int u = g.wg; u < units; u += g.G) attention_unit(a, kring, u, step, att_lds, cs, lds_flag + 1);
    }
    TRACE(5);
    release_results();
    TRACE(6);
    grid_barrier(g, lds_flag);
    TRACE(7);
    // ---- o_proj + residual.  Requests the remaining gate/up units and the RMSNorm weights of the MLP.
    f16 res;
    f16x8 nw;
    stage_request(st, a.ctx, M, a.d, KT_D);
    res = residual_at(a.x, g.wg, a.d, M);
    stage_commit(st, M, a.d, KT_D, xs, xstride, nullptr, 0.f, scratch);
    nw = normw_request(L.get<const f16>(P_N2), a.d);
#pragma unroll
    for (int k = 2; k < U_F; ++k) load_unit(t_gu[k], mgu, g.wg + k * g.G, nb_f, a.ffn, KT_D);
    TRACE(8);
    {
      f16* const o1[1] = {a.x};
      gemv_unit<FmtW4, 1, TPW_D, EPI_RESIDUAL>(t_o, o1, a.d, res, g.wg, nb_d, a.d, KT_D, M, xs, xstride, red, red_buf);
    }
    normw_commit(nw, normw, a.d);
    TRACE(9);
    release_results();
    TRACE(10);
    grid_barrier(g, lds_flag);
    TRACE(11);
    // ---- RMSNorm + gate/up + SwiGLU.  Requests down.
    stage_request(st, a.x, M, a.d, KT_D);
    stage_commit(st, M, a.d, KT_D, xs, xstride, normw, a.eps, scratch);
    {
      const Mat md[1] = {layer_mat(L, P_WD, P_SD)};
      load_unit(t_d, md, g.wg, nb_d, a.d, KT_F);
    }
    TRACE(12);
    {
      f16* const o2[2] = {a.act, a.act};
#pragma unroll
      for (int k = 0; k < U_F; ++k)
        gemv_unit<FmtW4, 2, TPW_D, EPI_SWIGLU>(t_gu[k], o2, a.ffn, (f16)0.0f, g.wg + k * g.G, nb_f, a.ffn, KT_D, M, xs,
                                               xstride, red, red_buf);
    }
    TRACE(13);
    release_results();
    TRACE(14);
    grid_barrier(g, lds_flag);
    TRACE(15);
    // ---- down + residual.  Requests the q/k/v of the next layer and the next RMSNorm weights.
    stage_request(st_f, a.act, M, a.ffn, KT_F);
    res = residual_at(a.x, g.wg, a.d, M);
    stage_commit(st_f, M, a.ffn, KT_F, xs, xstride, nullptr, 0.f, scratch);
    {
      const bool more = li + 1 < a.n_layer;
      const LayerPtrs Ln = layer_ptrs(lds_layers, more ? li + 1 : li);   // the last layer's own tiles again: never used
      nw = normw_request(more ? Ln.get<const f16>(P_N1) : a.final_norm, a.d);
      const Mat m3[3] = {layer_mat(Ln, P_WQ, P_SQ), layer_mat(Ln, P_WK, P_SK), layer_mat(Ln, P_WV, P_SV)};
      load_unit(t_qkv, m3, g.wg, nb_d, a.d, KT_D);
    }
    TRACE(16);
    {
      f16* const o1[1] = {a.x};
      gemv_unit<FmtW4, 1, TPW_F, EPI_RESIDUAL>(t_d, o1, a.d, res, g.wg, nb_d, a.d, KT_F, M, xs, xstride, red, red_buf);
    }
    normw_commit(nw, normw, a.d);
    TRACE(17);
    release_results();
    TRACE(18);
    grid_barrier(g, lds_flag);
    TRACE(19);
  }
  // ---- final RMSNorm + lm_head, streamed unit by unit with the next unit's tiles in flight
  if (!g.dead) {
    const Mat m1[1] = {{a.head, nullptr}};
    f16* const o1[1] = {a.logits};
    Staged<NS_D> st;
    stage_request(st, a.x, M, a.d, KT_D);
    Unit<FmtF16, 1, TPW_D> cur;
    load_unit(cur, m1, g.wg, nb_v, a.vocab, KT_D);
    stage_commit(st, M, a.d, KT_D, xs, xstride, normw, a.eps, scratch);
    for (int u = g.wg; u < nb_v; u += g.G) {
      Unit<FmtF16, 1, TPW_D> nxt;
      load_unit(nxt, m1, u + g.G, nb_v, a.vocab, KT_D);
      gemv_unit<FmtF16, 1, TPW_D, EPI_STORE>(cur, o1, a.vocab, (f16)0.0f, u, nb_v, a.vocab, KT_D, M, xs, xstride, red,
                                             red_buf);
      cur = nxt;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  grid_barrier(g, lds_flag);
  // ---- selection and bookkeeping
  if (g.wg == 0) {
    if (!g.dead) select_and_advance(a, scratch + DS_WAVES * DS_MAXB);
    if (thread_id() == 0)   // epoch base of the next launch
      __hip_atomic_store(a.sync, g.epoch - 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

struct Variant {
  int tpw_d, tpw_f, u_f, maxb;
  void (*kern)(DsArgs);
  bool ready;
};
Variant g_variants[] = {
    {1, 1, 1, 4, decode_step_kernel<1, 1, 1, 4>, false},   // small test shapes
    {2, 6, 3, 1, decode_step_kernel<2, 6, 3, 1>, false},   // 7B: hidden 4096, ffn 11008, batch 1
    {2, 6, 3, 4, decode_step_kernel<2, 6, 3, 4>, false},   // 7B, batch 2..4
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

int device_cus(int* cus) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  if (hipDeviceGetAttribute(cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || *cus <= 0) return -1;
  return 0;
}

}  // namespace

extern "C" size_t pta_decode_step_workspace_bytes(int batch, int n_head, int head_dim) {
  int cus = 0;
  if (batch <= 0 || batch > DS_MAXB || n_head <= 0 || head_dim != DS_D || device_cus(&cus) != 0) return 0;
  // sync words | tickets | attention partials | per-workgroup timestamps of instrumented builds
  return align256((size_t)(16 + cus) * 4) + align256((size_t)batch * n_head * 4) +
         align256((size_t)batch * n_head * DS_MAX_SPLIT * (DS_D + 2) * 4) + (size_t)cus * 256;
}

extern "C" int pta_llama_decode_step(const pta_decode_model* mdl, const pta_decode_state* st, void* workspace,
                                     pta_stream_t stream) {
  PTA_REQUIRE(mdl && st && workspace, "pta_llama_decode_step: null pointer");
  PTA_REQUIRE(mdl->layers && mdl->n_layer > 0 && mdl->embed && mdl->final_norm && mdl->head && mdl->inv_freq,
              "pta_llama_decode_step: incomplete model");
  PTA_REQUIRE(st->container && st->mask && st->stop_mask && st->step && st->keep_going && st->next_ids && st->x &&
                  st->qkv && st->ctx && st->act && st->logits,
              "pta_llama_decode_step: incomplete state");
  const int B = mdl->batch, d = mdl->hidden, H = mdl->n_head, ffn = mdl->ffn;
  PTA_REQUIRE(B >= 1 && d > 0 && H > 0 && ffn > 0 && mdl->vocab > 0 && mdl->max_len > 0,
              "pta_llama_decode_step: empty shape");
  int cus = 0;
  PTA_REQUIRE(device_cus(&cus) == 0, "pta_llama_decode_step: cannot read the compute-unit count of the current device");
  const int KT_D = (d + 127) / 128, KT_F = (ffn + 127) / 128;
  const int tpw_d = (KT_D + DS_WAVES - 1) / DS_WAVES, tpw_f = (KT_F + DS_WAVES - 1) / DS_WAVES;
  const int nb_d = (d + 15) / 16, nb_f = (ffn + 15) / 16;
  const int u_f = (nb_f + cus - 1) / cus;
  Variant* var = nullptr;
  for (Variant& v : g_variants)
    if (v.tpw_d == tpw_d && v.tpw_f == tpw_f && u_f <= v.u_f && B <= v.maxb && !var) var = &v;
  if (B > DS_MAXB || mdl->head_dim != DS_D || d != H * DS_D || ffn % 8 != 0 || mdl->vocab % 8 != 0 || nb_d > cus || !var) {
    pta_set_error("pta_llama_decode_step: supports batch <= %d, head size %d, hidden = heads * head size <= %d, ffn "
                  "and vocabulary sizes that are multiples of 8, and the (hidden, ffn) of the 7B model or small test shapes "
                  "(got batch %d, head size %d, hidden %d, heads %d, ffn %d)",
                  DS_MAXB, DS_D, 16 * cus, B, mdl->head_dim, d, H, ffn);
    return PTA_EUNSUPPORTED;
  }

  DsArgs a{};
  a.layers = reinterpret_cast<const uint32_t*>(mdl->layers);
  a.n_layer = mdl->n_layer;
  a.embed = (const f16*)mdl->embed; a.final_norm = (const f16*)mdl->final_norm;
  a.head = (const u32x4*)mdl->head; a.inv_freq = (const f16*)mdl->inv_freq;
  a.B = B; a.d = d; a.H = H; a.ffn = ffn; a.vocab = mdl->vocab; a.max_len = mdl->max_len; a.eps = mdl->eps;
  a.container = st->container; a.mask = (f16*)st->mask; a.stop_mask = st->stop_mask; a.step = st->step;
  a.keep_going = st->keep_going; a.next_ids = st->next_ids;
  a.pad_id = mdl->pad_id; a.eos_id = mdl->eos_id; a.early_stop = mdl->early_stop;
  a.x = (f16*)st->x; a.qkv = (f16*)st->qkv; a.ctx = (f16*)st->ctx; a.act = (f16*)st->act; a.logits = (f16*)st->logits;
  const size_t sync_b = align256((size_t)(16 + cus) * 4), tick_b = align256((size_t)B * H * 4);
  a.sync = (unsigned*)workspace;
  a.tickets = (unsigned*)((char*)workspace + sync_b);
  a.attn_part = (float*)((char*)workspace + sync_b + tick_b);
  a.trace = (unsigned long long*)((char*)workspace + sync_b + tick_b +
                                  align256((size_t)B * H * DS_MAX_SPLIT * (DS_D + 2) * 4));
  int nsplit = cus / (B * H);
  a.nsplit = nsplit < 1 ? 1 : (nsplit > DS_MAX_SPLIT ? DS_MAX_SPLIT : nsplit);
  const int xstride = (KT_D > KT_F ? KT_D : KT_F) * 128 + 8;
  size_t region0 = (size_t)B * xstride * 2;
  if (region0 < (size_t)DS_ATT_FLOATS * 4) region0 = (size_t)DS_ATT_FLOATS * 4;
  region0 = (region0 + 15) & ~(size_t)15;
  a.region0 = (int)region0;
  const size_t lds = region0 + (size_t)(2 * DS_RED + DS_TAIL_FLOATS) * 4 + (size_t)((d + 7) & ~7) * 2 + DS_D * 2 +
                     (size_t)mdl->n_layer * sizeof(pta_decode_layer);
  PTA_REQUIRE(lds <= 160 * 1024, "pta_llama_decode_step: %zu bytes of LDS exceed a compute unit's 160 KiB", lds);

  if (!var->ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)var->kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) ==
                    hipSuccess,
                "pta_llama_decode_step: cannot reserve dynamic LDS");
    // every workgroup must be resident at once: one per compute unit, so the kernel must fit one
    int per_cu = 0;
    PTA_REQUIRE(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)var->kern, DS_THREADS, lds) ==
                        hipSuccess && per_cu >= 1,
                "pta_llama_decode_step: the kernel does not fit a compute unit");
    var->ready = true;
  }
  hipLaunchKernelGGL(var->kern, dim3(cus), dim3(DS_THREADS), lds, (hipStream_t)stream, a);
  PTA_CHECK_LAUNCH("pta_llama_decode_step");
  return PTA_OK;
}

extern "C" int pta_decode_step_failed(const void* workspace, int* failed, pta_stream_t stream) {
  PTA_REQUIRE(workspace && failed, "pta_decode_step_failed: null pointer");
  unsigned word = 0;
  hipError_t e = hipMemcpyAsync(&word, (const unsigned*)workspace + 1, 4, hipMemcpyDeviceToHost, (hipStream_t)stream);
  if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess) {
    pta_set_error("pta_decode_step_failed: %s", hipGetErrorString(e));
    return PTA_EHIP;
  }
  *failed = word != 0;
  return PTA_OK;
}
