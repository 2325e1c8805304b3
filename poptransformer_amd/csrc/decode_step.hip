// One decode-loop iteration of a Llama-2-shaped INT4 model as ONE persistent kernel.
//
// The loop body of the reference (models/base_model.py:271-355 around models/llama2/model.py:162-197)
// is a chain of phases each of which needs ALL results of the previous one: [RMSNorm + q/k/v] ->
// [rotary + KV append + attention] -> [o_proj + residual] -> [RMSNorm + gate/up + SwiGLU] ->
// [down + residual], once per layer, then [RMSNorm + lm_head] -> [top-1 + container update].
// Launched as separate kernels, every phase pays a launch boundary and a cold start of the weight
// stream; at batch 1 a 7B layer's 101 MB of weights stream in 13 us and the boundaries take longer
// than that.  Here one workgroup per compute unit stays resident for the whole iteration and every
// wave holds the weight tiles of the next phase(s) in registers: they are requested a phase or
// more before they are used, so HBM streams while the phases wait for each other's results.
//
// Numerics are those of the per-operator entry points (norm.hip, attention.hip, select.hip), which
// the parity tests compare against the CPU restatement, with two differences: the order in which
// attention partials are merged, and the INT4 products, which apply the scale once to the fp32 sum
// instead of multiplying by fp16(q * s) (see gemv_slots).  The lm_head (fp16) is as in formats.h.
//
// How phases hand over results.  Every intermediate vector of the iteration (the residual stream
// after each half layer, q|k|v, the attention output, the SwiGLU output, attention partials, the
// logits) has a slot of its own in the workspace.  At the start of a launch all slots are filled
// with a bit pattern no result can have (all ones: a NaN that the stores below never write), one
// grid barrier follows, and from then on a consumer simply loads the values it needs until none
// of them is the filler: data and "ready" travel in the same load, there is no flag to wait for
// first and no barrier between phases.  Producers write with agent-scope stores (through the
// writer's L2 to memory), consumers read with agent-scope loads (no stale lines), so neither side
// needs a cache write-back or invalidation, which cost 5-20 us per use here.  Every wait is
// bounded: after DS_SPIN_LIMIT polls a wave sets the sticky error word of the workspace, every
// workgroup that sees it stops, and the loop state is left as it was.
//
// A compute unit returns loads in the order it received them from all of its waves, so a small
// activation load issued behind a burst of weight requests waits for those.  Each phase therefore
// first obtains its activations and only then requests weights for later phases.  A compute unit
// also accepts only a few tens of KiB of requests at a time: a wave that requests more is held at
// the request until earlier data has arrived, and the workgroup's barrier behind the phase's product
// waits for that wave.  The requests are therefore spread over the phases (64-96 KiB per workgroup
// and phase at the 7B shape) instead of being issued where registers first become free.  Every
// tile has a fixed place in one register array for the whole layer loop, so that no requested tile
// is ever moved between registers (a move waits for the load and for the burst around it).
#include <cstdlib>
#include <mutex>

#include "common.h"
#include "formats.h"

namespace {

constexpr int DS_WAVES = 16;
constexpr int DS_THREADS = DS_WAVES * 64;
constexpr unsigned DS_SPIN_LIMIT = 1u << 20;
constexpr unsigned long long DS_LAUNCH_TICKS = 20000000ull;   // a launch gives up 200 ms after it started (constant 100 MHz clock)
constexpr int DS_REPLICAS = 16;                             // copies of a row of arrival words, see grid_barrier
constexpr int DS_MAXB = 4;
constexpr int DS_D = 128;                                   // head size
constexpr int DS_MAX_SPLIT = 16;
constexpr int DS_PART = DS_D + 2;                           // floats of one attention partial
constexpr int DS_RED = DS_WAVES * 6 * 16 * DS_MAXB;         // floats in one reduction buffer (up to six matrices)
constexpr int DS_ATT_FLOATS = 3 * DS_D + 2 * DS_WAVES + DS_WAVES * DS_D;     // q | k | v of two units, per-wave softmax states
constexpr int DS_XSUM = DS_WAVES * DS_MAXB + 64 + 4;        // offset of the per-wave sums of the staged activations
constexpr int DS_TAIL_FLOATS = DS_XSUM + DS_WAVES * DS_MAXB; // norm sums | selection scratch | flags | activation sums
constexpr int DS_LAYER_WORDS = sizeof(pta_decode_layer) / 4;
constexpr uint16_t DS_EMPTY16 = 0xFFFFu;                    // filler of fp16 slots
constexpr uint32_t DS_EMPTY32 = 0xFFFFFFFFu;                // filler of fp32 slots

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
  f16* logits;
  // slots in the workspace
  f16* xres;             // [2 n_layer + 1][B, d]: residual stream after the embedding and after each half layer
  f16* qkv;              // [n_layer][B, 3d]
  f16* ctx;              // [n_layer][B, d]
  f16* act;              // [n_layer][B, ffn]
  float* part;           // [n_layer][B*H, nsplit, DS_PART]
  size_t fill_bytes;     // qkv .. end of part, contiguous from xres + B*d (the first residual is not filled)
  unsigned* flags;       // [4 n_layer + 1][DW_REPLICAS][flag_words] arrival words of decode_step_wide_kernel, behind part
  int flag_words;        // words of one row: the workgroups, rounded up to a KiB
  uint32_t* best;        // [workgroups][16 rows][2]: value bits and index of each workgroup's largest logit per row (wide kernel)
  unsigned* sync;
  int nsplit;
  int kv_scale;          // KV8 kernels: the rings hold F143 bytes of value * 2^-kv_scale (custom_ops/kv_cache.cpp:43-74)
  int region0;           // bytes of the activation / attention area at the start of LDS
  int xcd_groups;        // workgroups take their work by die: see logical_workgroup
  unsigned long long* trace;
};

#ifdef DS_TRACE
constexpr int DS_TRACE_WORDS = 128;      // per workgroup: 32 of the first thread, then 6 per wave
#define TRACE(i) do { if (li == 1 && thread_id() == 0) a.trace[g.wg * DS_TRACE_WORDS + (i)] = wall_clock64(); } while (0)
#define TRACE_AT(i) (li == 1 ? a.trace + g.wg * DS_TRACE_WORDS + (i) : nullptr)
#define TRACE_STEP(i) do { if (thread_id() == 0) a.trace[g.wg * DS_TRACE_WORDS + (i)] = wall_clock64(); } while (0)
#define WTRACE(k) do { if (li == 1 && lane_id() == 0) a.trace[g.wg * DS_TRACE_WORDS + 32 + wave_id() * 6 + (k)] = wall_clock64(); } while (0)
#else
constexpr int DS_TRACE_WORDS = 32;
#define WTRACE(k) do {} while (0)
#define TRACE(i) do {} while (0)
#define TRACE_AT(i) nullptr
#define TRACE_STEP(i) do {} while (0)
#endif

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

// results: agent-scope stores that never write the filler (a NaN with another payload replaces it)
__device__ __forceinline__ void put(f16* p, f16 v) {
  uint16_t bits = bitcast<uint16_t>(v);
  bits = bits == DS_EMPTY16 ? (uint16_t)0xFE00u : bits;
  __hip_atomic_store((DS_GLOBAL uint16_t*)p, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void put(float* p, float v) {
  uint32_t bits = bitcast<uint32_t>(v);
  bits = bits == DS_EMPTY32 ? 0xFFC00000u : bits;
  __hip_atomic_store((DS_GLOBAL uint32_t*)p, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t get_bits(const float* p) {
  return __hip_atomic_load((const DS_GLOBAL uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint16_t get_bits(const f16* p) {
  return __hip_atomic_load((const DS_GLOBAL uint16_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 bytes at agent scope, through a buffer descriptor because only buffer accesses take the scope
// bits together with a 128-bit width
__device__ __forceinline__ u32x4 get16(const void* base, size_t bytes, size_t byte_offset) {
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_offset, 0, 16 /* sc1 */);
}
__device__ __forceinline__ void put16(void* base, size_t bytes, size_t byte_offset, u32x4 v) {
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)bytes, 0x00020000);
  __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)byte_offset, 0, 16 /* sc1 */);
}
__device__ __forceinline__ bool has_empty16(u32x4 v) {
  bool e = false;
#pragma unroll
  for (int i = 0; i < 4; ++i) e = e || (v[i] & 0xFFFFu) == DS_EMPTY16 || (v[i] >> 16) == DS_EMPTY16;
  return e;
}

// Bounded waiting of one wave.  `give_up` turns true when the wave has polled DS_SPIN_LIMIT times,
// when the launch has run for DS_LAUNCH_TICKS (a launch whose workgroups cannot all be resident ends
// within a quarter of a second instead of spinning through every wait), or when another workgroup has
// reported a failure; the wave then sets the error word and the
// workgroup-wide flag in LDS and stops waiting.
struct Waiter {
  unsigned* err;     // sync[1]
  int* lds_dead;
  unsigned spins;
  unsigned long long deadline;     // of the launch, on the constant-rate clock
  __device__ __forceinline__ bool give_up() {
    ++spins;
    bool stop = spins > DS_SPIN_LIMIT;
    if ((spins & 63u) == 0)
      stop = stop || wall_clock64() > deadline ||
             __hip_atomic_load((DS_GLOBAL unsigned*)err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
    if (stop) {
      __hip_atomic_store((DS_GLOBAL unsigned*)err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *lds_dead = 1;
    }
    return stop;
  }
};

// wave-uniform wait for one fp16 / fp32 value per lane (lanes with on == false do not wait)
__device__ __forceinline__ f16 wait_value(const f16* p, bool on, Waiter& w) {
  uint16_t bits = 0;
  for (;;) {
    if (on) bits = get_bits(p);
    if (!__any(on && bits == DS_EMPTY16) || w.give_up()) break;
  }
  return bitcast<f16>(bits);
}
__device__ __forceinline__ float wait_value(const float* p, bool on, Waiter& w) {
  uint32_t bits = 0;
  for (;;) {
    if (on) bits = get_bits(p);
    if (!__any(on && bits == DS_EMPTY32) || w.give_up()) break;
  }
  return bitcast<float>(bits);
}

// the same for two fp16 values per lane whose loads travel together (one round trip, not two)
__device__ __forceinline__ void wait_pair(const f16* p0, bool on0, const f16* p1, bool on1, f16& v0, f16& v1, Waiter& w) {
  uint16_t b0 = 0, b1 = 0;
  for (;;) {
    if (on0) b0 = get_bits(p0);
    if (on1) b1 = get_bits(p1);
    if (!__any((on0 && b0 == DS_EMPTY16) || (on1 && b1 == DS_EMPTY16)) || w.give_up()) break;
  }
  v0 = bitcast<f16>(b0);
  v1 = bitcast<f16>(b1);
}
// and for three fp32 values per lane
__device__ __forceinline__ void wait_triple(const float* p0, const float* p1, const float* p2, bool on2, float& v0, float& v1,
                                            float& v2, Waiter& w) {
  uint32_t b0 = 0, b1 = 0, b2 = 0;
  for (;;) {
    b0 = get_bits(p0);
    b1 = get_bits(p1);
    if (on2) b2 = get_bits(p2);
    if (!__any(b0 == DS_EMPTY32 || b1 == DS_EMPTY32 || (on2 && b2 == DS_EMPTY32)) || w.give_up()) break;
  }
  v0 = bitcast<float>(b0);
  v1 = bitcast<float>(b1);
  v2 = bitcast<float>(b2);
}

// The one grid barrier of a launch (after the slots have been filled).  sync[0] holds the epoch
// base, sync[1] the error word, sync[16 + r * G + g] copy r of the arrival word of workgroup g: the
// words of one copy share a memory channel, and G workgroups polling one copy queue there for
// microseconds, so every workgroup writes DS_REPLICAS copies and polls copy g % DS_REPLICAS.
__device__ __forceinline__ void grid_barrier(unsigned* sync, unsigned epoch, int G, int wg, Waiter& w) {
  const int wave = wave_id(), lane = lane_id();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's agent-scope stores have completed
  wg_sync();
  if (wave == 0) {
    if (lane < DS_REPLICAS)
      __hip_atomic_store((DS_GLOBAL unsigned*)(sync + 16 + lane * G + wg), epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned* mine = sync + 16 + (wg % DS_REPLICAS) * G;
    for (;;) {
      bool ok = true;
      for (int i = lane; i < G; i += 64) {
        const unsigned v = __hip_atomic_load((DS_GLOBAL unsigned*)(mine + i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = ok && ((int)(v - epoch) >= 0);
      }
      if (__all(ok) || w.give_up()) break;
    }
  }
  wg_sync();
}

// Which share of the work the workgroup with hardware index `block` takes.  The device hands workgroups to its eight
// dies (each with an L2 of its own) in turn: block b runs on die b % 8.  A head's q | k | v channels, the splits of
// its attention and the merge of their partials all belong to eight consecutive logical indices, so giving the 32
// blocks of a die 32 consecutive logical indices keeps those hand-overs inside one L2 - a store followed by a load
// that hits there - where a hand-over between dies goes through memory.  Any permutation is correct; this one is
// only faster.
__device__ __forceinline__ int logical_workgroup(int block, int G, int xcd_groups) {
  return xcd_groups && G % 8 == 0 ? (block % 8) * (G / 8) + block / 8 : block;
}

// Sum over the sixteen lanes of a row (lanes 16 k .. 16 k + 15), left in every lane of the row: data-parallel moves
// inside the row, no LDS.
__device__ __forceinline__ float row_sum16(float v) {
  v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0xB1, 0xF, 0xF, true));    // quad_perm [1, 0, 3, 2]
  v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x4E, 0xF, 0xF, true));    // quad_perm [2, 3, 0, 1]
  v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x140, 0xF, 0xF, true));   // row_mirror
  return v;
}

// Sum over all 64 lanes, the same in every lane: the rows' sums by data-parallel moves, then the four rows' totals
// through scalar registers (a shuffle through the LDS crossbar per step takes several times as long).
__device__ __forceinline__ float wave_total(float v) {
  v = row_sum16(v);
  const int b = bitcast<int>(v);
  return bitcast<float>(__builtin_amdgcn_readlane(b, 0)) + bitcast<float>(__builtin_amdgcn_readlane(b, 16)) +
         (bitcast<float>(__builtin_amdgcn_readlane(b, 32)) + bitcast<float>(__builtin_amdgcn_readlane(b, 48)));
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

// The partial sums of the useful accumulator columns (activation rows m < M) of all waves meet in
// LDS; `res` is the residual element of this thread (EPI_RESIDUAL), and the value the thread
// stored is returned (it is the residual of the same thread in the next residual phase).
struct NoScales {};
// SCALED: the sums are over stored codes q + 8; 8 * sum(x) (xsum: per-wave partial sums of the staged
// activations) comes off and the channel's scale (SC[scbase + r] of the finishing lane, whose
// channel is lane % 16) is applied before the rounding to fp16.
template <int NRB, int EPI, bool SCALED = false, class Scales = NoScales, int MB = DS_MAXB, int RED = DS_RED>
__device__ __forceinline__ f16 finish_unit(const f32x4 (&acc)[NRB], f16* const (&out)[NRB], int ostride, f16 res, int u,
                                           int N, int M, float* red, int& red_buf, const float* xsum = nullptr,
                                           const Scales& SC = Scales{}, int scbase = 0) {
  constexpr int DS_MAXB = MB;      // rows a reduction buffer has room for (shadows the narrow kernel's constant)
  const int wave = wave_id(), lane = lane_id();
  float* rb = red + red_buf * RED;
  if ((lane & 15) < M) {
#pragma unroll
    for (int r = 0; r < NRB; ++r)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        rb[((wave * NRB + r) * 16 + (lane >> 4) * 4 + q) * DS_MAXB + (lane & 15)] = acc[r][q];
  }
  wg_sync();
  f16 y = res;
  {
    // thread (r * M + m_) * 16 + ch finishes channel ch of row m_ of matrix r (M <= 4: no division)
    const int tid = thread_id();
    const int total = (EPI == EPI_SWIGLU ? 1 : NRB) * 16 * M;
    if (tid < total) {
      const int q = tid >> 4, ch = tid & 15;
      const int r = (q >= M ? 1 : 0) + (q >= 2 * M ? 1 : 0);
      const int m_ = q - r * M;
      const int n = u * 16 + ch;
      if (n < N) {
        float off = 0.f, scale[NRB];
        if constexpr (SCALED) {
#pragma unroll 8
          for (int w = 0; w < DS_WAVES; ++w) off += xsum[w * DS_MAXB + m_];
          off *= 8.0f;
#pragma unroll
          for (int i = 0; i < NRB; ++i) scale[i] = (float)SC[scbase + i][0];
        }
        if (EPI == EPI_SWIGLU) {
          float sg = 0.f, su = 0.f;
#pragma unroll 4
          for (int w = 0; w < DS_WAVES; ++w) {
            sg += rb[((w * NRB + 0) * 16 + ch) * DS_MAXB + m_];
            su += rb[((w * NRB + (NRB > 1 ? 1 : 0)) * 16 + ch) * DS_MAXB + m_];
          }
          if constexpr (SCALED) { sg = (sg - off) * scale[0]; su = (su - off) * scale[NRB > 1 ? 1 : 0]; }
          put(out[0] + (size_t)m_ * ostride + n, (f16)su * swish_f16((f16)sg));
        } else {
          float s = 0.f;
#pragma unroll 8
          for (int w = 0; w < DS_WAVES; ++w) s += rb[((w * NRB + r) * 16 + ch) * DS_MAXB + m_];
          if constexpr (SCALED) {
            float sc = scale[0];
#pragma unroll
            for (int i = 1; i < NRB; ++i) sc = r == i ? scale[i] : sc;
            s = (s - off) * sc;
          }
          y = (f16)s;
          if (EPI == EPI_RESIDUAL) y = y + res;
          put(out[r] + (size_t)m_ * ostride + n, y);
        }
      }
    }
  }
  red_buf ^= 1;
  return y;
}

// finish_unit with the sixteen waves' partial sums of an output met by the sixteen lanes of a row: lane w of the row
// reads wave w's sum, the row adds up in registers, and the lane whose index in the row is the output's channel
// finishes it (so the scale it holds, SC of lane % 16, is the channel's).  Output o of a pass is row o of the
// workgroup's threads: o = (r * M + m) * 16 + ch; more than 64 outputs take several passes.  The residual element of
// (row m, channel ch) therefore lives in thread (m * 16 + ch) * 16 + ch (see residual_thread).
template <int NRB, int EPI, bool SCALED = false, class Scales = NoScales, int MB = DS_MAXB, int RED = DS_RED>
__device__ __forceinline__ f16 finish_unit_rows(const f32x4 (&acc)[NRB], f16* const (&out)[NRB], int ostride, f16 res, int u,
                                                int N, int M, float* red, int& red_buf, const float* xsum = nullptr,
                                                const Scales& SC = Scales{}, int scbase = 0) {
  static_assert(EPI != EPI_SWIGLU, "the gate / up pairs finish in finish_gate_up");
  const int wave = wave_id(), lane = lane_id();
  float* rb = red + red_buf * RED;
  if ((lane & 15) < M) {
#pragma unroll
    for (int r = 0; r < NRB; ++r)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        rb[((wave * NRB + r) * 16 + (lane >> 4) * 4 + q) * MB + (lane & 15)] = acc[r][q];
  }
  wg_sync();
  f16 y = res;
  const int total = NRB * 16 * M * 16;      // sixteen lanes per output
  for (int base = 0; base < total; base += DS_THREADS) {
    const int idx = base + thread_id();
    if (idx < total) {                       // whole rows: total is a multiple of 16
      const int o = idx >> 4, w = idx & 15;
      const int q = o >> 4, ch = o & 15;
      const int r = (q >= M ? 1 : 0) + (q >= 2 * M ? 1 : 0);
      const int m_ = q - r * M;
      float s = row_sum16(rb[((w * NRB + r) * 16 + ch) * MB + m_]);
      float off = 0.f;
      if constexpr (SCALED) off = 8.0f * row_sum16(xsum[w * DS_MAXB + m_]);
      const int n = u * 16 + ch;
      if (w == ch && n < N) {
        if constexpr (SCALED) {
          float sc = (float)SC[scbase][0];
#pragma unroll
          for (int i = 1; i < NRB; ++i) sc = r == i ? (float)SC[scbase + i][0] : sc;
          s = (s - off) * sc;
        }
        y = (f16)s;
        if (EPI == EPI_RESIDUAL) y = y + res;
        put(out[r] + (size_t)m_ * ostride + n, y);
      }
    }
  }
  red_buf ^= 1;
  return y;
}
// the thread that finishes (row m, channel ch) of a one-matrix unit in finish_unit_rows, as (m, ch, whether this thread is one)
__device__ __forceinline__ bool residual_thread(int& m_, int& ch) {
  const int tid = thread_id();
  const int o = tid >> 4;
  m_ = o >> 4;
  ch = o & 15;
  return (tid & 15) == ch;
}

// out[r][m, n] = sum_k xs[m, k] * W_r[n, k] for unit u, whose tiles are in t.  `res` is the residual
// element of this thread (EPI_RESIDUAL); the value the thread stored is returned (it is the
// residual of the same thread in the next residual phase).
template <class Fmt, int NRB, int TPW, int EPI, int MAXB>
__device__ __forceinline__ f16 gemv_unit(const Unit<Fmt, NRB, TPW>& t, f16* const (&out)[NRB], int ostride, f16 res,
                                         int u, int n_units, int N, int KT, int M, const f16* xs, int xstride,
                                         float* red, int& red_buf) {
  if (u >= n_units) return res;
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
  return finish_unit_rows<NRB, EPI>(acc, out, ostride, res, u, N, M, red, red_buf);
}

// The INT4 tiles of the layer phases live in ONE register array with a fixed place for every unit
// (the map is in the kernel), and so do their scales.  A place is written by the loads of the unit
// that owns it at that point of the layer and read by that unit's products, always under the same
// compile-time index, so no value ever has to move between registers: a move of a requested tile
// would have to wait for its load, and with it for the whole burst of requests around it.
// Requests tiles [FIRST, FIRST + COUNT) of unit u (tile r * TPW + i is tile i of matrix r), and the
// scales of the matrices whose first tile is among them.
template <int NRB, int TPW, int BASE, int SCBASE, int FIRST = 0, int COUNT = NRB * TPW, int NSLOT, int NSC>
__device__ __forceinline__ void load_slots(u32x4 (&S)[NSLOT], f16x2 (&SC)[NSC], const Mat (&m)[NRB], int u, int n_units,
                                           int N, int KT) {
  static_assert(BASE + NRB * TPW <= NSLOT && SCBASE + NRB <= NSC, "unit outside the register array");
  static_assert(FIRST >= 0 && COUNT >= 0 && FIRST + COUNT <= NRB * TPW, "tiles outside the unit");
  const int wave = wave_id(), lane = lane_id();
  u = u < n_units ? u : n_units - 1;
#pragma unroll
  for (int t = FIRST; t < FIRST + COUNT; ++t) {
    const int r = t / TPW, i = t % TPW;
    int kt = wave + i * DS_WAVES;
    kt = kt < KT ? kt : KT - 1;
    S[BASE + t] = __builtin_nontemporal_load(as_global(m[r].tiled) + ((size_t)u * KT + kt) * 64 + lane);
    if (i == 0) {
      int row = u * 16 + (lane & 15);
      row = row < N ? row : N - 1;
      const f16 sv = as_global(m[r].scale)[row];
      SC[SCBASE + r] = f16x2{sv, sv};
    }
  }
}

// out[r][m, n] = fp16(s_r[n] * sum_k xs[m, k] * q_r[n, k]) for unit u: the scale is applied once, to
// the fp32 sum, where the per-operator kernels multiply by fp16(q * s) (the reference materialises
// that matrix, ops/customized.py:115-125 into ops/popart.py:55-67); the two differ by the rounding of
// the 4096..11008 products q * s to fp16, far below the rounding of the fp16 result.  It makes the
// weights cost 5 VALU instructions per 8 instead of 13, and this phase is bound by exactly those.
// A stored code c = q + 8 masked in place is the fp16 subnormal c * 2^-24 (nibble 0 or 2 of a
// half, after a shift by 8 for the latter) or c * 2^-20 (nibble 1 or 3); the matrix unit takes
// subnormal operands at their exact value.  Steps of equal weight share an accumulator;
// sum_k x * (c - 8) = 2^24 acc_even + 2^20 acc_odd - 8 sum_k x, with sum_k x from `stage`.
template <int NRB, int TPW, int BASE, int NSLOT>
__device__ __forceinline__ void slots_product(const u32x4 (&S)[NSLOT], f32x4 (&sum)[NRB], int u, int n_units, int KT, int M,
                                              const f16* xs, int xstride) {
#pragma unroll
  for (int r = 0; r < NRB; ++r) sum[r] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (u >= n_units) return;
  const int wave = wave_id(), lane = lane_id();
  int mrow = lane & 15;
  mrow = mrow < M ? mrow : M - 1;
  const f16* xl = xs + (size_t)mrow * xstride + (lane >> 4) * 8;
  f32x4 acc[NRB][2];
#pragma unroll
  for (int r = 0; r < NRB; ++r) acc[r][0] = acc[r][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < TPW; ++i) {
    const int kt = wave + i * DS_WAVES;
    if (kt < KT) {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const f16x8 xb = *reinterpret_cast<const f16x8*>(xl + kt * 128 + m * 32);
#pragma unroll
        for (int r = 0; r < NRB; ++r) {
          const u32x4 w = S[BASE + r * TPW + i];
          u32x4 c;
#pragma unroll
          for (int d = 0; d < 4; ++d) c[d] = (m >= 2 ? w[d] >> 8 : w[d]) & ((m & 1) ? 0x00f000f0u : 0x000f000fu);
          acc[r][m & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<f16x8>(c), xb, acc[r][m & 1], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < NRB; ++r) sum[r] = acc[r][0] * 16777216.0f + acc[r][1] * 1048576.0f;
}

template <int NRB, int TPW, int EPI, int MAXB, int BASE, int SCBASE, int NSLOT, int NSC>
__device__ __forceinline__ f16 gemv_slots(const u32x4 (&S)[NSLOT], const f16x2 (&SC)[NSC], f16* const (&out)[NRB],
                                          int ostride, f16 res, int u, int n_units, int N, int KT, int M, const f16* xs,
                                          int xstride, float* red, int& red_buf, const float* xsum,
                                          unsigned long long* trace = nullptr, unsigned long long* wtrace = nullptr) {
  if (u >= n_units) return res;
  f32x4 sum[NRB];
  slots_product<NRB, TPW, BASE>(S, sum, u, n_units, KT, M, xs, xstride);
#ifdef DS_TRACE
  if (trace) { asm volatile("" :: "v"(sum[0][0])); if (thread_id() == 0) *trace = wall_clock64(); }
  if (wtrace && lane_id() == 0) { asm volatile("" :: "v"(sum[0][0])); wtrace[wave_id() * 6 + 1] = wall_clock64(); }
  const f16 y = finish_unit_rows<NRB, EPI, true>(sum, out, ostride, res, u, N, M, red, red_buf, xsum, SC, SCBASE);
  if (wtrace && lane_id() == 0) wtrace[wave_id() * 6 + 2] = wall_clock64();
  return y;
#endif
  return finish_unit_rows<NRB, EPI, true>(sum, out, ostride, res, u, N, M, red, red_buf, xsum, SC, SCBASE);
}

// The gate/up units of a workgroup (units wg, wg + G, ...) finish together: one meeting of the partial
// sums in LDS and one round of stores for all of them.  A wave puts the gate / up sums of unit k into
// LDS as soon as it has them (stash_gate_up); sg[k] / su[k] are the scales of this lane's channel.
template <int U_F>
__device__ __forceinline__ void stash_gate_up(const f32x4 (&sum)[2], int k, int M, float* red, int red_buf) {
  const int wave = wave_id(), lane = lane_id();
  float* rb = red + red_buf * DS_RED;
  if ((lane & 15) < M) {
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        rb[((wave * (2 * U_F) + 2 * k + r) * 16 + (lane >> 4) * 4 + q) * DS_MAXB + (lane & 15)] = sum[r][q];
  }
}

template <int U_F, int MAXB>
__device__ __forceinline__ void finish_gate_up(const float (&sg)[U_F], const float (&su)[U_F], f16* act, int ffn, int wg, int G,
                                               int nb_f, int M, float* red, int& red_buf, const float* xsum) {
  float* rb = red + red_buf * DS_RED;
  wg_sync();
  // as finish_unit_rows: output o = (k * M + m) * 16 + ch of a pass is row o of the threads, lane w of the row brings
  // wave w's gate and up sums, the lane with index ch in the row finishes the output (it holds the channel's scales)
  const int per = 16 * M, total = U_F * per * 16;
  for (int base = 0; base < total; base += DS_THREADS) {
    const int idx = base + thread_id();
    if (idx < total) {
      const int o = idx >> 4, w = idx & 15;
      const int k = (o >= per ? 1 : 0) + (o >= 2 * per ? 1 : 0);
      const int m_ = (o - k * per) >> 4, ch = o & 15;
      float g = row_sum16(rb[((w * (2 * U_F) + 2 * k) * 16 + ch) * DS_MAXB + m_]);
      float v = row_sum16(rb[((w * (2 * U_F) + 2 * k + 1) * 16 + ch) * DS_MAXB + m_]);
      const float off = 8.0f * row_sum16(xsum[w * DS_MAXB + m_]);
      const int u = wg + k * G, n = u * 16 + ch;
      if (w == ch && u < nb_f && n < ffn) {
        float cg = sg[0], cu = su[0];
#pragma unroll
        for (int i = 1; i < U_F; ++i) { cg = k == i ? sg[i] : cg; cu = k == i ? su[i] : cu; }
        g = (g - off) * cg;
        v = (v - off) * cu;
        put(act + (size_t)m_ * ffn + n, (f16)v * swish_f16((f16)g));
      }
    }
  }
  red_buf ^= 1;
}

// i / per for i < 4 * per, without a division
__device__ __forceinline__ int row_of(int i, int per) { return (i >= per ? 1 : 0) + (i >= 2 * per ? 1 : 0) + (i >= 3 * per ? 1 : 0); }

// Activations of a phase.  Every thread loads its 16-byte vectors of X (fp16 [M, K]) until none of
// their elements is the filler, then the vectors go to LDS (zero from K up to KT*128), RMS-
// normalised on the way when norm_w (in LDS) is given, as pta_rmsnorm does it
// (layers/rms_layer_norm.py:26-36).  Returns false when the wait was given up.
template <int NS, int MAXB>
__device__ __forceinline__ bool stage(const f16* X, int M, int K, int KT, f16* xs, int xstride, const f16* norm_w,
                                      float eps, float* scratch, Waiter& w, unsigned long long* trace = nullptr) {
  const int vec_per_row = KT * 16, total = M * vec_per_row;
  const int lane = lane_id(), wave = wave_id();
  u32x4 v[NS];
  bool need[NS];
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const int i = thread_id() + k * DS_THREADS;
    v[k] = u32x4{0, 0, 0, 0};
    need[k] = i < total && (i - row_of(i, vec_per_row) * vec_per_row) * 8 < K;
  }
  for (;;) {
    bool pending = false;
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      if (need[k]) {
        const int i = thread_id() + k * DS_THREADS;
        const int m = row_of(i, vec_per_row);
        v[k] = get16(X, (size_t)M * K * 2, ((size_t)m * K + (size_t)(i - m * vec_per_row) * 8) * 2);
      }
    }
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      if (need[k]) {
        if (has_empty16(v[k])) pending = true;
        else need[k] = false;
      }
    }
#ifdef DS_TRACE
    if (trace && thread_id() == 0) { trace[2] = trace[2] + 1; if (trace[2] == 1) trace[0] = wall_clock64(); }
#endif
    if (!__any(pending) || w.give_up()) break;
  }
#ifdef DS_TRACE
  if (trace && thread_id() == 0) trace[1] = wall_clock64();
#endif
  float pq[MAXB];
#pragma unroll
  for (int mm = 0; mm < MAXB; ++mm) pq[mm] = 0.f;
  if (norm_w) {
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const int i = thread_id() + k * DS_THREADS;
      if (i < total) {
        const int m = row_of(i, vec_per_row);
        const f16x8 h = bitcast<f16x8>(v[k]);
        float s2 = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float f = (float)h[e]; s2 = __builtin_fmaf(f, f, s2); }
#pragma unroll
        for (int mm = 0; mm < MAXB; ++mm) if (mm == m) pq[mm] += s2;
      }
    }
#pragma unroll
    for (int mm = 0; mm < MAXB; ++mm) pq[mm] = wave_total(pq[mm]);
    if (lane == 0) {
#pragma unroll
      for (int mm = 0; mm < MAXB; ++mm) scratch[wave * DS_MAXB + mm] = pq[mm];
    }
    wg_sync();
  }
  const float inv_n = 1.0f / (float)K;
  float ps[MAXB];      // sums of the values this thread puts into LDS, per activation row
#pragma unroll
  for (int mm = 0; mm < MAXB; ++mm) ps[mm] = 0.f;
#pragma unroll
  for (int k = 0; k < NS; ++k) {
    const int i = thread_id() + k * DS_THREADS;
    if (i < total) {
      const int m = row_of(i, vec_per_row), c = i - m * vec_per_row;
      f16x8 h = bitcast<f16x8>(v[k]);
      if (norm_w && c * 8 < K) {
        float sq = 0.f;
#pragma unroll
        for (int ww = 0; ww < DS_WAVES; ++ww) sq += scratch[ww * DS_MAXB + m];
        const f16 r16 = (f16)(1.0f / sqrtf(sq * inv_n + eps));
        const f16x8 gm = *reinterpret_cast<const f16x8*>(norm_w + c * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = (h[e] * r16) * gm[e];
      }
      *reinterpret_cast<f16x8*>(xs + (size_t)m * xstride + c * 8) = h;
      float s1 = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s1 += (float)h[e];
#pragma unroll
      for (int mm = 0; mm < MAXB; ++mm) if (mm == m) ps[mm] += s1;
    }
  }
  // The INT4 products below multiply by the stored codes q + 8 and take 8 * sum(x) off at the end.
#pragma unroll
  for (int mm = 0; mm < MAXB; ++mm) ps[mm] = wave_total(ps[mm]);
  if (lane == 0) {
#pragma unroll
    for (int mm = 0; mm < MAXB; ++mm) scratch[DS_XSUM + wave * DS_MAXB + mm] = ps[mm];
  }
  wg_sync();
  return *w.lds_dead == 0;
}

// RMSNorm weights go from global memory straight into LDS (no registers), requested at the end of
// the phase before the one that normalises with them; the wait of that phase's `stage` covers them,
// because a wave's loads complete in order.  Wave w moves weights [512 w, 512 w + 512): a whole KiB of
// LDS per wave (lanes beyond d repeat the last vector), so the LDS array is d rounded up to 512.
__device__ __forceinline__ void normw_fetch(const f16* w, f16* lds_w, int d) {
  const int wave = wave_id(), lane = lane_id();
  if (wave * 512 < d) {
    int i = wave * 512 + lane * 8;
    i = i + 8 <= d ? i : d - 8;      // d is a multiple of 128
    __builtin_amdgcn_global_load_lds((const DS_GLOBAL void*)(as_global(w) + i),
                                     (__attribute__((address_space(3))) void*)(lds_w + wave * 512), 16, 0, 0);
  }
}

// ------------------------------------------------------------------------------------------ attention phase
// Element (row m, feature n) of an activation slot of decode_step_wide_kernel, in halves: the slot is
// [features / 8][16 rows][8 features], so that the 64 lanes of a wave (lane = 16 * (eight-feature group
// % 4) + row) read one contiguous KiB per 32-feature step - whole cache lines, which the memory pipeline
// delivers at twice the rate of sixteen 64-byte pieces of sixteen rows.
__device__ __forceinline__ size_t grouped_at(int m, int n) { return (size_t)(n >> 3) * 128 + m * 8 + (n & 7); }

// merges the online-softmax state of the lane O (16 or 32) lanes away into this lane's
template <int O>
__device__ __forceinline__ void merge_lanes(float& m, float& l, float (&acc)[8]) {
  static_assert(O == 16 || O == 32, "row or half of the wave");
  // (the row / half swaps of gfx950 in place of these shuffles were measured: 2 % slower per step at batch 1)
  auto other = [](float v) { return __shfl_xor(v, O, 64); };
  const float mo = other(m), lo = other(l);
  const float mn = fmaxf(m, mo);
  const float ca = m == -INFINITY ? 0.f : __expf(m - mn);
  const float cb = mo == -INFINITY ? 0.f : __expf(mo - mn);
  l = l * ca + lo * cb;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = acc[e] * ca + other(acc[e]) * cb;
  m = mn;
}

// One (sequence, head, split) unit: rotary of q and of the new k (rotate-half, as rope_llama in
// attention.hip, models/llama2/attention.py:83-97; cs holds fp16 cos and sin of this step's
// angles), append of the new K/V row to the ring by the split whose range holds it, online-softmax
// attention over this split's rows.  Split 0 of a head collects the partials of the other splits
// that have rows and writes the head's output.
// FP8 KV rings (KVCacheOp with fp8 = true, custom_ops/kv_cache.cpp:43-74,103-105), as in attention.hip: a row is
// stored as the F143 bytes of value * 2^-kv_scale; the kernels take decode(byte) as the row, multiply the fp32 score
// by 2^kv_scale before it is rounded to fp16 and the weighted sum of the values by 2^kv_scale at the end (powers of
// two: exact).  This step's own row enters LDS as decode(byte) too, so the pass sees what the cache will hold.
__device__ __forceinline__ uint8_t ring_code(f16 v, int kv_scale) { return F8<0>::encode(ldexpf((float)v, -kv_scale)); }
template <bool KV8> struct RingRow;
template <> struct RingRow<false> {
  typedef f16x8 type;
  static __device__ __forceinline__ f16x8 values(f16x8 r) { return r; }
};
template <> struct RingRow<true> {
  typedef u32x2 type;
  static __device__ __forceinline__ f16x8 values(u32x2 r) { return f143_decode8(r[0], r[1]); }
};
template <bool KV8>
__device__ __forceinline__ void ring_rows(const f16* kring, const f16* vring, size_t at, f16x8& k8, f16x8& v8) {
  if constexpr (KV8) {
    const u32x2 kr = *reinterpret_cast<const DS_GLOBAL u32x2*>(as_global(reinterpret_cast<const uint8_t*>(kring)) + at);
    const u32x2 vr = *reinterpret_cast<const DS_GLOBAL u32x2*>(as_global(reinterpret_cast<const uint8_t*>(vring)) + at);
    k8 = f143_decode8(kr[0], kr[1]);
    v8 = f143_decode8(vr[0], vr[1]);
  } else {
    k8 = *reinterpret_cast<const DS_GLOBAL f16x8*>(as_global(kring) + at);
    v8 = *reinterpret_cast<const DS_GLOBAL f16x8*>(as_global(vring) + at);
  }
}
// the rings of (sequence b, head h): element pointers (fp16) or byte pointers carried as f16* (KV8)
template <bool KV8>
__device__ __forceinline__ void ring_of(const DsArgs& a, f16* kring_base, int b, int h, f16*& kring, f16*& vring) {
  const size_t head = ((size_t)b * a.H + h) * a.max_len * DS_D, all = (size_t)a.B * a.H * a.max_len * DS_D;
  if constexpr (KV8) {
    kring = reinterpret_cast<f16*>(reinterpret_cast<uint8_t*>(kring_base) + head);
    vring = reinterpret_cast<f16*>(reinterpret_cast<uint8_t*>(kring) + all);
  } else {
    kring = kring_base + head;
    vring = kring + all;
  }
}
// element d of row pos of a ring: y goes in, what the cache holds of it comes back
template <bool KV8>
__device__ __forceinline__ f16 ring_put(f16* ring, size_t at, f16 y, int kv_scale) {
  if constexpr (KV8) {
    const uint8_t code = ring_code(y, kv_scale);
    as_global(reinterpret_cast<uint8_t*>(ring))[at] = code;
    return (f16)F8<0>::decode(code);
  } else {
    as_global(ring)[at] = y;
    return y;
  }
}
template <bool KV8>
__device__ __forceinline__ f16 ring_value(f16 y, int kv_scale) {
  if constexpr (KV8) return (f16)F8<0>::decode(ring_code(y, kv_scale));
  else return y;
}

template <bool GROUPED = false, bool KV8 = false>
__device__ __forceinline__ void attention_unit(const DsArgs& a, int li, f16* kring_base, int unit, int step, float* lds,
                                               const f16* cs, Waiter& w) {
  constexpr int D = DS_D, LPP = D / 8, PPW = 64 / LPP, HALF = D / 2;
  const int wave = wave_id(), lane = lane_id();
#ifdef DS_TRACE
  struct { int wg; } g{logical_workgroup(blockIdx.x, gridDim.x, a.xcd_groups)};
#endif
  const int bh = unit / a.nsplit, split = unit % a.nsplit;
  const int b = bh / a.H, h = bh % a.H;
  const int valid = step + 1 < a.max_len ? step + 1 : a.max_len;
  const int pos = step % a.max_len;
  const int chunk = ((valid + a.nsplit - 1) / a.nsplit + 63) & ~63;
  const int nact = (valid + chunk - 1) / chunk;       // splits that have rows
  const int c0 = split * chunk;
  if (c0 >= valid) return;
  const int c1 = c0 + chunk < valid ? c0 + chunk : valid;
  f16* q_s = reinterpret_cast<f16*>(lds);            // [D] rotated q
  f16* k_s = q_s + D;                                 // [D] rotated new k
  f16* v_s = k_s + D;                                 // [D] new v
  float* sm_m = lds + 3 * D / 2;                      // [DS_WAVES]
  float* sm_l = sm_m + DS_WAVES;
  float* sm_acc = sm_l + DS_WAVES;                    // [DS_WAVES][D]
  const f16* qrow = a.qkv + ((size_t)li * a.B + b) * 3 * a.d + h * D;
  f16 *kring, *vring;
  ring_of<KV8>(a, kring_base, b, h, kring, vring);
  const float kv_mul = KV8 ? ldexpf(1.0f, a.kv_scale) : 1.0f;
  const bool owner = pos >= c0 && pos < c0 + chunk;
  {
    // waves 0-1: q, waves 2-3: k, waves 4-5: v; a rotated element needs x[d] and x[d +- D/2]
    const int tid = thread_id();
    const int which = tid / D, d_ = tid % D;
    const bool on = tid < 3 * D;
    const f16* row = qrow + (size_t)(which < 3 ? which : 0) * a.d;
    f16 x0, x1;
    wait_pair(row + d_, on, row + (d_ < HALF ? d_ + HALF : d_ - HALF), on && which < 2, x0, x1, w);
    if (on) {
      f16 y = x0;
      if (which < 2) {
        const int i = d_ < HALF ? d_ : d_ - HALF;
        const f16 rot = d_ < HALF ? -x1 : x1;
        y = x0 * cs[i] + rot * cs[HALF + i];
      }
      if (which == 1) y = owner ? ring_put<KV8>(kring, (size_t)pos * D + d_, y, a.kv_scale) : ring_value<KV8>(y, a.kv_scale);
      if (which == 2) y = owner ? ring_put<KV8>(vring, (size_t)pos * D + d_, y, a.kv_scale) : ring_value<KV8>(y, a.kv_scale);
      q_s[which * D + d_] = y;
    }
  }
  TRACE(10);
  wg_sync();
  {
    const int grp = lane / LPP, sub = lane % LPP, d0 = sub * 8;
    float qf[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[e] = (float)q_s[d0 + e];
    const f16 scale = (f16)0.08838834764831845f;   // fp16(1/sqrt(128))
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    // The rows of the next visit are requested before those of the current one are used (two sets of registers in
    // turn).  Every request issues the same loads: a row past the end of the range repeats its last row, and this
    // step's own row, whose ring copy is being written, is loaded like any other and replaced by its LDS copy at
    // the visit - so the wait before a visit leaves the next request on its way.
    typedef typename RingRow<KV8>::type Row;
    auto request = [&](Row& kr, Row& vr, int p0) {
      const int p = p0 + grp;
      const size_t at = ((size_t)(p < c1 ? p : c1 - 1) * D + d0) * (KV8 ? 1 : 2);
      kr = *reinterpret_cast<const DS_GLOBAL Row*>(as_global(reinterpret_cast<const uint8_t*>(kring)) + at);
      vr = *reinterpret_cast<const DS_GLOBAL Row*>(as_global(reinterpret_cast<const uint8_t*>(vring)) + at);
    };
    auto visit = [&](const Row& kr, const Row& vr, int p0) {
      const int p = p0 + grp;
      const bool on = p < c1;
      f16x8 k8 = RingRow<KV8>::values(kr), v8 = RingRow<KV8>::values(vr);
      if ((on ? p : c1 - 1) == pos) {      // this step's row: taken from LDS, its global copy is being written
        k8 = *reinterpret_cast<const f16x8*>(k_s + d0);
        v8 = *reinterpret_cast<const f16x8*>(v_s + d0);
      }
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s = __builtin_fmaf(qf[e], (float)k8[e], s);
#pragma unroll
      for (int o = LPP / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
      if (KV8) s *= kv_mul;
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
    };
    {
      constexpr int VISIT = DS_WAVES * PPW;
      Row ka, va, kb, vb;
      int p0 = c0 + wave * PPW;
      request(ka, va, p0);
      if (c1 - c0 <= VISIT) {              // one visit (batch 1 up to 512 rows of context): nothing to request ahead
        if (p0 < c1) visit(ka, va, p0);
      } else {
        for (; p0 < c1; p0 += 2 * VISIT) {
          request(kb, vb, p0 + VISIT);
          visit(ka, va, p0);
          if (p0 + VISIT >= c1) break;
          request(ka, va, p0 + 2 * VISIT);
          visit(kb, vb, p0 + VISIT);
        }
      }
    }
    // the four row groups of a wave merge in registers, the sixteen waves in LDS
    merge_lanes<16>(m, l, acc);
    merge_lanes<32>(m, l, acc);
    if (lane == 0) { sm_m[wave] = m; sm_l[wave] = l; }
    if (lane < LPP) {
#pragma unroll
      for (int e = 0; e < 8; ++e) sm_acc[wave * D + d0 + e] = acc[e];
    }
  }
  TRACE(11);
  wg_sync();
  float Mx = -INFINITY, Ls = 0.f, As = 0.f;
  float* part = a.part + (((size_t)li * a.B * a.H + bh) * a.nsplit) * DS_PART;
  if (thread_id() < D) {      // waves 0 and 1: this workgroup's own partial
    const int d_ = thread_id();
#pragma unroll
    for (int i = 0; i < DS_WAVES; ++i) Mx = fmaxf(Mx, sm_m[i]);
#pragma unroll
    for (int i = 0; i < DS_WAVES; ++i) {
      const float wgt = sm_m[i] == -INFINITY ? 0.f : __expf(sm_m[i] - Mx);
      Ls = __builtin_fmaf(sm_l[i], wgt, Ls);
      As = __builtin_fmaf(sm_acc[i * D + d_], wgt, As);
    }
    if (split != 0) {
      float* mine = part + (size_t)split * DS_PART;
      put(mine + 2 + d_, As);
      if (d_ == 0) { put(mine, Mx); put(mine + 1, Ls); }
    }
  }
  if (split == 0) {
    // The partials of the other splits that have rows: wave s fetches split s (all at the same time:
    // one round trip for all of them), they meet in LDS and merge in ascending order of split.
    static_assert(DS_MAX_SPLIT <= DS_WAVES && D == 128, "one wave per split, two numerator elements per lane");
    wg_sync();                // the per-wave state in LDS has been read
    if (wave >= 1 && wave < nact) {
      const float* ps = part + (size_t)wave * DS_PART;
      float a0, a1, ml;
      wait_triple(ps + 2 + lane, ps + 2 + 64 + lane, ps + (lane & 1), lane < 2, a0, a1, ml, w);
      sm_acc[wave * D + lane] = a0;
      sm_acc[wave * D + 64 + lane] = a1;
      if (lane == 0) sm_m[wave] = ml;
      if (lane == 1) sm_l[wave] = ml;
    }
    wg_sync();
    TRACE(12);
    if (thread_id() < D) {
      const int d_ = thread_id();
      for (int s = 1; s < nact; ++s) {
        const float ms = sm_m[s], ls = sm_l[s], as = sm_acc[s * D + d_];
        const float mn = fmaxf(Mx, ms);
        const float ca = __expf(Mx - mn), cb = __expf(ms - mn);
        Ls = Ls * ca + ls * cb;
        As = As * ca + as * cb;
        Mx = mn;
      }
      if (KV8) As *= kv_mul;
      if constexpr (GROUPED) put(a.ctx + (size_t)li * 16 * a.d + grouped_at(b, h * D + d_), (f16)(As / Ls));
      else put(a.ctx + ((size_t)li * a.B + b) * a.d + h * D + d_, (f16)(As / Ls));
    }
  }
  wg_sync();
}

// Two (sequence, head) units at a time, eight waves each, for launches without splits (nsplit == 1: at least as many
// units as workgroups): the same arithmetic as attention_unit per unit - the online-softmax state of a row group
// depends on the rows it visits, so the outputs differ from a sixteen-wave pass in the last bits, as they do between
// split counts.  bh1 < 0: the second half of the workgroup has no unit.
template <bool KV8 = false>
__device__ __forceinline__ void attention_two(const DsArgs& a, int li, f16* kring_base, int bh0, int bh1, int step, float* lds,
                                              const f16* cs, Waiter& w) {
  constexpr int D = DS_D, LPP = D / 8, PPW = 64 / LPP, HALF = D / 2, WPU = DS_WAVES / 2;
  const int wave = wave_id(), lane = lane_id();
  const int half = wave / WPU, wv = wave % WPU;
  const int bh = half ? bh1 : bh0;
  const bool active = bh >= 0;
  const int b = active ? bh / a.H : 0, h = active ? bh % a.H : 0;
  const int valid = step + 1 < a.max_len ? step + 1 : a.max_len;
  const int pos = step % a.max_len;
  f16* q_s = reinterpret_cast<f16*>(lds) + half * 3 * D;      // [D] rotated q | [D] rotated new k | [D] new v, per unit
  f16* k_s = q_s + D;
  f16* v_s = k_s + D;
  float* sm_m = lds + 3 * D;                                   // [DS_WAVES]
  float* sm_l = sm_m + DS_WAVES;
  float* sm_acc = sm_l + DS_WAVES;                             // [DS_WAVES][D]
  const f16* qrow = a.qkv + ((size_t)li * a.B + b) * 3 * a.d + h * D;
  f16 *kring, *vring;
  ring_of<KV8>(a, kring_base, b, h, kring, vring);
  const float kv_mul = KV8 ? ldexpf(1.0f, a.kv_scale) : 1.0f;
  // A window of NPRE rounds of cache rows (a round: four rows per wave) travels ahead of the visits: the first NPRE
  // rounds are requested before q, k and v are waited for - the rows are known, and they travel while the producers'
  // values do - and every visit of a round requests the round NPRE later into the registers it frees.  Every
  // request issues the same loads (a row past the end repeats the last one; this step's own row, whose ring copy is
  // being written, is loaded like any other and replaced by its LDS copy at the visit), so the wait before a visit
  // counts the requests issued after that round's and leaves them on their way.
  constexpr int NPRE = 4;
  typedef typename RingRow<KV8>::type Row;       // eight elements of a cache row as they are stored (decoded at the visit)
  Row kp[NPRE], vp[NPRE];
  const int att_grp = lane / LPP, att_d0 = (lane % LPP) * 8;
  auto request = [&](Row& kr, Row& vr, int round) {
    const int p = wv * PPW + att_grp + round * WPU * PPW;
    const size_t at = ((size_t)(p < valid ? p : valid - 1) * D + att_d0) * (KV8 ? 1 : 2);
    kr = *reinterpret_cast<const DS_GLOBAL Row*>(as_global(reinterpret_cast<const uint8_t*>(kring)) + at);
    vr = *reinterpret_cast<const DS_GLOBAL Row*>(as_global(reinterpret_cast<const uint8_t*>(vring)) + at);
  };
#pragma unroll
  for (int it = 0; it < NPRE; ++it) request(kp[it], vp[it], it);
  {
    const int t = thread_id() - half * WPU * 64;
    const int which = t / D, d_ = t % D;
    const bool on = active && t < 3 * D;
    const f16* row = qrow + (size_t)(which < 3 ? which : 0) * a.d;
    f16 x0, x1;
    wait_pair(row + d_, on, row + (d_ < HALF ? d_ + HALF : d_ - HALF), on && which < 2, x0, x1, w);
    if (on) {
      f16 y = x0;
      if (which < 2) {
        const int i = d_ < HALF ? d_ : d_ - HALF;
        const f16 rot = d_ < HALF ? -x1 : x1;
        y = x0 * cs[i] + rot * cs[HALF + i];
      }
      if (which == 1) y = ring_put<KV8>(kring, (size_t)pos * D + d_, y, a.kv_scale);
      if (which == 2) y = ring_put<KV8>(vring, (size_t)pos * D + d_, y, a.kv_scale);
      q_s[which * D + d_] = y;
    }
  }
  wg_sync();
  if (active) {
    const int grp = lane / LPP, sub = lane % LPP, d0 = sub * 8;
    float qf[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[e] = (float)q_s[d0 + e];
    const f16 scale = (f16)0.08838834764831845f;   // fp16(1/sqrt(128))
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    auto visit = [&](f16x8 k8, f16x8 v8, bool on) {
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s = __builtin_fmaf(qf[e], (float)k8[e], s);
#pragma unroll
      for (int o = LPP / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
      if (KV8) s *= kv_mul;
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
    };
    const int rounds = (valid + WPU * PPW - 1) / (WPU * PPW);
    for (int r0 = 0; r0 < rounds; r0 += NPRE) {
#pragma unroll
      for (int it = 0; it < NPRE; ++it) {
        const int p0 = wv * PPW + (r0 + it) * WPU * PPW;
        if (p0 < valid) {
          const int p = p0 + grp;
          const bool on = p < valid;
          f16x8 k8 = RingRow<KV8>::values(kp[it]), v8 = RingRow<KV8>::values(vp[it]);
          if ((on ? p : valid - 1) == pos) {      // this step's row: taken from LDS, its global copy is being written
            k8 = *reinterpret_cast<const f16x8*>(k_s + d0);
            v8 = *reinterpret_cast<const f16x8*>(v_s + d0);
          }
          visit(k8, v8, on);
        }
        request(kp[it], vp[it], r0 + it + NPRE);
      }
    }
    merge_lanes<16>(m, l, acc);
    merge_lanes<32>(m, l, acc);
    if (lane == 0) { sm_m[wave] = m; sm_l[wave] = l; }
    if (lane < LPP) {
#pragma unroll
      for (int e = 0; e < 8; ++e) sm_acc[wave * D + d0 + e] = acc[e];
    }
  }
  wg_sync();
  {
    const int d_ = thread_id() - half * WPU * 64;
    if (active && d_ < D) {      // the first two waves of each half
      float Mx = -INFINITY, Ls = 0.f, As = 0.f;
#pragma unroll
      for (int i = 0; i < WPU; ++i) Mx = fmaxf(Mx, sm_m[half * WPU + i]);
#pragma unroll
      for (int i = 0; i < WPU; ++i) {
        const float wgt = sm_m[half * WPU + i] == -INFINITY ? 0.f : __expf(sm_m[half * WPU + i] - Mx);
        Ls = __builtin_fmaf(sm_l[half * WPU + i], wgt, Ls);
        As = __builtin_fmaf(sm_acc[(half * WPU + i) * D + d_], wgt, As);
      }
      if (KV8) As *= kv_mul;
      put(a.ctx + (size_t)li * 16 * a.d + grouped_at(b, h * D + d_), (f16)(As / Ls));      // the layout of decode_step_wide_kernel
    }
  }
  wg_sync();
}

// ------------------------------------------------------------------------------------------ selection and bookkeeping
// The container / mask / stop-mask update of models/base_model.py:313-355 exactly as step_update_kernel in
// select.hip, from the rows' picks in ids (LDS); the first wave, one lane per row.
__device__ __forceinline__ void advance_rows(const DsArgs& a, const int* ids) {
  if (wave_id() == 0) {      // lane b takes row b: the rows' loads travel together
    const int b = lane_id();
    const bool on = b < a.B;
    const int ns = *a.step + 1;
    const bool stopped = on && a.stop_mask[on ? b : 0] != 0;
    const int stopped_before = __popcll(__ballot(stopped));
    if (on) {
      int id = ids[b];
      a.next_ids[b] = id;
      if (ns < a.max_len) {
        a.mask[(size_t)b * a.max_len + ns] = (f16)0.0f;
        const int slot = a.container[(size_t)b * a.max_len + ns];
        id = slot == a.pad_id ? id : slot;
        a.container[(size_t)b * a.max_len + ns] = id;
      }
      if (id == a.eos_id) a.stop_mask[b] |= 1;
    }
    if (b == 0) {
      *a.keep_going = a.early_stop ? (stopped_before < a.B ? 1 : 0) : 1;
      *a.step = ns;
    }
  }
}

// Top-1 per sequence (lowest index among equals) over the logits, then advance_rows; workgroup 0 only.
// Returns false when the wait for the logits was given up (nothing is updated then).
__device__ __forceinline__ bool select_and_advance(const DsArgs& a, float* lds, Waiter& w) {
  float* sv = lds;
  int* si = reinterpret_cast<int*>(lds + DS_WAVES);
  int* ids = si + DS_WAVES;
  const int lane = lane_id(), wave = wave_id();
  // All rows at once: 16, 8, 4, 2 or 1 waves per row for up to 1, 2, 4, 8, 16 rows.  A wave takes the 512-element
  // pieces part, part + wpr, ... of its row, eight pieces per round trip.
  constexpr int U = 8;
  const int wpr = a.B <= 1 ? 16 : a.B <= 2 ? 8 : a.B <= 4 ? 4 : a.B <= 8 ? 2 : 1;
  const int row = wave / wpr, part = wave % wpr;
  const bool active = row < a.B;
  const f16* xr = a.logits + (size_t)(active ? row : 0) * a.vocab;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = part * 512; c < a.vocab; c += wpr * 512 * U) {
    u32x4 v[U];
    bool need[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v[u] = u32x4{0, 0, 0, 0};
      need[u] = active && c + u * wpr * 512 + lane * 8 < a.vocab;      // vocab is a multiple of 8
    }
    for (;;) {
      bool pending = false;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (need[u]) v[u] = get16(xr, (size_t)a.vocab * 2, (size_t)(c + u * wpr * 512 + lane * 8) * 2);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (need[u]) {
          if (has_empty16(v[u])) pending = true;
          else need[u] = false;
        }
      if (!__any(pending) || w.give_up()) break;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i0 = c + u * wpr * 512 + lane * 8;
      if (active && i0 < a.vocab) {
        const f16x8 h = bitcast<f16x8>(v[u]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float f = (float)h[e];
          if (f > best) { best = f; bi = i0 + e; }
        }
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
  if (thread_id() < a.B) {
    const int b = thread_id();
    best = sv[b * wpr];
    bi = si[b * wpr];
    for (int ww = 1; ww < wpr; ++ww)
      if (sv[b * wpr + ww] > best || (sv[b * wpr + ww] == best && si[b * wpr + ww] < bi)) { best = sv[b * wpr + ww]; bi = si[b * wpr + ww]; }
    ids[b] = bi == 0x7fffffff ? 0 : bi;
  }
  wg_sync();
  if (*w.lds_dead != 0) return false;
  advance_rows(a, ids);
  return true;
}

// ------------------------------------------------------------------------------------------ the kernel
// TPW_D / TPW_F: K tiles per wave for K = hidden / ffn; U_F: gate/up row-blocks per workgroup;
// MAXB: largest batch the instance serves.  Hidden row-blocks (q/k/v, o_proj, down) are at most
// one per workgroup.
template <int TPW_D, int TPW_F, int U_F, int MAXB, bool KV8 = false>
__global__ __launch_bounds__(DS_THREADS) void decode_step_kernel(DsArgs a) {
  constexpr int NS_D = (MAXB * TPW_D * DS_WAVES * 16 + DS_THREADS - 1) / DS_THREADS;
  constexpr int NS_F = (MAXB * TPW_F * DS_WAVES * 16 + DS_THREADS - 1) / DS_THREADS;
  extern __shared__ __align__(16) unsigned char smem[];
  // once the loop condition has gone false a further iteration leaves everything as it is; so does
  // every launch after one that failed (the error word is sticky)
  if (*a.keep_going == 0) return;
  if (__hip_atomic_load((DS_GLOBAL unsigned*)(a.sync + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
  const int KT_D = (a.d + 127) / 128, KT_F = (a.ffn + 127) / 128;
  const int xstride = (KT_D > KT_F ? KT_D : KT_F) * 128 + 8;
  f16* xs = reinterpret_cast<f16*>(smem);
  float* att_lds = reinterpret_cast<float*>(smem);           // the attention phase reuses the activation area
  float* red = reinterpret_cast<float*>(smem + a.region0);
  float* scratch = red + 2 * DS_RED;                          // norm sums, then selection scratch, then flags
  int* lds_dead = reinterpret_cast<int*>(scratch + DS_WAVES * DS_MAXB + 64);
  f16* normw = reinterpret_cast<f16*>(scratch + DS_TAIL_FLOATS);   // [d rounded up to 512]: normw_fetch writes whole KiB
  f16* cs = normw + ((a.d + 511) & ~511);                          // [D]: cos, sin of this step's angles
  uint32_t* lds_layers = reinterpret_cast<uint32_t*>(cs + DS_D);   // [n_layer] descriptors

  const int M = a.B;
  const int step = *a.step;
  const int nb_d = (a.d + 15) / 16, nb_f = (a.ffn + 15) / 16, nb_v = (a.vocab + 15) / 16;
  const int G = gridDim.x, wg = logical_workgroup(blockIdx.x, G, a.xcd_groups);
  struct { int wg; } g{wg};       // for TRACE
  (void)g;
  const unsigned epoch = __hip_atomic_load((DS_GLOBAL unsigned*)a.sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
  Waiter w{a.sync + 1, lds_dead, 0, wall_clock64() + DS_LAUNCH_TICKS};
  int red_buf = 0;
  const size_t xslot = (size_t)M * a.d;      // halves of one residual-stream slot

  // ---- set-up: fill the slots, descriptors and this step's rotary factors into LDS, embedding rows
  {
    const int tid = thread_id();
    if (tid == 0) *lds_dead = 0;
    const u32x4 filler = {DS_EMPTY32, DS_EMPTY32, DS_EMPTY32, DS_EMPTY32};
    char* fill = reinterpret_cast<char*>(a.xres + xslot);
    for (size_t off = ((size_t)wg * DS_THREADS + tid) * 16; off < a.fill_bytes; off += (size_t)G * DS_THREADS * 16) {
      const size_t win = off & ~(((size_t)1 << 30) - 1);     // a buffer descriptor spans less than 4 GiB
      put16(fill + win, a.fill_bytes - win < ((size_t)1 << 31) ? a.fill_bytes - win : ((size_t)1 << 31), off - win, filler);
    }
    for (size_t i = ((size_t)wg * DS_THREADS + tid) * 8; i < (size_t)M * a.vocab; i += (size_t)G * DS_THREADS * 8)
      put16(a.logits, (size_t)M * a.vocab * 2, i * 2, filler);
    for (int i = tid; i < a.n_layer * DS_LAYER_WORDS; i += DS_THREADS) lds_layers[i] = a.layers[i];
    if (tid < DS_D / 2) {
      const f16 ang = (f16)((float)(f16)(float)step * (float)a.inv_freq[tid]);
      cs[tid] = (f16)cosf((float)ang);
      cs[DS_D / 2 + tid] = (f16)sinf((float)ang);
    }
    // xres[0][b] = embed[container[b, step]] (layers/embedding.py:34-36)
    const int col = step < a.max_len ? step : a.max_len - 1;
    for (int i = wg * DS_THREADS + tid; i < M * a.d; i += G * DS_THREADS) {
      const int b = i / a.d, c = i % a.d;
      int id = a.container[(size_t)b * a.max_len + col];
      id = id < 0 ? 0 : (id >= a.vocab ? a.vocab - 1 : id);
      put(a.xres + i, a.embed[(size_t)id * a.d + c]);
    }
  }
  wg_sync();

  // Places of the units in the tile array (T = TPW_D tiles per wave and matrix): q | k | v at
  // [0, 3T), o_proj at [3T, 4T), the first and second gate/up units at [4T, 6T) and [6T, 8T); the
  // third gate/up unit takes [0, 2T) once q/k/v have been multiplied, down takes [3T, 3T + TPW_F)
  // (o_proj's place and the start of the first gate/up unit's) as those are multiplied, and the
  // next layer's v, q, k return to their places as these become free.  No request point asks for
  // more than 2T tiles per wave (64 KiB per workgroup at the 7B shape): that is what a compute unit
  // accepts without holding the requesting waves.
  constexpr int T = TPW_D;
  constexpr int NSLOT = 8 * T;
  constexpr int S_QKV = 0, S_O = 3 * T, S_GU0 = 4 * T, S_GU1 = 6 * T, S_GU2 = 0, S_D = 3 * T;
  constexpr int NSC = 9;
  constexpr int C_QKV = 0, C_O = 3, C_GU0 = 4, C_GU1 = 6, C_GU2 = 0, C_D = 8;
  constexpr int D_EARLY = TPW_F < T ? TPW_F : T;        // down tiles that fit o_proj's place
  static_assert(U_F <= 3, "at most three gate/up units per workgroup");
  static_assert(TPW_F <= 3 * T, "the down tiles end where the first gate/up unit ends");
  u32x4 S[NSLOT];
  f16x2 SC[NSC];
  {
    const LayerPtrs L0 = layer_ptrs(lds_layers, 0);
    normw_fetch(L0.get<const f16>(P_N1), normw, a.d);
    const Mat m3[3] = {layer_mat(L0, P_WQ, P_SQ), layer_mat(L0, P_WK, P_SK), layer_mat(L0, P_WV, P_SV)};
    load_slots<3, T, S_QKV, C_QKV>(S, SC, m3, wg, nb_d, a.d, KT_D);
  }
  grid_barrier(a.sync, epoch, G, wg, w);
  bool alive = *lds_dead == 0;

  // the residual element of this thread's output channel (epilogue mapping of gemv_unit, N = d)
  f16 res = (f16)0.0f;
  if (alive) {
    int m_, ch;
    const bool mine = residual_thread(m_, ch);
    const int n = wg * 16 + ch;
    const bool on = mine && m_ < M && n < a.d;
    res = wait_value(a.xres + (on ? (size_t)m_ * a.d + n : 0), on, w);
  }

  for (int li = 0; li < a.n_layer && alive; ++li) {
    const LayerPtrs L = layer_ptrs(lds_layers, li);
    const bool more = li + 1 < a.n_layer;
    const LayerPtrs Ln = layer_ptrs(lds_layers, more ? li + 1 : li);   // the last layer's own tiles again: never used
    const Mat mgu[2] = {layer_mat(L, P_WG, P_SG), layer_mat(L, P_WU, P_SU)};
    const Mat md[1] = {layer_mat(L, P_WD, P_SD)};
    const Mat m3n[3] = {layer_mat(Ln, P_WQ, P_SQ), layer_mat(Ln, P_WK, P_SK), layer_mat(Ln, P_WV, P_SV)};
    f16* const x_in = a.xres + (size_t)(2 * li) * xslot;        // residual stream entering the layer
    f16* const x_mid = x_in + xslot;                             // after attention
    f16* const x_out = x_mid + xslot;                            // after the MLP
    // ---- RMSNorm + q/k/v; a row of the [B, 3d] slot holds q | k | v.
    //      Requests o_proj and the gate half of the first gate/up unit before the product, the up half after it.
    TRACE(0);
    alive = stage<NS_D, MAXB>(x_in, M, a.d, KT_D, xs, xstride, normw, a.eps, scratch, w);
    if (!alive) break;
    TRACE(21);
    {
      const Mat mo[1] = {layer_mat(L, P_WO, P_SO)};
      load_slots<1, T, S_O, C_O>(S, SC, mo, wg, nb_d, a.d, KT_D);
      load_slots<2, T, S_GU0, C_GU0, 0, T>(S, SC, mgu, wg, nb_f, a.ffn, KT_D);
    }
    TRACE(1);
    WTRACE(0);
    {
      f16* q = a.qkv + (size_t)li * M * 3 * a.d;
      f16* const o3[3] = {q, q + a.d, q + 2 * a.d};
      gemv_slots<3, T, EPI_STORE, MAXB, S_QKV, C_QKV>(S, SC, o3, 3 * a.d, (f16)0.0f, wg, nb_d, a.d, KT_D, M, xs, xstride,
                                                      red, red_buf, scratch + DS_XSUM, TRACE_AT(13), TRACE_AT(32));
    }
    TRACE(14);
    load_slots<2, T, S_GU0, C_GU0, T, T>(S, SC, mgu, wg, nb_f, a.ffn, KT_D);
    TRACE(2);
    // ---- rotary + KV append + attention.  Requests the second gate/up unit when it is done.
    {
      f16* kring = L.get<f16>(P_KV);
      const int units = M * a.H * a.nsplit;
      // With as many units as workgroups, the M * nsplit units of head h go to the workgroups that produce the
      // head's q | k | v (unit index: (sequence * H + head) * nsplit + split).
      const int per = M * a.nsplit;
      const bool by_head = per * a.H == G;
      for (int u0 = wg; u0 < units; u0 += G) {
        const int r = wg % per;
        const int u = by_head ? ((r / a.nsplit) * a.H + wg / per) * a.nsplit + r % a.nsplit : u0;
        attention_unit<false, KV8>(a, li, kring, u, step, att_lds, cs, w);
      }
      if constexpr (U_F > 1) load_slots<2, T, S_GU1, C_GU1>(S, SC, mgu, wg + G, nb_f, a.ffn, KT_D);
    }
    TRACE(3);
    // ---- o_proj + residual.  Requests the third gate/up unit before the product; after it the first
    //      down tiles (o_proj's place), the next layer's v and the RMSNorm weights of the MLP.
    alive = stage<NS_D, MAXB>(a.ctx + (size_t)li * xslot, M, a.d, KT_D, xs, xstride, nullptr, 0.f, scratch, w);
    if (!alive) break;
    TRACE(20);
    if constexpr (U_F > 2) load_slots<2, T, S_GU2, C_GU2>(S, SC, mgu, wg + 2 * G, nb_f, a.ffn, KT_D);
    TRACE(4);
    {
      f16* const o1[1] = {x_mid};
      res = gemv_slots<1, T, EPI_RESIDUAL, MAXB, S_O, C_O>(S, SC, o1, a.d, res, wg, nb_d, a.d, KT_D, M, xs, xstride, red,
                                                           red_buf, scratch + DS_XSUM, TRACE_AT(15));
    }
    TRACE(16);
    load_slots<1, TPW_F, S_D, C_D, 0, D_EARLY>(S, SC, md, wg, nb_d, a.d, KT_F);
    load_slots<3, T, S_QKV, C_QKV, 2 * T, T>(S, SC, m3n, wg, nb_d, a.d, KT_D);
    normw_fetch(L.get<const f16>(P_N2), normw, a.d);
    TRACE(5);
    // ---- RMSNorm + gate/up + SwiGLU.  Requests the remaining down tiles once the first unit has been
    //      multiplied (they take its place), and the next layer's q after the last unit.
#ifdef DS_TRACE
    if (li == 1 && thread_id() == 0) a.trace[g.wg * DS_TRACE_WORDS + 25] = 0;
#endif
    alive = stage<NS_D, MAXB>(x_mid, M, a.d, KT_D, xs, xstride, normw, a.eps, scratch, w, TRACE_AT(23));
    if (!alive) break;
    TRACE(6);
    {
      f16* act = a.act + (size_t)li * M * a.ffn;
      f32x4 gsum[2];
      slots_product<2, T, S_GU0>(S, gsum, wg, nb_f, KT_D, M, xs, xstride);
      stash_gate_up<U_F>(gsum, 0, M, red, red_buf);
      load_slots<1, TPW_F, S_D, C_D, D_EARLY, TPW_F - D_EARLY>(S, SC, md, wg, nb_d, a.d, KT_F);
      if constexpr (U_F > 1) {
        slots_product<2, T, S_GU1>(S, gsum, wg + G, nb_f, KT_D, M, xs, xstride);
        stash_gate_up<U_F>(gsum, 1, M, red, red_buf);
      }
      if constexpr (U_F > 2) {
        slots_product<2, T, S_GU2>(S, gsum, wg + 2 * G, nb_f, KT_D, M, xs, xstride);
        stash_gate_up<U_F>(gsum, 2, M, red, red_buf);
      }
      float sg[U_F], su[U_F];
      sg[0] = (float)SC[C_GU0][0]; su[0] = (float)SC[C_GU0 + 1][0];
      if constexpr (U_F > 1) { sg[1] = (float)SC[C_GU1][0]; su[1] = (float)SC[C_GU1 + 1][0]; }
      if constexpr (U_F > 2) { sg[2] = (float)SC[C_GU2][0]; su[2] = (float)SC[C_GU2 + 1][0]; }
      TRACE(17);
      finish_gate_up<U_F, MAXB>(sg, su, act, a.ffn, wg, G, nb_f, M, red, red_buf, scratch + DS_XSUM);
    }
    TRACE(18);
    load_slots<3, T, S_QKV, C_QKV, 0, T>(S, SC, m3n, wg, nb_d, a.d, KT_D);
    TRACE(7);
    // ---- down + residual.  Requests the next layer's k and the next RMSNorm weights.
#ifdef DS_TRACE
    if (li == 1 && thread_id() == 0) a.trace[g.wg * DS_TRACE_WORDS + 28] = 0;
#endif
    alive = stage<NS_F, MAXB>(a.act + (size_t)li * M * a.ffn, M, a.ffn, KT_F, xs, xstride, nullptr, 0.f, scratch, w, TRACE_AT(26));
    if (!alive) break;
    TRACE(22);
    load_slots<3, T, S_QKV, C_QKV, T, T>(S, SC, m3n, wg, nb_d, a.d, KT_D);
    TRACE(8);
    {
      f16* const o1[1] = {x_out};
      res = gemv_slots<1, TPW_F, EPI_RESIDUAL, MAXB, S_D, C_D>(S, SC, o1, a.d, res, wg, nb_d, a.d, KT_F, M, xs, xstride,
                                                               red, red_buf, scratch + DS_XSUM, TRACE_AT(19));
    }
    normw_fetch(more ? Ln.get<const f16>(P_N1) : a.final_norm, normw, a.d);
    TRACE(9);
  }
  // ---- final RMSNorm + lm_head, streamed unit by unit with the next unit's tiles in flight
  if (alive) alive = stage<NS_D, MAXB>(a.xres + (size_t)(2 * a.n_layer) * xslot, M, a.d, KT_D, xs, xstride, normw, a.eps,
                                       scratch, w);
  if (alive) {
    const Mat m1[1] = {{a.head, nullptr}};
    f16* const o1[1] = {a.logits};
    // two units in turn, each requested while the other is multiplied, each in registers of its own
    Unit<FmtF16, 1, TPW_D> even, odd;
    load_unit(even, m1, wg, nb_v, a.vocab, KT_D);
    for (int u = wg; u < nb_v; u += 2 * G) {
      load_unit(odd, m1, u + G, nb_v, a.vocab, KT_D);
      gemv_unit<FmtF16, 1, TPW_D, EPI_STORE, MAXB>(even, o1, a.vocab, (f16)0.0f, u, nb_v, a.vocab, KT_D, M, xs, xstride,
                                                   red, red_buf);
      load_unit(even, m1, u + 2 * G, nb_v, a.vocab, KT_D);
      gemv_unit<FmtF16, 1, TPW_D, EPI_STORE, MAXB>(odd, o1, a.vocab, (f16)0.0f, u + G, nb_v, a.vocab, KT_D, M, xs, xstride,
                                                   red, red_buf);
    }
  }
  // ---- selection and bookkeeping
  if (wg == 0) {
    if (alive) select_and_advance(a, scratch + DS_WAVES * DS_MAXB, w);
    if (thread_id() == 0)   // epoch base of the next launch
      __hip_atomic_store((DS_GLOBAL unsigned*)a.sync, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ------------------------------------------------------------------------------------------ 5..16 sequences
// The same iteration for up to 16 sequences.  Sixteen activation rows no longer fit in LDS next to the reduction
// buffers (16 x 4096 halves are 128 KiB, 16 x 11008 are 344), so nothing is staged: a wave multiplies K tiles
// wave, wave + 16, ... and therefore needs, of every activation row, exactly the features of ITS tiles - it loads
// them itself, as the B operands of its products (lane l: row l % 16, features (l / 16) * 8 + 0..7 of each 32-feature
// step), straight from the producer's slot, polling until no element is the filler.  Every element of a slot is read
// by exactly one wave of the workgroup.  RMS statistics and the sums of the rows (for the offset of the stored INT4
// codes) are partial per wave and meet in LDS.
constexpr int DW_MAXB = 16;
constexpr int DW_RED = DS_WAVES * 3 * 256;                  // floats of one reduction buffer: up to three matrices
constexpr int DW_SCL = 6 * 16;                                // channel scales of one phase: up to three gate / up pairs
constexpr int DW_TAIL_FLOATS = 2 * DS_WAVES * DW_MAXB + 64 + 4 + 2 * DW_SCL;   // norm sums | row sums | selection scratch | flags | scales

struct XTile {
  f16x8 v[4];      // the four 32-feature steps of one K tile
};

// Arrival words.  Workgroup g sets word g of a phase's row once everything it stored for the phase has reached
// memory: its stores are agent-scope, written through, and a wave's memory counter reaching zero says that wave's have
// arrived; the storing waves wait for that, the workgroup meets, the first wave writes the word.  A row exists in
// DW_REPLICAS copies, 1 KiB or more apart, and a consumer polls copy (its index % DW_REPLICAS): 256 compute units
// polling one KiB would all queue at one memory channel.  The launch cleared the rows before its grid barrier.  Only
// the first wave of a consumer polls, at agent scope; the workgroup meets, and only then are the phase's values read -
// with ordinary loads.
constexpr int DW_REPLICAS = DS_REPLICAS;
__device__ __forceinline__ void announce(unsigned* rows, int row_words, int wg, bool stored) {
  if (stored) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  wg_sync();
  if (wave_id() == 0 && lane_id() < DW_REPLICAS)
    __hip_atomic_store((DS_GLOBAL unsigned*)(rows + (size_t)lane_id() * row_words + wg), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// false when the wait was given up (by this or an earlier wait of the workgroup)
__device__ __forceinline__ bool await_row(const unsigned* rows, int row_words, int G, int wg, Waiter& w) {
  if (wave_id() == 0) {
    const unsigned* row = rows + (size_t)(wg % DW_REPLICAS) * row_words;
    const int lane = lane_id();
    for (;;) {
      bool ok = true;
      for (int o = lane * 4; o < G; o += 256) {
        const u32x4 v = get16(row, (size_t)G * 4, (size_t)o * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) ok = ok && (o + i >= G || v[i] == 1u);
      }
      if (__all(ok) || w.give_up()) break;
    }
  }
  wg_sync();
  asm volatile("" ::: "memory");      // the values are requested after the row has been seen complete
  return *w.lds_dead == 0;
}

// This wave's fragments of K tile kt of X (fp16 [M, K], a slot whose arrival row has been seen complete), through the
// caches: the 256 workgroups read the same values, and all but the first read of a line in each L2 stay out of the
// fabric.  Nothing of a slot is in a cache before its arrival: the launch starts with an agent-scope acquire (no
// line of the previous launch survives), no slot of this protocol is written with the filler, and every address is
// written once per launch.  The slot is laid out for this read (grouped_at): a wave's 64 loads of a step are one
// contiguous KiB.  Features beyond K (also: a tile beyond the last) and rows beyond M read as zero.
// The four loads are issued whatever the lane, the row count or the tile: through a buffer descriptor, with an
// offset beyond its range where the fragment does not exist (that reads zero and touches no memory).  With the
// loads under a condition the compiler cannot count them, and a wait for an OLDER load - the fragments of the
// current tile while those of the next are on their way - becomes a wait for all of them.
__device__ __forceinline__ void load_xtile(const f16* X, int M, int K, int kt, XTile& t) {
  const int lane = lane_id();
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<f16*>(X), 0, ((K + 127) / 128) * (16 * 128 * 2), 0x00020000);
  int no_row = (lane & 15) < M ? 0 : -1;      // rows beyond M are never written
  asm volatile("" : "+v"(no_row));            // (kept a value: as a condition the compiler turns it into two copies of the loads under branches)
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int no_k = kt * 128 + j * 32 + (lane >> 4) * 8 < K ? 0 : -1;
    t.v[j] = bitcast<f16x8>(__builtin_amdgcn_raw_buffer_load_b128(xr, ((kt * 4 + j) * 64 + lane) * 16 | no_row | no_k, 0, 0));
  }
}

// The same fragments requested into a wave's 4 KiB of LDS instead of registers (no register is held while they are
// on their way), and read back from there: vector j of lane l lies at j KiB + 16 l.
__device__ __forceinline__ void load_xtile_lds(const f16* X, int M, int K, int kt, float* slot) {
  const int lane = lane_id();
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<f16*>(X), 0, ((K + 127) / 128) * (16 * 128 * 2), 0x00020000);
  int no_row = (lane & 15) < M ? 0 : -1;
  asm volatile("" : "+v"(no_row));
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int no_k = kt * 128 + j * 32 + (lane >> 4) * 8 < K ? 0 : -1;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (__attribute__((address_space(3))) void*)(slot + j * 256), 16,
                                             ((kt * 4 + j) * 64 + lane) * 16 | no_row | no_k, 0, 0, 0);
  }
}
__device__ __forceinline__ void read_xtile_lds(const float* slot, XTile& t) {
  const int lane = lane_id();
#pragma unroll
  for (int j = 0; j < 4; ++j) t.v[j] = *reinterpret_cast<const f16x8*>(slot + j * 256 + lane * 4);
}
// waits until at most n of this wave's vector memory loads are in flight (n: 0, 4 or 8 - a constant wherever the
// caller's loop is unrolled)
__device__ __forceinline__ void wait_loads_but(int n) {
  if (n >= 8) __builtin_amdgcn_s_waitcnt(0x0f70 | 8);
  else if (n >= 4) __builtin_amdgcn_s_waitcnt(0x0f70 | 4);
  else __builtin_amdgcn_s_waitcnt(0x0f70);
}

// sums over the lane groups that share a row: afterwards lanes 0..15 (and their images) hold the row's total of the wave
__device__ __forceinline__ float rows_of_wave(float v) {
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// sum over the eight elements of v of v[e] * u[e], added to s in fp32: four two-element dot products
__device__ __forceinline__ float dot8(f16x8 v, f16x8 u, float s) {
  s = __builtin_amdgcn_fdot2(__builtin_shufflevector(v, v, 0, 1), __builtin_shufflevector(u, u, 0, 1), s, false);
  s = __builtin_amdgcn_fdot2(__builtin_shufflevector(v, v, 2, 3), __builtin_shufflevector(u, u, 2, 3), s, false);
  s = __builtin_amdgcn_fdot2(__builtin_shufflevector(v, v, 4, 5), __builtin_shufflevector(u, u, 4, 5), s, false);
  s = __builtin_amdgcn_fdot2(__builtin_shufflevector(v, v, 6, 7), __builtin_shufflevector(u, u, 6, 7), s, false);
  return s;
}

// RMSNorm of the rows whose fragments the waves hold (layers/rms_layer_norm.py:26-36, as pta_rmsnorm): the sums of
// squares meet in LDS, every lane then scales its own fragments by the weights normw_fetch brought to LDS.  NT tiles
// per wave; tiles beyond KT hold zeros.
template <int NT>
__device__ __forceinline__ void norm_xtiles(XTile (&t)[NT], const f16* lds_w, int K, int KT, float eps, float* sums) {
  const int lane = lane_id(), wave = wave_id();
  // sixteen rows of K features are 6 lane operations per element when done one element at a time - microseconds
  // per phase on the four SIMDs; two-element dot products and packed fp16 multiplies take a third of that
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) sq = dot8(t[i].v[j], t[i].v[j], sq);
  sq = rows_of_wave(sq);
  if (lane < 16) sums[wave * DW_MAXB + lane] = sq;
  wg_sync();
  float tot = 0.f;
#pragma unroll
  for (int ww = 0; ww < DS_WAVES; ++ww) tot += sums[ww * DW_MAXB + (lane & 15)];
  const f16 r16 = (f16)(1.0f / sqrtf(tot * (1.0f / (float)K) + eps));
  const f16x8 r8 = {r16, r16, r16, r16, r16, r16, r16, r16};
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int kt = wave + i * DS_WAVES;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = kt * 128 + j * 32 + (lane >> 4) * 8;
      if (kt < KT && k < K) {
        const f16x8 gm = *reinterpret_cast<const f16x8*>(lds_w + k);
        t[i].v[j] = (t[i].v[j] * r8) * gm;      // fp16(fp16(x * r) * g), element by element
      }
    }
  }
}

// The rows' sums over this wave's fragments (the INT4 products multiply by the stored codes q + 8 and take
// 8 * sum(x) off at the end), in fp32.
template <int NT>
__device__ __forceinline__ float xtiles_rowsum(const XTile (&t)[NT]) {
  const f16 one = (f16)1.0f;
  const f16x8 ones = {one, one, one, one, one, one, one, one};
  float s1 = 0.f;
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s1 = dot8(t[i].v[j], ones, s1);
  return rows_of_wave(s1);
}

// acc[r][0 / 1] += the products of tile `i` of unit u's NRB matrices (places base + r * TPW + i; constants once the
// callers' loops are unrolled) with the fragments x
template <int NRB, int TPW, int NSLOT>
__device__ __forceinline__ void wide_tile_product(const u32x4 (&S)[NSLOT], f32x4 (&acc)[NRB][2], int base, int i, const XTile& x) {
#pragma unroll
  for (int m = 0; m < 4; ++m) {
#pragma unroll
    for (int r = 0; r < NRB; ++r) {
      const u32x4 wv = S[base + r * TPW + i];
      u32x4 c;
#pragma unroll
      for (int d = 0; d < 4; ++d) c[d] = (m >= 2 ? wv[d] >> 8 : wv[d]) & ((m & 1) ? 0x00f000f0u : 0x000f000fu);
      acc[r][m & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<f16x8>(c), x.v[m], acc[r][m & 1], 0, 0, 0);
    }
  }
}

// Requests tiles [FIRST, FIRST + COUNT) of unit u's NRB matrices into places BASE + t (tile t = r * TPW + i is tile i of
// this wave of matrix r), as load_slots does, without the scales.
template <int NRB, int TPW, int BASE, int FIRST = 0, int COUNT = NRB * TPW, int NSLOT>
__device__ __forceinline__ void load_tiles(u32x4 (&S)[NSLOT], const Mat (&m)[NRB], int u, int n_units, int KT) {
  static_assert(BASE + NRB * TPW <= NSLOT, "unit outside the register array");
  static_assert(FIRST >= 0 && COUNT >= 0 && FIRST + COUNT <= NRB * TPW, "tiles outside the unit");
  const int wave = wave_id(), lane = lane_id();
  u = u < n_units ? u : n_units - 1;
#pragma unroll
  for (int t = FIRST; t < FIRST + COUNT; ++t) {
    const int r = t / TPW, i = t % TPW;
    int kt = wave + i * DS_WAVES;
    kt = kt < KT ? kt : KT - 1;
    S[BASE + t] = __builtin_nontemporal_load(as_global(m[r].tiled) + ((size_t)u * KT + kt) * 64 + lane);
  }
}

// The scales of unit u's channels (channel lane % 16) of NRB matrices: requested by the first wave before it requests
// its activation fragments and written to LDS once those have arrived (a wave's loads complete in order), so that no
// wave waits for a load of its own in the epilogue, behind the tiles requested ahead.
template <int NRB>
__device__ __forceinline__ void request_scales(const Mat (&m)[NRB], int u, int n_units, int N, f16 (&v)[NRB]) {
  u = u < n_units ? u : n_units - 1;
  int row = u * 16 + (lane_id() & 15);
  row = row < N ? row : N - 1;
#pragma unroll
  for (int r = 0; r < NRB; ++r) v[r] = as_global(m[r].scale)[row];
}
template <int NRB>
__device__ __forceinline__ void keep_scales(const f16 (&v)[NRB], float* scl) {
  const int lane = lane_id();
  if (lane < 16) {
#pragma unroll
    for (int r = 0; r < NRB; ++r) scl[r * 16 + lane] = (float)v[r];
  }
}

// This wave's partial sums of matrix r of a unit (accumulator layout: lane l holds channels (l / 16) * 4 + 0..3 of
// row l % 16) go to the reduction buffer: [wave][r][lane] vectors of four channels.
template <int NRB>
__device__ __forceinline__ void wide_stash(const f32x4& sum, int r, float* rb) {
  const int wave = wave_id(), lane = lane_id();
  *reinterpret_cast<f32x4*>(rb + ((wave * NRB + r) * 64 + lane) * 4) = sum;
}

// The partial sums of all waves meet: thread (r * 16 + m) * 16 + ch finishes channel ch of row m of matrix r
// (EPI_SWIGLU: of the gate / up pair).  xsum: the waves' sums of the rows (8 * sum(x) comes off, the stored codes are
// q + 8); scl[r * 16 + ch]: the channels' scales.  EPI_STORE writes row-major outputs (q/k/v, read by the attention
// phase), the others activation slots in the layout of grouped_at.  Returns the value stored (the thread's residual element in the next
// residual phase).
template <int NRB, int EPI>
__device__ __forceinline__ f16 wide_finish(f16* const (&out)[NRB], int ostride, f16 res, int u, int N, int M, const float* rb,
                                           const float* xsum, const float* scl) {
  wg_sync();
  f16 y = res;
  const int tid = thread_id();
  constexpr int MATS = EPI == EPI_SWIGLU ? 1 : NRB;
  if (tid < MATS * 256) {
    const int r = tid >> 8, m_ = (tid >> 4) & 15, ch = tid & 15;
    const int n = u * 16 + ch;
    if (m_ < M && n < N) {
      float off = 0.f;
#pragma unroll 8
      for (int w = 0; w < DS_WAVES; ++w) off += xsum[w * DW_MAXB + m_];
      off *= 8.0f;
      const int at = ((ch >> 2) * 16 + m_) * 4 + (ch & 3);
      if (EPI == EPI_SWIGLU) {
        float sg = 0.f, su = 0.f;
#pragma unroll 4
        for (int w = 0; w < DS_WAVES; ++w) {
          sg += rb[(w * NRB + 0) * 256 + at];
          su += rb[(w * NRB + (NRB > 1 ? 1 : 0)) * 256 + at];
        }
        sg = (sg - off) * scl[ch];
        su = (su - off) * scl[(NRB > 1 ? 16 : 0) + ch];
        put(out[0] + grouped_at(m_, n), (f16)su * swish_f16((f16)sg));
      } else {
        float s = 0.f;
#pragma unroll 8
        for (int w = 0; w < DS_WAVES; ++w) s += rb[(w * NRB + r) * 256 + at];
        s = (s - off) * scl[r * 16 + ch];
        y = (f16)s;
        if (EPI == EPI_RESIDUAL) {
          y = y + res;
          put(out[r] + grouped_at(m_, n), y);
        } else {
          put(out[r] + (size_t)m_ * ostride + n, y);
        }
      }
    }
  }
  return y;
}

// out = fp16(scale * sum) of unit u, from the tiles in places [BASE, BASE + NRB * TPW) and the fragments xt (tile i of
// this wave in xt[i]); see gemv_slots for the numerics.  One matrix at a time: its accumulators are stored before the
// next one's are started.
template <int NRB, int TPW, int EPI, int BASE, int NSLOT>
__device__ __forceinline__ f16 wide_unit(const u32x4 (&S)[NSLOT], const float* scl, f16* const (&out)[NRB], int ostride,
                                         f16 res, int u, int n_units, int N, int KT, int M, const XTile (&xt)[TPW], float* red,
                                         int& red_buf, const float* xsum) {
  if (u >= n_units) return res;
  const int wave = wave_id();
  float* rb = red + red_buf * DW_RED;
#pragma unroll
  for (int r = 0; r < NRB; ++r) {
    f32x4 acc[1][2];
    acc[0][0] = acc[0][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < TPW; ++i)
      if (wave + i * DS_WAVES < KT) wide_tile_product<1, TPW>(S, acc, BASE + r * TPW, i, xt[i]);
    wide_stash<NRB>(acc[0][0] * 16777216.0f + acc[0][1] * 1048576.0f, r, rb);
  }
  red_buf ^= 1;
  return wide_finish<NRB, EPI>(out, ostride, res, u, N, M, rb, xsum, scl);
}

template <int TPW_D, int TPW_F, int U_F, bool KV8 = false>
__global__ __launch_bounds__(DS_THREADS) void decode_step_wide_kernel(DsArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  if (*a.keep_going == 0) return;
  if (__hip_atomic_load((DS_GLOBAL unsigned*)(a.sync + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
  const int KT_D = (a.d + 127) / 128, KT_F = (a.ffn + 127) / 128;
  float* att_lds = reinterpret_cast<float*>(smem);
  float* red = reinterpret_cast<float*>(smem + a.region0);
  float* scratch = red + 2 * DW_RED;                               // [16 waves][16 rows] sums of squares
  float* xsum = scratch + DS_WAVES * DW_MAXB;                      // [16 waves][16 rows] sums of the rows
  float* sel = xsum + DS_WAVES * DW_MAXB;                          // selection scratch (64 floats), then flags
  int* lds_dead = reinterpret_cast<int*>(sel + 64);
  float* scl = sel + 64 + 4;                                       // [2][6][16] channel scales, the phases in turn
  f16* normw = reinterpret_cast<f16*>(scratch + DW_TAIL_FLOATS);   // [d rounded up to 512]: normw_fetch writes whole KiB
  f16* cs = normw + ((a.d + 511) & ~511);                          // [D]: cos, sin of this step's angles
  uint32_t* lds_layers = reinterpret_cast<uint32_t*>(cs + DS_D);   // [n_layer] descriptors

  const int M = a.B;
  const int step = *a.step;
  const int nb_d = (a.d + 15) / 16, nb_f = (a.ffn + 15) / 16, nb_v = (a.vocab + 15) / 16;
  const int G = gridDim.x, wg = logical_workgroup(blockIdx.x, G, a.xcd_groups);
  struct { int wg; } g{wg};       // for TRACE
  (void)g;
  const unsigned epoch = __hip_atomic_load((DS_GLOBAL unsigned*)a.sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
  Waiter w{a.sync + 1, lds_dead, 0, wall_clock64() + DS_LAUNCH_TICKS};
  int red_buf = 0;
  const size_t xslot = (size_t)DW_MAXB * a.d;      // halves of one residual-stream slot: always sixteen rows

  // ---- set-up: as in decode_step_kernel, except that only the slots the attention phase and the selection poll
  //      (q/k/v, attention partials, logits) are filled; the arrival rows are cleared
  TRACE_STEP(26);
  if (wave_id() == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");      // no cache holds a line of an earlier launch
  TRACE_STEP(25);
  {
    const int tid = thread_id();
    if (tid == 0) *lds_dead = 0;
    const u32x4 filler = {DS_EMPTY32, DS_EMPTY32, DS_EMPTY32, DS_EMPTY32};
    const u32x4 zero = {0, 0, 0, 0};
    const size_t first = ((size_t)wg * DS_THREADS + tid) * 16, stride = (size_t)G * DS_THREADS * 16;
    const size_t qkv_bytes = (size_t)a.n_layer * M * 3 * a.d * 2;
    const size_t part_bytes = (size_t)(reinterpret_cast<unsigned char*>(a.flags) - reinterpret_cast<unsigned char*>(a.part));
    const size_t flag_bytes = (size_t)(4 * a.n_layer + 1) * DW_REPLICAS * a.flag_words * 4;
    for (size_t off = first; off < qkv_bytes; off += stride) put16(a.qkv, qkv_bytes, off, filler);
    for (size_t off = first; off < part_bytes; off += stride) put16(a.part, part_bytes, off, filler);
    for (size_t off = first; off < flag_bytes; off += stride) put16(a.flags, flag_bytes, off, zero);
    for (size_t off = first; off < (size_t)G * 128; off += stride) put16(a.best, (size_t)G * 128, off, filler);
    for (size_t i = ((size_t)wg * DS_THREADS + tid) * 8; i < (size_t)M * a.vocab; i += (size_t)G * DS_THREADS * 8)
      put16(a.logits, (size_t)M * a.vocab * 2, i * 2, filler);
    for (int i = tid; i < a.n_layer * DS_LAYER_WORDS; i += DS_THREADS) lds_layers[i] = a.layers[i];
    if (tid < DS_D / 2) {
      const f16 ang = (f16)((float)(f16)(float)step * (float)a.inv_freq[tid]);
      cs[tid] = (f16)cosf((float)ang);
      cs[DS_D / 2 + tid] = (f16)sinf((float)ang);
    }
    const int col = step < a.max_len ? step : a.max_len - 1;
    for (int i = wg * DS_THREADS + tid; i < M * a.d; i += G * DS_THREADS) {
      const int b = i / a.d, c = i % a.d;
      int id = a.container[(size_t)b * a.max_len + col];
      id = id < 0 ? 0 : (id >= a.vocab ? a.vocab - 1 : id);
      put(a.xres + grouped_at(b, c), a.embed[(size_t)id * a.d + c]);
    }
  }
  wg_sync();

  // Places of the units in the tile array: as in decode_step_kernel.  The tiles are requested later than there, so
  // that at most 12 places hold tiles at any time: activation fragments and tiles share the 128 registers of a wave,
  // and a value that does not fit is reloaded from scratch memory behind every tile requested ahead.
  constexpr int T = TPW_D;
  constexpr int NSLOT = 8 * T;
  constexpr int S_QKV = 0, S_O = 3 * T, S_GU0 = 4 * T, S_GU1 = 6 * T, S_GU2 = 0, S_D = 3 * T;
  constexpr int D_EARLY = TPW_F < T ? TPW_F : T;
  static_assert(U_F <= 3 && TPW_F <= 3 * T, "see decode_step_kernel");
  u32x4 S[NSLOT];
  {
    const LayerPtrs L0 = layer_ptrs(lds_layers, 0);
    normw_fetch(L0.get<const f16>(P_N1), normw, a.d);
    const Mat m3[3] = {layer_mat(L0, P_WQ, P_SQ), layer_mat(L0, P_WK, P_SK), layer_mat(L0, P_WV, P_SV)};
    load_tiles<3, T, S_QKV>(S, m3, wg, nb_d, KT_D);
  }
  TRACE_STEP(27);
  grid_barrier(a.sync, epoch, G, wg, w);
  bool alive = *lds_dead == 0;
  TRACE_STEP(28);

  // the residual element of this thread's output (epilogue mapping of wide_finish: row tid / 16, channel tid % 16)
  f16 res = (f16)0.0f;
  if (alive) {
    const int tid = thread_id();
    const int m_ = tid >> 4, n = wg * 16 + (tid & 15);
    const bool on = m_ < M && n < a.d;
    res = wait_value(a.xres + (on ? grouped_at(m_, n) : 0), on, w);
  }
  const int wave = wave_id();
  auto phase_rows = [&](int phase) { return a.flags + (size_t)phase * DW_REPLICAS * a.flag_words; };

  for (int li = 0; li < a.n_layer && alive; ++li) {
    const LayerPtrs L = layer_ptrs(lds_layers, li);
    const bool more = li + 1 < a.n_layer;
    const LayerPtrs Ln = layer_ptrs(lds_layers, more ? li + 1 : li);
    // the matrices' pointers are rebuilt from the descriptor words where they are used (a few lane reads each): held
    // across the layer they would not fit the scalar registers
#define M3 {layer_mat(L, P_WQ, P_SQ), layer_mat(L, P_WK, P_SK), layer_mat(L, P_WV, P_SV)}
#define MO {layer_mat(L, P_WO, P_SO)}
#define MGU {layer_mat(L, P_WG, P_SG), layer_mat(L, P_WU, P_SU)}
#define MD {layer_mat(L, P_WD, P_SD)}
#define M3N {layer_mat(Ln, P_WQ, P_SQ), layer_mat(Ln, P_WK, P_SK), layer_mat(Ln, P_WV, P_SV)}
    f16* const x_in = a.xres + (size_t)(2 * li) * xslot;
    f16* const x_mid = x_in + xslot;
    f16* const x_out = x_mid + xslot;
    XTile xt[T];
    // ---- RMSNorm + q/k/v (scales in the first of the two LDS places, which the phases take in turn)
    TRACE(0);
    {
      f16 sv[3] = {};
      if (wave == 0) { const Mat mm[3] = M3; request_scales<3>(mm, wg, nb_d, a.d, sv); }
      // the first layer's input is the embedding rows, complete since the grid barrier
      if (li > 0) await_row(phase_rows(4 * li), a.flag_words, G, wg, w);
#pragma unroll
      for (int i = 0; i < T; ++i) {
        xt[i] = XTile{};
        load_xtile(x_in, M, a.d, wave + i * DS_WAVES, xt[i]);
      }
      if (wave == 0) keep_scales<3>(sv, scl);
    }
    { const Mat mm[1] = MO; load_tiles<1, T, S_O>(S, mm, wg, nb_d, KT_D); }
    { const Mat mm[2] = MGU; load_tiles<2, T, S_GU0, 0, T>(S, mm, wg, nb_f, KT_D); }
    TRACE(1);
    norm_xtiles<T>(xt, normw, a.d, KT_D, a.eps, scratch);
    alive = *lds_dead == 0;      // behind the barrier of the norm: the same answer in every wave
    if (!alive) break;
    {
      const float s1 = xtiles_rowsum<T>(xt);
      if (lane_id() < 16) xsum[wave * DW_MAXB + lane_id()] = s1;
      f16* q = a.qkv + (size_t)li * M * 3 * a.d;
      f16* const o3[3] = {q, q + a.d, q + 2 * a.d};
      wide_unit<3, T, EPI_STORE, S_QKV>(S, scl, o3, 3 * a.d, (f16)0.0f, wg, nb_d, a.d, KT_D, M, xt, red, red_buf, xsum);
    }
    { const Mat mm[2] = MGU; load_tiles<2, T, S_GU0, T, T>(S, mm, wg, nb_f, KT_D); }
    TRACE(2);
    // ---- rotary + KV append + attention
    {
      f16* kring = L.get<f16>(P_KV);
      const int units = M * a.H * a.nsplit;
      if (a.nsplit == 1 && a.H * 8 == G) {
        // sequences wg % 8 and wg % 8 + 8 of head wg / 8: the workgroups that produce the head's q | k | v
        const int b0 = wg % 8, h = wg / 8;
        if (b0 < M) attention_two<KV8>(a, li, kring, b0 * a.H + h, b0 + 8 < M ? (b0 + 8) * a.H + h : -1, step, att_lds, cs, w);
      } else if (a.nsplit == 1) {
        for (int u = wg; u < units; u += 2 * G) attention_two<KV8>(a, li, kring, u, u + G < units ? u + G : -1, step, att_lds, cs, w);
      } else {
        for (int u = wg; u < units; u += G) attention_unit<true, KV8>(a, li, kring, u, step, att_lds, cs, w);
      }
      // the head outputs are stored by waves 0, 1 and (second unit of attention_two) 8, 9
      announce(phase_rows(4 * li + 1), a.flag_words, wg, wave < 2 || wave == 8 || wave == 9);
      if constexpr (U_F > 1) { const Mat mm[2] = MGU; load_tiles<2, T, S_GU1>(S, mm, wg + G, nb_f, KT_D); }
    }
    TRACE(3);
    // ---- o_proj + residual
    {
      f16 sv[1] = {};
      if (wave == 0) { const Mat mm[1] = MO; request_scales<1>(mm, wg, nb_d, a.d, sv); }
      await_row(phase_rows(4 * li + 1), a.flag_words, G, wg, w);
#pragma unroll
      for (int i = 0; i < T; ++i) {
        xt[i] = XTile{};
        load_xtile(a.ctx + (size_t)li * xslot, M, a.d, wave + i * DS_WAVES, xt[i]);
      }
      if (wave == 0) keep_scales<1>(sv, scl + DW_SCL);
    }
    wg_sync();      // the row sums of the previous phase have been read; every wave knows whether one gave up
    alive = *lds_dead == 0;
    if (!alive) break;
    TRACE(4);
    {
      const float s1 = xtiles_rowsum<T>(xt);
      if (lane_id() < 16) xsum[wave * DW_MAXB + lane_id()] = s1;
      f16* const o1[1] = {x_mid};
      res = wide_unit<1, T, EPI_RESIDUAL, S_O>(S, scl + DW_SCL, o1, a.d, res, wg, nb_d, a.d, KT_D, M, xt, red, red_buf, xsum);
    }
    announce(phase_rows(4 * li + 2), a.flag_words, wg, wave < 4);
    if constexpr (U_F > 2) { const Mat mm[2] = MGU; load_tiles<2, T, S_GU2>(S, mm, wg + 2 * G, nb_f, KT_D); }
    normw_fetch(L.get<const f16>(P_N2), normw, a.d);
    TRACE(5);
    // ---- RMSNorm + gate/up + SwiGLU, one unit after the other
    {
      f16 sv[U_F][2] = {};
      if (wave == 0) {
#pragma unroll
        for (int k = 0; k < U_F; ++k) { const Mat mm[2] = MGU; request_scales<2>(mm, wg + k * G, nb_f, a.ffn, sv[k]); }
      }
      await_row(phase_rows(4 * li + 2), a.flag_words, G, wg, w);
#pragma unroll
      for (int i = 0; i < T; ++i) {
        xt[i] = XTile{};
        load_xtile(x_mid, M, a.d, wave + i * DS_WAVES, xt[i]);
      }
      if (wave == 0) {
#pragma unroll
        for (int k = 0; k < U_F; ++k) keep_scales<2>(sv[k], scl + k * 32);
      }
    }
    TRACE(6);
    norm_xtiles<T>(xt, normw, a.d, KT_D, a.eps, scratch);
    alive = *lds_dead == 0;
    if (!alive) break;
    {
      const float s1 = xtiles_rowsum<T>(xt);
      if (lane_id() < 16) xsum[wave * DW_MAXB + lane_id()] = s1;
      f16* act = a.act + (size_t)li * DW_MAXB * a.ffn;
      f16* const o2[2] = {act, act};
      wide_unit<2, T, EPI_SWIGLU, S_GU0>(S, scl, o2, a.ffn, (f16)0.0f, wg, nb_f, a.ffn, KT_D, M, xt, red, red_buf, xsum);
      if constexpr (U_F > 1)
        wide_unit<2, T, EPI_SWIGLU, S_GU1>(S, scl + 32, o2, a.ffn, (f16)0.0f, wg + G, nb_f, a.ffn, KT_D, M, xt, red, red_buf, xsum);
      if constexpr (U_F > 2)
        wide_unit<2, T, EPI_SWIGLU, S_GU2>(S, scl + 64, o2, a.ffn, (f16)0.0f, wg + 2 * G, nb_f, a.ffn, KT_D, M, xt, red, red_buf, xsum);
    }
    announce(phase_rows(4 * li + 3), a.flag_words, wg, wave < 4);
    { const Mat mm[1] = MD; load_tiles<1, TPW_F, S_D>(S, mm, wg, nb_d, KT_F); }
    TRACE(7);
    // ---- down + residual: the fragments of one K tile at a time, the next tile's requested before the wait
    {
      f32x4 acc[1][2];
      acc[0][0] = acc[0][1] = f32x4{0.f, 0.f, 0.f, 0.f};
      float s1 = 0.f;
      const f16* actx = a.act + (size_t)li * DW_MAXB * a.ffn;
      f16 sv[1] = {};
      if (wave == 0) { const Mat mm[1] = MD; request_scales<1>(mm, wg, nb_d, a.d, sv); }
      await_row(phase_rows(4 * li + 3), a.flag_words, G, wg, w);
      // Two tiles' fragments are on their way at any time: the even tiles into registers, the odd ones into 4 KiB
      // of LDS per wave - the reduction buffer the last gate/up unit used and the part of the current one beyond
      // this phase's single matrix, both idle here.  (One tile ahead, in registers alone, left the phase waiting a
      // round trip per tile.)  A wave's loads return in order, so a wait names how many younger loads may still
      // be out: the next even tile's four and, at the third tile, the next layer's four weight tiles as well.
      XTile ahead;
      float* const slot = wave < 12 ? red + (red_buf ^ 1) * DW_RED + wave * 1024 : red + red_buf * DW_RED + 4096 + (wave - 12) * 1024;
      load_xtile(actx, M, a.ffn, wave, ahead);
      if constexpr (TPW_F > 1) load_xtile_lds(actx, M, a.ffn, wave + DS_WAVES, slot);
      if (wave == 0) keep_scales<1>(sv, scl + DW_SCL);      // requested before the arrival row: here by now
      if constexpr (TPW_F == 1) {
        { const Mat mm[3] = M3N; load_tiles<3, T, S_QKV, 2 * T, T>(S, mm, wg, nb_d, KT_D); }      // the next layer's v and q
        { const Mat mm[3] = M3N; load_tiles<3, T, S_QKV, 0, T>(S, mm, wg, nb_d, KT_D); }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TPW_F; ++i) {
        XTile x1;
        if (i % 2 == 0) {
          x1 = ahead;
          if (i + 2 < TPW_F) load_xtile(actx, M, a.ffn, wave + (i + 2) * DS_WAVES, ahead);      // (a tile beyond the last: zeros)
        } else {
          wait_loads_but((i + 1 < TPW_F ? 4 : 0) + (i == 3 ? 2 * T : 0));
          read_xtile_lds(slot, x1);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // read before the slot is requested again
          if (i + 2 < TPW_F) load_xtile_lds(actx, M, a.ffn, wave + (i + 2) * DS_WAVES, slot);
          if (i == 1) {
            { const Mat mm[3] = M3N; load_tiles<3, T, S_QKV, 2 * T, T>(S, mm, wg, nb_d, KT_D); }      // the next layer's v and q
            { const Mat mm[3] = M3N; load_tiles<3, T, S_QKV, 0, T>(S, mm, wg, nb_d, KT_D); }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (wave + i * DS_WAVES < KT_F) {
          const XTile one[1] = {x1};
          s1 += xtiles_rowsum<1>(one);
          wide_tile_product<1, TPW_F>(S, acc, S_D, i, x1);
        }
      }
      wg_sync();      // the row sums of the previous phase have been read; every wave knows whether one gave up
      alive = *lds_dead == 0;
      if (!alive) break;
      TRACE(8);
      if (lane_id() < 16) xsum[wave * DW_MAXB + lane_id()] = s1;
      f16* const o1[1] = {x_out};
      if (wg < nb_d) {
        float* rb = red + red_buf * DW_RED;
        wide_stash<1>(acc[0][0] * 16777216.0f + acc[0][1] * 1048576.0f, 0, rb);
        red_buf ^= 1;
        res = wide_finish<1, EPI_RESIDUAL>(o1, a.d, res, wg, a.d, M, rb, xsum, scl + DW_SCL);
      }
      announce(phase_rows(4 * li + 4), a.flag_words, wg, wave < 4);
      { const Mat mm[3] = M3N; load_tiles<3, T, S_QKV, T, T>(S, mm, wg, nb_d, KT_D); }
      normw_fetch(more ? Ln.get<const f16>(P_N1) : a.final_norm, normw, a.d);
      TRACE(9);
    }
  }
  TRACE_STEP(29);
#undef M3
#undef MO
#undef MGU
#undef MD
#undef M3N
  // ---- final RMSNorm + lm_head, streamed unit by unit with the next unit's tiles in flight
  if (alive) {
    XTile xt[T];
    alive = await_row(phase_rows(4 * a.n_layer), a.flag_words, G, wg, w);
#pragma unroll
    for (int i = 0; i < T; ++i) {
      xt[i] = XTile{};
      load_xtile(a.xres + (size_t)(2 * a.n_layer) * xslot, M, a.d, wave + i * DS_WAVES, xt[i]);
    }
    wg_sync();
    alive = *lds_dead == 0;
    if (alive) {
      norm_xtiles<T>(xt, normw, a.d, KT_D, a.eps, scratch);
      const Mat m1[1] = {{a.head, nullptr}};
      f16* const o1[1] = {a.logits};
      Unit<FmtF16, 1, T> even, odd;
      // thread 16 m + ch finishes channel ch of row m of every unit and keeps the row's largest logit among them (the
      // lowest index among equals: the units come in ascending order, NaN is never larger)
      float top = -INFINITY;
      int top_at = 0x7fffffff;
      auto head_unit = [&](const Unit<FmtF16, 1, T>& t, int u) {
        if (u >= nb_v) return;
        f32x4 acc[1] = {f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int i = 0; i < T; ++i)
          if (wave + i * DS_WAVES < KT_D) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(FmtF16::a_operand(t.w[0][i], j, t.sc[0]), xt[i].v[j], acc[0], 0, 0, 0);
          }
        const f16 y = finish_unit<1, EPI_STORE, false, NoScales, DW_MAXB, DW_RED>(acc, o1, a.vocab, (f16)0.0f, u, a.vocab, M, red, red_buf);
        const int tid = thread_id(), n = u * 16 + (tid & 15);
        if (tid < 16 * M && n < a.vocab && (float)y > top) { top = (float)y; top_at = n; }
      };
      load_unit(even, m1, wg, nb_v, a.vocab, KT_D);
      for (int u = wg; u < nb_v; u += 2 * G) {
        load_unit(odd, m1, u + G, nb_v, a.vocab, KT_D);
        head_unit(even, u);
        load_unit(even, m1, u + 2 * G, nb_v, a.vocab, KT_D);
        head_unit(odd, u + G);
      }
      // the sixteen channels of a row meet; the row's pair goes to this workgroup's place
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) {
        const float ov = __shfl_xor(top, o, 64);
        const int oi = __shfl_xor(top_at, o, 64);
        if (ov > top || (ov == top && oi < top_at)) { top = ov; top_at = oi; }
      }
      const int tid = thread_id();
      if (tid < 16 * M && (tid & 15) == 0) {
        uint32_t* mine = a.best + ((size_t)wg * 16 + (tid >> 4)) * 2;
        __hip_atomic_store((DS_GLOBAL uint32_t*)mine, bitcast<uint32_t>(top), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store((DS_GLOBAL uint32_t*)(mine + 1), (uint32_t)top_at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  TRACE_STEP(30);
  // ---- selection and bookkeeping
  if (wg == 0) {
    if (alive) {
      // wave r gathers row r's pairs of all workgroups (neither word of a pair is ever the filler)
      int* ids = reinterpret_cast<int*>(sel);
      const int lane = lane_id();
      float top = -INFINITY;
      int top_at = 0x7fffffff;
      if (wave < M) {
        for (int g0 = 0; g0 < G; g0 += 256) {      // four pairs per lane travel together
          uint32_t vb[4], ib[4];
          for (;;) {
            bool pending = false;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int gg = g0 + k * 64 + lane;
              const uint32_t* p = a.best + ((size_t)(gg < G ? gg : G - 1) * 16 + wave) * 2;
              vb[k] = get_bits(reinterpret_cast<const float*>(p));
              ib[k] = get_bits(reinterpret_cast<const float*>(p + 1));
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) pending = pending || vb[k] == DS_EMPTY32 || ib[k] == DS_EMPTY32;
            if (!__any(pending) || w.give_up()) break;
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const float v = bitcast<float>(vb[k]);
            if (g0 + k * 64 + lane < G && (v > top || (v == top && (int)ib[k] < top_at))) { top = v; top_at = (int)ib[k]; }
          }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
          const float ov = __shfl_xor(top, o, 64);
          const int oi = __shfl_xor(top_at, o, 64);
          if (ov > top || (ov == top && oi < top_at)) { top = ov; top_at = oi; }
        }
        if (lane == 0) ids[wave] = top_at == 0x7fffffff ? 0 : top_at;
      }
      wg_sync();
      if (*lds_dead == 0) advance_rows(a, ids);
    }
    if (thread_id() == 0)
      __hip_atomic_store((DS_GLOBAL unsigned*)a.sync, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  TRACE_STEP(31);
}

struct Variant {
  int tpw_d, tpw_f, u_f, minb, maxb;
  bool kv8;              // FP8 (F143) KV rings
  void (*kern)(DsArgs);
  bool ready;
};
Variant g_variants[] = {
    {1, 1, 1, 1, 4, false, decode_step_kernel<1, 1, 1, 4>, false},        // small test shapes
    {2, 6, 3, 1, 1, false, decode_step_kernel<2, 6, 3, 1>, false},        // 7B: hidden 4096, ffn 11008, batch 1
    {2, 6, 3, 2, 4, false, decode_step_kernel<2, 6, 3, 4>, false},        // 7B, batch 2..4
    {1, 1, 1, 5, 16, false, decode_step_wide_kernel<1, 1, 1>, false},     // small test shapes, batch 5..16
    {2, 6, 3, 5, 16, false, decode_step_wide_kernel<2, 6, 3>, false},     // 7B, batch 5..16
    {1, 1, 1, 1, 4, true, decode_step_kernel<1, 1, 1, 4, true>, false},   // the same with FP8 KV rings
    {2, 6, 3, 1, 1, true, decode_step_kernel<2, 6, 3, 1, true>, false},
    {2, 6, 3, 2, 4, true, decode_step_kernel<2, 6, 3, 4, true>, false},
    {1, 1, 1, 5, 16, true, decode_step_wide_kernel<1, 1, 1, true>, false},
    {2, 6, 3, 5, 16, true, decode_step_wide_kernel<2, 6, 3, true>, false},
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

int device_cus(int* cus) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  if (hipDeviceGetAttribute(cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || *cus <= 0) return -1;
  return 0;
}

int splits_for(int cus, int B, int H) {
  const int n = cus / (B * H);
  return n < 1 ? 1 : (n > DS_MAX_SPLIT ? DS_MAX_SPLIT : n);
}

size_t flag_words_for(int cus) { return ((size_t)cus + 255) & ~(size_t)255; }

// byte offsets of the workspace parts
struct Layout {
  size_t sync, xres, qkv, ctx, act, part, flags, best, trace, total;
};
Layout layout_for(const pta_decode_model* m, int cus) {
  const size_t B = m->batch, d = m->hidden, L = m->n_layer, f = m->ffn, H = m->n_head;
  const size_t R = B > DS_MAXB ? DW_MAXB : B;      // rows of an activation slot: decode_step_wide_kernel's hold sixteen
  Layout l;
  l.sync = 0;
  l.xres = align256((size_t)(16 + DS_REPLICAS * cus) * 4);
  l.qkv = l.xres + align256((2 * L + 1) * R * d * 2);
  l.ctx = l.qkv + align256(L * B * 3 * d * 2);
  l.act = l.ctx + align256(L * R * d * 2);
  l.part = l.act + align256(L * R * f * 2);
  l.flags = l.part + align256(L * B * H * splits_for(cus, (int)B, (int)H) * DS_PART * 4);
  // arrival words and per-workgroup best logits: decode_step_wide_kernel only
  l.best = l.flags + (B > DS_MAXB ? align256((4 * L + 1) * DS_REPLICAS * flag_words_for(cus) * 4) : 0);
  l.trace = l.best + (B > DS_MAXB ? align256((size_t)cus * 16 * 2 * 4) : 0);
  l.total = l.trace + (size_t)cus * DS_TRACE_WORDS * 8;
  return l;
}

bool shape_ok(const pta_decode_model* m) {
  return m && m->batch >= 1 && m->batch <= DW_MAXB && m->hidden > 0 && m->n_head > 0 && m->ffn > 0 && m->vocab > 0 &&
         m->max_len > 0 && m->n_layer > 0 && m->head_dim == DS_D && m->hidden == m->n_head * DS_D && m->ffn % 8 == 0 &&
         m->vocab % 8 == 0;
}

}  // namespace

extern "C" size_t pta_decode_step_workspace_bytes(const pta_decode_model* model) {
  int cus = 0;
  if (!shape_ok(model) || device_cus(&cus) != 0) return 0;
  return layout_for(model, cus).total;
}

// `who`: the entry point's name, for its messages
static int decode_step_launch(const char* who, const pta_decode_model* mdl, const pta_decode_state* st, void* workspace,
                              pta_stream_t stream, bool kv8 = false, int kv_scale = 0) {
  PTA_REQUIRE(mdl && st && workspace, "%s: null pointer", who);
  PTA_REQUIRE(mdl->layers && mdl->n_layer > 0 && mdl->embed && mdl->final_norm && mdl->head && mdl->inv_freq,
              "%s: incomplete model", who);
  PTA_REQUIRE(st->container && st->mask && st->stop_mask && st->step && st->keep_going && st->next_ids && st->logits,
              "%s: incomplete state", who);
  PTA_REQUIRE(pta_aligned(workspace, 256) && pta_aligned(st->logits, 16),
              "%s: the workspace must be 256-byte aligned and the logits 16-byte aligned", who);
  const int B = mdl->batch, d = mdl->hidden, H = mdl->n_head, ffn = mdl->ffn;
  PTA_REQUIRE(B >= 1 && d > 0 && H > 0 && ffn > 0 && mdl->vocab > 0 && mdl->max_len > 0,
              "%s: empty shape", who);
  int cus = 0;
  PTA_REQUIRE(device_cus(&cus) == 0, "%s: cannot read the compute-unit count of the current device", who);
  const int KT_D = (d + 127) / 128, KT_F = (ffn + 127) / 128;
  const int tpw_d = (KT_D + DS_WAVES - 1) / DS_WAVES, tpw_f = (KT_F + DS_WAVES - 1) / DS_WAVES;
  const int nb_d = (d + 15) / 16, nb_f = (ffn + 15) / 16;
  const int u_f = (nb_f + cus - 1) / cus;
  Variant* var = nullptr;
  for (Variant& v : g_variants)
    if (v.tpw_d == tpw_d && v.tpw_f == tpw_f && u_f <= v.u_f && B >= v.minb && B <= v.maxb && v.kv8 == kv8 && !var) var = &v;
  if (!shape_ok(mdl) || nb_d > cus || !var) {
    pta_set_error("%s: supports batch <= %d, head size %d, hidden = heads * head size <= %d, ffn "
                  "and vocabulary sizes that are multiples of 8, and the (hidden, ffn) of the 7B model or small test "
                  "shapes (got batch %d, head size %d, hidden %d, heads %d, ffn %d, vocabulary %d)", who,
                  DW_MAXB, DS_D, 16 * cus, B, mdl->head_dim, d, H, ffn, mdl->vocab);
    return PTA_EUNSUPPORTED;
  }

  const Layout lay = layout_for(mdl, cus);
  char* ws = (char*)workspace;
  DsArgs a{};
  a.layers = reinterpret_cast<const uint32_t*>(mdl->layers);
  a.n_layer = mdl->n_layer;
  a.embed = (const f16*)mdl->embed; a.final_norm = (const f16*)mdl->final_norm;
  a.head = (const u32x4*)mdl->head; a.inv_freq = (const f16*)mdl->inv_freq;
  a.B = B; a.d = d; a.H = H; a.ffn = ffn; a.vocab = mdl->vocab; a.max_len = mdl->max_len; a.eps = mdl->eps;
  a.container = st->container; a.mask = (f16*)st->mask; a.stop_mask = st->stop_mask; a.step = st->step;
  a.keep_going = st->keep_going; a.next_ids = st->next_ids;
  a.pad_id = mdl->pad_id; a.eos_id = mdl->eos_id; a.early_stop = mdl->early_stop;
  a.logits = (f16*)st->logits;
  a.sync = (unsigned*)(ws + lay.sync);
  a.xres = (f16*)(ws + lay.xres);
  a.qkv = (f16*)(ws + lay.qkv);
  a.ctx = (f16*)(ws + lay.ctx);
  a.act = (f16*)(ws + lay.act);
  a.part = (float*)(ws + lay.part);
  a.trace = (unsigned long long*)(ws + lay.trace);
  a.fill_bytes = lay.flags - (lay.xres + (size_t)B * d * 2);   // everything after the first residual slot, up to the flags
  a.flags = (unsigned*)(ws + lay.flags);
  a.flag_words = (int)flag_words_for(cus);
  a.best = (uint32_t*)(ws + lay.best);
  a.nsplit = splits_for(cus, B, H);
  a.kv_scale = kv_scale;
  {
    static const int by_die = [] { const char* v = getenv("PTA_DS_XCD_GROUPS"); return v && v[0] == '1' ? 1 : 0; }();
    a.xcd_groups = by_die;
  }
  const bool wide = B > DS_MAXB;                 // nothing is staged: the head of LDS is the attention area only
  const int xstride = (KT_D > KT_F ? KT_D : KT_F) * 128 + 8;
  size_t region0 = wide ? 0 : (size_t)B * xstride * 2;
  if (region0 < (size_t)DS_ATT_FLOATS * 4) region0 = (size_t)DS_ATT_FLOATS * 4;
  region0 = (region0 + 15) & ~(size_t)15;
  a.region0 = (int)region0;
  const size_t lds = wide ? region0 + (size_t)(2 * DW_RED + DW_TAIL_FLOATS) * 4 + (size_t)((d + 511) & ~511) * 2 + DS_D * 2 +
                                (size_t)mdl->n_layer * sizeof(pta_decode_layer)
                          : region0 + (size_t)(2 * DS_RED + DS_TAIL_FLOATS) * 4 + (size_t)((d + 511) & ~511) * 2 + DS_D * 2 +
                                (size_t)mdl->n_layer * sizeof(pta_decode_layer);
  PTA_REQUIRE(lds <= 160 * 1024, "%s: %zu bytes of LDS exceed a compute unit's 160 KiB", who, lds);

  if (!var->ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)var->kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) ==
                    hipSuccess,
                "%s: cannot reserve dynamic LDS", who);
    // every workgroup must be resident at once: one per compute unit, so the kernel must fit one
    int per_cu = 0;
    PTA_REQUIRE(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)var->kern, DS_THREADS, lds) ==
                        hipSuccess && per_cu >= 1,
                "%s: the kernel does not fit a compute unit", who);
    var->ready = true;
  }
  hipLaunchKernelGGL(var->kern, dim3(cus), dim3(DS_THREADS), lds, (hipStream_t)stream, a);
  PTA_CHECK_LAUNCH(who);
  return PTA_OK;
}

extern "C" int pta_llama_decode_step(const pta_decode_model* mdl, const pta_decode_state* st, void* workspace,
                                     pta_stream_t stream) {
  return decode_step_launch("pta_llama_decode_step", mdl, st, workspace, stream);
}

extern "C" int pta_llama_decode_step_f8(const pta_decode_model* mdl, const pta_decode_state* st, int kv_scale, void* workspace,
                                        pta_stream_t stream) {
  PTA_REQUIRE(kv_scale >= -16 && kv_scale <= 16, "pta_llama_decode_step_f8: kv_scale %d outside [-16, 16]", kv_scale);
  return decode_step_launch("pta_llama_decode_step_f8", mdl, st, workspace, stream, true, kv_scale);
}

// ------------------------------------------------------------------------------------------ the same step without a workspace argument
// The workspace of pta_llama_decode_step (result slots, attention partials, synchronisation words) in a
// file-scope device array, for callers that cannot allocate.  Every device holds its own copy of the
// array at its own address; the name `scratch` is only a host-side handle, so the address is looked up
// once per device with hipGetSymbolAddress and kept.  The array starts zeroed (epoch 0, no failure), which
// is the state the kernel expects of a fresh workspace; later launches continue the epoch of the one before,
// whatever model they serve, because the synchronisation words sit at the same offsets for every shape.
namespace {
constexpr size_t DS_STATIC_BYTES = (size_t)16 << 20;
constexpr int DS_MAX_DEVICES = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[DS_STATIC_BYTES];

namespace {
std::mutex g_static_mutex;
void* g_static_ptr[DS_MAX_DEVICES] = {};

__global__ void clear_failure_kernel(unsigned* sync) {
  if (threadIdx.x == 0 && blockIdx.x == 0)
    __hip_atomic_store((DS_GLOBAL unsigned*)(sync + 1), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
}  // namespace

extern "C" int pta_llama_decode_step_static(const pta_decode_model* mdl, const pta_decode_state* st, int clear_failure,
                                            pta_stream_t stream) {
  PTA_REQUIRE(mdl && st, "pta_llama_decode_step_static: null pointer");
  int dev = 0;
  PTA_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < DS_MAX_DEVICES,
              "pta_llama_decode_step_static: cannot identify the current device");
  int cus = 0;
  PTA_REQUIRE(device_cus(&cus) == 0, "pta_llama_decode_step_static: cannot read the compute-unit count of the current device");
  if (!shape_ok(mdl)) {
    pta_set_error("pta_llama_decode_step_static: unsupported shape (see pta_llama_decode_step)");
    return PTA_EUNSUPPORTED;
  }
  const size_t need = layout_for(mdl, cus).total;
  PTA_REQUIRE(need <= DS_STATIC_BYTES,
              "pta_llama_decode_step_static: this model needs %zu bytes of workspace, the built-in array holds %zu; use "
              "pta_llama_decode_step with a workspace of its own", need, (size_t)DS_STATIC_BYTES);
  void* ws = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
      void* p = nullptr;
      const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !p) {
        pta_set_error("pta_llama_decode_step_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        return PTA_EHIP;
      }
      g_static_ptr[dev] = p;
    }
    ws = g_static_ptr[dev];
  }
  if (clear_failure) {
    hipLaunchKernelGGL(clear_failure_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (unsigned*)ws);
    PTA_CHECK_LAUNCH("pta_llama_decode_step_static");
  }
  return decode_step_launch("pta_llama_decode_step_static", mdl, st, ws, stream);
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
