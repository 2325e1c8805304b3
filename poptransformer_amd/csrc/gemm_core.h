// Epilogue shared by the fused GEMV/GEMM kernels (INT4, FP16 and FP8 weights).
//
// The reference builds these as separate fp16 graph ops after the MatMul: the bias `ops.add`
// of poptransformer/layers/linear.py:42-46, the activation of layers/mlp.py:34-41 /
// models/rwkv/ffn.py:47-59, and the residual `ops.add` of the transformer blocks
// (e.g. models/llama2/model.py:38-46).  Each step therefore rounds to fp16.
#pragma once
#include "common.h"
#include "f8codec.h"

struct GemmEpilogue {
  const f16* bias;
  const f16* residual;
  int act;
  const f16* mul;
  float post_scale;
  int norm;                 // PTA_NORM_*, applied to the rows of X before the product
  const f16* norm_weight;
  const f16* norm_bias;
  float norm_eps;
  const int32_t* out_fp8_scale;   // when set: the result is left on the FP8 grid of this exponent (unscaled)
  int out_fp8_format;
  f16* mix_state;                 // [2][M, K] or null: the previous token's rows for the token-shift mixes (gemv_lds_kernel)
  const int32_t* mix_step;
};

__device__ __forceinline__ f16 sigmoid_f16(f16 x) {
  return (f16)(1.0f / (1.0f + __expf(-(float)x)));
}

// x * sigmoid(x), evaluated in fp32 from the fp16 input and rounded once.
__device__ __forceinline__ f16 swish_f16(f16 x) {
  const float v = (float)x;
  return (f16)(v / (1.0f + __expf(-v)));
}

// tanh-form GELU, evaluated in fp32 from the fp16 input and rounded once.
__device__ __forceinline__ f16 gelu_tanh_f16(f16 x) {
  const float v = (float)x;
  const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
  return (f16)(0.5f * v * (1.0f + tanhf(u)));
}

__device__ __forceinline__ f16 apply_act(int act, f16 y) {
  switch (act) {
    case PTA_ACT_GELU_TANH: return gelu_tanh_f16(y);
    case PTA_ACT_RELU_SQUARE: { f16 r = y > (f16)0.0f ? y : (f16)0.0f; return r * r; }
    case PTA_ACT_SIGMOID: return sigmoid_f16(y);
    default: return y;
  }
}

__device__ __forceinline__ f16 apply_epilogue(const GemmEpilogue& e, f16 y, int m, int n, int N) {
  if (e.bias) y = y + e.bias[n];
  y = apply_act(e.act, y);
  if (e.mul) y = y * e.mul[(size_t)m * N + n];
  if (e.residual) y = y + e.residual[(size_t)m * N + n];
  if (e.post_scale != 0.0f) y = y * (f16)e.post_scale;
  if (e.out_fp8_scale) y = f8_grid_value(y, e.out_fp8_scale[0], e.out_fp8_format);
  return y;
}

// the SwiGLU pair's result: up * swish(gate), then the optional cast of the epilogue
__device__ __forceinline__ f16 swiglu_out(const GemmEpilogue& e, f16 gate, f16 up) {
  f16 y = up * swish_f16(gate);
  if (e.out_fp8_scale) y = f8_grid_value(y, e.out_fp8_scale[0], e.out_fp8_format);
  return y;
}

static inline int make_epilogue(const pta_fusion* in, GemmEpilogue* out, const char* name) {
  *out = GemmEpilogue{nullptr, nullptr, PTA_ACT_NONE, nullptr, 0.f, PTA_NORM_NONE, nullptr, nullptr, 0.f, nullptr, PTA_F143, nullptr, nullptr};
  if (!in) return PTA_OK;
  PTA_REQUIRE(in->act >= PTA_ACT_NONE && in->act <= PTA_ACT_SIGMOID, "%s: unknown activation %d", name, in->act);
  PTA_REQUIRE(in->norm >= PTA_NORM_NONE && in->norm <= PTA_NORM_LAYER, "%s: unknown norm %d", name, in->norm);
  PTA_REQUIRE(in->norm == PTA_NORM_NONE || in->norm_weight, "%s: fused norm needs norm_weight", name);
  PTA_REQUIRE(in->norm != PTA_NORM_LAYER || in->norm_bias, "%s: fused LayerNorm needs norm_bias", name);
  out->bias = (const f16*)in->bias; out->residual = (const f16*)in->residual; out->act = in->act;
  out->mul = (const f16*)in->mul; out->post_scale = in->post_scale;
  out->norm = in->norm; out->norm_weight = (const f16*)in->norm_weight; out->norm_bias = (const f16*)in->norm_bias;
  out->norm_eps = in->norm_eps;
  PTA_REQUIRE(!in->out_fp8_scale || in->out_fp8_format == PTA_F143 || in->out_fp8_format == PTA_F152,
              "%s: unsupported fp8 format %d, it must be F143 or F152", name, in->out_fp8_format);
  out->out_fp8_scale = in->out_fp8_scale; out->out_fp8_format = in->out_fp8_format;
  PTA_REQUIRE(!in->mix_state == !in->mix_step, "%s: mix_state and mix_step come together", name);
  out->mix_state = (f16*)in->mix_state; out->mix_step = in->mix_step;
  return PTA_OK;
}

// ------------------------------------------------------------------------------------------
// Small-M GEMM core: Y[M,N] = fp16(X[M,K] @ W^T) for M <= 64, weights streamed once.
//
// Weights are stored tiled (see the *_tile entry points): a tile is 16 output channels x 128
// input features, made of Fmt::kVec vectors of 1 KiB; in each vector lane l owns the 16 bytes
// at offset 16*l.  The tiles of one 16-channel block are contiguous over the feature axis.
// One workgroup owns one 16-channel block; its NW waves take feature tiles round-robin, each
// wave feeding the 16x16x32 fp16 MFMA with A = 16 channels x 32 features of weights (decoded
// in registers) and B = 32 features x 16 activation rows read straight from X, and the
// partial sums meet in LDS.  HBM traffic is the weight bytes, once; X comes from L2.
// ------------------------------------------------------------------------------------------
struct GemmMat {
  const void* tiled;
  const void* scale;   // fp16 [N] (INT4), device int32 exponent (FP8), unused (FP16)
  const f16* bias;     // [N] or null; used when the launch holds several matrices
  const f16* X;        // this matrix's own input, or null for the shared one
  const f16* mix;      // this matrix's token-shift mixing vector [K], or null (with GemmEpilogue::mix_state)
  int act;             // activation of this matrix's output when the launch holds several
  f16* Y;
  int N;
  int nb_begin;        // first 16-channel block of this matrix in the launch grid
};

struct GemmArgs {
  GemmMat mat[4];
  int count;
  const f16* X;
  const int32_t* x_scale;  // device exponent of X when X holds unscaled FP8 grid values, else null
  int M, K, KT;
  GemmEpilogue epi;
  // PAIR mode (SwiGLU): mat[0] is the gate weight, mat[1] the up weight, output in mat[0].Y.
  // K split across workgroups (gemm_tile_kernel, one matrix): slice blockIdx.y of `ksplit` writes its fp32
  // sums to part[slice][M][N]; splitk_finish_kernel adds the slices and applies the epilogue.
  float* part;
  size_t part_bytes;
  int ksplit;          // 0 or 1: no split
  int prefer_stream;   // host side: up to 16 rows go to gemv_stream_kernel wherever it fits
};
static inline int device_compute_units();
constexpr int GEMM_MAX_KSPLIT = 4;
constexpr int GEMM_MAX_ROWS = 4096;

template <class Fmt, int MT, int NW, bool PAIR>
__global__ __launch_bounds__(NW * 64) void gemv_mfma_kernel(GemmArgs a) {
  constexpr int NACC = PAIR ? 2 : 1;
  constexpr int KV = Fmt::kVec;
  __shared__ float red[NW * NACC * MT * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int mi = 0;
  if (!PAIR) {
#pragma unroll
    for (int i = 1; i < 4; ++i)
      if (i < a.count && (int)blockIdx.x >= a.mat[i].nb_begin) mi = i;
  }
  const int nb = blockIdx.x - a.mat[mi].nb_begin;
  const int N = a.mat[mi].N;
  const int row = nb * 16 + (lane & 15);
  const int K = a.K, KT = a.KT;

  typename Fmt::Scale sc[NACC];
  const u32x4* wp[NACC];
#pragma unroll
  for (int g = 0; g < NACC; ++g) {
    const GemmMat& m = a.mat[PAIR ? g : mi];
    sc[g] = Fmt::load_scale(m.scale, a.x_scale, row, N);
    wp[g] = reinterpret_cast<const u32x4*>(m.tiled) + (size_t)nb * KT * (64 * KV) + lane;
  }
  // B operand source: row (mt*16 + lane%16) of X, clamped into range; lanes of padding rows
  // compute values that are never stored.
  const f16* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + (lane & 15);
    m = m < a.M ? m : a.M - 1;
    xrow[mt] = (a.mat[mi].X ? a.mat[mi].X : a.X) + (size_t)m * K + (lane >> 4) * 8;
  }

  f32x4 acc[NACC][MT];
#pragma unroll
  for (int g = 0; g < NACC; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll 2
  for (int kt = wave; kt < KT; kt += NW) {
    u32x4 w[NACC][KV];
#pragma unroll
    for (int g = 0; g < NACC; ++g)
#pragma unroll
      for (int v = 0; v < KV; ++v)
        w[g][v] = __builtin_nontemporal_load(wp[g] + ((size_t)kt * KV + v) * 64);
    f16x8 xb[4][MT];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = kt * 128 + j * 32;
      const bool in = k + (lane >> 4) * 8 < K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        xb[j][mt] = in ? *reinterpret_cast<const f16x8*>(xrow[mt] + k) : z;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int g = 0; g < NACC; ++g) {
        const f16x8 av = Fmt::a_operand(w[g], j, sc[g]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[g][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, xb[j][mt], acc[g][mt], 0, 0, 0);
      }
    }
  }

  // Cross-wave reduction through LDS, then the epilogue.  The accumulator of lane l holds
  // channels (l/16)*4 + r, r = 0..3, for activation row l%16.
#pragma unroll
  for (int g = 0; g < NACC; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        red[(((wave * NACC + g) * MT + mt) * 4 + r) * 64 + lane] = acc[g][mt][r];
  __syncthreads();
  for (int idx = threadIdx.x; idx < MT * 256; idx += NW * 64) {
    const int nn = idx & 15;  // channel inside the block
    const int m = idx >> 4;   // activation row
    const int n = nb * 16 + nn;
    if (m >= a.M || n >= N) continue;
    const int mt = m >> 4, r = nn & 3, ln = (nn >> 2) * 16 + (m & 15);
    float sum[NACC];
#pragma unroll
    for (int g = 0; g < NACC; ++g) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) t += red[(((w * NACC + g) * MT + mt) * 4 + r) * 64 + ln];
      sum[g] = Fmt::finish(t, sc[g]);
    }
    if (PAIR) {
      const f16 gate = (f16)sum[0];
      const f16 up = (f16)sum[1];
      a.mat[0].Y[(size_t)m * N + n] = swiglu_out(a.epi, gate, up);
    } else {
      f16 y0 = (f16)sum[0];
      if (a.mat[mi].bias) y0 = y0 + a.mat[mi].bias[n];
      y0 = apply_act(a.mat[mi].act, y0);
      a.mat[mi].Y[(size_t)m * N + n] = apply_epilogue(a.epi, y0, m, n, N);
    }
  }
}


// ------------------------------------------------------------------------------------------
// Variant for very small M (M <= 4): the activation rows are staged once per workgroup in LDS
// (M*K*2 bytes) and the B operand comes from LDS reads, which are broadcasts when M == 1.
// The first weight tile is requested before the staging so that HBM latency overlaps it.
// ------------------------------------------------------------------------------------------
template <class Fmt, int NW, bool PAIR>
__global__ __launch_bounds__(NW * 64) void gemv_lds_kernel(GemmArgs a) {
  constexpr int NACC = PAIR ? 2 : 1;
  constexpr int KV = Fmt::kVec;
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int mi = 0;
  if (!PAIR) {
#pragma unroll
    for (int i = 1; i < 4; ++i)
      if (i < a.count && (int)blockIdx.x >= a.mat[i].nb_begin) mi = i;
  }
  const int nb = blockIdx.x - a.mat[mi].nb_begin;
  const int N = a.mat[mi].N;
  const int row = nb * 16 + (lane & 15);
  const int K = a.K, KT = a.KT, M = a.M;
  const int xstride = KT * 128 + 8;                 // +8 halves: rows land in different banks
  f16* xs = reinterpret_cast<f16*>(smem);
  float* red = reinterpret_cast<float*>(smem + (((size_t)M * xstride * 2 + 15) & ~(size_t)15));

  typename Fmt::Scale sc[NACC];
  const u32x4* wp[NACC];
#pragma unroll
  for (int g = 0; g < NACC; ++g) {
    const GemmMat& m = a.mat[PAIR ? g : mi];
    sc[g] = Fmt::load_scale(m.scale, a.x_scale, row, N);
    wp[g] = reinterpret_cast<const u32x4*>(m.tiled) + (size_t)nb * KT * (64 * KV) + lane;
  }
  // first tile of this wave: requested before anything else
  u32x4 wcur[NACC][KV];
  int kt = wave;
  if (kt < KT) {
#pragma unroll
    for (int g = 0; g < NACC; ++g)
#pragma unroll
      for (int v = 0; v < KV; ++v) wcur[g][v] = __builtin_nontemporal_load(wp[g] + ((size_t)kt * KV + v) * 64);
  }
  // stage X (zero beyond K), normalising its rows on the way when a norm is fused
  {
    const int vec_per_row = KT * 16;               // 8-half vectors per padded row
    float ps[4] = {0.f, 0.f, 0.f, 0.f}, pq[4] = {0.f, 0.f, 0.f, 0.f};
    for (int i = threadIdx.x; i < M * vec_per_row; i += NW * 64) {
      const int m = i / vec_per_row, c = i % vec_per_row;
      f16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (c * 8 < K) v = *reinterpret_cast<const f16x8*>((a.mat[mi].X ? a.mat[mi].X : a.X) + (size_t)m * K + c * 8);
      *reinterpret_cast<f16x8*>(xs + (size_t)m * xstride + c * 8) = v;
      if (a.epi.norm != PTA_NORM_NONE) {
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float f = (float)v[e]; s1 += f; s2 = __builtin_fmaf(f, f, s2); }
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) if (mm == m) { ps[mm] += s1; pq[mm] += s2; }
      }
    }
    if (a.epi.norm != PTA_NORM_NONE) {
      // per-row sums over the workgroup: over the wave by data-parallel moves (a chain of six LDS-crossbar shuffles
      // per sum took longer than the norm launch this replaces), then LDS (the reduction buffer is free here)
#pragma unroll
      for (int mm = 0; mm < 4; ++mm)
        if (mm < M) { ps[mm] = wave_total_dpp(ps[mm]); pq[mm] = wave_total_dpp(pq[mm]); }
      if (lane == 0) {
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) { red[(wave * 4 + mm) * 2] = ps[mm]; red[(wave * 4 + mm) * 2 + 1] = pq[mm]; }
      }
      __syncthreads();
      const float inv_n = 1.0f / (float)K;
      for (int i = threadIdx.x; i < M * vec_per_row; i += NW * 64) {
        const int m = i / vec_per_row, c = i % vec_per_row;
        if (c * 8 >= K) continue;
        float sum = 0.f, sq = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) { sum += red[(w * 4 + m) * 2]; sq += red[(w * 4 + m) * 2 + 1]; }
        f16x8 v = *reinterpret_cast<f16x8*>(xs + (size_t)m * xstride + c * 8);
        const f16x8 gm = *reinterpret_cast<const f16x8*>(a.epi.norm_weight + c * 8);
        if (a.epi.norm == PTA_NORM_RMS) {
          const f16 r16 = (f16)(1.0f / sqrtf(sq * inv_n + a.epi.norm_eps));
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = (v[e] * r16) * gm[e];
        } else {
          const f16x8 bt = *reinterpret_cast<const f16x8*>(a.epi.norm_bias + c * 8);
          const float mean = sum * inv_n;
          const f16 mean16 = (f16)mean;
          float var;
          if (M == 1) var = sq * inv_n - mean * mean + a.epi.norm_eps;          // single-row NormCE
          else { const float mf = (float)mean16; var = fmaxf(sq * inv_n - mf * mf, 0.0f) + a.epi.norm_eps; }
          const f16 r16 = (f16)(1.0f / sqrtf(var));
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = ((v[e] - mean16) * r16) * gm[e] + bt[e];
        }
        *reinterpret_cast<f16x8*>(xs + (size_t)m * xstride + c * 8) = v;
      }
    }
    if (a.epi.mix_state) {
      // token shift: this matrix's input is x * w + (1 - w) * prev, each step an fp16 operation as in pta_rwkv_mix;
      // prev is the copy of the state that the previous token's launch wrote, x goes to the other one (first
      // workgroup) - no workgroup of this launch reads the copy that is written
      // (a thread mixes the vectors it staged and normalised itself: no barrier in between)
      const int parity = a.epi.mix_step[0] & 1;
      const f16* prev = a.epi.mix_state + (size_t)parity * M * K;
      f16* next = a.epi.mix_state + (size_t)(parity ^ 1) * M * K;
      const f16* mw = a.mat[mi].mix;
      const f16 one = (f16)1.0f;
      for (int i = threadIdx.x; i < M * vec_per_row; i += NW * 64) {
        const int m = i / vec_per_row, c = i % vec_per_row;
        if (c * 8 >= K) continue;
        f16x8 v = *reinterpret_cast<f16x8*>(xs + (size_t)m * xstride + c * 8);
        if (blockIdx.x == 0) *reinterpret_cast<f16x8*>(next + (size_t)m * K + c * 8) = v;
        if (mw) {
          const f16x8 pv = *reinterpret_cast<const f16x8*>(prev + (size_t)m * K + c * 8);
          const f16x8 wv = *reinterpret_cast<const f16x8*>(mw + c * 8);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = v[e] * wv[e] + (one - wv[e]) * pv[e];
          *reinterpret_cast<f16x8*>(xs + (size_t)m * xstride + c * 8) = v;
        }
      }
    }
  }
  __syncthreads();
  int mrow = lane & 15;
  mrow = mrow < M ? mrow : M - 1;
  const f16* xl = xs + (size_t)mrow * xstride + (lane >> 4) * 8;

  f32x4 acc[NACC];
#pragma unroll
  for (int g = 0; g < NACC; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};

  while (kt < KT) {
    const int ktn = kt + NW;
    u32x4 wnext[NACC][KV];
    if (ktn < KT) {
#pragma unroll
      for (int g = 0; g < NACC; ++g)
#pragma unroll
        for (int v = 0; v < KV; ++v) wnext[g][v] = __builtin_nontemporal_load(wp[g] + ((size_t)ktn * KV + v) * 64);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f16x8 xb = *reinterpret_cast<const f16x8*>(xl + kt * 128 + j * 32);
#pragma unroll
      for (int g = 0; g < NACC; ++g) {
        const f16x8 av = Fmt::a_operand(wcur[g], j, sc[g]);
        acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, xb, acc[g], 0, 0, 0);
      }
    }
    if (ktn < KT) {
#pragma unroll
      for (int g = 0; g < NACC; ++g)
#pragma unroll
        for (int v = 0; v < KV; ++v) wcur[g][v] = wnext[g][v];
    }
    kt = ktn;
  }

#pragma unroll
  for (int g = 0; g < NACC; ++g)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((wave * NACC + g) * 4 + r) * 64 + lane] = acc[g][r];
  __syncthreads();
  for (int idx = threadIdx.x; idx < 256; idx += NW * 64) {
    const int nn = idx & 15, m = idx >> 4;
    const int n = nb * 16 + nn;
    if (m >= M || n >= N) continue;
    const int r = nn & 3, ln = (nn >> 2) * 16 + m;
    float sum[NACC];
#pragma unroll
    for (int g = 0; g < NACC; ++g) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) t += red[((w * NACC + g) * 4 + r) * 64 + ln];
      sum[g] = Fmt::finish(t, sc[g]);
    }
    if (PAIR) {
      const f16 gate = (f16)sum[0];
      const f16 up = (f16)sum[1];
      a.mat[0].Y[(size_t)m * N + n] = swiglu_out(a.epi, gate, up);
    } else {
      f16 y0 = (f16)sum[0];
      if (a.mat[mi].bias) y0 = y0 + a.mat[mi].bias[n];
      y0 = apply_act(a.mat[mi].act, y0);
      a.mat[mi].Y[(size_t)m * N + n] = apply_epilogue(a.epi, y0, m, n, N);
    }
  }
}

// ------------------------------------------------------------------------------------------
// Variant for 4 < M <= 64 when all matrices of the launch share X: one workgroup of 16 waves per
// compute unit's worth of work.  A workgroup owns NB 16-channel blocks (blocks g, g + G, ... of
// the launch's G workgroups); wave w takes the feature tiles w, w + 16, ... of ALL of them, so the
// activation fragments of a tile (the B operands: 4 KiB per 16 rows, against 1 KiB of INT4
// weights) are read once and used NB times, and every wave has NB weight tiles per feature tile
// in flight.  MT = number of 16-row groups of X.
// ------------------------------------------------------------------------------------------
constexpr int WIDE_WAVES = 16;

template <class Fmt, int MT, int NB, bool PAIR, bool NORM = false>
__global__ __launch_bounds__(WIDE_WAVES * 64) void gemv_wide_kernel(GemmArgs a, int total_nb) {
  static_assert(!NORM || MT == 1, "the fused norm covers up to 16 rows");
  constexpr int NACC = PAIR ? 2 : 1;
  constexpr int KV = Fmt::kVec;
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);          // [WIDE_WAVES][NB][NACC][MT][256]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int G = gridDim.x;
  const int K = a.K, KT = a.KT;

  int mi[NB], nb[NB];
  typename Fmt::Scale sc[NB][NACC];
  const u32x4* wp[NB][NACC];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    int blk = blockIdx.x + b * G;
    blk = blk < total_nb ? blk : total_nb - 1;          // a duplicate whose results are not stored
    int m_ = 0;
    if (!PAIR) {
#pragma unroll
      for (int i = 1; i < 4; ++i)
        if (i < a.count && blk >= a.mat[i].nb_begin) m_ = i;
    }
    mi[b] = m_;
    nb[b] = blk - a.mat[m_].nb_begin;
    const int row = nb[b] * 16 + (lane & 15);
#pragma unroll
    for (int g = 0; g < NACC; ++g) {
      const GemmMat& m = a.mat[PAIR ? g : m_];
      sc[b][g] = Fmt::load_scale(m.scale, a.x_scale, row, m.N);
      wp[b][g] = reinterpret_cast<const u32x4*>(m.tiled) + (size_t)nb[b] * KT * (64 * KV) + lane;
    }
  }
  const f16* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int mrow = mt * 16 + (lane & 15);
    mrow = mrow < a.M ? mrow : a.M - 1;                 // padding rows compute values that are never stored
    xrow[mt] = a.X + (size_t)mrow * K + (lane >> 4) * 8;
  }

  f32x4 acc[NB][NACC][MT];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int g = 0; g < NACC; ++g)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[b][g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Fused norm (MT == 1): a first pass over this wave's activation fragments gives the row sums (lane l
  // holds row l % 16, features (l / 16) * 8 + 0..7 of every 32), they meet over the lane groups and, in
  // LDS, over the waves; the product pass then normalises every fragment it loads, with the numerics of
  // pta_rmsnorm / pta_layer_norm_ce (rows > 1 variant).
  f16 n_mean = (f16)0.0f, n_r = (f16)1.0f;
  auto norm_statistics = [&]() {
    float s1 = 0.f, s2 = 0.f;
    for (int kt = wave; kt < KT; kt += WIDE_WAVES)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = kt * 128 + j * 32;
        if (k + (lane >> 4) * 8 < K) {
          const f16x8 v = *reinterpret_cast<const f16x8*>(xrow[0] + k);
#pragma unroll
          for (int e = 0; e < 8; ++e) { const float f = (float)v[e]; s1 += f; s2 = __builtin_fmaf(f, f, s2); }
        }
      }
    s1 += __shfl_xor(s1, 16, 64); s2 += __shfl_xor(s2, 16, 64);
    s1 += __shfl_xor(s1, 32, 64); s2 += __shfl_xor(s2, 32, 64);
    if (lane < 16) { red[(wave * 16 + lane) * 2] = s1; red[(wave * 16 + lane) * 2 + 1] = s2; }
    __syncthreads();
    float sum = 0.f, sq = 0.f;
#pragma unroll
    for (int w = 0; w < WIDE_WAVES; ++w) { sum += red[(w * 16 + (lane & 15)) * 2]; sq += red[(w * 16 + (lane & 15)) * 2 + 1]; }
    __syncthreads();      // the buffer is reused for the partial sums of the product
    const float inv_n = 1.0f / (float)K;
    if (a.epi.norm == PTA_NORM_RMS) {
      n_r = (f16)(1.0f / sqrtf(sq * inv_n + a.epi.norm_eps));
    } else {
      const float mean = sum * inv_n;
      n_mean = (f16)mean;
      float var;
      if (a.M == 1) var = sq * inv_n - mean * mean + a.epi.norm_eps;          // single-row NormCE
      else { const float mf = (float)n_mean; var = fmaxf(sq * inv_n - mf * mf, 0.0f) + a.epi.norm_eps; }
      n_r = (f16)(1.0f / sqrtf(var));
    }
  };
  if constexpr (MT == 1) {
    // UN feature tiles per step, all of their loads requested before the first product (a tile
    // beyond KT repeats the last one with zero activations)
    constexpr int UN = NB * NACC * KV <= 4 ? 2 : 1;
    u32x4 w[UN][NB][NACC][KV];
    f16x8 xb[UN][4];
    auto load_w = [&](int kt0) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int kt_ = kt0 + u * WIDE_WAVES;
        const int kt = kt_ < KT ? kt_ : KT - 1;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
          for (int g = 0; g < NACC; ++g)
#pragma unroll
            for (int v = 0; v < KV; ++v)
              w[u][b][g][v] = __builtin_nontemporal_load(wp[b][g] + ((size_t)kt * KV + v) * 64);
      }
    };
    auto load_x = [&](int kt0) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int kt_ = kt0 + u * WIDE_WAVES;
        const bool there = kt_ < KT;
        const int kt = there ? kt_ : KT - 1;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int k = kt * 128 + j * 32;
          const f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
          const bool in = there && k + (lane >> 4) * 8 < K;
          xb[u][j] = in ? *reinterpret_cast<const f16x8*>(xrow[0] + k) : z;
          if (NORM && in) {
            const f16x8 gm = *reinterpret_cast<const f16x8*>(a.epi.norm_weight + k + (lane >> 4) * 8);
            if (a.epi.norm == PTA_NORM_RMS) {
#pragma unroll
              for (int e = 0; e < 8; ++e) xb[u][j][e] = (xb[u][j][e] * n_r) * gm[e];
            } else {
              const f16x8 bt = *reinterpret_cast<const f16x8*>(a.epi.norm_bias + k + (lane >> 4) * 8);
#pragma unroll
              for (int e = 0; e < 8; ++e) xb[u][j][e] = ((xb[u][j][e] - n_mean) * n_r) * gm[e] + bt[e];
            }
          }
        }
      }
    };
    auto products = [&]() {
#pragma unroll
      for (int u = 0; u < UN; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int g = 0; g < NACC; ++g)
              acc[b][g][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Fmt::a_operand(w[u][b][g], j, sc[b][g]), xb[u][j],
                                                                    acc[b][g][0], 0, 0, 0);
    };
    int kt0 = wave;
    if constexpr (NORM) {
      // Fused norm: the first weight tiles are requested before the pass over the activations that gives the
      // row statistics (lane l holds row l % 16, features (l / 16) * 8 + 0..7 of every 32; the sums meet over
      // the lane groups and, in LDS, over the waves), so that pass runs while they are on their way.  The
      // product pass then normalises every fragment it loads, with the numerics of pta_rmsnorm /
      // pta_layer_norm_ce (rows > 1 variant).
      if (kt0 < KT) load_w(kt0);
      norm_statistics();
      if (kt0 < KT) {
        load_x(kt0);
        products();
        kt0 += WIDE_WAVES * UN;
      }
    }
    for (; kt0 < KT; kt0 += WIDE_WAVES * UN) {
      load_w(kt0);
      load_x(kt0);
      products();
    }
  } else {
    // several row groups: the activation fragments of one 32-feature slice at a time (16 bytes per
    // lane and row group), each used for all blocks before the next slice is read
    for (int kt = wave; kt < KT; kt += WIDE_WAVES) {
      u32x4 w[NB][NACC][KV];
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g = 0; g < NACC; ++g)
#pragma unroll
          for (int v = 0; v < KV; ++v) w[b][g][v] = __builtin_nontemporal_load(wp[b][g] + ((size_t)kt * KV + v) * 64);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = kt * 128 + j * 32;
        const f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        f16x8 xb[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          xb[mt] = k + (lane >> 4) * 8 < K ? *reinterpret_cast<const f16x8*>(xrow[mt] + k) : z;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
          for (int g = 0; g < NACC; ++g) {
            const f16x8 av = Fmt::a_operand(w[b][g], j, sc[b][g]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[b][g][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, xb[mt], acc[b][g][mt], 0, 0, 0);
          }
      }
    }
  }

  // The accumulator of lane l holds channels (l/16)*4 + r, r = 0..3, for activation row l%16 of its group.
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int g = 0; g < NACC; ++g)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          red[((((wave * NB + b) * NACC + g) * MT + mt) * 4 + r) * 64 + lane] = acc[b][g][mt][r];
  __syncthreads();
  // The 256 outputs (16 rows x 16 channels) of (block b, row group mt) are finished by the quarter
  // (b * MT + mt) % 4 of the workgroup, thread t of it taking row (t / 16) % 16, channel t % 16.
  const int quarter = threadIdx.x >> 8;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (((b * MT + mt) & 3) != quarter) continue;
      const int nn = threadIdx.x & 15, m = mt * 16 + ((threadIdx.x >> 4) & 15);
      const GemmMat& mat = a.mat[PAIR ? 0 : mi[b]];
      const int N = mat.N, n = nb[b] * 16 + nn;
      if ((int)blockIdx.x + b * G >= total_nb || m >= a.M || n >= N) continue;
      const int r = nn & 3, ln = (nn >> 2) * 16 + (m & 15);
      float sum[NACC];
#pragma unroll
      for (int g = 0; g < NACC; ++g) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < WIDE_WAVES; ++w) t += red[((((w * NB + b) * NACC + g) * MT + mt) * 4 + r) * 64 + ln];
        sum[g] = Fmt::finish(t, sc[b][g]);      // no format's finish uses the per-channel part of the scale
      }
      if (PAIR) {
        const f16 gate = (f16)sum[0];
        const f16 up = (f16)sum[1];
        mat.Y[(size_t)m * N + n] = swiglu_out(a.epi, gate, up);
      } else {
        f16 y0 = (f16)sum[0];
        if (mat.bias) y0 = y0 + mat.bias[n];
        y0 = apply_act(mat.act, y0);
        mat.Y[(size_t)m * N + n] = apply_epilogue(a.epi, y0, m, n, N);
      }
    }
  }
}

template <class Fmt, int MT, int NB, bool PAIR, bool NORM = false>
static int launch_gemv_wide(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  static bool ready = false;
  const size_t smem = (size_t)WIDE_WAVES * NB * (PAIR ? 2 : 1) * MT * 256 * sizeof(float);
  static_assert(WIDE_WAVES * NB * (PAIR ? 2 : 1) * MT * 1024 <= 128 * 1024, "reduction buffer beyond 128 KiB of LDS");
  if (!ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)gemv_wide_kernel<Fmt, MT, NB, PAIR, NORM>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess,
                "%s: cannot reserve %zu bytes of LDS", name, smem);
    ready = true;
  }
  hipLaunchKernelGGL((gemv_wide_kernel<Fmt, MT, NB, PAIR, NORM>), dim3((total_nb + NB - 1) / NB), dim3(WIDE_WAVES * 64), smem, s,
                     a, total_nb);
  return PTA_OK;
}

// blocks per workgroup: the launch's share per compute unit, capped by what the registers of a wave
// (weight tiles in flight) and the LDS reduction buffer (8 KiB-groups of partial sums) hold
// the longest chain of channel blocks a compute unit multiplies under launch_gemv_wide_for (M <= 16)
template <class Fmt, bool PAIR>
static int wide_block_times(int total_nb, int per_cu);

template <class Fmt, int MT, bool PAIR, bool NORM = false>
static int launch_gemv_wide_for(const GemmArgs& a, int total_nb, int per_cu, hipStream_t s, const char* name) {
  constexpr int NACC = PAIR ? 2 : 1;
  constexpr int cap_regs = Fmt::kVec * NACC <= 4 ? 3 : 2;
  constexpr int cap_lds = 8 / (NACC * MT) >= 1 ? 8 / (NACC * MT) : 1;
  constexpr int cap = cap_regs < cap_lds ? cap_regs : cap_lds;
  if (per_cu <= 1 || cap == 1) return launch_gemv_wide<Fmt, MT, 1, PAIR, NORM>(a, total_nb, s, name);
  if (per_cu == 2 || cap == 2) return launch_gemv_wide<Fmt, MT, cap >= 2 ? 2 : 1, PAIR, NORM>(a, total_nb, s, name);
  return launch_gemv_wide<Fmt, MT, cap >= 3 ? 3 : 1, PAIR, NORM>(a, total_nb, s, name);
}

template <class Fmt, bool PAIR>
static int wide_block_times(int total_nb, int per_cu) {
  constexpr int NACC = PAIR ? 2 : 1;
  constexpr int cap_regs = Fmt::kVec * NACC <= 4 ? 3 : 2;
  constexpr int cap_lds = 8 / NACC;
  constexpr int cap = cap_regs < cap_lds ? cap_regs : cap_lds;
  const int nb = per_cu < cap ? per_cu : cap;
  const int cus = device_compute_units();
  const int wgs = (total_nb + nb - 1) / nb;
  return (wgs + cus - 1) / cus * nb;
}

// ------------------------------------------------------------------------------------------
// Variant for up to 16 rows, one shared X, K <= 4096 and several channel blocks per compute unit: one workgroup
// of 8 waves per compute unit walks a contiguous range of the launch's 16-channel blocks.  Wave w takes the
// feature tiles w, w + 8, ... of every block, U at a time (a step; a block is up to 4 / U steps long).  The
// weights of the next D - 1 steps are on their way while those of the current one are multiplied, across block
// boundaries as well, so the stream does not pause for a reduction or for a change of workgroups; the partial
// sums of a block meet in LDS (two buffers in turn, one barrier per block) and 256 threads finish its 16 x 16
// outputs while the others go on.  The activation fragments of a wave's tiles are the same for every block
// and stay in registers (x[p]: those of a block's step p).
// ------------------------------------------------------------------------------------------
constexpr int STREAM_WAVES = 8;
constexpr int STREAM_TILES = 4;          // feature tiles of a block per wave, at most: K <= 8 * 4 * 128

template <class Fmt, int U, int D, bool PAIR>
__global__ __launch_bounds__(STREAM_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemv_stream_kernel(GemmArgs a, int total_nb) {
  constexpr int XP = STREAM_TILES / U;     // steps of a block, at most
  static_assert(D % XP == 0, "a step's place in the ring of weight sets tells its place in the block");
  constexpr int NACC = PAIR ? 2 : 1;
  constexpr int KV = Fmt::kVec;
  __shared__ float red[2][STREAM_WAVES][NACC][256];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int K = a.K, KT = a.KT;
  const int G = gridDim.x;
  const int b0 = (int)((long)total_nb * blockIdx.x / G), b1 = (int)((long)total_nb * (blockIdx.x + 1) / G);
  // steps per block: 1, 2 or 4 (a divisor of the ring's length; a step past the end of K multiplies zeros)
  const int spb = KT <= STREAM_WAVES * U ? 1 : KT <= 2 * STREAM_WAVES * U ? 2 : XP;
  const int steps = (b1 - b0) * spb;
  if (steps == 0) return;

  struct Set {
    u32x4 w[U][NACC][KV];
    typename Fmt::Scale sc[NACC];
    uint16_t e[4];      // epilogue operands of the output this thread finishes: the matrix's bias, then bias, mul, residual
  };
  Set ring[D];
  typename Fmt::Scale sc[NACC];
  f32x4 acc[NACC];
#pragma unroll
  for (int g = 0; g < NACC; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto matrix_of = [&](int blk) {
    int m_ = 0;
    if (!PAIR) {
#pragma unroll
      for (int i = 1; i < 4; ++i)
        if (i < a.count && blk >= a.mat[i].nb_begin) m_ = i;
    }
    return m_;
  };

  // The requesting side runs D - 1 steps ahead of the multiplying side.  Every step issues the same loads whatever
  // the data (a wait for one set of weights then counts the loads issued after it): they go through a buffer
  // descriptor of the block's matrix, and a tile past the end of K, or a step past the end of the workgroup's
  // range, is given an offset beyond the descriptor's range - it reads as zero and touches no memory.
  const uint32_t blk_bytes = (uint32_t)KT * (KV * 1024);
  int fb = b0, fs = 0;
  auto fetch = [&](Set& st, bool live) {
    const int m_ = matrix_of(fb);
    const int nb = fb - a.mat[m_].nb_begin;
#pragma unroll
    for (int g = 0; g < NACC; ++g) {
      const GemmMat& m = a.mat[PAIR ? g : m_];
      const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<void*>(m.tiled), 0, (int)((uint32_t)((m.N + 15) / 16) * blk_bytes), 0x00020000);
      st.sc[g] = Fmt::load_scale(m.scale, a.x_scale, nb * 16 + (lane & 15), m.N);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kt = (fs * U + u) * STREAM_WAVES + wave;
        const int voff = live && kt < KT ? lane * 16 : -1;
#pragma unroll
        for (int v = 0; v < KV; ++v)
          st.w[u][g][v] = __builtin_amdgcn_raw_buffer_load_b128(wr, voff, (int)((uint32_t)nb * blk_bytes + (uint32_t)(kt * KV + v) * 1024), 2);
      }
    }
    if constexpr (!PAIR) {
      // The operands of the epilogue travel with the weights of the block's last step: a load issued when the block
      // is finished would wait for every set of weights requested before it.  Absent operands have an empty range.
      const GemmMat& mat = a.mat[m_];
      const int nn = threadIdx.x & 15, m = threadIdx.x >> 4, n = nb * 16 + nn;
      const bool mine = live && fs == spb - 1 && threadIdx.x < 256 && m < a.M && n < mat.N;
      const f16* ptr[4] = {mat.bias, a.epi.bias, a.epi.mul, a.epi.residual};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<f16*>(ptr[i]), 0, ptr[i] ? (i < 2 ? mat.N : a.M * mat.N) * 2 : 0, 0x00020000);
        st.e[i] = __builtin_amdgcn_raw_buffer_load_b16(r, mine ? (i < 2 ? n : m * mat.N + n) * 2 : -1, 0, 0);
      }
    }
    if (++fs == spb) { fs = 0; ++fb; }
  };

  // B operands: row lane % 16 of X (clamped: padding rows compute values that are never stored), features
  // (lane / 16) * 8 + 0..7 of every 32; x[p] holds them for the tiles of a block's step p (of its only step, when
  // a block is one step long).  Requested before the first weights: loads return in the order of their issue, and
  // the first products need these and one set of weights only.
  f16x8 x[XP][U][4];
  {
    int mrow = lane & 15;
    mrow = mrow < a.M ? mrow : a.M - 1;
    const f16* xrow = a.X + (size_t)mrow * K + (lane >> 4) * 8;
#pragma unroll
    for (int p = 0; p < XP; ++p)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int kt = ((p % spb) * U + u) * STREAM_WAVES + wave;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int k = kt * 128 + j * 32;
          const f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
          x[p][u][j] = kt < KT && k + (lane >> 4) * 8 < K ? *reinterpret_cast<const f16x8*>(xrow + k) : z;
        }
      }
  }

#pragma unroll
  for (int i = 0; i < D - 1; ++i) fetch(ring[i], i < steps);

  int cb = b0, cs = 0, par = 0;
  auto multiply = [&](Set& st, const f16x8 (&xs)[U][4]) {
    if (cs == 0) {
#pragma unroll
      for (int g = 0; g < NACC; ++g) sc[g] = st.sc[g];
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int g = 0; g < NACC; ++g)
          acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Fmt::a_operand(st.w[u][g], j, sc[g]), xs[u][j], acc[g], 0, 0, 0);
    if (++cs < spb) return;
    // the block is complete: lane l holds channels (l/16)*4 + r, r = 0..3, for activation row l%16
#pragma unroll
    for (int g = 0; g < NACC; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        red[par][wave][g][r * 64 + lane] = acc[g][r];
        acc[g][r] = 0.f;
      }
    __syncthreads();
    if (threadIdx.x < 256) {
      const int m_ = matrix_of(cb);
      const GemmMat& mat = a.mat[PAIR ? 0 : m_];
      const int nn = threadIdx.x & 15, m = threadIdx.x >> 4;
      const int N = mat.N, n = (cb - a.mat[m_].nb_begin) * 16 + nn;
      if (m < a.M && n < N) {
        const int r = nn & 3, ln = (nn >> 2) * 16 + m;
        float sum[NACC];
#pragma unroll
        for (int g = 0; g < NACC; ++g) {
          float t = 0.f;
#pragma unroll
          for (int w = 0; w < STREAM_WAVES; ++w) t += red[par][w][g][r * 64 + ln];
          sum[g] = Fmt::finish(t, sc[g]);        // no format's finish uses the per-channel part of the scale
        }
        if (PAIR) {
          mat.Y[(size_t)m * N + n] = swiglu_out(a.epi, (f16)sum[0], (f16)sum[1]);
        } else {
          // as apply_epilogue, with the operands that came with the weights
          f16 y0 = (f16)sum[0];
          if (mat.bias) y0 = y0 + bitcast<f16>(st.e[0]);
          y0 = apply_act(mat.act, y0);
          if (a.epi.bias) y0 = y0 + bitcast<f16>(st.e[1]);
          y0 = apply_act(a.epi.act, y0);
          if (a.epi.mul) y0 = y0 * bitcast<f16>(st.e[2]);
          if (a.epi.residual) y0 = y0 + bitcast<f16>(st.e[3]);
          if (a.epi.post_scale != 0.0f) y0 = y0 * (f16)a.epi.post_scale;
          if (a.epi.out_fp8_scale) y0 = f8_grid_value(y0, a.epi.out_fp8_scale[0], a.epi.out_fp8_format);
          mat.Y[(size_t)m * N + n] = y0;
        }
      }
    }
    par ^= 1;
    cs = 0;
    ++cb;
  };

  int t = 0;
  for (; t + D <= steps; t += D) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      fetch(ring[(i + D - 1) % D], t + i + D - 1 < steps);
      multiply(ring[i], x[i % XP]);
    }
  }
  // fewer than D steps are left and their weights are on their way
#pragma unroll
  for (int i = 0; i < D - 1; ++i)
    if (t + i < steps) multiply(ring[i], x[i % XP]);
}

// the shapes the streaming kernel takes
static inline bool stream_fits(const GemmArgs& a) {
  if (a.M > 16 || a.KT < 8 || a.KT > STREAM_WAVES * STREAM_TILES || a.epi.norm != PTA_NORM_NONE) return false;
  for (int i = 0; i < a.count; ++i) {
    if (a.mat[i].X) return false;
    // a matrix's tiles sit behind one buffer descriptor (32-bit range and offsets; four vectors per tile at most)
    if ((size_t)((a.mat[i].N + 15) / 16) * (size_t)a.KT * 4096 > 0x7fffffffu) return false;
  }
  return true;
}

template <class Fmt, bool PAIR>
static int launch_gemv_stream(const GemmArgs& a, int total_nb, int cus, hipStream_t s, const char* name) {
  // tiles per step, and four steps in the ring: 96 KiB on their way per compute unit, a ring of 64 registers
  constexpr int V = Fmt::kVec * (PAIR ? 2 : 1);
  constexpr int U = V >= 4 ? 1 : V >= 2 ? 2 : 4, D = 4;
  hipLaunchKernelGGL((gemv_stream_kernel<Fmt, U, D, PAIR>), dim3(total_nb < cus ? total_nb : cus), dim3(STREAM_WAVES * 64), 0, s, a,
                     total_nb);
  return PTA_OK;
}

// ------------------------------------------------------------------------------------------
// Variant for 16 < M <= 64: the activation rows of a feature tile are staged in LDS once per
// workgroup and shared by its waves, so that the B operands (4 KiB per 16 rows and tile, against
// 1 KiB of INT4 weights) come from LDS and not from the L2.
// A workgroup of 8 waves owns 2 * (8 / KQ) weight streams of 16 channels (consecutive channel blocks
// of one matrix; or, for a SwiGLU pair, the gate and the up weights of 8 / KQ channel blocks) and
// all rows; its waves form KQ groups that take the feature tiles g, g + KQ, ... each; a wave
// multiplies two streams, so every B fragment it reads from LDS feeds two MFMAs.  The X tiles of
// step i + 1 are fetched (global -> registers -> LDS, double-buffered) while step i is multiplied,
// and so are the weight tiles.  The partial sums of the KQ groups meet in LDS (the staging area).
// ------------------------------------------------------------------------------------------
constexpr int TILE_WAVES = 8;
constexpr int TILE_XSTRIDE = 128 + 8;      // halves per staged row: 16 consecutive rows hit 16 different bank groups

template <class Fmt, int MT, int KQ, bool PAIR, int NWV = TILE_WAVES>
__global__ __launch_bounds__(NWV * 64) void gemm_tile_kernel(GemmArgs a) {
  constexpr int KV = Fmt::kVec;
  constexpr int WPG = NWV / KQ;          // waves per K group
  constexpr int ROWS = MT * 16;
  constexpr int XBUF = ROWS * TILE_XSTRIDE;     // halves of one staged tile
  constexpr int VPT = ROWS * 16 / (WPG * 64);   // 16-byte vectors of a tile per thread of its group
  static_assert(VPT >= 1 && ROWS * 16 % (WPG * 64) == 0, "staging must divide evenly");
  extern __shared__ __align__(16) unsigned char smem[];
  f16* xs = reinterpret_cast<f16*>(smem);       // [KQ][2][ROWS][TILE_XSTRIDE]
  float* red = reinterpret_cast<float*>(smem);  // after the product: [NWV][2][MT][256]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kq = wave / WPG, wg_ = wave % WPG;  // K group, wave within the group
  const int tig = wg_ * 64 + lane;              // thread index within the group
  const int K = a.K, M = a.M;
  // feature tiles of this workgroup: all of them, or slice blockIdx.y of a K split
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  const int per_slice = (a.KT + nsl - 1) / nsl;
  const int kt_first = (int)blockIdx.y * per_slice;
  const int KT = kt_first + per_slice < a.KT ? kt_first + per_slice : a.KT;     // end of the slice

  // the two weight streams of this wave
  int mi = 0;
  const int first_blk = PAIR ? (int)blockIdx.x * WPG : (int)blockIdx.x * 2 * WPG;
  if (!PAIR) {
#pragma unroll
    for (int i = 1; i < 4; ++i)
      if (i < a.count && first_blk >= a.mat[i].nb_begin) mi = i;
  }
  int nb[2];
  typename Fmt::Scale sc[2];
  const u32x4* wp[2];
#pragma unroll
  for (int st = 0; st < 2; ++st) {
    const GemmMat& m = a.mat[PAIR ? st : mi];
    nb[st] = PAIR ? first_blk + wg_ : first_blk - m.nb_begin + 2 * wg_ + st;
    sc[st] = Fmt::load_scale(m.scale, a.x_scale, nb[st] * 16 + (lane & 15), m.N);
    wp[st] = reinterpret_cast<const u32x4*>(m.tiled) + (size_t)nb[st] * a.KT * (64 * KV) + lane;
  }
  const f16* X = a.mat[mi].X ? a.mat[mi].X : a.X;

  f32x4 acc[2][MT];
#pragma unroll
  for (int st = 0; st < 2; ++st)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[st][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // thread tig of a group stages vectors tig, tig + WPG*64, ... of the tile: vector v = row * 16 + c
  auto fetch_x = [&](int kt, u32x4 (&xv)[VPT]) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = tig + i * WPG * 64;
      const int row = v >> 4, c = v & 15;
      const int k = kt * 128 + c * 8;
      xv[i] = (row < M && k < K && kt < KT) ? *reinterpret_cast<const u32x4*>(X + (size_t)row * K + k) : u32x4{0, 0, 0, 0};
    }
  };
  auto store_x = [&](f16* buf, const u32x4 (&xv)[VPT]) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = tig + i * WPG * 64;
      *reinterpret_cast<u32x4*>(buf + (v >> 4) * TILE_XSTRIDE + (v & 15) * 8) = xv[i];
    }
  };
  auto fetch_w = [&](int kt, u32x4 (&w)[2][KV]) {
    const int ktc = kt < KT ? kt : KT - 1;
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int v = 0; v < KV; ++v) w[st][v] = __builtin_nontemporal_load(wp[st] + ((size_t)ktc * KV + v) * 64);
  };

  f16* xbuf = xs + (size_t)kq * 2 * XBUF;
  const int steps = (KT - kt_first + KQ - 1) / KQ;
  u32x4 w_cur[2][KV], w_nxt[2][KV], xv[VPT];
  fetch_w(kt_first + kq, w_cur);
  fetch_x(kt_first + kq, xv);
  store_x(xbuf, xv);
  __syncthreads();
  for (int i = 0; i < steps; ++i) {
    const int kt = kt_first + kq + i * KQ, ktn = kt + KQ;
    const bool more = i + 1 < steps;
    if (more) { fetch_w(ktn, w_nxt); fetch_x(ktn, xv); }
    const f16* cur = xbuf + (i & 1) * XBUF + (lane & 15) * TILE_XSTRIDE + (lane >> 4) * 8;
    if (kt < KT) {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        if constexpr (MT <= 4) {
          f16x8 xb[MT];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) xb[mt] = *reinterpret_cast<const f16x8*>(cur + mt * 16 * TILE_XSTRIDE + m * 32);
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            const f16x8 av = Fmt::a_operand(w_cur[st], m, sc[st]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[st][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, xb[mt], acc[st][mt], 0, 0, 0);
          }
        } else {
          // many row groups: both weight fragments decoded once, then one activation fragment at a time feeds both
          const f16x8 av0 = Fmt::a_operand(w_cur[0], m, sc[0]), av1 = Fmt::a_operand(w_cur[1], m, sc[1]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const f16x8 xb = *reinterpret_cast<const f16x8*>(cur + mt * 16 * TILE_XSTRIDE + m * 32);
            acc[0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av0, xb, acc[0][mt], 0, 0, 0);
            acc[1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av1, xb, acc[1][mt], 0, 0, 0);
          }
        }
      }
    }
    if (more) {
      store_x(xbuf + ((i + 1) & 1) * XBUF, xv);
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int v = 0; v < KV; ++v) w_cur[st][v] = w_nxt[st][v];
    }
    __syncthreads();
  }

  if constexpr (KQ == 1) {
    // one K group: every wave holds finished sums.  Lane l has channels (l / 16) * 4 + r, r = 0..3, of row l % 16 of
    // each row group, for both of its streams.
    const GemmMat& mat = a.mat[PAIR ? 0 : mi];
    const int N = mat.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + (lane & 15);
      if (m >= M) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (PAIR) {
          const int n = nb[0] * 16 + (lane >> 4) * 4 + r;
          if (n >= N) continue;
          const f16 gate = (f16)Fmt::finish(acc[0][mt][r], sc[0]), up = (f16)Fmt::finish(acc[1][mt][r], sc[1]);
          mat.Y[(size_t)m * N + n] = swiglu_out(a.epi, gate, up);
        } else {
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            const int n = nb[st] * 16 + (lane >> 4) * 4 + r;
            if (n >= N) continue;
            if (nsl > 1) { a.part[((size_t)blockIdx.y * M + m) * N + n] = acc[st][mt][r]; continue; }
            f16 y0 = (f16)Fmt::finish(acc[st][mt][r], sc[st]);
            if (mat.bias) y0 = y0 + mat.bias[n];
            y0 = apply_act(mat.act, y0);
            mat.Y[(size_t)m * N + n] = apply_epilogue(a.epi, y0, m, n, N);
          }
        }
      }
    }
    return;
  }
  // partial sums of the K groups meet in LDS (the staging area is free after the last barrier)
#pragma unroll
  for (int st = 0; st < 2; ++st)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(((wave * 2 + st) * MT + mt) * 4 + r) * 64 + lane] = acc[st][mt][r];
  __syncthreads();
  // outputs of the workgroup: WPG wave slots x 2 streams x MT row groups x 256; PAIR: one output per stream pair
  constexpr int OUTS = WPG * (PAIR ? 1 : 2) * MT * 256;
  for (int o = threadIdx.x; o < OUTS; o += NWV * 64) {
    const int nn = o & 15, m16 = (o >> 4) & 15;
    int rest = o >> 8;
    const int mt = rest % MT; rest /= MT;
    const int st = PAIR ? 0 : rest & 1;
    const int wslot = PAIR ? rest : rest >> 1;
    const int m = mt * 16 + m16;
    const GemmMat& mat = a.mat[PAIR ? 0 : mi];
    const int N = mat.N;
    const int blk = PAIR ? first_blk + wslot : first_blk - mat.nb_begin + 2 * wslot + st;
    const int n = blk * 16 + nn;
    if (m >= M || n >= N) continue;
    const int r = nn & 3, ln = (nn >> 2) * 16 + m16;
    float sum[2] = {0.f, 0.f};
#pragma unroll
    for (int g = 0; g < (PAIR ? 2 : 1); ++g) {
      float t = 0.f;
#pragma unroll
      for (int q = 0; q < KQ; ++q) t += red[((((q * WPG + wslot) * 2 + (PAIR ? g : st)) * MT + mt) * 4 + r) * 64 + ln];
      sum[g] = t;
    }
    if (!PAIR && nsl > 1) {                // a slice of a K split: the raw fp32 sum; the finishing kernel does the rest
      a.part[((size_t)blockIdx.y * M + m) * N + n] = sum[0];
      continue;
    }
#pragma unroll
    for (int g = 0; g < (PAIR ? 2 : 1); ++g) sum[g] = Fmt::finish(sum[g], sc[0]);   // no format's finish uses the per-channel part
    if (PAIR) {
      const f16 gate = (f16)sum[0];
      const f16 up = (f16)sum[1];
      mat.Y[(size_t)m * N + n] = swiglu_out(a.epi, gate, up);
    } else {
      f16 y0 = (f16)sum[0];
      if (mat.bias) y0 = y0 + mat.bias[n];
      y0 = apply_act(mat.act, y0);
      mat.Y[(size_t)m * N + n] = apply_epilogue(a.epi, y0, m, n, N);
    }
  }
}

// Second half of a K split: adds the slices' fp32 sums of one matrix and applies what the one-kernel form
// applies to its sum (the format's scale, bias, activation, epilogue).
template <class Fmt>
__global__ __launch_bounds__(256) void splitk_finish_kernel(GemmArgs a) {
  const GemmMat& mat = a.mat[0];
  const int N = mat.N;
  const size_t total = (size_t)a.M * N;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int m = (int)(i / N), n = (int)(i % N);
  float t = 0.f;
  for (int sl = 0; sl < a.ksplit; ++sl) t += a.part[(size_t)sl * total + i];
  f16 y0 = (f16)Fmt::finish(t, Fmt::load_scale(mat.scale, a.x_scale, n, N));
  if (mat.bias) y0 = y0 + mat.bias[n];
  y0 = apply_act(mat.act, y0);
  mat.Y[i] = apply_epilogue(a.epi, y0, m, n, N);
}

template <class Fmt, int MT, int KQ, bool PAIR, int NWV = TILE_WAVES>
static int launch_gemm_tile(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  static bool ready = false;
  constexpr int WPG = NWV / KQ;
  const size_t stage = (size_t)KQ * 2 * MT * 16 * TILE_XSTRIDE * 2;
  const size_t redb = KQ == 1 ? 0 : (size_t)NWV * 2 * MT * 256 * 4;      // one K group: no meeting in LDS
  const size_t smem = stage > redb ? stage : redb;
  static_assert((size_t)KQ * 2 * MT * 16 * TILE_XSTRIDE * 2 <= 160 * 1024, "staging beyond the LDS of a compute unit");
  if (!ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)gemm_tile_kernel<Fmt, MT, KQ, PAIR, NWV>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess,
                "%s: cannot reserve %zu bytes of LDS", name, smem);
    ready = true;
  }
  const int per_wg = PAIR ? WPG : 2 * WPG;
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  hipLaunchKernelGGL((gemm_tile_kernel<Fmt, MT, KQ, PAIR, NWV>), dim3(total_nb / per_wg, nsl), dim3(NWV * 64), smem, s, a);
  if (nsl > 1) {
    const size_t total = (size_t)a.M * a.mat[0].N;
    hipLaunchKernelGGL(splitk_finish_kernel<Fmt>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a);
  }
  return PTA_OK;
}

// ------------------------------------------------------------------------------------------
// Variant for many rows (prompt passes): the activation fragments live in registers, the weights go through
// LDS decoded.  A workgroup of 8 waves owns 8 weight streams of 16 channels (8 channel blocks of one matrix,
// or the gate and up weights of 4 blocks) and 8 * RG * 16 rows.  Per 128-feature tile, wave w
//   - fetches the tile of stream w, decodes it ONCE into the four fp16 A operands of its MFMA steps and puts
//     them into LDS (double-buffered, one barrier per tile) - every weight is decoded once per workgroup, not
//     once per wave and row group: with the decode in the product loop a wave spends 13 VALU instructions per
//     step for RG MFMAs and the kernel is bound by those (measured: 262 TFLOP/s at 256 rows);
//   - holds the B operands of ITS RG row groups in registers (fetched with whole-row loads, turned into
//     fragment order through a strip of LDS of its own) and multiplies them with every stream's operands.
// ------------------------------------------------------------------------------------------
constexpr int ROWS_WAVES = 8;
constexpr int ROWS_CB = 8;                  // streams per workgroup: one per wave
constexpr int ROWS_XSTRIDE = 128 + 8;
constexpr int ROWS_AVEC = ROWS_CB * 4 * 64; // A operands (16 bytes each) of one feature tile: [stream][step][lane]

// (two waves per SIMD: the whole register file of 256 per lane is this kernel's to use)
template <class Fmt, int RG, bool PAIR>
__global__ __launch_bounds__(ROWS_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_rows_kernel(GemmArgs a, int groups, int row_blocks) {
  constexpr int KV = Fmt::kVec;
  constexpr int XROWS = RG * 16;
  static_assert(ROWS_CB == ROWS_WAVES, "wave w decodes stream w");
  extern __shared__ __align__(16) unsigned char smem[];
  f16x8* abuf = reinterpret_cast<f16x8*>(smem);                                          // [2][ROWS_AVEC]
  f16* xbuf = reinterpret_cast<f16*>(smem + (size_t)2 * ROWS_AVEC * 16);                 // [waves][XROWS][ROWS_XSTRIDE]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int K = a.K, M = a.M;
  // Workgroups are dealt to the eight XCDs (each with an L2 of its own) in turn: workgroup id of the launch takes
  // tile (id % 8) * per + id / 8 of the list (row block, channel group), row block slowest - so an XCD works through
  // a contiguous stretch of the list, i.e. on one row block at a time, whose activations stay in its L2.
  const int per = (int)gridDim.x / 8;
  const int tile = ((int)blockIdx.x % 8) * per + (int)blockIdx.x / 8;
  if (tile >= groups * row_blocks) return;
  const int group = tile % groups, row_block = tile / groups;
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  const int per_slice = (a.KT + nsl - 1) / nsl;
  const int kt_first = (int)blockIdx.y * per_slice;
  const int kt_end = kt_first + per_slice < a.KT ? kt_first + per_slice : a.KT;
  const int steps = kt_end - kt_first;

  int mi = 0;
  const int first_blk = group * (PAIR ? ROWS_CB / 2 : ROWS_CB);
  if (!PAIR) {
#pragma unroll
    for (int i = 1; i < 4; ++i)
      if (i < a.count && first_blk >= a.mat[i].nb_begin) mi = i;
  }
  // stream st: its matrix and channel block
  auto stream_mat = [&](int st) -> const GemmMat& { return a.mat[PAIR ? (st < ROWS_CB / 2 ? 0 : 1) : mi]; };
  auto stream_blk = [&](int st) { return PAIR ? first_blk + st % (ROWS_CB / 2) : first_blk - a.mat[mi].nb_begin + st; };
  const GemmMat& own = stream_mat(wave);
  const typename Fmt::Scale own_sc = Fmt::load_scale(own.scale, a.x_scale, stream_blk(wave) * 16 + (lane & 15), own.N);
  const u32x4* own_w = reinterpret_cast<const u32x4*>(own.tiled) + (size_t)stream_blk(wave) * a.KT * (KV * 64) + lane;
  const f16* X = a.mat[mi].X ? a.mat[mi].X : a.X;
  const int row0 = (row_block * ROWS_WAVES + wave) * XROWS;      // first row of this wave
  f16* xw = xbuf + (size_t)wave * XROWS * ROWS_XSTRIDE;

  auto fetch_w = [&](int kt, u32x4 (&wv)[KV]) {
#pragma unroll
    for (int v = 0; v < KV; ++v) wv[v] = __builtin_nontemporal_load(own_w + ((size_t)kt * KV + v) * 64);
  };
  auto decode_w = [&](f16x8* buf, const u32x4 (&wv)[KV]) {
#pragma unroll
    for (int m = 0; m < 4; ++m) buf[(wave * 4 + m) * 64 + lane] = Fmt::a_operand(wv, m, own_sc);
  };
  // whole-row loads: instruction j covers rows 4 j .. 4 j + 3 of the wave, 256 bytes each
  auto fetch_x = [&](int kt, u32x4 (&xr)[RG * 4]) {
#pragma unroll
    for (int j = 0; j < RG * 4; ++j) {
      const int row = row0 + j * 4 + (lane >> 4), k = kt * 128 + (lane & 15) * 8;
      xr[j] = (row < M && k < K) ? *reinterpret_cast<const u32x4*>(X + (size_t)row * K + k) : u32x4{0, 0, 0, 0};
    }
  };
  // through the wave's own strip of LDS into fragment order (a wave's LDS accesses complete in order)
  auto to_fragments = [&](const u32x4 (&xr)[RG * 4], f16x8 (&xf)[RG][4]) {
#pragma unroll
    for (int j = 0; j < RG * 4; ++j)
      *reinterpret_cast<u32x4*>(xw + (j * 4 + (lane >> 4)) * ROWS_XSTRIDE + (lane & 15) * 8) = xr[j];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
      for (int m = 0; m < 4; ++m)
        xf[rg][m] = *reinterpret_cast<const f16x8*>(xw + (rg * 16 + (lane & 15)) * ROWS_XSTRIDE + m * 32 + (lane >> 4) * 8);
  };

  f32x4 acc[RG][ROWS_CB];
#pragma unroll
  for (int rg = 0; rg < RG; ++rg)
#pragma unroll
    for (int st = 0; st < ROWS_CB; ++st) acc[rg][st] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 wv[KV], xr[RG * 4];
  f16x8 xf[RG][4];
  if (steps > 0) {
    fetch_w(kt_first, wv);
    fetch_x(kt_first, xr);
    decode_w(abuf, wv);
    to_fragments(xr, xf);
  }
  __syncthreads();
  for (int i = 0; i < steps; ++i) {
    const bool more = i + 1 < steps;
    if (more) { fetch_w(kt_first + i + 1, wv); fetch_x(kt_first + i + 1, xr); }
    const f16x8* cur = abuf + (size_t)(i & 1) * ROWS_AVEC;
    // the operands of stream st + 1 are read while stream st is multiplied (left to itself the compiler reads two
    // operands, waits, multiplies, and the LDS latency shows after every fourth MFMA)
    f16x8 av[4], avn[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) av[m] = cur[m * 64 + lane];
#pragma unroll
    for (int st = 0; st < ROWS_CB; ++st) {
      if (st + 1 < ROWS_CB) {
#pragma unroll
        for (int m = 0; m < 4; ++m) avn[m] = cur[((st + 1) * 4 + m) * 64 + lane];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) acc[rg][st] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[m], xf[rg][m], acc[rg][st], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < 4; ++m) av[m] = avn[m];
    }
    if (more) {
      decode_w(abuf + (size_t)((i + 1) & 1) * ROWS_AVEC, wv);
      to_fragments(xr, xf);
    }
    __syncthreads();
  }

  // Lane l holds channels (l / 16) * 4 + r, r = 0..3, of row l % 16 of each row group, for every stream.  The sums
  // go to the wave's strip of LDS first (the operand buffers are free after the last barrier) and one copy of the
  // epilogue walks over them: unrolled RG * 8 * 4 times the epilogue is too large to unroll, and an accumulator
  // array that is indexed by a loop counter lives in scratch memory - for the whole kernel.
  f32x4* sums = reinterpret_cast<f32x4*>(smem) + (size_t)wave * (RG * ROWS_CB * 64);
#pragma unroll
  for (int rg = 0; rg < RG; ++rg)
#pragma unroll
    for (int st = 0; st < ROWS_CB; ++st) sums[(rg * ROWS_CB + st) * 64 + lane] = acc[rg][st];
  if constexpr (PAIR) {
    const GemmMat& mat = a.mat[0];
    const typename Fmt::Scale sg = Fmt::load_scale(a.mat[0].scale, a.x_scale, 0, 1), su = Fmt::load_scale(a.mat[1].scale, a.x_scale, 0, 1);
#pragma unroll 1
    for (int i = 0; i < RG * ROWS_CB / 2; ++i) {
      const int rg = i / (ROWS_CB / 2), st = i % (ROWS_CB / 2);
      const int m = row0 + rg * 16 + (lane & 15);
      const f32x4 g4 = sums[(rg * ROWS_CB + st) * 64 + lane], u4 = sums[(rg * ROWS_CB + st + ROWS_CB / 2) * 64 + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = (first_blk + st) * 16 + (lane >> 4) * 4 + r;
        if (m >= M || n >= mat.N) continue;
        mat.Y[(size_t)m * mat.N + n] = swiglu_out(a.epi, (f16)Fmt::finish(g4[r], sg), (f16)Fmt::finish(u4[r], su));
      }
    }
  } else {
    const GemmMat& mat = a.mat[mi];
    const int N = mat.N;
    const typename Fmt::Scale s1 = Fmt::load_scale(mat.scale, a.x_scale, 0, 1);      // no format's finish uses the per-channel part
#pragma unroll 1
    for (int i = 0; i < RG * ROWS_CB; ++i) {
      const int rg = i / ROWS_CB, st = i % ROWS_CB;
      const int m = row0 + rg * 16 + (lane & 15);
      const f32x4 v4 = sums[i * 64 + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = stream_blk(st) * 16 + (lane >> 4) * 4 + r;
        if (m >= M || n >= N) continue;
        if (nsl > 1) { a.part[((size_t)blockIdx.y * M + m) * N + n] = v4[r]; continue; }
        f16 y0 = (f16)Fmt::finish(v4[r], s1);
        if (mat.bias) y0 = y0 + mat.bias[n];
        y0 = apply_act(mat.act, y0);
        mat.Y[(size_t)m * N + n] = apply_epilogue(a.epi, y0, m, n, N);
      }
    }
  }
}

template <class Fmt, int RG, bool PAIR>
static int launch_gemm_rows(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  static bool ready = false;
  const size_t smem = (size_t)2 * ROWS_AVEC * 16 + (size_t)ROWS_WAVES * RG * 16 * ROWS_XSTRIDE * 2;
  static_assert((size_t)2 * ROWS_AVEC * 16 + (size_t)ROWS_WAVES * RG * 16 * ROWS_XSTRIDE * 2 <= 160 * 1024, "LDS");
  if (!ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)gemm_rows_kernel<Fmt, RG, PAIR>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem) == hipSuccess,
                "%s: cannot reserve %zu bytes of LDS", name, smem);
    ready = true;
  }
  const int groups = total_nb / (PAIR ? ROWS_CB / 2 : ROWS_CB);
  const int row_blocks = (a.M + ROWS_WAVES * RG * 16 - 1) / (ROWS_WAVES * RG * 16);
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  const int per = (groups * row_blocks + 7) / 8;
  hipLaunchKernelGGL((gemm_rows_kernel<Fmt, RG, PAIR>), dim3(per * 8, nsl), dim3(ROWS_WAVES * 64), smem, s, a, groups, row_blocks);
  if (nsl > 1) {
    const size_t total = (size_t)a.M * a.mat[0].N;
    hipLaunchKernelGGL((splitk_finish_kernel<Fmt>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a);
  }
  return PTA_OK;
}

// The sums of a wave's tile (RG row groups x NST channel blocks; lane l holds channels st * 16 + (l / 16) * 4 + r of
// row l % 16 of each row group) go out: unit cw of the workgroup, first block blk0 of matrix mi, rows from row0.
template <class Fmt, int NST, int RG, bool PAIR>
__device__ __forceinline__ void panel_store(const GemmArgs& a, f32x4 (&acc)[RG][NST], unsigned char* smem, int cw, int mi, int blk0,
                                            int row0, int nsl, typename Fmt::Scale s0, typename Fmt::Scale s1) {
  constexpr int SW = NST * 16 + 4;                // floats per row of a wave's epilogue strip
  const int lane = threadIdx.x & 63;
  const int M = a.M;
  // Lane l holds channels st * 16 + (l / 16) * 4 + r of row l % 16 of each row group.  Row group by row group the
  // sums pass through a strip of LDS of the wave's own (the row buffers are free after the last barrier) and come
  // back with eight consecutive channels of one row per lane: one 16-byte store per lane, whole 128-byte stretches
  // of a row per wave.  (A wave's LDS accesses complete in order.)
  float* strip = reinterpret_cast<float*>(smem) + (size_t)cw * (16 * SW);
  const GemmMat& mat = a.mat[PAIR ? 0 : mi];
  const int N = mat.N;
  const bool direct = !mat.bias && mat.act == PTA_ACT_NONE && !a.epi.bias && a.epi.act == PTA_ACT_NONE && !a.epi.mul &&
                      a.epi.post_scale == 0.0f && !a.epi.out_fp8_scale;
  auto put = [&](const f32x4 (&sums)[NST]) {
#pragma unroll
    for (int st = 0; st < NST; ++st)
      *reinterpret_cast<f32x4*>(strip + (lane & 15) * SW + st * 16 + (lane >> 4) * 4) = sums[st];
  };
  // (one copy of the epilogue code: unrolled over the row groups it is too large to unroll, and an accumulator
  // array indexed by a loop counter lives in scratch memory for the whole kernel - hence the chain of comparisons)
#pragma unroll 1
  for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
    for (int r = 0; r < RG; ++r)
      if (r == rg) put(acc[r]);
    if constexpr (PAIR) {
      constexpr int LPR = NST / 2 * 16 / 8;                      // lanes per row: eight output channels each
      constexpr int RPP = 64 / LPR;                              // rows per pass
#pragma unroll 1
      for (int it = 0; it < 16 / RPP; ++it) {
        const int rr = it * RPP + lane / LPR, c0 = (lane % LPR) * 8;
        const int m = row0 + rg * 16 + rr, n = blk0 * 16 + c0;
        if (rr >= 16) continue;
        const f32x4 g0 = *reinterpret_cast<const f32x4*>(strip + rr * SW + c0), g1 = *reinterpret_cast<const f32x4*>(strip + rr * SW + c0 + 4);
        const f32x4 u0 = *reinterpret_cast<const f32x4*>(strip + rr * SW + NST / 2 * 16 + c0), u1 = *reinterpret_cast<const f32x4*>(strip + rr * SW + NST / 2 * 16 + c0 + 4);
        if (m >= M) continue;
        f16x8 y;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          y[j] = swiglu_out(a.epi, (f16)Fmt::finish(j < 4 ? g0[j & 3] : g1[j & 3], s0), (f16)Fmt::finish(j < 4 ? u0[j & 3] : u1[j & 3], s1));
        if (n + 8 <= N && (N & 7) == 0) {
          *reinterpret_cast<f16x8*>(mat.Y + (size_t)m * N + n) = y;
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (n + j < N) mat.Y[(size_t)m * N + n + j] = y[j];
        }
      }
    } else {
      constexpr int LPR = NST * 16 / 8;
      constexpr int RPP = 64 / LPR;
#pragma unroll 1
      for (int it = 0; it < (16 + RPP - 1) / RPP; ++it) {
        const int rr = it * RPP + lane / LPR, c0 = (lane % LPR) * 8;
        const int m = row0 + rg * 16 + rr, n = blk0 * 16 + c0;
        if (rr >= 16) continue;
        const f32x4 v0 = *reinterpret_cast<const f32x4*>(strip + rr * SW + c0), v1 = *reinterpret_cast<const f32x4*>(strip + rr * SW + c0 + 4);
        if (m >= M) continue;
        if (nsl > 1) {
          float* p = a.part + ((size_t)blockIdx.y * M + m) * N + n;
          if (n + 8 <= N && (N & 3) == 0) {
            *reinterpret_cast<f32x4*>(p) = v0;
            *reinterpret_cast<f32x4*>(p + 4) = v1;
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (n + j < N) p[j] = j < 4 ? v0[j & 3] : v1[j & 3];
          }
          continue;
        }
        f16x8 y;
        if (direct && n + 8 <= N && (N & 7) == 0) {                // nothing but the residual stream to add: whole vectors
          f16x8 res;
          if (a.epi.residual) res = *reinterpret_cast<const f16x8*>(a.epi.residual + (size_t)m * N + n);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            y[j] = (f16)Fmt::finish(j < 4 ? v0[j & 3] : v1[j & 3], s0);
            if (a.epi.residual) y[j] = y[j] + res[j];
          }
          *reinterpret_cast<f16x8*>(mat.Y + (size_t)m * N + n) = y;
          continue;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          f16 y0 = (f16)Fmt::finish(j < 4 ? v0[j & 3] : v1[j & 3], s0);
          if (n + j < N) {
            if (mat.bias) y0 = y0 + mat.bias[n + j];
            y0 = apply_act(mat.act, y0);
            y0 = apply_epilogue(a.epi, y0, m, n + j, N);
          }
          y[j] = y0;
        }
        if (n + 8 <= N && (N & 7) == 0) {
          *reinterpret_cast<f16x8*>(mat.Y + (size_t)m * N + n) = y;
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (n + j < N) mat.Y[(size_t)m * N + n + j] = y[j];
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Variant for hundreds of rows: the roles turned round.  The tiled weight format IS the A operand order, so a
// wave fetches the tiles of its own NST channel blocks straight into registers (1 KiB per instruction, no LDS)
// and decodes them there; the 128 activation rows of the workgroup go through LDS once per 128-feature tile
// (whole-row loads, double-buffered, one barrier per tile) and every wave reads all of them as B operands.
// A wave's tile is 128 rows x NST * 16 channels: one B operand read from LDS feeds NST MFMAs and one decoded
// A operand feeds 8, which is what keeps both LDS (128 bytes per clock and compute unit) and the vector ALU
// behind the matrix unit.  (With the weights through LDS and the rows in registers - gemm_rows_kernel - every
// wave reads every decoded weight: 1 KiB of LDS per 2 MFMAs, more than the LDS delivers.)
// PAIR: a wave owns NST / 2 gate blocks and the same blocks of the up weight.
// ------------------------------------------------------------------------------------------
constexpr int PANEL_WAVES = 8;

// RG: row groups of 16 per workgroup (every wave multiplies all of them); KH: parts of K inside the workgroup - the
// waves are 8 / KH channel units x KH parts, part kh takes the feature tiles kh, kh + KH, ... of the workgroup's
// range and the parts' sums meet in LDS at the end.  KH > 1 is for launches with few channels: it halves or
// quarters the channels of a workgroup tile, so more workgroups, without the fp32 round trip through memory that
// slices of workgroups (ksplit) cost.
template <class Fmt, int NST, int RG, int KH, bool PAIR>
__global__ __launch_bounds__(PANEL_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_panel_kernel(GemmArgs a, int groups, int row_blocks, int unit0, int units) {
  constexpr int KV = Fmt::kVec;
  constexpr int CW = PANEL_WAVES / KH;            // channel units (waves side by side) per workgroup
  constexpr int ROWS = RG * 16;
  constexpr int XPART = ROWS * 128;               // halves of one feature tile of the workgroup's rows
  constexpr int XSTAGE = KH * XPART;              // one stage: a tile per part
  constexpr int QN = KH * RG / 2;                 // row loads (4 rows each) per wave and stage
  constexpr int SW = NST * 16 + 4;                // floats per row of a wave's epilogue strip
  static_assert(!PAIR || NST % 2 == 0, "gate and up blocks in equal numbers");
  static_assert(KH == 1 || KH == 2 || KH == 4, "parts of K");
  static_assert((KH * RG) % 2 == 0 && RG <= 8, "row loads per wave");
  static_assert(KH == 1 || (KH - 1) * CW * RG * NST * 1024 <= 2 * XSTAGE * 2, "the parts' sums meet in the row buffers");
  extern __shared__ __align__(16) unsigned char smem[];
  f16* xbuf = reinterpret_cast<f16*>(smem);                                              // [2][KH][ROWS][128], pieces exchanged (see fetch_x)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int cw = wave % CW, kh = wave / CW;
  const int K = a.K, M = a.M;
  // workgroup id -> tile as in gemm_rows_kernel (contiguous stretches of the tile list per XCD); the row block runs
  // fastest, so the workgroups that are resident together multiply the same weights and those come from L2
  const int per = (int)gridDim.x / 8;
  const int tile = ((int)blockIdx.x % 8) * per + (int)blockIdx.x / 8;
  if (tile >= groups * row_blocks) return;
  const int row_block = tile % row_blocks, group = tile / row_blocks;
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  const int per_slice = (a.KT + nsl - 1) / nsl;
  const int kt_first = (int)blockIdx.y * per_slice;
  const int kt_end = kt_first + per_slice < a.KT ? kt_first + per_slice : a.KT;
  const int steps = kt_end > kt_first ? (kt_end - kt_first + KH - 1) / KH : 0;      // a tile per part and step

  // this wave's channel blocks: unit `wu` of the matrices (the launch covers units unit0 .. units - 1); waves past the
  // last unit only help with the rows
  const int wu = unit0 + group * CW + cw;
  const bool active = wu < units;
  const int gb = (active ? wu : 0) * (PAIR ? NST / 2 : NST);      // first block (of the launch; of the pair's matrices)
  int mi = 0;
  if (!PAIR) {
#pragma unroll
    for (int i = 1; i < 4; ++i)
      if (i < a.count && gb >= a.mat[i].nb_begin) mi = i;
  }
  const int blk0 = PAIR ? gb : gb - a.mat[mi].nb_begin;           // first block within its matrix
  // Loads through buffer descriptors: the descriptor and the tile's offset travel in scalar registers and one
  // 32-bit offset per lane serves all streams, another all rows (with 64-bit addresses per lane the loop keeps a
  // pointer per stream and row in vector registers, which this kernel does not have).  Rows past M lie past
  // the end of the rows' descriptor and read as zero.
  constexpr int NBW = PAIR ? NST / 2 : NST;                        // consecutive blocks behind one descriptor
  const uint32_t blk_bytes = (uint32_t)a.KT * (KV * 1024);
  const unsigned char* w0 = reinterpret_cast<const unsigned char*>(a.mat[PAIR ? 0 : mi].tiled) + (size_t)blk0 * blk_bytes;
  const unsigned char* w1 = reinterpret_cast<const unsigned char*>(a.mat[PAIR ? 1 : mi].tiled) + (size_t)blk0 * blk_bytes;
  const __amdgpu_buffer_rsrc_t wr0 = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(w0), 0, (int)(NBW * blk_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t wr1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(w1), 0, (int)(NBW * blk_bytes), 0x00020000);
  const int wlane = lane * 16;
  const int row0 = row_block * ROWS;
  const int rows_here = M - row0 < ROWS ? M - row0 : ROWS;
  const __amdgpu_buffer_rsrc_t xr0 = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<f16*>(a.X + (size_t)row0 * K), 0, (int)((size_t)rows_here * K * 2), 0x00020000);

  // this wave's weight tiles of step i (past the end of the range: zeros - the rows of that tile are zeros too)
  auto fetch_w = [&](int i, u32x4 (&wv)[NST][KV]) {
    const int kt = kt_first + i * KH + kh;
#pragma unroll
    for (int st = 0; st < NST; ++st)
#pragma unroll
      for (int v = 0; v < KV; ++v)
        wv[st][v] = kt < kt_end ? __builtin_amdgcn_raw_buffer_load_b128(PAIR && st >= NST / 2 ? wr1 : wr0, wlane,
                                      (int)((PAIR ? st % (NST / 2) : st) * blk_bytes + (uint32_t)(kt * KV + v) * 1024), 0)
                                : u32x4{0, 0, 0, 0};
  };
  // The rows go from memory into LDS without passing through registers: load q = 8 j + w (w: the wave) of a stage
  // brings rows 4 (q % (4 RG)) .. + 3 of the tile of part q / (4 RG), 256 bytes each, lane l the 16 bytes that
  // belong at position l % 16 of row l / 16 - LDS receives the lanes' data one after the other, so a row takes 256
  // bytes and its 16-byte pieces are stored exchanged among themselves: piece c of row r at position c ^ (r % 16).
  // The sixteen rows of a B operand read then fall into sixteen different groups of four banks, without padding.
  auto fetch_x = [&](int i, f16* stage) {
#pragma unroll
    for (int j = 0; j < QN; ++j) {
      const int q = j * PANEL_WAVES + wave;
      const int part = q / (4 * RG), rb = q % (4 * RG);
      const int row = rb * 4 + (lane >> 4);
      const int piece = (lane & 15) ^ (row & 15);
      const int kt = kt_first + i * KH + part;
      const bool in_k = kt < kt_end && kt * 128 + piece * 8 < K;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xr0, (__attribute__((address_space(3))) void*)(stage + part * XPART + rb * 4 * 128), 16,
                                               in_k ? row * K * 2 + piece * 16 : -1, kt * 256, 0, 0);
    }
  };

  f32x4 acc[RG][NST];
#pragma unroll
  for (int rg = 0; rg < RG; ++rg)
#pragma unroll
    for (int st = 0; st < NST; ++st) acc[rg][st] = f32x4{0.f, 0.f, 0.f, 0.f};

  // The product runs as one pipeline over all steps: 4 * NST blocks of RG MFMAs per tile (one decoded A operand
  // each); the A operand of the next block is decoded among the MFMAs of this one, and during the last block of a
  // 32-feature step every B operand is replaced by the next one's as soon as its MFMA has been issued - across the
  // tile boundary too.  So the tile's one barrier stands before its last 32 features: by then every wave has read
  // the last B operands from this stage (which the loads of the stage after next may then overwrite) and the next
  // stage's rows, requested when this one began, must have landed.
  u32x4 wa[NST][KV], wb[NST][KV];
  f16x8 xf[RG];
  f16x8 avc;
  const int xat = kh * XPART + (lane & 15) * 128;                  // this lane's row within a row group of its part, in halves
  auto b_piece = [&](int m) { return ((m * 4 + (lane >> 4)) ^ (lane & 15)) * 8; };
  if (steps > 0) {
    if (active) fetch_w(0, wa);
    fetch_x(0, xbuf);
  }
  typename Fmt::Scale sc[NST];             // (requested behind the first tile: one round trip to memory, not two)
#pragma unroll
  for (int st = 0; st < NST; ++st) {
    const GemmMat& mt = a.mat[PAIR ? (st < NST / 2 ? 0 : 1) : mi];
    sc[st] = Fmt::load_scale(mt.scale, a.x_scale, (blk0 + (PAIR ? st % (NST / 2) : st)) * 16 + (lane & 15), mt.N);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);      // vmcnt(0): the rows have landed in LDS
  __syncthreads();
  if (active && steps > 0) {
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) xf[rg] = *reinterpret_cast<const f16x8*>(xbuf + xat + rg * 16 * 128 + b_piece(0));
    avc = Fmt::a_operand(wa[0], 0, sc[0]);
  }
  auto feature_tile = [&](int i, const u32x4 (&wc)[NST][KV], u32x4 (&wn)[NST][KV]) {
    const bool more = i + 1 < steps;
    const f16* xc = xbuf + (size_t)(i & 1) * XSTAGE + xat;
    const f16* xn = xbuf + (size_t)((i + 1) & 1) * XSTAGE + xat;
    if (more) {
      if (active) fetch_w(i + 1, wn);
      fetch_x(i + 1, xbuf + (size_t)((i + 1) & 1) * XSTAGE);
    }
    auto blocks = [&](int first, int last) {
#pragma unroll
      for (int blk = first; blk < last; ++blk) {
        const int m = blk / NST, st = blk % NST;
        f16x8 avn = avc;
        if (blk + 1 < 4 * NST) avn = Fmt::a_operand(wc[(blk + 1) % NST], (blk + 1) / NST, sc[(blk + 1) % NST]);
        else if (more) avn = Fmt::a_operand(wn[0], 0, sc[0]);
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
          acc[rg][st] = __builtin_amdgcn_mfma_f32_16x16x32_f16(avc, xf[rg], acc[rg][st], 0, 0, 0);
          if (st == NST - 1) {
            if (m < 3) xf[rg] = *reinterpret_cast<const f16x8*>(xc + rg * 16 * 128 + b_piece(m + 1));
            else if (more) xf[rg] = *reinterpret_cast<const f16x8*>(xn + rg * 16 * 128 + b_piece(0));
          }
        }
        avc = avn;
      }
    };
    if (active) blocks(0, 3 * NST);
    __builtin_amdgcn_s_waitcnt(0x0f70);    // vmcnt(0): the next stage's rows have landed (and its weights)
    __syncthreads();
    if (active) blocks(3 * NST, 4 * NST);
  };
  for (int i = 0; i < steps; i += 2) {
    feature_tile(i, wa, wb);
    if (i + 1 < steps) feature_tile(i + 1, wb, wa);
  }
  __syncthreads();                         // (what follows reuses the row buffers)
  if constexpr (KH > 1) {
    // the sums of parts 1 .. KH - 1 go to part 0's wave of the same channel unit
    f32x4* ex = reinterpret_cast<f32x4*>(smem);                   // [(KH - 1) * CW][RG * NST][64]
    if (kh > 0 && active) {
#pragma unroll
      for (int rg = 0; rg < RG; ++rg)
#pragma unroll
        for (int st = 0; st < NST; ++st) ex[(((kh - 1) * CW + cw) * (RG * NST) + rg * NST + st) * 64 + lane] = acc[rg][st];
    }
    __syncthreads();
    if (kh == 0 && active) {
#pragma unroll
      for (int k = 1; k < KH; ++k)
#pragma unroll
        for (int rg = 0; rg < RG; ++rg)
#pragma unroll
          for (int st = 0; st < NST; ++st) {
            const f32x4 other = ex[(((k - 1) * CW + cw) * (RG * NST) + rg * NST + st) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[rg][st][r] += other[r];
          }
    }
    __syncthreads();
    if (kh > 0) return;
  }
  if (!active) return;

  const typename Fmt::Scale s0 = Fmt::load_scale(a.mat[PAIR ? 0 : mi].scale, a.x_scale, 0, 1);   // no format's finish uses the per-channel part
  const typename Fmt::Scale s1 = Fmt::load_scale(a.mat[PAIR ? 1 : mi].scale, a.x_scale, 0, 1);
  panel_store<Fmt, NST, RG, PAIR>(a, acc, smem, cw, mi, blk0, row0, nsl, s0, s1);
}

// whether every matrix of the launch is a whole number of wave tiles of `nst` channel blocks and all share one input
static inline bool panel_fits(const GemmArgs& a, int nst, bool pair) {
  if (a.epi.norm != PTA_NORM_NONE || a.KT < 2) return false;
  if (pair) return ((a.mat[0].N + 15) / 16) % (nst / 2) == 0;
  for (int i = 0; i < a.count; ++i) {
    if (((a.mat[i].N + 15) / 16) % nst != 0) return false;
    if (a.mat[i].X && a.mat[i].X != a.X) return false;
  }
  return true;
}

// units [unit0, unit1) of the launch's matrices (a unit: NST channel blocks, or NST / 2 gate and up blocks)
template <class Fmt, int NST, int RG, int KH, bool PAIR>
static int launch_gemm_panel(const GemmArgs& a, int unit0, int unit1, hipStream_t s, const char* name) {
  static bool ready = false;
  constexpr int CW = PANEL_WAVES / KH;
  constexpr size_t rows_bytes = (size_t)2 * KH * RG * 16 * 128 * 2, strips = (size_t)CW * 16 * (NST * 16 + 4) * 4;
  constexpr size_t smem = rows_bytes > strips ? rows_bytes : strips;
  static_assert(smem <= 160 * 1024, "LDS");
  if (!ready) {
    PTA_REQUIRE(hipFuncSetAttribute((const void*)gemm_panel_kernel<Fmt, NST, RG, KH, PAIR>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem) == hipSuccess,
                "%s: cannot reserve %zu bytes of LDS", name, smem);
    ready = true;
  }
  const int groups = (unit1 - unit0 + CW - 1) / CW;
  const int row_blocks = (a.M + RG * 16 - 1) / (RG * 16);
  const int nsl = a.ksplit > 1 ? a.ksplit : 1;
  const int per = (groups * row_blocks + 7) / 8;
  hipLaunchKernelGGL((gemm_panel_kernel<Fmt, NST, RG, KH, PAIR>), dim3(per * 8, nsl), dim3(PANEL_WAVES * 64), smem, s, a, groups, row_blocks, unit0, unit1);
  if (nsl > 1) {
    const size_t total = (size_t)a.M * a.mat[0].N;
    hipLaunchKernelGGL((splitk_finish_kernel<Fmt>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a);
  }
  return PTA_OK;
}

// whether the launch fits gemm_tile_kernel with `per_wg` channel blocks per workgroup: every matrix
// a whole number of workgroups, enough feature tiles for the K groups
static inline bool tile_fits(const GemmArgs& a, int per_wg, int kq, bool pair) {
  if (a.KT < 2 * kq) return false;
  if (pair) return ((a.mat[0].N + 15) / 16) % per_wg == 0;
  for (int i = 0; i < a.count; ++i)
    if (((a.mat[i].N + 15) / 16) % per_wg != 0) return false;
  return true;
}

static inline int device_compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

template <class Fmt, int NW, bool PAIR>
static void launch_gemv_lds(const GemmArgs& a, int total_nb, hipStream_t s) {
  const size_t xbytes = (((size_t)a.M * (a.KT * 128 + 8) * 2) + 15) & ~(size_t)15;
  const size_t smem = xbytes + (size_t)NW * (PAIR ? 2 : 1) * 256 * sizeof(float);
  hipLaunchKernelGGL((gemv_lds_kernel<Fmt, NW, PAIR>), dim3(total_nb), dim3(NW * 64), smem, s, a);
}

template <class Fmt, int MT, bool PAIR>
static void launch_gemv(const GemmArgs& a, int total_nb, hipStream_t s) {
  // Waves per block: enough to split K finely when there are few channel blocks, fewer when
  // the grid alone already fills the machine.  The LDS reduction buffer caps the wide cases.
  if constexpr (MT == 4 && PAIR) {
    hipLaunchKernelGGL((gemv_mfma_kernel<Fmt, MT, 4, PAIR>), dim3(total_nb), dim3(4 * 64), 0, s, a);
  } else if constexpr (MT == 4 || PAIR) {
    hipLaunchKernelGGL((gemv_mfma_kernel<Fmt, MT, 8, PAIR>), dim3(total_nb), dim3(8 * 64), 0, s, a);
  } else {
    if (a.KT >= 16 && total_nb <= 1024)
      hipLaunchKernelGGL((gemv_mfma_kernel<Fmt, MT, 16, PAIR>), dim3(total_nb), dim3(16 * 64), 0, s, a);
    else
      hipLaunchKernelGGL((gemv_mfma_kernel<Fmt, MT, 8, PAIR>), dim3(total_nb), dim3(8 * 64), 0, s, a);
  }
}

template <class Fmt, bool PAIR>
static int dispatch_gemv(const GemmArgs& a, int total_nb, hipStream_t s, const char* name);

// More than 64 rows.  Beyond 128 rows gemm_panel_kernel, up to 128 (fp16 weights: any number) gemm_rows_kernel, where
// the channel blocks divide into their workgroup tiles; a single matrix with few channels also splits K when a workspace is at hand.  Otherwise
// the rows go through the smaller paths in turn, 64 at a time.
template <class Fmt, bool PAIR>
static int dispatch_many_rows(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  const int cus = device_compute_units();
  const int per_wg = PAIR ? 4 : 8;
  const bool tiles = a.epi.norm == PTA_NORM_NONE && tile_fits(a, per_wg, 2, PAIR);
  // More than 128 rows (measured on whole prompt passes of the 7B shape, gemm_rows_kernel against this: 6.5 against
  // 7.2 ms at 128 rows, 7.7 against 7.3 at 192, 8.1 against 7.5 at 256): 128-row panels through LDS, the weights
  // straight into registers.  Formats of up to two vectors per tile only - with four (fp16) two tiles of four
  // streams do not fit the registers.
  if constexpr (Fmt::kVec <= 2) {
    if (a.M > 128 && panel_fits(a, 4, PAIR)) {
      const int units = PAIR ? total_nb / 2 : total_nb / 4;
      const int row_blocks = (a.M + 127) / 128;
      // few workgroup tiles (4096 channels: 8 per row block): K in halves inside the workgroup, tiles of half the channels
      const int groups = (units + 7) / 8, tiles_all = groups * row_blocks;
      const bool halves = tiles_all * 2 <= cus && a.KT >= 16;
      const int wgs = ((units + (halves ? 3 : 7)) / (halves ? 4 : 8)) * row_blocks;
      GemmArgs b = a;
      int nsl = wgs > 0 ? cus / wgs : 1;
      nsl = nsl > GEMM_MAX_KSPLIT ? GEMM_MAX_KSPLIT : nsl;
      while (nsl > 1 && a.KT < nsl * 16) --nsl;
      if (!PAIR && a.count == 1 && a.part && nsl > 1 && a.part_bytes >= (size_t)nsl * a.M * a.mat[0].N * sizeof(float)) b.ksplit = nsl;
      // More tiles than compute units and a last round that fills at most half of them (344 tiles are 1.34 rounds
      // of 256 and would take 2): the channel groups of the whole rounds in one launch, the rest with K in halves -
      // twice the workgroups, each half as long.
      const int whole = (tiles_all / cus) * cus / row_blocks;             // channel groups within the whole rounds
      const int rest = (groups - whole) * row_blocks;
      int rc;
      if (!halves && whole > 0 && rest > 0 && rest * 2 <= cus && a.KT >= 16 && b.ksplit <= 1) {
        rc = launch_gemm_panel<Fmt, 4, 8, 1, PAIR>(b, 0, whole * 8, s, name);
        if (!rc) rc = launch_gemm_panel<Fmt, 4, 8, 2, PAIR>(b, whole * 8, units, s, name);
      } else {
        rc = halves ? launch_gemm_panel<Fmt, 4, 8, 2, PAIR>(b, 0, units, s, name) : launch_gemm_panel<Fmt, 4, 8, 1, PAIR>(b, 0, units, s, name);
      }
      if (rc) return rc;
      PTA_CHECK_LAUNCH(name);
      return PTA_OK;
    }
  }
  if (tiles) {
    // fragments in registers, weights through LDS: 256 rows per workgroup where that still fills the machine,
    // else 128; few workgroups and one matrix: K in slices as well
    const int groups = total_nb / per_wg;
    const bool two = a.M > 128 && (long)groups * ((a.M + 255) / 256) * 2 >= (long)cus;
    const int wgs = groups * (two ? (a.M + 255) / 256 : (a.M + 127) / 128);
    GemmArgs b = a;
    int nsl = wgs > 0 ? cus / wgs : 1;
    nsl = nsl > GEMM_MAX_KSPLIT ? GEMM_MAX_KSPLIT : nsl;
    while (nsl > 1 && a.KT < nsl * 8) --nsl;
    if (!PAIR && a.count == 1 && a.part && nsl > 1 && a.part_bytes >= (size_t)nsl * a.M * a.mat[0].N * sizeof(float)) b.ksplit = nsl;
    const int rc = two ? launch_gemm_rows<Fmt, 2, PAIR>(b, total_nb, s, name) : launch_gemm_rows<Fmt, 1, PAIR>(b, total_nb, s, name);
    if (rc) return rc;
    PTA_CHECK_LAUNCH(name);
    return PTA_OK;
  }
  const int chunk = 64;
  for (int m0 = 0; m0 < a.M; m0 += chunk) {
    GemmArgs b = a;
    b.M = a.M - m0 < chunk ? a.M - m0 : chunk;
    if (b.X) b.X += (size_t)m0 * a.K;
    for (int i = 0; i < a.count; ++i) {
      if (b.mat[i].X) b.mat[i].X += (size_t)m0 * a.K;
      if (!PAIR || i == 0) b.mat[i].Y += (size_t)m0 * a.mat[i].N;
    }
    if (PAIR) b.mat[1].Y = b.mat[0].Y;
    if (b.epi.residual) b.epi.residual += (size_t)m0 * a.mat[0].N;
    if (b.epi.mul) b.epi.mul += (size_t)m0 * a.mat[0].N;
    const int rc = dispatch_gemv<Fmt, PAIR>(b, total_nb, s, name);
    if (rc) return rc;
  }
  return PTA_OK;
}

template <class Fmt, bool PAIR>
static int dispatch_gemv(const GemmArgs& a, int total_nb, hipStream_t s, const char* name) {
  if (a.M > 64) return dispatch_many_rows<Fmt, PAIR>(a, total_nb, s, name);
  const size_t xbytes = (size_t)a.M * (a.KT * 128 + 8) * 2;
  bool all_shared_x = true;
  for (int i = 0; i < a.count; ++i) all_shared_x = all_shared_x && a.mat[i].X == nullptr;
  const bool norm_small = a.M <= 4 && xbytes <= 40 * 1024;
  const bool norm_wide = a.M <= 16 && all_shared_x && a.KT >= 8;
  if (a.epi.norm != PTA_NORM_NONE && !norm_small && !norm_wide) {
    pta_set_error("%s: the fused norm needs M <= 4 with M*K <= 20480, or M <= 16 with one shared X and K >= 1024 "
                  "(got M=%d K=%d)", name, a.M, a.K);
    return PTA_EUNSUPPORTED;
  }
  if (a.M <= 4 && xbytes <= 40 * 1024) {
    if (a.KT >= 16 && total_nb <= 1024 && !PAIR) launch_gemv_lds<Fmt, 16, PAIR>(a, total_nb, s);
    else launch_gemv_lds<Fmt, 8, PAIR>(a, total_nb, s);
  } else {
    bool shared_x = true;
    for (int i = 0; i < a.count; ++i) shared_x = shared_x && a.mat[i].X == nullptr;
    const int per_cu = (total_nb + device_compute_units() - 1) / device_compute_units();
    if (a.M > 16 && a.epi.norm == PTA_NORM_NONE) {
      // the staged kernel where its workgroups fill the machine: 2 streams x 4 K groups (4 channel blocks,
      // or 2 SwiGLU pairs, per workgroup); for M <= 32 also 8 K groups (half as many blocks per workgroup)
      const int cus = device_compute_units();
      const int wgs4 = total_nb / (PAIR ? 2 : 4), wgs8 = total_nb / (PAIR ? 1 : 2);
      int rc = 1;
      // one matrix, too few channel blocks to fill the machine, scratch at hand: split K too
      int nsl = wgs4 > 0 ? cus / wgs4 : 1;
      nsl = nsl > GEMM_MAX_KSPLIT ? GEMM_MAX_KSPLIT : nsl;
      while (nsl > 1 && a.KT < nsl * 8) --nsl;
      if (!PAIR && a.count == 1 && a.part && nsl > 1 && tile_fits(a, 4, 4, false) &&
          a.part_bytes >= (size_t)nsl * a.M * a.mat[0].N * sizeof(float)) {
        GemmArgs b = a;
        b.ksplit = nsl;
        rc = a.M <= 32 ? launch_gemm_tile<Fmt, 2, 4, PAIR>(b, total_nb, s, name) : launch_gemm_tile<Fmt, 4, 4, PAIR>(b, total_nb, s, name);
      } else if (tile_fits(a, PAIR ? 2 : 4, 4, PAIR) && 2 * wgs4 >= cus) {
        // What bounds these launches is the bytes through the busiest compute unit: a workgroup reads all rows of X
        // beside its weights.  More workgroups than compute units (20480 channels: 320 of 64 channels): workgroups
        // of 16 waves and 128 channels where their rounds come out shorter - 160 of 768 KiB against two rounds of
        // 640 at 64 rows.  Measured, 4096 x 20480: 26.0 against 40.7 us at 64 rows, 24.7 against 38.2 at 48, 18.8
        // against 20.8 at 32; in a single round they lose (4096 x 11008 at 64 rows: 24.9 against 21.5 us).
        bool wide = false;
        if constexpr (!PAIR && Fmt::kVec <= 2) {
          // (beyond 32 rows with INT4 weights only: with two vectors per tile the 16 waves' registers do not hold it)
          if (tile_fits(a, 8, 4, false) && wgs4 > cus && (a.M <= 32 || Fmt::kVec == 1)) {
            const double xb = (double)a.M * a.K * 2, wb = (double)a.KT * Fmt::kVec * 1024;
            const int wgs_wide = total_nb / 8;
            wide = ((wgs_wide + cus - 1) / cus) * (xb + 8 * wb) < ((wgs4 + cus - 1) / cus) * (xb + 4 * wb);
          }
          if (wide) {
            if (a.M <= 32) rc = launch_gemm_tile<Fmt, 2, 4, false, 16>(a, total_nb, s, name);
            else if constexpr (Fmt::kVec == 1) rc = launch_gemm_tile<Fmt, 4, 4, false, 16>(a, total_nb, s, name);
          }
        }
        if (!wide)
        rc = a.M <= 32 ? launch_gemm_tile<Fmt, 2, 4, PAIR>(a, total_nb, s, name) : launch_gemm_tile<Fmt, 4, 4, PAIR>(a, total_nb, s, name);
      } else if (a.M <= 32 && tile_fits(a, PAIR ? 1 : 2, 8, PAIR) && 2 * wgs8 >= cus) {
        rc = launch_gemm_tile<Fmt, 2, 8, PAIR>(a, total_nb, s, name);
      }
      if (rc < 0) return rc;
      if (rc == 0) { PTA_CHECK_LAUNCH(name); return PTA_OK; }
    }
    if (shared_x && a.KT >= 8) {
      int rc;
      bool streamed = false;
      if constexpr (Fmt::kVec * (PAIR ? 2 : 1) <= 4) {
        // gemv_stream_kernel where gemv_wide_kernel's rounds of workgroups come out longer than an even share of the
        // blocks (856 blocks: 286 workgroups of 3 = two rounds = 6 block times, against 4), or on request
        if (stream_fits(a) && total_nb >= device_compute_units() && (a.prefer_stream || wide_block_times<Fmt, PAIR>(total_nb, per_cu) > per_cu)) {
          rc = launch_gemv_stream<Fmt, PAIR>(a, total_nb, device_compute_units(), s, name);
          streamed = true;
        }
      }
      if (streamed) {}
      else if (a.M <= 16 && a.epi.norm != PTA_NORM_NONE) rc = launch_gemv_wide_for<Fmt, 1, PAIR, true>(a, total_nb, per_cu, s, name);
      else if (a.M <= 16) rc = launch_gemv_wide_for<Fmt, 1, PAIR>(a, total_nb, per_cu, s, name);
      else if (a.M <= 32) rc = launch_gemv_wide_for<Fmt, 2, PAIR>(a, total_nb, per_cu, s, name);
      else rc = launch_gemv_wide_for<Fmt, 4, PAIR>(a, total_nb, per_cu, s, name);
      if (rc) return rc;
    } else if (a.M <= 16) launch_gemv<Fmt, 1, PAIR>(a, total_nb, s);
    else if (a.M <= 32) launch_gemv<Fmt, 2, PAIR>(a, total_nb, s);
    else launch_gemv<Fmt, 4, PAIR>(a, total_nb, s);
  }
  PTA_CHECK_LAUNCH(name);
  return PTA_OK;
}

static inline int check_gemv_common(const char* name, const void* X, int M, int K) {
  PTA_REQUIRE(X, "%s: null X", name);
  PTA_REQUIRE(M >= 1 && M <= GEMM_MAX_ROWS, "%s: M must be in [1, %d], got %d", name, GEMM_MAX_ROWS, M);
  PTA_REQUIRE(K > 0 && (K % 8) == 0, "%s: K must be a positive multiple of 8, got %d", name, K);
  PTA_REQUIRE(pta_aligned(X, 16), "%s: X must be 16-byte aligned", name);
  return PTA_OK;
}

static inline size_t gemv_tiled_bytes(int N, int K, int kvec) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)((N + 15) / 16) * (size_t)((K + 127) / 128) * 1024 * kvec;
}
