// Decode attention (one query position per sequence) over the ring KV cache, and the
// query/key preparation that precedes it.
//
// Reference graphs: models/gpt2/attention.py:50-90, models/llama2/attention.py:28-114,
// models/chatglm2/attention.py:77-302.  They compute q.K^T over all max_len cache rows, add a
// mask of 0 / -10000, apply the non-stable SoftmaxV3 and multiply by V.  A masked row
// contributes exp(-10000 + s) = 0 exactly (in fp16 and in fp32), so attending to the valid rows
// only gives the same sums; subtracting the running maximum before exp is the same function
// without the overflow.  Roundings that the reference performs on the scores (fp16 MatMul
// output, fp16 multiply by 1/sqrt(D)) are reproduced; probabilities stay fp32 up to the final
// fp16 rounding of the context vector.
#include "common.h"
#include "formats.h"
#include "f8codec.h"

// ------------------------------------------------------------------------------------------
// q/k rotary embedding + KV ring append.
// ------------------------------------------------------------------------------------------
struct QkvArgs {
  const f16* q; const f16* k; const f16* v;   // rows of the projection outputs
  int q_stride, k_stride, v_stride;           // elements between batch rows
  f16* q_out;                                 // [B, Hq, D]
  f16* kring; f16* vring;                     // [B*Hkv, max_len, D] each
  const int32_t* step;
  const void* inv_freq;                       // fp16 [D/2] (PTA_ROPE_LLAMA) or fp32 [D/4] (PTA_ROPE_GLM2)
  int B, Hq, Hkv, D, max_len, rope;
  int rows;                                   // consecutive positions per sequence (1 in the decode step)
  int kv8, kv_scale;                          // kv8: the rings hold F143 bytes (kring / vring point at bytes)
};

// Llama: angle = fp16(fp16(step) * inv_freq16) (an fp16 MatMul of a 1x1 by a 1xD/2 matrix,
// llama2/attention.py:28-38), sin/cos rounded to fp16, rotate-half over the whole head
// (llama2/attention.py:40-56): y = fp16(fp16(x*cos) + fp16(rot(x)*sin)).
__device__ __forceinline__ f16 rope_mix(f16 x, f16 rot, f16 c, f16 s) { return x * c + rot * s; }
__device__ __forceinline__ f16 rope_llama_angle(int step, f16 inv_freq) { return (f16)((float)(f16)(float)step * (float)inv_freq); }
__device__ __forceinline__ f16 rope_llama_value(const f16* x, int d, int D, int step, const f16* inv_freq) {
  const int half = D >> 1;
  const int i = d < half ? d : d - half;
  const f16 ang = rope_llama_angle(step, inv_freq[i]);
  const f16 c = (f16)cosf((float)ang), s = (f16)sinf((float)ang);
  const f16 rot = d < half ? -x[d + half] : x[d - half];
  return rope_mix(x[d], rot, c, s);
}
__device__ __forceinline__ void rope_llama(const f16* x, f16* y, int d, int D, int step, const f16* inv_freq) {
  y[d] = rope_llama_value(x, d, D, step, inv_freq);
}

// ChatGLM2: only the first D/2 features of a head rotate, as interleaved pairs (2j, 2j+1) with
// angle fp16(fp32(step) * inv_freq32[j]) (chatglm2/attention.py:77-164).
__device__ __forceinline__ f16 rope_glm2_value(const f16* x, int d, int D, int step, const float* inv_freq) {
  const int rot_dim = D >> 1;
  if (d >= rot_dim) return x[d];
  const int j = d >> 1;
  const f16 ang = (f16)((float)step * inv_freq[j]);
  const f16 c = (f16)cosf((float)ang), s = (f16)sinf((float)ang);
  const f16 rot = (d & 1) ? x[d - 1] : -x[d + 1];
  return rope_mix(x[d], rot, c, s);
}
__device__ __forceinline__ void rope_glm2(const f16* x, f16* y, int d, int D, int step, const float* inv_freq) {
  y[d] = rope_glm2_value(x, d, D, step, inv_freq);
}

__device__ __forceinline__ f16 rope_value(int rope, const f16* x, int d, int D, int step, const void* inv_freq) {
  if (rope == PTA_ROPE_LLAMA) return rope_llama_value(x, d, D, step, (const f16*)inv_freq);
  if (rope == PTA_ROPE_GLM2) return rope_glm2_value(x, d, D, step, (const float*)inv_freq);
  return x[d];
}

// FP8 KV cache (KVCacheOp with fp8 = true, custom_ops/kv_cache.cpp:43-74,103-105): rows are stored as F143
// bytes of value * 2^-kv_scale (the reference's metadata scale is the constant 1) and read back as
// decode(byte) * 2^kv_scale, which fp16 holds exactly.
__device__ __forceinline__ uint8_t kv8_encode(f16 v, int kv_scale) { return F8<0>::encode(ldexpf((float)v, -kv_scale)); }
__device__ __forceinline__ f16 kv8_round(f16 v, int kv_scale) {
  return (f16)ldexpf(F8<0>::decode(kv8_encode(v, kv_scale)), kv_scale);
}

__global__ __launch_bounds__(256) void qkv_rope_append_kernel(QkvArgs a) {
  const int D = a.D;
  const int per_b = (a.Hq + 2 * a.Hkv) * D;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.B * a.rows * per_b) return;
  const int row = idx / per_b;                // row of the projection outputs: sequence-major, then position
  const int b = row / a.rows;
  int r = idx % per_b;
  const int step = *a.step + row % a.rows;
  const int pos = step % a.max_len;
  if (r < a.Hq * D) {
    const int h = r / D, d = r % D;
    const f16* x = a.q + (size_t)row * a.q_stride + h * D;
    f16* y = a.q_out + ((size_t)row * a.Hq + h) * D;
    if (a.rope == PTA_ROPE_LLAMA) rope_llama(x, y, d, D, step, (const f16*)a.inv_freq);
    else if (a.rope == PTA_ROPE_GLM2) rope_glm2(x, y, d, D, step, (const float*)a.inv_freq);
    else y[d] = x[d];
    return;
  }
  r -= a.Hq * D;
  if (r < a.Hkv * D) {
    const int h = r / D, d = r % D;
    const f16* x = a.k + (size_t)row * a.k_stride + h * D;
    const size_t at = (((size_t)b * a.Hkv + h) * a.max_len + pos) * D + d;
    const f16 y = rope_value(a.rope, x, d, D, step, a.inv_freq);
    if (a.kv8) reinterpret_cast<uint8_t*>(a.kring)[at] = kv8_encode(y, a.kv_scale);
    else a.kring[at] = y;
    return;
  }
  r -= a.Hkv * D;
  const int h = r / D, d = r % D;
  const size_t at = (((size_t)b * a.Hkv + h) * a.max_len + pos) * D + d;
  const f16 y = a.v[(size_t)row * a.v_stride + h * D + d];
  if (a.kv8) reinterpret_cast<uint8_t*>(a.vring)[at] = kv8_encode(y, a.kv_scale);
  else a.vring[at] = y;
}

// The same for many rows (prompt passes): one workgroup per row.  The angles of a position are the same for every
// head, so their cosines and sines are worked out once per row into LDS (the kernel above evaluates both for every
// element), and every thread moves vectors of eight features.  The arithmetic per element is that of the kernel
// above, so both leave the same bits.
__global__ __launch_bounds__(256) void qkv_rope_append_rows_kernel(QkvArgs a) {
  __shared__ f16 cs[2][256];
  const int D = a.D, tid = threadIdx.x;
  const int row = blockIdx.x;
  const int b = row / a.rows;
  const int step = *a.step + row % a.rows;
  const int pos = step % a.max_len;
  if (a.rope == PTA_ROPE_LLAMA && tid < (D >> 1)) {
    const f16 ang = rope_llama_angle(step, ((const f16*)a.inv_freq)[tid]);
    cs[0][tid] = (f16)cosf((float)ang); cs[1][tid] = (f16)sinf((float)ang);
  } else if (a.rope == PTA_ROPE_GLM2 && tid < (D >> 2)) {
    const f16 ang = (f16)((float)step * ((const float*)a.inv_freq)[tid]);
    cs[0][tid] = (f16)cosf((float)ang); cs[1][tid] = (f16)sinf((float)ang);
  }
  __syncthreads();
  const int nq = a.Hq * D, nk = a.Hkv * D;
  for (int r = tid * 8; r < nq + 2 * nk; r += 256 * 8) {
    const int sect = r < nq ? 0 : (r < nq + nk ? 1 : 2);
    const int e = r - (sect == 0 ? 0 : (sect == 1 ? nq : nq + nk));
    const int h = e / D, d0 = e % D;
    const f16* x = sect == 0 ? a.q + (size_t)row * a.q_stride + h * D
                 : sect == 1 ? a.k + (size_t)row * a.k_stride + h * D : a.v + (size_t)row * a.v_stride + h * D;
    f16x8 y = *reinterpret_cast<const f16x8*>(x + d0);
    if (sect < 2 && a.rope == PTA_ROPE_LLAMA) {
      const int half = D >> 1;
      const bool low = d0 < half;
      const f16x8 o = *reinterpret_cast<const f16x8*>(x + (low ? d0 + half : d0 - half));
      const int i0 = low ? d0 : d0 - half;
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = rope_mix(y[j], low ? -o[j] : o[j], cs[0][i0 + j], cs[1][i0 + j]);
    } else if (sect < 2 && a.rope == PTA_ROPE_GLM2 && d0 < (D >> 1)) {
      const f16x8 xin = y;
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = rope_mix(xin[j], (j & 1) ? xin[j - 1] : -xin[j + 1], cs[0][(d0 + j) >> 1], cs[1][(d0 + j) >> 1]);
    }
    if (sect == 0) {
      *reinterpret_cast<f16x8*>(a.q_out + ((size_t)row * a.Hq + h) * D + d0) = y;
      continue;
    }
    const size_t at = (((size_t)b * a.Hkv + h) * a.max_len + pos) * D + d0;
    f16* ring = sect == 1 ? a.kring : a.vring;
    if (a.kv8) {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        lo |= (uint32_t)kv8_encode(y[j], a.kv_scale) << (8 * j);
        hi |= (uint32_t)kv8_encode(y[4 + j], a.kv_scale) << (8 * j);
      }
      *reinterpret_cast<uint2*>(reinterpret_cast<uint8_t*>(ring) + at) = make_uint2(lo, hi);
    } else {
      *reinterpret_cast<f16x8*>(ring + at) = y;
    }
  }
}

static int rope_append_rows(const char* name, const pta_half* q, const pta_half* k, const pta_half* v, int q_stride,
                            int k_stride, int v_stride, pta_half* q_out, pta_half* kv_ring, const int32_t* step,
                            const void* inv_freq, int B, int rows, int Hq, int Hkv, int D, int max_len, int rope,
                            int kv8, int kv_scale, pta_stream_t stream) {
  PTA_REQUIRE(q && k && v && q_out && kv_ring && step, "%s: null pointer", name);
  PTA_REQUIRE(!kv8 || (kv_scale >= -16 && kv_scale <= 16), "%s: kv_scale %d outside [-16, 16]", name, kv_scale);
  PTA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0, "%s: bad head counts %d/%d", name, Hq, Hkv);
  PTA_REQUIRE(D > 0 && D % 4 == 0 && max_len > 0, "%s: bad head size %d or max_len %d", name, D, max_len);
  PTA_REQUIRE(rows > 0 && rows <= max_len, "%s: rows = %d must lie in [1, max_len = %d]", name, rows, max_len);
  PTA_REQUIRE(rope == PTA_ROPE_NONE || rope == PTA_ROPE_LLAMA || rope == PTA_ROPE_GLM2, "%s: unknown rope mode %d", name, rope);
  PTA_REQUIRE(rope == PTA_ROPE_NONE || inv_freq, "%s: inv_freq is required for rotary modes", name);
  const size_t ring_elems = (size_t)B * Hkv * max_len * D;
  f16* vring = kv8 ? (f16*)((uint8_t*)kv_ring + ring_elems) : (f16*)kv_ring + ring_elems;
  QkvArgs a{(const f16*)q, (const f16*)k, (const f16*)v, q_stride, k_stride, v_stride, (f16*)q_out,
            (f16*)kv_ring, vring, step, inv_freq, B, Hq, Hkv, D, max_len, rope, rows, kv8 ? 1 : 0, kv_scale};
  const long total = (long)B * rows * (Hq + 2 * Hkv) * D;
  const bool vectors = D % 16 == 0 && D <= 512 && q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 &&
                       (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)q_out | (uintptr_t)kv_ring) & 15) == 0 &&
                       (!kv8 || ring_elems % 8 == 0);
  if (vectors && (long)B * rows >= 64)
    hipLaunchKernelGGL(qkv_rope_append_rows_kernel, dim3((unsigned)(B * rows)), dim3(256), 0, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL(qkv_rope_append_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, a);
  PTA_CHECK_LAUNCH(name);
  return PTA_OK;
}

extern "C" int pta_qkv_rope_append(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride,
                                   int k_stride, int v_stride, pta_half* q_out, pta_half* kv_ring,
                                   const int32_t* step, const void* inv_freq, int B, int Hq, int Hkv, int D,
                                   int max_len, int rope, pta_stream_t stream) {
  return rope_append_rows("pta_qkv_rope_append", q, k, v, q_stride, k_stride, v_stride, q_out, kv_ring, step, inv_freq, B, 1,
                          Hq, Hkv, D, max_len, rope, 0, 0, stream);
}

extern "C" int pta_prompt_rope_append(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride,
                                      int k_stride, int v_stride, pta_half* q_out, pta_half* kv_ring,
                                      const int32_t* step, const void* inv_freq, int B, int rows, int Hq, int Hkv,
                                      int D, int max_len, int rope, pta_stream_t stream) {
  return rope_append_rows("pta_prompt_rope_append", q, k, v, q_stride, k_stride, v_stride, q_out, kv_ring, step, inv_freq, B,
                          rows, Hq, Hkv, D, max_len, rope, 0, 0, stream);
}

extern "C" int pta_prompt_rope_append_f8(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride,
                                         int k_stride, int v_stride, pta_half* q_out, uint8_t* kv_ring,
                                         const int32_t* step, const void* inv_freq, int B, int rows, int Hq, int Hkv,
                                         int D, int max_len, int rope, int kv_scale, pta_stream_t stream) {
  return rope_append_rows("pta_prompt_rope_append_f8", q, k, v, q_stride, k_stride, v_stride, q_out, (pta_half*)kv_ring, step,
                          inv_freq, B, rows, Hq, Hkv, D, max_len, rope, 1, kv_scale, stream);
}

// ------------------------------------------------------------------------------------------
// Split-K decode attention with online softmax.
//
// The grid is fixed when the call is recorded (it may be replayed from a graph while the context
// grows), so the number of splits per (sequence, head) is chosen from the batch alone - enough
// workgroups to fill the machine, no more - and each split's range of cache rows is derived on the
// device from the current step: chunk = ceil(valid / nsplit), rounded up to a multiple of 16 rows
// and at least 64.  Splits beyond the valid rows exit at once.
// ------------------------------------------------------------------------------------------
constexpr int ATT_THREADS = 256;
constexpr int ATT_WAVES = ATT_THREADS / 64;
constexpr int ATT_UNROLL = 4;      // cache rows per lane group whose loads are in flight together

struct AttnArgs {
  const f16* q;       // [B, Hq, D]
  const f16* kring;   // [B*Hkv, max_len, D]
  const f16* vring;
  const int32_t* step;
  float* part;        // [B*Hq, nsplit, D + 2]: running max, denominator, numerator
  f16* out;           // [B, Hq*D]
  int B, Hq, Hkv, max_len, nsplit;
  int rows;           // consecutive positions per sequence (1 in the decode step): row r of a sequence sits at step + r
  int kv_scale;       // FP8 rings (KV8 kernels): rows hold F143 bytes of value * 2^-kv_scale
  int use_scale;
  f16 scale;
  // fused preparation (pta_decode_attention_qkv): raw projection rows instead of q [B, Hq, D]
  const f16* q_raw; const f16* k_raw; const f16* v_raw;
  int q_stride, k_stride, v_stride;
  f16* kring_w; f16* vring_w;
  const void* inv_freq;
  int rope;
  // when set: the context vector is left on the FP8 grid of this device exponent (the cast of the next Linear)
  const int32_t* out_fp8_scale;
  int out_fp8_format;
};

// the value stored for a context element: as computed, or rounded to the FP8 grid its consumer casts to
__device__ __forceinline__ f16 attn_result(const AttnArgs& a, f16 y) {
  return a.out_fp8_scale ? f8_grid_value(y, a.out_fp8_scale[0], a.out_fp8_format) : y;
}

__device__ __forceinline__ int attn_chunk(int valid, int nsplit) {
  int c = (valid + nsplit - 1) / nsplit;
  c = (c + 15) & ~15;
  return c < 64 ? 64 : c;
}

// Partial attention of one (sequence, query head) over one chunk of cache rows.
// LPP = D/8 lanes share a cache row (16 bytes each); a wave covers 64/LPP rows per load, and
// requests ATT_UNROLL such loads of K and of V before it uses the first.
// FUSED: the workgroup prepares its own operands from the raw projection rows - the rotary embedding
// of its query head, and, when its range of rows holds this step's position, of the new key; that
// key and the new value are used from LDS and written to the ring (by the first query head of the
// KV group), so that no separate preparation pass runs before the attention.
// KV8: the rings hold F143 bytes (8 per lane and row); they are decoded in registers and the power of two of the
// cache scale is applied to the fp32 score and numerator, which is exact.
template <int D, bool FUSED, bool KV8>
__global__ __launch_bounds__(ATT_THREADS) void attn_partial_kernel(AttnArgs a) {
  constexpr int LPP = D / 8;
  constexpr int PPW = 64 / LPP;
  constexpr int STRIDE = ATT_WAVES * PPW;
  __shared__ float sm_m[ATT_WAVES], sm_l[ATT_WAVES];
  __shared__ float sm_acc[ATT_WAVES][D];
  __shared__ __align__(16) f16 sm_qkv[FUSED ? 3 * D : 8];
  __shared__ __align__(16) uint8_t sm_code[FUSED && KV8 ? 2 * D : 16];
  const float kv_mul = KV8 ? ldexpf(1.0f, a.kv_scale) : 1.0f;
  const int split = blockIdx.x, bh = blockIdx.y;      // bh = (sequence * rows + row) * Hq + head
  const int step = *a.step + (bh / a.Hq) % a.rows;
  const int valid = step + 1 < a.max_len ? step + 1 : a.max_len;
  const int chunk = attn_chunk(valid, a.nsplit);
  const int c0 = split * chunk;
  if (c0 >= valid) return;
  const int c1 = c0 + chunk < valid ? c0 + chunk : valid;
  const int b = bh / (a.Hq * a.rows), h = bh % a.Hq;
  const int hk = h / (a.Hq / a.Hkv);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = lane / LPP, sub = lane % LPP;
  const int d0 = sub * 8;

  const int pos = step % a.max_len;
  bool owner = false;
  if constexpr (FUSED) {
    owner = pos >= c0 && pos < c1;
    for (int t = threadIdx.x; t < (owner ? 3 * D : D); t += ATT_THREADS) {
      const int which = t / D, d = t % D;
      const f16* x = which == 0 ? a.q_raw + (size_t)b * a.q_stride + h * D
                                : (which == 1 ? a.k_raw + (size_t)b * a.k_stride + hk * D : a.v_raw + (size_t)b * a.v_stride + hk * D);
      f16 y = which == 2 ? x[d] : rope_value(a.rope, x, d, D, step, a.inv_freq);
      if (KV8 && which != 0) {          // the new row as the cache will hold it: its byte, and decode(byte) for this pass
        const uint8_t code = kv8_encode(y, a.kv_scale);
        sm_code[t - D] = code;
        y = (f16)F8<0>::decode(code);
      }
      sm_qkv[t] = y;
    }
    __syncthreads();
    if (owner && h % (a.Hq / a.Hkv) == 0) {
      for (int t = threadIdx.x; t < 2 * D; t += ATT_THREADS) {
        const size_t at = (((size_t)b * a.Hkv + hk) * a.max_len + pos) * D + t % D;
        if (KV8) reinterpret_cast<uint8_t*>(t < D ? a.kring_w : a.vring_w)[at] = sm_code[t];
        else (t < D ? a.kring_w : a.vring_w)[at] = sm_qkv[D + t];
      }
    }
  }
  float qf[8];
  {
    const f16x8 q8 = FUSED ? *reinterpret_cast<const f16x8*>(sm_qkv + d0)
                           : *reinterpret_cast<const f16x8*>(a.q + (size_t)bh * D + d0);
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[e] = (float)q8[e];
  }
  const size_t ring_at = ((size_t)b * a.Hkv + hk) * a.max_len * D + d0;
  const f16* kb = a.kring + ring_at;
  const f16* vb = a.vring + ring_at;
  const uint8_t* kb8 = reinterpret_cast<const uint8_t*>(a.kring) + ring_at;
  const uint8_t* vb8 = reinterpret_cast<const uint8_t*>(a.vring) + ring_at;

  float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;

  for (int p0 = c0 + wave * PPW + grp; p0 < c1 + grp; p0 += STRIDE * ATT_UNROLL) {
    f16x8 k8[ATT_UNROLL], v8[ATT_UNROLL];
    bool on[ATT_UNROLL];
#pragma unroll
    for (int u = 0; u < ATT_UNROLL; ++u) {
      const int p = p0 + u * STRIDE;
      on[u] = p < c1;
      const int pc = on[u] ? p : c1 - 1;
      if (FUSED && pc == pos) {      // this step's row: its ring copy is being written by this launch
        k8[u] = *reinterpret_cast<const f16x8*>(sm_qkv + D + d0);
        v8[u] = *reinterpret_cast<const f16x8*>(sm_qkv + 2 * D + d0);
      } else if constexpr (KV8) {
        const u32x2 kr = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(kb8 + (size_t)pc * D));
        const u32x2 vr = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(vb8 + (size_t)pc * D));
        k8[u] = f143_decode8(kr[0], kr[1]);
        v8[u] = f143_decode8(vr[0], vr[1]);
      } else {
        k8[u] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(kb + (size_t)pc * D));
        v8[u] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(vb + (size_t)pc * D));
      }
    }
    float x[ATT_UNROLL];
    float mn = m;
#pragma unroll
    for (int u = 0; u < ATT_UNROLL; ++u) {
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s = __builtin_fmaf(qf[e], (float)k8[u][e], s);
      s = lane_group_sum<LPP>(s);
      if (KV8) s *= kv_mul;
      f16 s16 = (f16)s;                       // fp16 output of the q.K^T MatMul
      if (a.use_scale) s16 = s16 * a.scale;   // fp16 multiply by fp16(1/sqrt(D))
      x[u] = on[u] ? (float)s16 : -INFINITY;
      mn = fmaxf(mn, x[u]);
    }
    if (mn != -INFINITY) {                    // some row of this group so far is valid
      const float corr = m == -INFINITY ? 0.f : __expf(m - mn);
      l *= corr;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] *= corr;
#pragma unroll
      for (int u = 0; u < ATT_UNROLL; ++u) {
        const float pe = on[u] ? __expf(x[u] - mn) : 0.f;
        l += pe;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(pe, (float)v8[u][e], acc[e]);
      }
      m = mn;
    }
  }

  // the row groups of a wave merge in registers, the waves in LDS
#pragma unroll
  for (int o = LPP; o < 64; o <<= 1) {
    const float mo = __shfl_xor(m, o, 64), lo = __shfl_xor(l, o, 64);
    const float mn = fmaxf(m, mo);
    const float ca = m == -INFINITY ? 0.f : __expf(m - mn);
    const float cb = mo == -INFINITY ? 0.f : __expf(mo - mn);
    l = l * ca + lo * cb;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = acc[e] * ca + __shfl_xor(acc[e], o, 64) * cb;
    m = mn;
  }
  if (lane == 0) { sm_m[wave] = m; sm_l[wave] = l; }
  if (lane < LPP) {
#pragma unroll
    for (int e = 0; e < 8; ++e) sm_acc[wave][d0 + e] = acc[e];
  }
  __syncthreads();
  float* out = a.part + ((size_t)bh * a.nsplit + split) * (D + 2);
  for (int d = threadIdx.x; d < D; d += ATT_THREADS) {
    float M = -INFINITY;
#pragma unroll
    for (int i = 0; i < ATT_WAVES; ++i) M = fmaxf(M, sm_m[i]);
    float L = 0.f, A = 0.f;
#pragma unroll
    for (int i = 0; i < ATT_WAVES; ++i) {
      const float w = sm_m[i] == -INFINITY ? 0.f : __expf(sm_m[i] - M);
      L = __builtin_fmaf(sm_l[i], w, L);
      A = __builtin_fmaf(sm_acc[i][d], w, A);
    }
    if (a.nsplit == 1) {                     // the only split of this (row, head): the context vector itself
      a.out[(size_t)bh * D + d] = attn_result(a, (f16)((KV8 ? A * kv_mul : A) / L));
      continue;
    }
    out[2 + d] = KV8 ? A * kv_mul : A;
    if (d == 0) { out[0] = M; out[1] = L; }
  }
}

template <int D>
__global__ __launch_bounds__(D) void attn_combine_kernel(AttnArgs a) {
  const int bh = blockIdx.x, d = threadIdx.x;
  const int step = *a.step + (bh / a.Hq) % a.rows;
  const int valid = step + 1 < a.max_len ? step + 1 : a.max_len;
  const int chunk = attn_chunk(valid, a.nsplit);
  const int nact = (valid + chunk - 1) / chunk;
  const float* p = a.part + (size_t)bh * a.nsplit * (D + 2);
  // eight chunks at a time: their maxima, denominators and numerators are requested together (a chunk past the last
  // reads the last one again and counts for nothing); the order of the sums is that of one chunk after the other
  float M = -INFINITY;
  for (int s0 = 0; s0 < nact; s0 += 8) {
    float mv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) mv[i] = p[(size_t)(s0 + i < nact ? s0 + i : nact - 1) * (D + 2)];
#pragma unroll
    for (int i = 0; i < 8; ++i) M = fmaxf(M, mv[i]);
  }
  float L = 0.f, A = 0.f;
  for (int s0 = 0; s0 < nact; s0 += 8) {
    float mv[8], lv[8], av[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float* ps = p + (size_t)(s0 + i < nact ? s0 + i : nact - 1) * (D + 2);
      mv[i] = ps[0]; lv[i] = ps[1]; av[i] = ps[2 + d];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (s0 + i < nact) {
        const float w = __expf(mv[i] - M);
        L = __builtin_fmaf(lv[i], w, L);
        A = __builtin_fmaf(av[i], w, A);
      }
    }
  }
  a.out[(size_t)bh * D + d] = attn_result(a, (f16)(A / L));
}

// splits per (sequence, head): about 1024 workgroups in all, never more than one per 64 cache rows
// (which is what the workspace is sized for); from 512 (sequence, head) pairs on, one workgroup each, which
// writes the context vector itself and saves the merging launch
static int attn_splits(int B, int Hq, int max_len) {
  const int cap = (max_len + 63) / 64;
  if (B * Hq >= 512) return 1;
  // a ring of up to 256 rows: one workgroup walks it in four rounds of loads, which costs less than the merging launch
  // (GPT-2 small, 12 heads, ring of 128: 0.312 -> 0.285 ms per token)
  if (max_len <= 256) return 1;
  int n = (1024 + B * Hq - 1) / (B * Hq);
  n = n < 1 ? 1 : n;
  return n > cap ? cap : n;
}

// ------------------------------------------------------------------------------------------
// Attention of many rows at once (the prompt passes) on the matrix unit, head size D = 64 or 128, fp16 or F143 cache.
// One workgroup of four waves per (sequence, query head, 64 or 128 rows of the pass); wave w owns one or two
// groups of 16 rows.  The cache rows go through LDS 32 at a time, K as it lies, V transposed; per step a wave computes,
// for each of its row groups,
//   S^T = K Q^T     (two 16 x 16 tiles, D / 32 MFMAs each: lane l then holds the scores of query row l % 16 for
//                    cache rows (l / 16) * 4 + 0..3 of each tile - which IS the layout of an A operand whose
//                    k index runs over those eight cache rows),
//   the roundings of the reference on the scores (fp16 MatMul output, fp16 multiply by 1/sqrt(D)), the online
//   softmax in fp32 per query row (partners: lanes l ^ 16, l ^ 32), probabilities rounded to fp16 (the
//   reference's softmax output is fp16),
//   O += P V        (D / 16 tiles of 16 x 16 over the head size, B operands from the transposed V rows);
// every K and V operand read from LDS serves all row groups of the wave.
// Row r of the pass sits at position step + r and attends to cache rows [0, min(step + r + 1, max_len)), as in
// attn_partial_kernel.  Outputs differ from that kernel in the last bits (another summation order, fp16
// probabilities); both are held to 1e-2 against the oracle.
// ------------------------------------------------------------------------------------------
constexpr int PA_THREADS = 256;
constexpr int PA_VSTRIDE = 32 + 8;       // halves per staged row of V^T

// V^T in LDS: feature d, cache row p (of the 32 staged) at d * PA_VSTRIDE + (((p / 2) ^ (2 * (d / 16))) * 2 + p % 2.
// Exchanging the dwords of a row by its feature group spreads the 2-byte stores of the transposition (which go
// down the features, 8 * PA_VSTRIDE halves apart) over the banks; pairs of dwords stay together for the 8-byte reads.
__device__ __forceinline__ int pa_vt_at(int d, int p) { return d * PA_VSTRIDE + ((((p >> 1) ^ ((d >> 4) << 1))) << 1) + (p & 1); }

// PA_RG: row groups of 16 per wave (a workgroup takes 4 * PA_RG * 16 rows of the pass).  Two where that still gives every
// compute unit two workgroups or more (a wave's dependent chains - MFMA, maximum, exponentials, MFMA - need company
// on their SIMD), else one.
// KV8: the rings hold F143 bytes of value * 2^-kv_scale (as in attn_partial_kernel): a thread loads eight bytes where
// it loads eight halves of an fp16 ring, decodes them on their way into LDS, and the power of two goes to the fp32
// scores before they are rounded and to the result.
template <int D, int PA_RG, bool KV8 = false>
__global__ __launch_bounds__(PA_THREADS) void prompt_attention_mfma_kernel(AttnArgs a) {
  static_assert(D == 64 || D == 128, "head size");
  constexpr int PA_KSTRIDE = D + 8;        // halves per staged K row
  constexpr int NV = D / 64;               // 16-byte vectors of K (and of V) per thread and step: 32 rows of D / 8
  const float kv_mul = KV8 ? ldexpf(1.0f, a.kv_scale) : 1.0f;
  constexpr int PA_ROWS = 4 * PA_RG * 16;
  __shared__ __align__(16) f16 ks[32 * PA_KSTRIDE];
  __shared__ __align__(16) f16 vt[D * PA_VSTRIDE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int h = blockIdx.y, b = blockIdx.z;
  const int kvh = h / (a.Hq / a.Hkv);
  const int step0 = *a.step;
  const int r0 = (int)blockIdx.x * PA_ROWS + wave * (PA_RG * 16);          // first row of this wave within the pass
  auto valid_of = [&](int row) { const int v = step0 + row + 1; return row < a.rows ? (v < a.max_len ? v : a.max_len) : 0; };
  f16x8 qf[PA_RG][D / 32];
  int my_valid[PA_RG];
#pragma unroll
  for (int g = 0; g < PA_RG; ++g) {
    const int qrow = r0 + g * 16 + (lane & 15);
    my_valid[g] = valid_of(qrow);
#pragma unroll
    for (int m = 0; m < D / 32; ++m) {
      qf[g][m] = f16x8{};
      if (qrow < a.rows) qf[g][m] = *reinterpret_cast<const f16x8*>(a.q + (((size_t)b * a.rows + qrow) * a.Hq + h) * D + m * 32 + (lane >> 4) * 8);
    }
  }
  const int last_of_wave = r0 + PA_RG * 16 - 1 < a.rows ? r0 + PA_RG * 16 - 1 : a.rows - 1;
  const int wave_valid = r0 < a.rows ? valid_of(last_of_wave) : 0;
  const int last_of_wg = (int)blockIdx.x * PA_ROWS + PA_ROWS - 1 < a.rows ? (int)blockIdx.x * PA_ROWS + PA_ROWS - 1 : a.rows - 1;
  const int wg_valid = valid_of(last_of_wg);
  const f16* kbase = a.kring + ((size_t)b * a.Hkv + kvh) * a.max_len * D;
  const f16* vbase = a.vring + ((size_t)b * a.Hkv + kvh) * a.max_len * D;
  const uint8_t* kbase8 = reinterpret_cast<const uint8_t*>(a.kring) + ((size_t)b * a.Hkv + kvh) * a.max_len * D;
  const uint8_t* vbase8 = reinterpret_cast<const uint8_t*>(a.vring) + ((size_t)b * a.Hkv + kvh) * a.max_len * D;

  float run_m[PA_RG], run_l[PA_RG];
  f32x4 o[PA_RG][D / 16];
#pragma unroll
  for (int g = 0; g < PA_RG; ++g) {
    run_m[g] = -INFINITY; run_l[g] = 0.f;
#pragma unroll
    for (int jd = 0; jd < D / 16; ++jd) o[g][jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // cache rows p .. p + 31: 32 * D / 8 vectors of 16 bytes each of K and V, NV per thread; they are requested one step
  // ahead, so that their way from memory runs beside the step's arithmetic
  f16x8 kv[NV], vv[NV];
  u32x2 kq[NV], vq[NV];       // KV8: the bytes as stored
  auto request = [&](int p) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = (int)threadIdx.x + i * PA_THREADS;
      const int row = c / (D / 8), col = (c % (D / 8)) * 8;
      kv[i] = f16x8{}; vv[i] = f16x8{};
      kq[i] = u32x2{0, 0}; vq[i] = u32x2{0, 0};      // (the byte 0 is the value 0)
      if (p + row < wg_valid) {
        if constexpr (KV8) {
          kq[i] = *reinterpret_cast<const u32x2*>(kbase8 + (size_t)(p + row) * D + col);
          vq[i] = *reinterpret_cast<const u32x2*>(vbase8 + (size_t)(p + row) * D + col);
        } else {
          kv[i] = *reinterpret_cast<const f16x8*>(kbase + (size_t)(p + row) * D + col);
          vv[i] = *reinterpret_cast<const f16x8*>(vbase + (size_t)(p + row) * D + col);
        }
      }
    }
  };
  request(0);
  for (int p0 = 0; p0 < wg_valid; p0 += 32) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = (int)threadIdx.x + i * PA_THREADS;
      const int row = c / (D / 8), col = (c % (D / 8)) * 8;
      if constexpr (KV8) {
        kv[i] = f143_decode8(kq[i][0], kq[i][1]);
        vv[i] = f143_decode8(vq[i][0], vq[i][1]);
      }
      *reinterpret_cast<f16x8*>(ks + row * PA_KSTRIDE + col) = kv[i];
#pragma unroll
      for (int e = 0; e < 8; ++e) vt[pa_vt_at(col + e, row)] = vv[i][e];
    }
    if (p0 + 32 < wg_valid) request(p0 + 32);
    __syncthreads();
    if (p0 >= wave_valid) continue;
    f32x4 sc[PA_RG][2];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
      for (int g = 0; g < PA_RG; ++g) sc[g][hh] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int m = 0; m < D / 32; ++m) {
        const f16x8 kf = *reinterpret_cast<const f16x8*>(ks + (hh * 16 + (lane & 15)) * PA_KSTRIDE + m * 32 + (lane >> 4) * 8);
#pragma unroll
        for (int g = 0; g < PA_RG; ++g) sc[g][hh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[g][m], sc[g][hh], 0, 0, 0);
      }
    }
    f16x8 pa[PA_RG];
    float cr[PA_RG][4];
#pragma unroll
    for (int g = 0; g < PA_RG; ++g) {
      float x[8];
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          f16 s16 = (f16)(KV8 ? sc[g][hh][r] * kv_mul : sc[g][hh][r]);      // fp16 output of the q.K^T MatMul
          if (a.use_scale) s16 = s16 * a.scale;       // fp16 multiply by fp16(1/sqrt(D))
          const int pos = p0 + hh * 16 + (lane >> 4) * 4 + r;
          x[hh * 4 + r] = pos < my_valid[g] ? (float)s16 : -INFINITY;
        }
      float mx = x[0];
#pragma unroll
      for (int e = 1; e < 8; ++e) mx = fmaxf(mx, x[e]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float new_m = fmaxf(run_m[g], mx);
      const float corr = run_m[g] == -INFINITY ? 0.f : __expf(run_m[g] - new_m);
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pe = x[e] == -INFINITY ? 0.f : __expf(x[e] - new_m);
        psum += pe;
        pa[g][e] = (f16)pe;
      }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      run_l[g] = run_l[g] * corr + psum;
      run_m[g] = new_m;
      // the accumulators' rows are query rows (lane / 16) * 4 + r: their correction factors sit in lanes of that index
#pragma unroll
      for (int r = 0; r < 4; ++r) cr[g][r] = __shfl(corr, (lane >> 4) * 4 + r, 64);
    }
#pragma unroll
    for (int jd = 0; jd < D / 16; ++jd) {
      // cache rows (lane / 16) * 4 + 0..3 and 16 + the same of feature jd * 16 + lane % 16
      const int d = jd * 16 + (lane & 15);
      const f16x4 v0 = *reinterpret_cast<const f16x4*>(vt + pa_vt_at(d, (lane >> 4) * 4));
      const f16x4 v1 = *reinterpret_cast<const f16x4*>(vt + pa_vt_at(d, 16 + (lane >> 4) * 4));
      const f16x8 vb = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
      for (int g = 0; g < PA_RG; ++g) {
#pragma unroll
        for (int r = 0; r < 4; ++r) o[g][jd][r] *= cr[g][r];
        o[g][jd] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa[g], vb, o[g][jd], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int g = 0; g < PA_RG; ++g) {
    float lr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) lr[r] = __shfl(run_l[g], (lane >> 4) * 4 + r, 64);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = r0 + g * 16 + (lane >> 4) * 4 + r;
      if (row >= a.rows) continue;
#pragma unroll
      for (int jd = 0; jd < D / 16; ++jd)
        a.out[(((size_t)b * a.rows + row) * a.Hq + h) * D + jd * 16 + (lane & 15)] =
            attn_result(a, (f16)((KV8 ? o[g][jd][r] * kv_mul : o[g][jd][r]) / lr[r]));
    }
  }
}

// ------------------------------------------------------------------------------------------
// Decode attention of grouped heads on the matrix unit: sixteen query heads share a KV head (ChatGLM2: 32 query
// heads on 2, chatglm2/attention.py:166-302), so the sixteen heads of a group are the sixteen columns of one MFMA
// tile and a workgroup reads the group's cache rows once for all of them - attn_partial_kernel reads them once per
// query head, sixteen times through the compute units.  One workgroup of four waves per (sequence, KV head, chunk of
// cache rows); wave w takes the chunk's rows 32 w .. 32 w + 31, then 128 further on.  Per step of 32 rows, as in
// prompt_attention_mfma_kernel with the query heads where that kernel has query rows:
//   S^T = K Q^T   (K rows straight from the ring as A operands: lane l holds row l % 16, features (l / 16) * 8 + 0..7
//                  of each 32; Q, rotated, from LDS), the reference's roundings of the scores, the online softmax per
//   head in fp32 (partners: lanes l ^ 16, l ^ 32), probabilities rounded to fp16,
//   O += P V      (V transposed through 10 KiB of LDS that belong to the wave).
// The waves' states meet in LDS; the chunk's (maximum, denominator, numerator) go to the workspace in
// attn_partial_kernel's layout, for attn_combine_kernel.  FUSED as there: the workgroup rotates its sixteen query
// heads itself, and the one whose chunk holds this step's position rotates the new key, uses it and the new value
// from LDS, and writes both to the ring.
// ------------------------------------------------------------------------------------------
constexpr int GQA_HEADS = 16;

template <int D, bool FUSED>
__global__ __launch_bounds__(256) void attn_gqa_partial_kernel(AttnArgs a) {
  static_assert(D == 64 || D == 128, "head size");
  constexpr int QS = D + 8;                         // halves per staged query row
  constexpr int VPR = D / 8;                        // 16-byte vectors per row
  __shared__ f16 cs[2][64];
  __shared__ __align__(16) f16 sm_q[GQA_HEADS * QS];
  __shared__ __align__(16) f16 sm_kv[2 * D];
  __shared__ __align__(16) f16 vt_all[4 * D * PA_VSTRIDE];       // per wave: V^T of its 32 rows; after the loop: the waves' numerators
  __shared__ float sm_m[4][GQA_HEADS], sm_l[4][GQA_HEADS];
  static_assert(4 * D * PA_VSTRIDE * 2 >= 4 * GQA_HEADS * D * 4, "the numerators fit the staging area");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.x, bg = blockIdx.y;
  const int b = bg / a.Hkv, g = bg % a.Hkv;
  const int step = *a.step;
  const int valid = step + 1 < a.max_len ? step + 1 : a.max_len;
  const int chunk = attn_chunk(valid, a.nsplit);
  const int c0 = split * chunk;
  if (c0 >= valid) return;
  const int c1 = c0 + chunk < valid ? c0 + chunk : valid;
  const int pos = step % a.max_len;
  const bool owner = FUSED && pos >= c0 && pos < c1;
  const size_t ring_at = ((size_t)b * a.Hkv + g) * a.max_len * D;
  const f16* kbase = a.kring + ring_at;
  const f16* vbase = a.vring + ring_at;

  // a step's rows: K as the A operands of its two tiles (lane l: row l % 16, features (l / 16) * 8 + 0..7 of each 32),
  // V for the transposition; rows past the chunk read its last row (finite values under a probability of zero).  The
  // first step's rows are requested before the queries are prepared: they do not depend on them.
  f16x8 kf[2][D / 32], vv[VPR / 2];
  auto request = [&](int p0) {
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int row = p0 + hh * 16 + (lane & 15);
      const int rc = row < c1 ? row : c1 - 1;
#pragma unroll
      for (int m = 0; m < D / 32; ++m)
        kf[hh][m] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(kbase + (size_t)rc * D + m * 32 + (lane >> 4) * 8));
    }
#pragma unroll
    for (int i = 0; i < VPR / 2; ++i) {
      const int c = lane + i * 64;
      const int row = c / VPR, col = (c % VPR) * 8;
      const int rc = p0 + row < c1 ? p0 + row : c1 - 1;
      vv[i] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(vbase + (size_t)rc * D + col));
    }
  };
  if (c0 + wave * 32 < c1) request(c0 + wave * 32);

  // the queries of the sixteen heads (and, in the chunk that holds this step's position, the new key and value): one
  // vector of eight per thread, a second one for 2 * D / 8 threads of that chunk; requested before the angles are
  // worked out
  const int nvec = GQA_HEADS * VPR + (owner ? 2 * VPR : 0);
  int p_sect[2], p_h[2], p_d0[2];
  bool p_on[2];
  f16x8 p_y[2], p_o[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int vi = tid + u * 256;
    p_on[u] = vi < nvec;
    p_sect[u] = vi < GQA_HEADS * VPR ? 0 : 1 + (vi - GQA_HEADS * VPR) / VPR;
    p_h[u] = p_sect[u] == 0 ? vi / VPR : 0;
    p_d0[u] = (vi % VPR) * 8;
    p_y[u] = f16x8{}; p_o[u] = f16x8{};
    if (!p_on[u]) continue;
    const f16* x;
    if constexpr (FUSED)
      x = p_sect[u] == 0 ? a.q_raw + (size_t)b * a.q_stride + (size_t)(g * GQA_HEADS + p_h[u]) * D
        : p_sect[u] == 1 ? a.k_raw + (size_t)b * a.k_stride + (size_t)g * D : a.v_raw + (size_t)b * a.v_stride + (size_t)g * D;
    else
      x = a.q + ((size_t)b * a.Hq + g * GQA_HEADS + p_h[u]) * D;
    p_y[u] = *reinterpret_cast<const f16x8*>(x + p_d0[u]);
    if (FUSED && p_sect[u] < 2 && a.rope == PTA_ROPE_LLAMA)
      p_o[u] = *reinterpret_cast<const f16x8*>(x + (p_d0[u] < (D >> 1) ? p_d0[u] + (D >> 1) : p_d0[u] - (D >> 1)));
  }
  if constexpr (FUSED) {
    // the angles of this position, once for all heads (the arithmetic of qkv_rope_append_rows_kernel: the same bits)
    if (a.rope == PTA_ROPE_LLAMA && tid < (D >> 1)) {
      const f16 ang = rope_llama_angle(step, ((const f16*)a.inv_freq)[tid]);
      cs[0][tid] = (f16)cosf((float)ang); cs[1][tid] = (f16)sinf((float)ang);
    } else if (a.rope == PTA_ROPE_GLM2 && tid < (D >> 2)) {
      const f16 ang = (f16)((float)step * ((const float*)a.inv_freq)[tid]);
      cs[0][tid] = (f16)cosf((float)ang); cs[1][tid] = (f16)sinf((float)ang);
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    if (!p_on[u]) continue;
    const int sect = p_sect[u], d0 = p_d0[u];
    f16x8 y = p_y[u];
    if constexpr (FUSED) {
      if (sect < 2 && a.rope == PTA_ROPE_LLAMA) {
        const bool low = d0 < (D >> 1);
        const int i0 = low ? d0 : d0 - (D >> 1);
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = rope_mix(y[j], low ? -p_o[u][j] : p_o[u][j], cs[0][i0 + j], cs[1][i0 + j]);
      } else if (sect < 2 && a.rope == PTA_ROPE_GLM2 && d0 < (D >> 1)) {
        const f16x8 xin = y;
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = rope_mix(xin[j], (j & 1) ? xin[j - 1] : -xin[j + 1], cs[0][(d0 + j) >> 1], cs[1][(d0 + j) >> 1]);
      }
    }
    if (sect == 0) {
      *reinterpret_cast<f16x8*>(sm_q + p_h[u] * QS + d0) = y;
    } else {
      *reinterpret_cast<f16x8*>(sm_kv + (sect - 1) * D + d0) = y;
      *reinterpret_cast<f16x8*>((sect == 1 ? a.kring_w : a.vring_w) + ring_at + (size_t)pos * D + d0) = y;
    }
  }
  __syncthreads();
  f16x8 qf[D / 32];
#pragma unroll
  for (int m = 0; m < D / 32; ++m) qf[m] = *reinterpret_cast<const f16x8*>(sm_q + (lane & 15) * QS + m * 32 + (lane >> 4) * 8);

  f16* vt = vt_all + wave * (D * PA_VSTRIDE);
  float run_m = -INFINITY, run_l = 0.f;
  f32x4 o[D / 16];
#pragma unroll
  for (int jd = 0; jd < D / 16; ++jd) o[jd] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int p0 = c0 + wave * 32; p0 < c1; p0 += 128) {
    // this step's position comes from LDS (its ring copy is being written by this launch)
    if (owner) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = p0 + hh * 16 + (lane & 15);
        if ((row < c1 ? row : c1 - 1) == pos) {
#pragma unroll
          for (int m = 0; m < D / 32; ++m) kf[hh][m] = *reinterpret_cast<const f16x8*>(sm_kv + m * 32 + (lane >> 4) * 8);
        }
      }
#pragma unroll
      for (int i = 0; i < VPR / 2; ++i) {
        const int c = lane + i * 64;
        const int row = c / VPR, col = (c % VPR) * 8;
        if ((p0 + row < c1 ? p0 + row : c1 - 1) == pos) vv[i] = *reinterpret_cast<const f16x8*>(sm_kv + D + col);
      }
    }
    f32x4 sc[2];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      sc[hh] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int m = 0; m < D / 32; ++m) sc[hh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[hh][m], qf[m], sc[hh], 0, 0, 0);
    }
    // (the wave's own staging area: its LDS accesses complete in the order of their issue)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < VPR / 2; ++i) {
      const int c = lane + i * 64;
      const int row = c / VPR, col = (c % VPR) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) vt[pa_vt_at(col + e, row)] = vv[i][e];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (p0 + 128 < c1) request(p0 + 128);           // the next step's rows travel during this step's softmax and products
    float x[8];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        f16 s16 = (f16)sc[hh][r];                   // fp16 output of the q.K^T MatMul
        if (a.use_scale) s16 = s16 * a.scale;       // fp16 multiply by fp16(1/sqrt(D))
        const int row = p0 + hh * 16 + (lane >> 4) * 4 + r;
        x[hh * 4 + r] = row < c1 ? (float)s16 : -INFINITY;
      }
    float mx = x[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) mx = fmaxf(mx, x[e]);
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float new_m = fmaxf(run_m, mx);           // (finite: the step's first row lies inside the chunk)
    const float corr = run_m == -INFINITY ? 0.f : __expf(run_m - new_m);
    float psum = 0.f;
    f16x8 pa;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = x[e] == -INFINITY ? 0.f : __expf(x[e] - new_m);
      psum += pe;
      pa[e] = (f16)pe;
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    run_l = run_l * corr + psum;
    run_m = new_m;
    // the accumulators' rows are heads (lane / 16) * 4 + r: their correction factors sit in the lanes of that index
    float cr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, (lane >> 4) * 4 + r, 64);
#pragma unroll
    for (int jd = 0; jd < D / 16; ++jd) {
      const int d = jd * 16 + (lane & 15);
      const f16x4 v0 = *reinterpret_cast<const f16x4*>(vt + pa_vt_at(d, (lane >> 4) * 4));
      const f16x4 v1 = *reinterpret_cast<const f16x4*>(vt + pa_vt_at(d, 16 + (lane >> 4) * 4));
      const f16x8 vb = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
      for (int r = 0; r < 4; ++r) o[jd][r] *= cr[r];
      o[jd] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vb, o[jd], 0, 0, 0);
    }
  }

  // the waves' states meet in LDS (the staging areas are done with)
  __syncthreads();
  float* sm_o = reinterpret_cast<float*>(vt_all);        // [4][GQA_HEADS][D]
  if (lane < GQA_HEADS) { sm_m[wave][lane] = run_m; sm_l[wave][lane] = run_l; }
#pragma unroll
  for (int jd = 0; jd < D / 16; ++jd)
#pragma unroll
    for (int r = 0; r < 4; ++r) sm_o[((size_t)wave * GQA_HEADS + (lane >> 4) * 4 + r) * D + jd * 16 + (lane & 15)] = o[jd][r];
  __syncthreads();
  for (int idx = tid; idx < GQA_HEADS * D; idx += 256) {
    const int h = idx / D, d = idx % D;
    float M = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) M = fmaxf(M, sm_m[i][h]);
    float L = 0.f, A = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float w = sm_m[i][h] == -INFINITY ? 0.f : __expf(sm_m[i][h] - M);
      L = __builtin_fmaf(sm_l[i][h], w, L);
      A = __builtin_fmaf(sm_o[((size_t)i * GQA_HEADS + h) * D + d], w, A);
    }
    const size_t bh = (size_t)b * a.Hq + g * GQA_HEADS + h;
    if (a.nsplit == 1) {                     // the only chunk: the context vector itself
      a.out[bh * D + d] = attn_result(a, (f16)(A / L));
      continue;
    }
    float* out = a.part + (bh * a.nsplit + split) * (D + 2);
    out[2 + d] = A;
    if (d == 0) { out[0] = M; out[1] = L; }
  }
}

// chunks per (sequence, KV head) for attn_gqa_partial_kernel: about 128 workgroups in all (ChatGLM2-6B, 8 sequences,
// contexts 512..1023: 2.27 ms per step with 128, 2.29 with 256, 2.33 with 512, 2.34 with 64), never more than one per
// 64 cache rows
static int attn_gqa_splits(int B, int Hkv, int max_len) {
  const int cap = (max_len + 63) / 64;
  if (max_len <= 256) return 1;
  int n = (128 + B * Hkv - 1) / (B * Hkv);
  n = n < 1 ? 1 : n;
  return n > cap ? cap : n;
}

extern "C" size_t pta_decode_attention_workspace_bytes(int B, int Hq, int D, int max_len) {
  if (B <= 0 || Hq <= 0 || D <= 0 || max_len <= 0) return 0;
  const int chunk = 64;
  const int nsplit = (max_len + chunk - 1) / chunk;
  return (size_t)B * Hq * nsplit * (D + 2) * sizeof(float);
}

// whether a decode-attention launch goes to attn_gqa_partial_kernel: one row per sequence, sixteen query heads per KV
// head, an fp16 ring, and 16-byte vectors wherever that kernel reads its operands
static bool attn_gqa_fits(const AttnArgs& a, bool kv8, bool fused) {
  if (kv8 || a.rows != 1 || a.Hq != GQA_HEADS * a.Hkv) return false;
  if (fused)
    return a.q_stride % 8 == 0 && a.k_stride % 8 == 0 && a.v_stride % 8 == 0 &&
           (((uintptr_t)a.q_raw | (uintptr_t)a.k_raw | (uintptr_t)a.v_raw) & 15) == 0;
  return true;
}

template <bool FUSED>
static void launch_attention(const AttnArgs& a_in, int D, bool kv8, int heads_rows, hipStream_t s) {
  if (attn_gqa_fits(a_in, kv8, FUSED)) {
    AttnArgs a = a_in;
    a.nsplit = attn_gqa_splits(a.B, a.Hkv, a.max_len);
    const dim3 grid(a.nsplit, a.B * a.Hkv);
    if (D == 128) {
      hipLaunchKernelGGL((attn_gqa_partial_kernel<128, FUSED>), grid, dim3(256), 0, s, a);
      if (a.nsplit > 1) hipLaunchKernelGGL(attn_combine_kernel<128>, dim3(heads_rows), dim3(128), 0, s, a);
    } else {
      hipLaunchKernelGGL((attn_gqa_partial_kernel<64, FUSED>), grid, dim3(256), 0, s, a);
      if (a.nsplit > 1) hipLaunchKernelGGL(attn_combine_kernel<64>, dim3(heads_rows), dim3(64), 0, s, a);
    }
    return;
  }
  const AttnArgs& a = a_in;
  dim3 grid(a.nsplit, heads_rows);
  if (D == 128) {
    if (kv8) hipLaunchKernelGGL((attn_partial_kernel<128, FUSED, true>), grid, dim3(ATT_THREADS), 0, s, a);
    else hipLaunchKernelGGL((attn_partial_kernel<128, FUSED, false>), grid, dim3(ATT_THREADS), 0, s, a);
    if (a.nsplit > 1) hipLaunchKernelGGL(attn_combine_kernel<128>, dim3(heads_rows), dim3(128), 0, s, a);
  } else {
    if (kv8) hipLaunchKernelGGL((attn_partial_kernel<64, FUSED, true>), grid, dim3(ATT_THREADS), 0, s, a);
    else hipLaunchKernelGGL((attn_partial_kernel<64, FUSED, false>), grid, dim3(ATT_THREADS), 0, s, a);
    if (a.nsplit > 1) hipLaunchKernelGGL(attn_combine_kernel<64>, dim3(heads_rows), dim3(64), 0, s, a);
  }
}

static int attention_rows(const char* name, const pta_half* q, const void* kv_ring, const int32_t* step, void* workspace,
                          pta_half* out, int B, int rows, int Hq, int Hkv, int D, int max_len, int use_scale,
                          int kv8, int kv_scale, pta_stream_t stream) {
  PTA_REQUIRE(q && kv_ring && step && workspace && out, "%s: null pointer", name);
  PTA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0, "%s: bad head counts %d/%d", name, Hq, Hkv);
  PTA_REQUIRE(D == 64 || D == 128, "%s: head size must be 64 or 128, got %d", name, D);
  PTA_REQUIRE(max_len > 0, "%s: max_len = %d", name, max_len);
  PTA_REQUIRE(rows > 0 && rows <= max_len, "%s: rows = %d must lie in [1, max_len = %d]", name, rows, max_len);
  PTA_REQUIRE(rows >= 16 || (long)B * rows * Hq <= 65535, "%s: rows = %d (B*rows*Hq must stay below 65536)", name, rows);
  PTA_REQUIRE(pta_aligned(q, 16) && pta_aligned(kv_ring, 16), "%s: q and kv_ring must be 16-byte aligned", name);
  PTA_REQUIRE(!kv8 || (kv_scale >= -16 && kv_scale <= 16), "%s: kv_scale %d outside [-16, 16]", name, kv_scale);
  const size_t ring_elems = (size_t)B * Hkv * max_len * D;
  AttnArgs a{};
  a.q = (const f16*)q; a.kring = (const f16*)kv_ring;
  a.vring = kv8 ? (const f16*)((const uint8_t*)kv_ring + ring_elems) : (const f16*)kv_ring + ring_elems;
  a.step = step; a.part = (float*)workspace; a.out = (f16*)out;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.max_len = max_len; a.nsplit = attn_splits(B * rows, Hq, max_len); a.rows = rows;
  a.kv_scale = kv_scale;
  a.use_scale = use_scale; a.scale = (f16)(1.0 / sqrt((double)D));
  if (rows >= 16) {        // many rows: on the matrix unit, no splits, no workspace
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    const bool two = (long)((rows + 127) / 128) * Hq * B >= 2L * cus;
    const dim3 grid(two ? (rows + 127) / 128 : (rows + 63) / 64, Hq, B);
    auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(PA_THREADS), 0, (hipStream_t)stream, a); };
    if (D == 128) {
      if (kv8) { if (two) go(prompt_attention_mfma_kernel<128, 2, true>); else go(prompt_attention_mfma_kernel<128, 1, true>); }
      else { if (two) go(prompt_attention_mfma_kernel<128, 2, false>); else go(prompt_attention_mfma_kernel<128, 1, false>); }
    } else {
      if (kv8) { if (two) go(prompt_attention_mfma_kernel<64, 2, true>); else go(prompt_attention_mfma_kernel<64, 1, true>); }
      else { if (two) go(prompt_attention_mfma_kernel<64, 2, false>); else go(prompt_attention_mfma_kernel<64, 1, false>); }
    }
    PTA_CHECK_LAUNCH(name);
    return PTA_OK;
  }
  launch_attention<false>(a, D, kv8 != 0, B * rows * Hq, (hipStream_t)stream);
  PTA_CHECK_LAUNCH(name);
  return PTA_OK;
}

extern "C" int pta_decode_attention(const pta_half* q, const pta_half* kv_ring, const int32_t* step, void* workspace,
                                    pta_half* out, int B, int Hq, int Hkv, int D, int max_len, int use_scale,
                                    pta_stream_t stream) {
  return attention_rows("pta_decode_attention", q, kv_ring, step, workspace, out, B, 1, Hq, Hkv, D, max_len, use_scale, 0, 0, stream);
}

extern "C" int pta_prompt_attention(const pta_half* q, const pta_half* kv_ring, const int32_t* step, void* workspace,
                                    pta_half* out, int B, int rows, int Hq, int Hkv, int D, int max_len, int use_scale,
                                    pta_stream_t stream) {
  return attention_rows("pta_prompt_attention", q, kv_ring, step, workspace, out, B, rows, Hq, Hkv, D, max_len, use_scale, 0, 0, stream);
}

extern "C" int pta_prompt_attention_f8(const pta_half* q, const uint8_t* kv_ring, const int32_t* step, void* workspace,
                                       pta_half* out, int B, int rows, int Hq, int Hkv, int D, int max_len, int use_scale,
                                       int kv_scale, pta_stream_t stream) {
  return attention_rows("pta_prompt_attention_f8", q, kv_ring, step, workspace, out, B, rows, Hq, Hkv, D, max_len, use_scale, 1,
                        kv_scale, stream);
}

static int attention_qkv(const char* name, const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                         int v_stride, void* kv_ring, const int32_t* step, const void* inv_freq, void* workspace,
                         pta_half* out, int B, int Hq, int Hkv, int D, int max_len, int rope, int use_scale, int kv8,
                         int kv_scale, pta_stream_t stream, const int32_t* out_fp8_scale = nullptr, int out_fp8_format = 0) {
  PTA_REQUIRE(q && k && v && kv_ring && step && workspace && out, "%s: null pointer", name);
  PTA_REQUIRE(!out_fp8_scale || out_fp8_format == PTA_F143 || out_fp8_format == PTA_F152,
              "%s: unsupported fp8 format %d, it must be F143 or F152", name, out_fp8_format);
  PTA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0, "%s: bad head counts %d/%d", name, Hq, Hkv);
  PTA_REQUIRE(D == 64 || D == 128, "%s: head size must be 64 or 128, got %d", name, D);
  PTA_REQUIRE(max_len > 0, "%s: max_len = %d", name, max_len);
  PTA_REQUIRE(rope == PTA_ROPE_NONE || rope == PTA_ROPE_LLAMA || rope == PTA_ROPE_GLM2, "%s: unknown rope mode %d", name, rope);
  PTA_REQUIRE(rope == PTA_ROPE_NONE || inv_freq, "%s: inv_freq is required for rotary modes", name);
  PTA_REQUIRE(pta_aligned(kv_ring, 16), "%s: kv_ring must be 16-byte aligned", name);
  PTA_REQUIRE(!kv8 || (kv_scale >= -16 && kv_scale <= 16), "%s: kv_scale %d outside [-16, 16]", name, kv_scale);
  const size_t ring_elems = (size_t)B * Hkv * max_len * D;
  AttnArgs a{};
  a.kring_w = (f16*)kv_ring;
  a.vring_w = kv8 ? (f16*)((uint8_t*)kv_ring + ring_elems) : (f16*)kv_ring + ring_elems;
  a.kring = a.kring_w; a.vring = a.vring_w;
  a.q_raw = (const f16*)q; a.k_raw = (const f16*)k; a.v_raw = (const f16*)v;
  a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride;
  a.inv_freq = inv_freq; a.rope = rope;
  a.step = step; a.part = (float*)workspace; a.out = (f16*)out;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.max_len = max_len; a.nsplit = attn_splits(B, Hq, max_len); a.rows = 1;
  a.kv_scale = kv_scale;
  a.out_fp8_scale = out_fp8_scale; a.out_fp8_format = out_fp8_format;
  a.use_scale = use_scale; a.scale = (f16)(1.0 / sqrt((double)D));
  launch_attention<true>(a, D, kv8 != 0, B * Hq, (hipStream_t)stream);
  PTA_CHECK_LAUNCH(name);
  return PTA_OK;
}

extern "C" int pta_decode_attention_qkv(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                                        int v_stride, pta_half* kv_ring, const int32_t* step, const void* inv_freq,
                                        void* workspace, pta_half* out, int B, int Hq, int Hkv, int D, int max_len, int rope,
                                        int use_scale, pta_stream_t stream) {
  return attention_qkv("pta_decode_attention_qkv", q, k, v, q_stride, k_stride, v_stride, kv_ring, step, inv_freq, workspace, out,
                       B, Hq, Hkv, D, max_len, rope, use_scale, 0, 0, stream);
}

extern "C" int pta_decode_attention_qkv_grid(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                                             int v_stride, pta_half* kv_ring, const int32_t* step, const void* inv_freq,
                                             void* workspace, pta_half* out, int B, int Hq, int Hkv, int D, int max_len,
                                             int rope, int use_scale, const int32_t* out_fp8_scale, int out_fp8_format,
                                             pta_stream_t stream) {
  PTA_REQUIRE(out_fp8_scale, "pta_decode_attention_qkv_grid: null pointer");
  return attention_qkv("pta_decode_attention_qkv_grid", q, k, v, q_stride, k_stride, v_stride, kv_ring, step, inv_freq, workspace,
                       out, B, Hq, Hkv, D, max_len, rope, use_scale, 0, 0, stream, out_fp8_scale, out_fp8_format);
}

extern "C" int pta_decode_attention_qkv_f8(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                                           int v_stride, uint8_t* kv_ring, const int32_t* step, const void* inv_freq,
                                           void* workspace, pta_half* out, int B, int Hq, int Hkv, int D, int max_len,
                                           int rope, int use_scale, int kv_scale, pta_stream_t stream) {
  return attention_qkv("pta_decode_attention_qkv_f8", q, k, v, q_stride, k_stride, v_stride, kv_ring, step, inv_freq, workspace,
                       out, B, Hq, Hkv, D, max_len, rope, use_scale, 1, kv_scale, stream);
}
