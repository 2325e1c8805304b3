/*
 * poptransformer_hip.h — C ABI of libpoptransformer_hip.so (gfx950 / MI355X).
 *
 * This library replaces PopTransformer's `custom_ops.so` (PopART custom ops whose bodies
 * are Poplar programs and IPU codelets) for the per-token decode path.  The reference
 * library exports no C symbols: its ops self-register with PopART when it is dlopen'ed at
 * poptransformer/ops/customized.py:17-18.  Here each op is one extern "C" function over raw
 * device pointers, called from the Python `ops` layer with ctypes.
 *
 * Rules common to every entry point
 *   - all pointers are DEVICE pointers unless the parameter name starts with `host_`;
 *   - fp16 tensors are passed as `pta_half*` (IEEE binary16 bit patterns);
 *   - `stream` is a hipStream_t (NULL = the default stream);
 *   - nothing is allocated, freed or synchronised: work is only enqueued on `stream`, so a
 *     call may be recorded into a HIP graph;
 *   - return value: PTA_OK (0) or a negative PTA_E* code; the message of the most recent
 *     failure on the calling thread is returned by pta_last_error().  Nothing throws.
 *     Shape/dtype predicates mirror the reference's setup()/grow() guards so that an
 *     invalid call fails where the reference would have refused to build its graph.
 */
#ifndef POPTRANSFORMER_HIP_H
#define POPTRANSFORMER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t pta_half;
typedef void* pta_stream_t;

enum {
  PTA_OK = 0,
  PTA_EINVAL = -1,       /* bad shape / dtype / alignment / null pointer            */
  PTA_EUNSUPPORTED = -2, /* valid in the reference but not implemented here         */
  PTA_EHIP = -3          /* the HIP runtime reported an error (see pta_last_error)  */
};

/* Library version (major*10000 + minor*100 + patch).  Stands in for the SDK-version
 * check custom_ops/compile_time_version.h:33-43 performs in a dlopen constructor. */
int pta_version(void);
const char* pta_last_error(void);

/* ------------------------------------------------------------------------------------
 * INT4 weights
 * ---------------------------------------------------------------------------------- */

/* Int4ToHalf (ops/customized.py:115-125; custom_ops/int4_to_half_custom_op.cpp:65-108,
 * 168-278, 280-380; codelets custom_ops/int4_to_half_codelets.cpp:18-74).
 * packed int8 [n, m]; every byte holds two signed 4-bit values, hi = b >> 4 (arithmetic),
 * lo = (int8)(b << 4) >> 4.
 *   axis == 1: scale fp16 [n]; out fp16 [2m, n]; out[2j,r] = hi(P[r,j])*scale[r],
 *              out[2j+1,r] = lo(P[r,j])*scale[r]
 *   axis == 0: scale fp16 [m]; out fp16 [2n, m]; out[2i,c] = hi(P[i,c])*scale[c],
 *              out[2i+1,c] = lo(P[i,c])*scale[c]
 * The product is one fp16 multiply (round to nearest even).  Bit-exact. */
int pta_int4_to_half(const int8_t* packed, const pta_half* scale, pta_half* out, int n, int m,
                     int axis, pta_stream_t stream);

/* Re-tiling of a packed INT4 weight for the fused GEMV/GEMM below.  The reference does the
 * same kind of load-time re-layout when it copies the unpacked matrix into the matmul-RHS
 * layout (custom_ops/int4_to_half_custom_op.cpp:366-378).  `packed` is the checkpoint layout
 * int8 [N, K/2] (N output channels, K input features); `tiled` receives
 * pta_w4_tiled_bytes(N, K) bytes.  K must be even. */
size_t pta_w4_tiled_bytes(int N, int K);
int pta_w4_tile(const int8_t* packed, void* tiled, int N, int K, pta_stream_t stream);

/* Operations fused around the product Y0 = fp16(X' @ W) of the GEMM entry points.  Each one is
 * a separate fp16 graph op in the reference and keeps its own fp16 rounding here.
 * Before: X' = norm(X) over the K features of every row -
 *   PTA_NORM_RMS:   pta_rmsnorm(X, norm_weight, norm_eps)               (layers/rms_layer_norm.py:26-36)
 *   PTA_NORM_LAYER: pta_layer_norm_ce(X, norm_weight, norm_bias, eps)   (ops/customized.py:69-102)
 *   The fused norm needs M <= 4 and K <= 20480 / M; otherwise the call returns PTA_EUNSUPPORTED and the
 *   caller runs the norm entry point first.
 * After, in this order: Y = Y0 + bias (layers/linear.py:42-46); Y = act(Y); Y = Y * mul (the
 * receptance gate of models/rwkv/ffn.py:58); Y = Y + residual (the blocks' residual `ops.add`, e.g.
 * models/llama2/model.py:38-46); Y = Y * post_scale when post_scale != 0 (the halving of
 * models/rwkv/model.py:115-116).
 * workspace (optional): scratch of pta_linear_workspace_bytes(M, N) bytes, 16-byte aligned.  With it, a
 * single-weight launch of more than 16 rows whose channel count alone cannot fill the machine also
 * splits K across workgroups (fp32 partial sums in the workspace, summed by a second kernel that
 * applies the epilogue).  Calls sharing one workspace must not overlap.
 * Last of all, with out_fp8_scale: Y = pta_half_to_fp8_grid(Y) - the cast of the next FP8 Linear
 * (precision_strategy.py:62-66) done where its input is produced; it also applies to the SwiGLU pair. */
typedef struct pta_fusion {
  const pta_half* bias;        /* [N] or NULL                                   */
  const pta_half* residual;    /* [M, N] or NULL; may alias Y                   */
  int act;                     /* PTA_ACT_*                                     */
  const pta_half* mul;         /* [M, N] or NULL                                */
  float post_scale;            /* 0 = none                                      */
  int norm;                    /* PTA_NORM_*                                    */
  const pta_half* norm_weight; /* [K]                                           */
  const pta_half* norm_bias;   /* [K], PTA_NORM_LAYER only                      */
  float norm_eps;
  void* workspace;             /* NULL, or scratch for a K split across workgroups */
  size_t workspace_bytes;
  const int32_t* out_fp8_scale;/* NULL, or: leave the result on the FP8 grid of this device exponent, as the
                                  half_to_uint8 of the Linear that consumes it would (pta_half_to_fp8_grid)   */
  int out_fp8_format;          /* PTA_F143 / PTA_F152                           */
  pta_half* mix_state;         /* NULL, or [2][M, K]: the (normalised) rows of the previous token, two copies used in
                                  turn - the token shift of models/rwkv/attention.py:59-72 and ffn.py:47-51 done
                                  inside the Linears that consume it: weight i with a `mix` vector w_i is fed
                                  x * w_i + (1 - w_i) * prev (fp16 operations in that order, as pta_rwkv_mix), x being
                                  X after the fused norm and prev copy (*mix_step & 1); the launch leaves x in the
                                  other copy, which the next token's launch reads.  Up to 4 rows with M * K <= 20480 */
  const int32_t* mix_step;     /* device int32: the loop's step counter (with mix_state)                              */
} pta_fusion;

size_t pta_linear_workspace_bytes(int M, int N);

enum { PTA_NORM_NONE = 0, PTA_NORM_RMS = 1, PTA_NORM_LAYER = 2 };
enum { PTA_ACT_NONE = 0, PTA_ACT_GELU_TANH = 1, PTA_ACT_RELU_SQUARE = 2, PTA_ACT_SIGMOID = 3 };

/* Fused Int4ToHalf(axis=1) + MatMul (utils/param_handler/precision_strategy.py:56-60,74-75):
 * Y[M,N] = fp16( X[M,K] @ W ), W[k,n] = fp16(nibble(k,n) * scale[n]) exactly as
 * pta_int4_to_half(axis=1) would produce, fp32 accumulation, never materialised.
 * `tiled` comes from pta_w4_tile.  1 <= M <= 4096.  `fuse` may be NULL. */
int pta_w4a16_gemm(const pta_half* X, const void* tiled, const pta_half* scale, pta_half* Y,
                   int M, int K, int N, const pta_fusion* fuse, pta_stream_t stream);

/* Up to 4 weights sharing the same X and K in one launch (q/k/v projections of
 * models/llama2/attention.py:65-67).  host_* arrays have `count` entries.  Of `fuse` only the
 * norm fields are used. */
int pta_w4a16_gemm_multi(const pta_half* X, int count, const void* const* host_tiled,
                         const pta_half* const* host_scale, pta_half* const* host_Y,
                         const int* host_N, int M, int K, const pta_fusion* fuse, pta_stream_t stream);

/* SwiGLU pair (models/llama2/mlp.py:20-28, models/chatglm2/mlp.py:51-59):
 * Y[M,F] = fp16( fp16(X@Wup) * fp16(swish(fp16(X@Wgate))) ), swish(g) = g*sigmoid(g).
 * Of `fuse` only the norm fields are used. */
int pta_w4a16_gemm_swiglu(const pta_half* X, const void* tiled_gate, const pta_half* scale_gate,
                          const void* tiled_up, const pta_half* scale_up, pta_half* Y, int M,
                          int K, int F, const pta_fusion* fuse, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * FP16 weights (embedding-tied heads, lm_head, GPT-2 linears): ops.matmul of
 * ops/popart.py:55-67 with an initializer on the right-hand side.
 * ---------------------------------------------------------------------------------- */

/* `w` is fp16 [N, K] (the [out, in] orientation of the state dict, layers/linear.py:30-33). */
size_t pta_f16_tiled_bytes(int N, int K);
int pta_f16_tile(const pta_half* w, void* tiled, int N, int K, pta_stream_t stream);
/* Y[M,N] = fp16(X[M,K] @ w^T), fp32 accumulation. 1 <= M <= 4096. */
int pta_f16_gemm(const pta_half* X, const void* tiled, pta_half* Y, int M, int K, int N,
                 const pta_fusion* fuse, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Normalisation
 * ---------------------------------------------------------------------------------- */

/* RMSNorm as composed by layers/rms_layer_norm.py:26-36: v = mean(fp32(x)^2) + eps;
 * r = fp16(1/sqrt(v)); y = fp16(fp16(x*r) * weight).  x, y fp16 [rows, cols]. cols % 8 == 0. */
int pta_rmsnorm(const pta_half* x, const pta_half* weight, pta_half* y, int rows, int cols, float eps,
                pta_stream_t stream);
/* pta_rmsnorm followed by pta_half_to_fp8_grid in one pass: y = grid(rmsnorm(x)) for the FP8 Linear
 * that consumes the normalised rows (the same two roundings, bit for bit). */
int pta_rmsnorm_fp8_grid(const pta_half* x, const pta_half* weight, pta_half* y, const int32_t* scale, int format,
                         int rows, int cols, float eps, pta_stream_t stream);

/* NormCE LayerNorm (ops/customized.py:69-102; custom_ops/NormCE.cpp:534-610).  fp16 in/out,
 * fp32 statistics.  rows == 1 follows calSmallBatchNorm + GetInPlaceNorm (NormCE.cpp:122-200,
 * NormCECodelets.cpp:65-112): var = E[x^2] - mean^2 + eps with the fp32 mean, no clamp.
 * rows > 1 follows normInfKernel (NormCE.S:243-423, NormCECodelets.cpp:181-211): the mean is
 * rounded to fp16 before it is squared and the variance is clamped at 0.  In both,
 * y = fp16(fp16(fp16(fp16(x - mean16) * rstd16) * gamma) + beta).  cols % 8 == 0, cols < 8192. */
int pta_layer_norm_ce(const pta_half* x, const pta_half* gamma, const pta_half* beta, pta_half* y, int rows,
                      int cols, float eps, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Softmax
 * ---------------------------------------------------------------------------------- */
enum { PTA_F16 = 0, PTA_F32 = 1 };

/* SoftmaxV3 over the last axis (ops/customized.py:57-65; custom_ops/softmax.cpp:41-83).
 * x, y are [rows, n] of `dtype`; stable_mode != 0 subtracts the row maximum first. */
int pta_softmax_ce(const void* x, void* y, int rows, int n, int dtype, int stable_mode, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * KV cache.  Shapes are [outer, seq, inner] (inner contiguous); with the models' layout
 * [2, B, H, seq, D] and sequence_axis = 3, outer = 2*B*H and inner = D.  `step` is a device
 * int32 scalar, as it is a graph tensor in the reference.
 * ---------------------------------------------------------------------------------- */

/* KVCache, literal (ops/customized.py:21-35; custom_ops/kv_cache.cpp:94-187):
 *   clone = (*step != 0) ? cache : 0;  cache = concat(updater, clone[:, 0 : max_len-step_len]).
 * cache and clone are [outer, max_len, inner]; updater is [outer, step_len, inner].  The
 * result (the op's output) is `cache` itself. */
int pta_kv_cache_update(void* cache, void* clone, const void* updater, const int32_t* step, int outer,
                        int max_len, int step_len, int inner, int elem_bytes, pta_stream_t stream);

/* The same cache kept as a ring in arrival order: one row written per call, nothing shifted.
 * cache is [max_bps, outer, max_len, inner]; the call at step s writes updater [outer, inner]
 * to row (s / max_bps) % max_len of register s % max_bps.  max_bps == 1 is KVCache; larger
 * values are KVCachePipeline (custom_ops/kv_cache_pipeline.cpp:374-451,
 * custom_ops/kv_cache_codelet.cpp:18-131) with step_len == 1 and the sequence axis at
 * rank - 2.  Calls must come with step = 0, 1, 2, ... as the generation loop issues them. */
int pta_kv_cache_append(void* cache, const void* updater, const int32_t* step, int outer, int max_len, int inner,
                        int elem_bytes, int max_bps, pta_stream_t stream);

/* Materialises the reference op's output from the ring after the append of the same step:
 * out [outer, max_len, inner], out[:, i] = i-th newest row of register step % max_bps, zero for
 * rows the shift register would not have received since step 0. */
int pta_kv_cache_read(const void* cache, void* out, const int32_t* step, int outer, int max_len, int inner,
                      int elem_bytes, int max_bps, pta_stream_t stream);

/* KVCachePipeline with transpose = 1, literal (custom_ops/kv_cache_pipeline.cpp:397-451; codelet
 * custom_ops/kv_cache_codelet.cpp:170-212): the max_bps persistent registers `caches`
 * [max_bps, outer, inner, max_len] keep the sequence as their last axis; all are zeroed when *step == 0;
 * register *step % max_bps is shifted by one element along that axis in place, with the new row
 * `updater` [outer, 1, inner] at index 0; `out` [outer, max_len, inner] receives that register in the
 * input's layout (the op's output).  step_len is 1, as the op itself requires (pipeline.cpp:410). */
int pta_kv_cache_pipeline_seq_last(void* caches, void* out, const void* updater, const int32_t* step, int outer,
                                   int max_len, int inner, int elem_bytes, int max_bps, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Attention for one new position per sequence
 * ---------------------------------------------------------------------------------- */
enum { PTA_ROPE_NONE = 0, PTA_ROPE_LLAMA = 1, PTA_ROPE_GLM2 = 2 };

/* Rotary embedding of q and k at position *step and append of (k, v) to the ring cache
 * (models/llama2/attention.py:28-94; models/chatglm2/attention.py:77-232;
 * models/gpt2/attention.py:50-66 with PTA_ROPE_NONE).
 * q/k/v point at the projection outputs, row b at q + b*q_stride etc.: heads are contiguous,
 * [Hq*D] for q and [Hkv*D] for k and v.  q_out is [B, Hq, D].  kv_ring is the cache of
 * pta_kv_cache_append with max_bps = 1, outer = 2*B*Hkv, inner = D: keys first, then values.
 * inv_freq: PTA_ROPE_LLAMA fp16 [D/2] (the graph constant of llama2/attention.py:29-31);
 *           PTA_ROPE_GLM2 fp32 [D/4] (chatglm2/attention.py:80-83). */
int pta_qkv_rope_append(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                        int v_stride, pta_half* q_out, pta_half* kv_ring, const int32_t* step, const void* inv_freq,
                        int B, int Hq, int Hkv, int D, int max_len, int rope, pta_stream_t stream);

/* softmax(q K^T [* fp16(1/sqrt(D))] + mask) V over the rows received so far, heads merged:
 * out [B, Hq*D] (forward_attention + forward_output up to the output projection,
 * models/llama2/attention.py:97-113, models/gpt2/attention.py:68-90,
 * models/chatglm2/attention.py:277-302).  The mask of models/base_model.py:258-262,321-325 is
 * implied by *step: rows 0..step are open.  Hq % Hkv == 0 (multi-query groups share a cache
 * head).  D is 64 or 128.  workspace: pta_decode_attention_workspace_bytes(...) bytes. */
size_t pta_decode_attention_workspace_bytes(int B, int Hq, int D, int max_len);
int pta_decode_attention(const pta_half* q, const pta_half* kv_ring, const int32_t* step, void* workspace,
                         pta_half* out, int B, int Hq, int Hkv, int D, int max_len, int use_scale,
                         pta_stream_t stream);

/* pta_qkv_rope_append and pta_decode_attention in one pass: every attention workgroup rotates its own
 * query head from the raw projection rows, and the workgroups whose rows hold this step's position
 * rotate the new key, use it and the new value directly and write them to the ring.  Arguments as in
 * those two calls; the result is bit-identical to calling them one after the other. */
int pta_decode_attention_qkv(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                             int v_stride, pta_half* kv_ring, const int32_t* step, const void* inv_freq,
                             void* workspace, pta_half* out, int B, int Hq, int Hkv, int D, int max_len, int rope,
                             int use_scale, pta_stream_t stream);

/* pta_decode_attention_qkv whose context vector is left on an FP8 grid: out = pta_half_to_fp8_grid(context,
 * out_fp8_scale, out_fp8_format), bit for bit - the cast with which the next FP8 Linear starts
 * (half_to_uint8, utils/param_handler/precision_strategy.py:62-66), done where the value is produced. */
int pta_decode_attention_qkv_grid(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                                  int v_stride, pta_half* kv_ring, const int32_t* step, const void* inv_freq,
                                  void* workspace, pta_half* out, int B, int Hq, int Hkv, int D, int max_len, int rope,
                                  int use_scale, const int32_t* out_fp8_scale, int out_fp8_format, pta_stream_t stream);

/* The same two operators over `rows` consecutive positions of every sequence at once - the prompt.
 * The reference feeds a prompt through its loop one token per iteration (the container keeps the
 * prompt's ids, models/base_model.py:313-318); its two-stage ChatGLM graphs run the same layers with
 * sequence_length > 1 for the prompt (models/chatglm/attention.py:89-140).  Row r of sequence b (row
 * b*rows + r of q, k, v, q_out, out) stands at position *step + r: it is rotated for that position,
 * appended there, and attends to positions 0 .. *step + r, which is what `rows` iterations of the loop
 * compute.  *step + rows must not exceed max_len (no wrap inside one call).  The attention workspace
 * is pta_decode_attention_workspace_bytes(B*rows, ...) bytes. */
int pta_prompt_rope_append(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                           int v_stride, pta_half* q_out, pta_half* kv_ring, const int32_t* step, const void* inv_freq,
                           int B, int rows, int Hq, int Hkv, int D, int max_len, int rope, pta_stream_t stream);
int pta_prompt_attention(const pta_half* q, const pta_half* kv_ring, const int32_t* step, void* workspace,
                         pta_half* out, int B, int rows, int Hq, int Hkv, int D, int max_len, int use_scale,
                         pta_stream_t stream);

/* The same with an FP8 KV cache: KVCacheOp with fp8 = true casts the rows to F143 bytes with the constant
 * metadata scale 1 before they are stored and casts the whole cache back to fp16 when it is read
 * (custom_ops/kv_cache.cpp:43-74,103-105; `fp8_cache` of models/llama2/attention.py:18-24).  kv_ring is
 * uint8 [2*B*Hkv, max_len, D]: a row holds encode_F143(value * 2^-kv_scale), attention uses
 * decode(byte) * 2^kv_scale.  rows = 1 is the decode step. */
int pta_prompt_rope_append_f8(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                              int v_stride, pta_half* q_out, uint8_t* kv_ring, const int32_t* step,
                              const void* inv_freq, int B, int rows, int Hq, int Hkv, int D, int max_len, int rope,
                              int kv_scale, pta_stream_t stream);
int pta_prompt_attention_f8(const pta_half* q, const uint8_t* kv_ring, const int32_t* step, void* workspace,
                            pta_half* out, int B, int rows, int Hq, int Hkv, int D, int max_len, int use_scale,
                            int kv_scale, pta_stream_t stream);
int pta_decode_attention_qkv_f8(const pta_half* q, const pta_half* k, const pta_half* v, int q_stride, int k_stride,
                                int v_stride, uint8_t* kv_ring, const int32_t* step, const void* inv_freq,
                                void* workspace, pta_half* out, int B, int Hq, int Hkv, int D, int max_len, int rope,
                                int use_scale, int kv_scale, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Token selection and loop bookkeeping
 * ---------------------------------------------------------------------------------- */

/* ops.topk(k=1) over the last axis (layers/lm_head.py:55; ops/popart.py:135-137): ids[r] = index
 * of the largest logit of row r, the lowest index among equals; values (optional) receives it. */
int pta_argmax(const pta_half* logits, int32_t* ids, pta_half* values, int rows, int n, pta_stream_t stream);

/* ops.topk(k) over the last axis (ops/popart.py:135-137; layers/lm_head.py:52-53,89): ids[r, j] and
 * values[r, j] (optional) are the j-th largest logit of row r; equal values come in ascending order of
 * index.  1 <= k <= n. */
int pta_topk(const pta_half* logits, int32_t* ids, pta_half* values, int rows, int n, int k, pta_stream_t stream);

/* The slice of ops.random_sample (ops/popart.py:25-29): out[r] = candidates[r, *pick] for candidates
 * int32 [rows, k] and a device index `pick` (clamped into [0, k)), the same column for every row. */
int pta_take_column(const int32_t* candidates, const int32_t* pick, int32_t* out, int rows, int k, pta_stream_t stream);

/* Bytes of the workspace of pta_beam_search_step (the per-beam candidates); 0 for beam_size outside [1, 64]. */
size_t pta_beam_search_workspace_bytes(int batch, int beam);

/* One call of the BeamSearch op (custom_ops/beam_search_custom_op.cpp:333-478; shape guards :103-177).
 * logits [batch, beam, vocab] and prob_container [batch, beam] of `dtype` (PTA_F16 / PTA_F32), hyp_container
 * int32 [batch, max_len, beam], `step` a device int32.  Per beam the `beam` best scores over the vocabulary;
 *   *step == 0: next_id = global_best_id = the ids of beam 0, hyp_container[:, 0] = next_id, prob_container =
 *     the scores of beam 0;
 *   otherwise: candidate (i, j) = prob_container[i] + score j of beam i (added in `dtype`); the `beam` best
 *     of the beam * beam candidates give global_best_id (flat index i * beam + j), next_id (their ids) and
 *     prob_container; every row of hyp_container is re-gathered from the parent hypotheses i and row *step
 *     (if inside the container) takes next_id.
 * Equal scores are taken in ascending order of index.  The containers are updated in place; next_id and
 * global_best_id are int32 [batch, beam]. */
int pta_beam_search_step(const void* logits, int dtype, int32_t* hyp_container, void* prob_container, const int32_t* step,
                         int32_t* next_id, int32_t* global_best_id, void* workspace, int batch, int beam, int vocab,
                         int max_len, pta_stream_t stream);

/* Embedding rows (layers/embedding.py:34-36); with pos_table also GPT-2's wte[id] + wpe[*pos]
 * (models/gpt2/embedding.py:31-36).  out [rows, cols].  Row b uses
 * id = ids[b*ids_stride + (ids_index ? *ids_index : 0)], so the `dynamic_slice(container, step)`
 * of the model graphs (e.g. models/llama2/model.py:168) needs no copy: pass the container,
 * ids_stride = max_length and ids_index = step.  For a plain id vector: ids_stride 1, NULL. */
int pta_embedding(const pta_half* table, const int32_t* ids, int ids_stride, const int32_t* ids_index,
                  const pta_half* pos_table, const int32_t* pos, pta_half* out, int rows, int cols, int vocab,
                  pta_stream_t stream);

/* step_containers + step_loop_cond of models/base_model.py:313-355 for one iteration; all
 * arrays on the device.  container int32 [B, max_len]; mask fp16 [B, max_len] or NULL;
 * stop_mask int32 [B]; step int32 scalar (advanced by one); next_ids int32 [B];
 * ids_out (optional) int32 [B] receives the ids written; keep_going (optional) int32 scalar. */
int pta_step_update(int32_t* container, pta_half* mask, int32_t* stop_mask, int32_t* step, const int32_t* next_ids,
                    int32_t* ids_out, int32_t* keep_going, int B, int max_len, int pad_id, int eos_id,
                    int early_stop, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * FP8 (Graphcore F143 / F152 bytes, value = decode(byte) * 2^scale).  Scales are device int32
 * tensors of which element 0 is read, as in custom_ops/matmul_fp8.cpp:890-891.
 * ---------------------------------------------------------------------------------- */
enum { PTA_F143 = 0, PTA_F152 = 1 };

/* CastToUint8 (ops/customized.py:127-135; custom_ops/cast_to_uint8.cpp:107-127): fp16 -> byte,
 * round to nearest even, saturating, NaN -> 0x80.  out has the shape of x (n elements). */
int pta_half_to_fp8(const pta_half* x, uint8_t* out, const int32_t* scale, size_t n, int format,
                    pta_stream_t stream);
/* The cast back (custom_ops/matmul_fp8.cpp:925-930, custom_ops/kv_cache.cpp:56-74). */
int pta_fp8_to_half(const uint8_t* in, pta_half* out, const int32_t* scale, size_t n, int format,
                    pta_stream_t stream);

/* Re-tiling of an FP8 weight.  `w` is uint8 [N, K] (w_is_kn == 0, state-dict orientation) or
 * [K, N] (w_is_kn != 0, the orientation the reference graph holds after layers/linear.py:32). */
size_t pta_fp8_tiled_bytes(int N, int K);
int pta_fp8_tile(const uint8_t* w, void* tiled, int N, int K, int w_is_kn, pta_stream_t stream);

/* FP8MatMul (ops/customized.py:137-148; custom_ops/matmul_fp8.cpp:177-250, 885-1003).
 * lhs is fp16 [M, K] (lhs_is_fp8 == 0: the weight is cast to fp16, then an fp16 MatMul) or uint8
 * [M, K] (both operands FP8).  Y fp16 [M, N], fp32 accumulation.  1 <= M <= 4096.
 * workspace: pta_fp8_gemm_workspace_bytes(M, K) bytes, 16-byte aligned.  `fuse` may be NULL. */
size_t pta_fp8_gemm_workspace_bytes(int M, int K);
int pta_fp8_gemm(const void* lhs, int lhs_is_fp8, const void* tiled_rhs, pta_half* Y, int M, int K, int N,
                 int format_lhs, int format_rhs, const int32_t* scale_lhs, const int32_t* scale_rhs,
                 void* workspace, const pta_fusion* fuse, pta_stream_t stream);

/* fp16 values on the FP8 grid: out = decode(encode(x * 2^-scale)) WITHOUT the scale, i.e. what an
 * FP8 operand contributes to a product before the power of two is applied.  Lets
 * half_to_uint8 + fp8_matmul (precision_strategy.py:62-66,77-81) run as one rounding pass plus
 * pta_linear with x_scale. */
int pta_half_to_fp8_grid(const pta_half* x, pta_half* out, const int32_t* scale, size_t n, int format,
                         pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Linear layers, general form (layers/linear.py:19-46 + precision_strategy.py:56-81)
 * ---------------------------------------------------------------------------------- */
enum { PTA_W_INT4 = 0, PTA_W_F16 = 1, PTA_W_F143 = 2, PTA_W_F152 = 3 };

typedef struct pta_weight {
  int kind;            /* PTA_W_*                                                              */
  const void* tiled;   /* from pta_w4_tile / pta_f16_tile / pta_fp8_tile                      */
  const void* scale;   /* INT4: fp16 [N]; FP8: device int32 exponent; FP16: NULL              */
  int N, K;
  const pta_half* x;   /* NULL, or this weight's own input [M, K] instead of X (the three token-shift
                          mixes of models/rwkv/attention.py:69-71 feed three Linears)          */
  int act;             /* PTA_ACT_* applied to this weight's output in a multi-weight launch  */
  const pta_half* mix; /* NULL, or this weight's token-shift mixing vector [K] (see pta_fusion.mix_state) */
} pta_weight;

/* Y_i[M, N_i] = fp16(X' @ W_i) + bias_i for `count` (1..4) weights of one kind and one K in one
 * launch; with swiglu != 0 (count == 2: gate, up) Y_0 = fp16(up * swish(gate)).  x_scale (FP8
 * weights only, may be NULL): X holds unscaled values on the weights' FP8 grid, whose device int32 exponent it is
 * (from 65 rows on, F143 weights and such an X are multiplied as bytes on the FP8 matrix instruction).
 * host_bias may be NULL.  With count == 1 all of `fuse` applies, otherwise its norm fields. */
int pta_linear(const pta_half* X, const int32_t* x_scale, int count, const pta_weight* host_w,
               const pta_half* const* host_bias, pta_half* const* host_Y, int M, int swiglu,
               const pta_fusion* fuse, pta_stream_t stream);

/* out = up * swish(gate), two fp16 ops (models/llama2/mlp.py:22-26): the unfused form of the
 * SwiGLU pair, for gate/up weights that cannot share a launch. */
int pta_swiglu(const pta_half* gate, const pta_half* up, pta_half* out, size_t n, pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * RWKV-4 recurrent step (models/rwkv/attention.py:59-105, models/rwkv/ffn.py:40-59)
 * ---------------------------------------------------------------------------------- */

/* Token-shift mixes o_i = x*w_i + (1 - w_i)*prev (fp16 ops of `gate`, attention.py:59-64) for one to
 * three mixing vectors w_i [cols] (w1/w2 may be NULL), then prev <- x.  x, prev, o_i: [rows, cols]. */
int pta_rwkv_mix(const pta_half* x, pta_half* prev, const pta_half* w0, const pta_half* w1, const pta_half* w2,
                 pta_half* o0, pta_half* o1, pta_half* o2, int rows, int cols, pta_stream_t stream);

/* pta_layer_norm_ce followed by pta_rwkv_mix in one launch (the LayerNorm before each token shift:
 * models/rwkv/attention.py:66-72, models/rwkv/ffn.py:44-51): h = LayerNorm(x); o_i = h*w_i + (1 - w_i)*prev;
 * prev <- h.  Bit-identical to the two calls.  y receives h, or may be NULL. */
int pta_layer_norm_ce_mix(const pta_half* x, const pta_half* gamma, const pta_half* beta, pta_half* y, pta_half* prev,
                          const pta_half* w0, const pta_half* w1, const pta_half* w2, pta_half* o0, pta_half* o1,
                          pta_half* o2, int rows, int cols, float eps, pta_stream_t stream);

/* The WKV recurrence in fp32 (attention.py:78-100) followed by y = r * fp16(out) (:101-103).
 * k, v, r, y fp16 [rows, cols]; time_decay, time_first fp16 [cols]; num, den, max_state fp32
 * [rows, cols], updated in place (initial values 0, 0, -1e30: models/rwkv/model.py:157-187). */
int pta_rwkv_wkv(const pta_half* k, const pta_half* v, const pta_half* r, const pta_half* time_decay,
                 const pta_half* time_first, float* num, float* den, float* max_state, pta_half* y, int rows, int cols,
                 pta_stream_t stream);

/* ------------------------------------------------------------------------------------
 * One whole loop iteration in one launch (models/base_model.py:271-355 driving
 * models/llama2/model.py:162-197: embedding, every decoder layer, final RMSNorm, lm_head,
 * top-1, container / mask / stop-mask update).  The reference compiles this loop body into one
 * Poplar program; this entry is its counterpart for INT4 Llama-2 shapes: a single persistent
 * kernel, one workgroup per compute unit; a phase hands its results to the next through slots of the
 * workspace that the consumers poll (no grid-wide barrier between phases), the weights of later phases
 * are requested early.  Results equal those of the per-operator entry points above run in the
 * reference's order, up to the order in which attention partial sums are merged.
 * ---------------------------------------------------------------------------------- */

typedef struct pta_decode_layer {
  const void *wq, *wk, *wv, *wo, *wg, *wu, *wd;       /* INT4 weights tiled by pta_w4_tile            */
  const pta_half *sq, *sk, *sv, *so, *sg, *su, *sd;   /* their per-output-channel scales              */
  const pta_half *norm1, *norm2;                      /* RMSNorm weights [hidden]                     */
  pta_half* kv_ring;                                  /* ring of pta_qkv_rope_append for this layer   */
} pta_decode_layer;

typedef struct pta_decode_model {
  const pta_decode_layer* layers;                     /* DEVICE array [n_layer]                       */
  int n_layer;
  const pta_half* embed;                              /* [vocab, hidden]                              */
  const pta_half* final_norm;                         /* [hidden]                                     */
  const void* head;                                   /* lm_head [vocab, hidden] tiled by pta_f16_tile */
  const pta_half* inv_freq;                           /* rotary inverse frequencies, fp16 [head_dim/2] */
  int batch, hidden, n_head, head_dim, ffn, vocab, max_len;
  float eps;
  int pad_id, eos_id, early_stop;                     /* as pta_step_update                           */
} pta_decode_model;

typedef struct pta_decode_state {
  int32_t* container;                                 /* [batch, max_len]                             */
  pta_half* mask;                                     /* [batch, max_len]                             */
  int32_t* stop_mask;                                 /* [batch]                                      */
  int32_t* step;                                      /* [1]                                          */
  int32_t* keep_going;                                /* [1]; 0 makes the launch a no-op              */
  int32_t* next_ids;                                  /* [batch] out: the selected tokens             */
  pta_half* logits;                                   /* [batch, vocab] out, 16-byte aligned          */
} pta_decode_state;

/* Bytes of the workspace of pta_llama_decode_step for this model on the current device; 0 for
 * unsupported shapes.  The workspace holds one slot per intermediate vector of an iteration (the
 * residual stream after each half layer, q|k|v, attention output and partials, SwiGLU output) and a
 * few synchronisation words.  The caller zeroes it once after allocating it (256-byte aligned). */
size_t pta_decode_step_workspace_bytes(const pta_decode_model* model);

/* Enqueues one loop iteration.  Supports batch <= 16, head_dim 128, hidden = n_head * 128 with
 * (hidden, ffn) of the 7B model or a small test shape; PTA_EUNSUPPORTED otherwise.  Batches of 5..16
 * run a second kernel of the same structure (activations as matrix-instruction fragments in registers
 * instead of staged in LDS).
 * Needs every compute unit of the device for itself while it runs: workgroups wait for each
 * other's results, every wait is bounded, and if one gives up it sets word 1 of the workspace
 * (sticky), the loop state is left untouched and the kernel ends; pta_decode_step_failed reports it.
 * Numerics: every rounding point is that of the per-operator entry points, except that an INT4
 * projection is fp16(scale * sum(x * q)) - the scale applied once to the fp32 sum - where
 * pta_w4a16_gemm computes fp16(sum(x * fp16(q * scale))); the results agree to the last fp16 bit or
 * differ in it. */
int pta_llama_decode_step(const pta_decode_model* model, const pta_decode_state* state, void* workspace,
                          pta_stream_t stream);

/* The same iteration with FP8 KV rings (KVCacheOp with fp8 = true, custom_ops/kv_cache.cpp:43-74,103-105;
 * the cache layout and numerics of pta_decode_attention_qkv_f8): every layer's kv_ring holds F143 bytes
 * [2 * batch * n_head, max_len, head_dim] of value * 2^-kv_scale, kv_scale in [-16, 16] (the reference's
 * metadata scale is the constant 1).  Same workspace, same conditions. */
int pta_llama_decode_step_f8(const pta_decode_model* model, const pta_decode_state* state, int kv_scale, void* workspace,
                             pta_stream_t stream);

/* Copies the failure word of the workspace to *failed (synchronises with `stream`). */
int pta_decode_step_failed(const void* workspace, int* failed, pta_stream_t stream);

/* pta_llama_decode_step for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The
 * workspace is an array built into the library, 16 MiB of device memory that every GPU the library runs on
 * holds until the process ends; a model whose workspace (pta_decode_step_workspace_bytes) is larger is
 * refused with PTA_EINVAL.  The call allocates and frees nothing.  Its first call on a device looks up
 * the array's address there: make that call outside any capture.  All calls on one GPU share the array:
 * calls that overlap on one GPU (two streams, two threads) race; calls in stream order do not, also when
 * they serve different models.  There is no workspace pointer to hand to pta_decode_step_failed: a launch
 * that gave up leaves `*state->step` as it was, which is how the caller sees it, and every later launch does
 * nothing until one is made with clear_failure != 0 (a one-thread kernel clears the failure word first). */
int pta_llama_decode_step_static(const pta_decode_model* model, const pta_decode_state* state, int clear_failure,
                                 pta_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* POPTRANSFORMER_HIP_H */
