// Linear layers of the decode step: Y = [act](X' @ W + bias) [+ residual] for INT4, FP16 and FP8
// weights, one or several weights per launch, optionally as a SwiGLU pair.
//
// Reference: poptransformer/layers/linear.py:19-46 with the precision hooks of
// poptransformer/utils/param_handler/precision_strategy.py:56-81 (int4: Int4ToHalf + MatMul;
// fp8: CastToUint8 + FP8MatMul; fp8_weight: FP8MatMul on fp16 activations; fp16: MatMul).
#include "common.h"
#include "formats.h"
#include "gemm_f8n.h"

int f8_decode_unscaled_launch(const uint8_t* in, f16* out, size_t n, int format, hipStream_t s);

template <class Fmt>
static int run_linear(GemmArgs& a, int total_nb, int swiglu, hipStream_t s, const char* name) {
  if (swiglu) return dispatch_gemv<Fmt, true>(a, total_nb, s, name);
  return dispatch_gemv<Fmt, false>(a, total_nb, s, name);
}

// PTA_FP8_NATIVE=0 in the environment keeps FP8 x FP8 products on the fp16 instruction (decode of both operands),
// for comparisons; read once.
static bool fp8_native_enabled() {
  static const bool on = [] {
    const char* v = getenv("PTA_FP8_NATIVE");
    return !(v && v[0] == '0');
  }();
  return on;
}

// The FP8 instruction's many-row kernel takes launches of more rows than this.  Up to 64 rows a launch is bound by
// the weights' way from memory and the fp16 instruction's kernels for few rows are as fast or faster (measured at
// 32 and 64 rows: 13 and 23 against 27 and 38 us for q | kv of the ChatGLM2-6B shape, 28 and 46 against 33 and 44
// for the gate / up pair).  PTA_FP8_PANEL_MIN_ROWS in the environment overrides it (for comparisons); read once.
static int f8n_panel_min_rows() {
  static const int rows = [] {
    const char* v = getenv("PTA_FP8_PANEL_MIN_ROWS");
    return v ? atoi(v) : 64;
  }();
  return rows;
}

// x_bytes: 1 - X holds F143 bytes [M, K] instead of fp16 values (FP8 weights of format F143 only); 2 - fp16 values with
// an exponent (x_scale) that are not known to lie on the F143 grid (they keep to the fp16 instruction)
static int linear_impl(const void* X, const int32_t* x_scale, int x_bytes, int count, const pta_weight* host_w,
                       const pta_half* const* host_bias, pta_half* const* host_Y, int M, int swiglu,
                       const pta_fusion* fuse, pta_stream_t stream) {
  PTA_REQUIRE(host_w && host_Y, "pta_linear: null pointer");
  PTA_REQUIRE(count >= 1 && count <= 4, "pta_linear: count must be in [1, 4], got %d", count);
  PTA_REQUIRE(!swiglu || count == 2, "pta_linear: a SwiGLU pair is exactly two weights (gate, up)");
  const int kind = host_w[0].kind, K = host_w[0].K;
  int rc = check_gemv_common("pta_linear", X ? (const void*)X : (const void*)host_w[0].x, M, K);
  if (rc) return rc;
  for (int i = 0; i < count; ++i) PTA_REQUIRE(X || host_w[i].x, "pta_linear: entry %d has no input", i);
  PTA_REQUIRE(kind >= PTA_W_INT4 && kind <= PTA_W_F152, "pta_linear: unknown weight kind %d", kind);
  GemmArgs a{};
  a.count = count; a.X = (const f16*)X; a.x_scale = x_scale; a.M = M; a.K = K; a.KT = (K + 127) / 128;
  PTA_REQUIRE(!x_scale || kind == PTA_W_F143 || kind == PTA_W_F152, "pta_linear: x_scale is only meaningful with FP8 weights");
  int nb = 0;
  for (int i = 0; i < count; ++i) {
    const pta_weight& w = host_w[i];
    PTA_REQUIRE(w.kind == kind && w.K == K, "pta_linear: weights of one call must share their kind and K");
    PTA_REQUIRE(w.tiled && host_Y[i] && w.N > 0, "pta_linear: entry %d is incomplete", i);
    PTA_REQUIRE(kind == PTA_W_F16 || w.scale, "pta_linear: entry %d needs its scale", i);
    PTA_REQUIRE(pta_aligned(w.tiled, 16), "pta_linear: tiled[%d] must be 16-byte aligned", i);
    PTA_REQUIRE(!swiglu || w.N == host_w[0].N, "pta_linear: the SwiGLU weights must have the same shape");
    PTA_REQUIRE(w.act >= PTA_ACT_NONE && w.act <= PTA_ACT_SIGMOID, "pta_linear: unknown activation %d in entry %d", w.act, i);
    PTA_REQUIRE(!swiglu || (!w.x && w.act == PTA_ACT_NONE), "pta_linear: the SwiGLU pair shares X and takes no activation");
    PTA_REQUIRE(!w.x || pta_aligned(w.x, 16), "pta_linear: x[%d] must be 16-byte aligned", i);
    a.mat[i] = GemmMat{w.tiled, w.scale, host_bias ? (const f16*)host_bias[i] : nullptr, (const f16*)w.x, (const f16*)w.mix, w.act,
                       (f16*)host_Y[i], w.N, swiglu ? 0 : nb};
    nb += (w.N + 15) / 16;
  }
  if (swiglu) {
    nb = (host_w[0].N + 15) / 16;
    PTA_REQUIRE(!a.mat[0].bias && !a.mat[1].bias, "pta_linear: the SwiGLU pair takes no bias");
  }
  rc = make_epilogue(fuse, &a.epi, "pta_linear");
  if (rc) return rc;
  {
    bool any_mix = false;
    for (int i = 0; i < count; ++i) any_mix = any_mix || host_w[i].mix;
    PTA_REQUIRE(!any_mix || a.epi.mix_state, "pta_linear: a mixing vector needs pta_fusion.mix_state and mix_step");
    if (a.epi.mix_state) {
      // the token shift runs where the rows are staged in LDS: gemv_lds_kernel's shapes, one shared input
      PTA_REQUIRE(X && M <= 4 && (size_t)M * (a.KT * 128 + 8) * 2 <= 40 * 1024 && K % 8 == 0 && !swiglu && !x_bytes && !x_scale,
                  "pta_linear: mix_state needs one shared fp16 X of up to 4 rows with M * K <= 20480 (got M=%d K=%d)", M, K);
      for (int i = 0; i < count; ++i) PTA_REQUIRE(!host_w[i].x, "pta_linear: mix_state and a weight's own input exclude each other");
      PTA_REQUIRE(pta_aligned(a.epi.mix_state, 16), "pta_linear: mix_state must be 16-byte aligned");
    }
  }
  if (fuse && fuse->workspace) {
    PTA_REQUIRE(pta_aligned(fuse->workspace, 16), "pta_linear: the workspace must be 16-byte aligned");
    a.part = (float*)fuse->workspace;
    a.part_bytes = fuse->workspace_bytes;
  }
  PTA_REQUIRE(count == 1 || (!a.epi.bias && !a.epi.residual && !a.epi.mul && a.epi.post_scale == 0.0f && a.epi.act == PTA_ACT_NONE),
              "pta_linear: with several weights only the norm fields and the output cast of `fuse` apply (use host_bias for biases)");
  PTA_REQUIRE(!a.epi.out_fp8_scale || count == 1 || swiglu, "pta_linear: the output cast applies to one weight or to a SwiGLU pair");
  hipStream_t s = (hipStream_t)stream;
  // Both operands F143: the FP8 matrix instruction.  fp16 grid values are turned into bytes by every workgroup that
  // reads them (about 60 vector instructions per 32-feature step), which pays only when the bytes feed several
  // products.  Measured at the ChatGLM2-6B shape, 8 rows, saturating activations (every step multiplied twice, 224
  // and 16): the SwiGLU pair 31.2 against 32.5 us for gemv_wide_kernel on the fp16 instruction with decoded weights
  // - and 25.0 us for gemv_stream_kernel, also with decoded weights, which therefore takes the pair wherever it
  // fits; one channel block per workgroup (4096 x 4096) 16.2 against 11.5 us, q | kv and the lm_head slower as well.
  // So fp16 grid values come here for a SwiGLU pair outside that kernel's shapes only; an uint8 left-hand side always.
  const bool several = swiglu != 0;
  const bool stream_pair = several && !x_bytes && stream_fits(a) && nb >= device_compute_units();
  if (kind == PTA_W_F143 && f8n_fits(a) && (x_bytes == 1 || (x_bytes == 0 && fp8_native_enabled() && several && !stream_pair))) {
    if (x_bytes) return swiglu ? dispatch_gemv_f8n<true, true>(a, nb, s, "pta_linear") : dispatch_gemv_f8n<false, true>(a, nb, s, "pta_linear");
    return swiglu ? dispatch_gemv_f8n<true, false>(a, nb, s, "pta_linear") : dispatch_gemv_f8n<false, false>(a, nb, s, "pta_linear");
  }
  a.prefer_stream = stream_pair && (kind == PTA_W_F143 || kind == PTA_W_F152);
  PTA_REQUIRE(x_bytes != 1, "pta_linear: an uint8 left-hand side needs F143 weights, M <= 16 and K >= 1024");
  // more than 16 rows of F143-grid values by F143 weights (a prompt pass): the 16x16x128 FP8 instruction
  if (kind == PTA_W_F143 && x_bytes == 0 && fp8_native_enabled() && f8n_panel_fits(a, swiglu != 0) && M > f8n_panel_min_rows())
    return swiglu ? dispatch_f8n_panel<true>(a, nb, s, "pta_linear") : dispatch_f8n_panel<false>(a, nb, s, "pta_linear");
  switch (kind) {
    case PTA_W_INT4: return run_linear<FmtW4>(a, nb, swiglu, s, "pta_linear");
    case PTA_W_F16: return run_linear<FmtF16>(a, nb, swiglu, s, "pta_linear");
    case PTA_W_F143: return run_linear<FmtF8<0>>(a, nb, swiglu, s, "pta_linear");
    default: return run_linear<FmtF8<1>>(a, nb, swiglu, s, "pta_linear");
  }
}

extern "C" int pta_linear(const pta_half* X, const int32_t* x_scale, int count, const pta_weight* host_w,
                          const pta_half* const* host_bias, pta_half* const* host_Y, int M, int swiglu,
                          const pta_fusion* fuse, pta_stream_t stream) {
  return linear_impl(X, x_scale, 0, count, host_w, host_bias, host_Y, M, swiglu, fuse, stream);
}

extern "C" size_t pta_linear_workspace_bytes(int M, int N) {
  if (M <= 0 || N <= 0) return 0;
  return (size_t)GEMM_MAX_KSPLIT * M * N * sizeof(float);
}

// ------------------------------------------------------------------------------------------
// Operator-shaped entry points over pta_linear.
// ------------------------------------------------------------------------------------------
extern "C" int pta_w4a16_gemm(const pta_half* X, const void* tiled, const pta_half* scale, pta_half* Y, int M, int K,
                              int N, const pta_fusion* fuse, pta_stream_t stream) {
  pta_weight w{PTA_W_INT4, tiled, scale, N, K, nullptr, PTA_ACT_NONE};
  return pta_linear(X, nullptr, 1, &w, nullptr, &Y, M, 0, fuse, stream);
}

extern "C" int pta_w4a16_gemm_multi(const pta_half* X, int count, const void* const* host_tiled,
                                    const pta_half* const* host_scale, pta_half* const* host_Y, const int* host_N,
                                    int M, int K, const pta_fusion* fuse, pta_stream_t stream) {
  PTA_REQUIRE(count >= 1 && count <= 4 && host_tiled && host_scale && host_N, "pta_w4a16_gemm_multi: bad arguments");
  pta_weight w[4];
  for (int i = 0; i < count; ++i) w[i] = pta_weight{PTA_W_INT4, host_tiled[i], host_scale[i], host_N[i], K, nullptr, PTA_ACT_NONE};
  return pta_linear(X, nullptr, count, w, nullptr, host_Y, M, 0, fuse, stream);
}

extern "C" int pta_w4a16_gemm_swiglu(const pta_half* X, const void* tiled_gate, const pta_half* scale_gate,
                                     const void* tiled_up, const pta_half* scale_up, pta_half* Y, int M, int K, int F,
                                     const pta_fusion* fuse, pta_stream_t stream) {
  pta_weight w[2] = {{PTA_W_INT4, tiled_gate, scale_gate, F, K, nullptr, PTA_ACT_NONE},
                     {PTA_W_INT4, tiled_up, scale_up, F, K, nullptr, PTA_ACT_NONE}};
  pta_half* ys[2] = {Y, Y};
  return pta_linear(X, nullptr, 2, w, nullptr, ys, M, 1, fuse, stream);
}

extern "C" int pta_f16_gemm(const pta_half* X, const void* tiled, pta_half* Y, int M, int K, int N,
                            const pta_fusion* fuse, pta_stream_t stream) {
  pta_weight w{PTA_W_F16, tiled, nullptr, N, K, nullptr, PTA_ACT_NONE};
  return pta_linear(X, nullptr, 1, &w, nullptr, &Y, M, 0, fuse, stream);
}

extern "C" size_t pta_fp8_gemm_workspace_bytes(int M, int K) {
  if (M <= 0 || K <= 0) return 0;
  return (size_t)M * K * 2;     // the left-hand side decoded to fp16
}

extern "C" int pta_fp8_gemm(const void* lhs, int lhs_is_fp8, const void* tiled_rhs, pta_half* Y, int M, int K, int N,
                            int format_lhs, int format_rhs, const int32_t* scale_lhs, const int32_t* scale_rhs,
                            void* workspace, const pta_fusion* fuse, pta_stream_t stream) {
  // dtype guards of FP8MatMulOp::setup (custom_ops/matmul_fp8.cpp:237-245) are the caller's to state
  // through lhs_is_fp8; formats must be F143 or F152 (:324-351).
  PTA_REQUIRE(format_rhs == PTA_F143 || format_rhs == PTA_F152, "pta_fp8_gemm: unsupported fp8 format %d, it must be F143 or F152", format_rhs);
  PTA_REQUIRE(lhs && scale_rhs, "pta_fp8_gemm: null pointer");
  const f16* X = (const f16*)lhs;
  const int32_t* xs = nullptr;
  if (lhs_is_fp8) {
    PTA_REQUIRE(format_lhs == PTA_F143 || format_lhs == PTA_F152, "pta_fp8_gemm: unsupported fp8 format %d, it must be F143 or F152", format_lhs);
    PTA_REQUIRE(scale_lhs && workspace && pta_aligned(workspace, 16), "pta_fp8_gemm: an fp8 left-hand side needs its scale and a 16-byte aligned workspace");
    PTA_REQUIRE(M >= 1 && K >= 1, "pta_fp8_gemm: empty left-hand side");
    if (format_lhs == PTA_F143 && format_rhs == PTA_F143 && M <= 16 && K >= 1024 && K % 8 == 0 && pta_aligned(lhs, 8) &&
        fp8_native_enabled() && !(fuse && fuse->norm != PTA_NORM_NONE)) {
      // the bytes go to the FP8 matrix instruction as they are
      pta_weight w8{PTA_W_F143, tiled_rhs, scale_rhs, N, K, nullptr, PTA_ACT_NONE};
      return linear_impl(lhs, scale_lhs, 1, 1, &w8, nullptr, &Y, M, 0, fuse, stream);
    }
    f8_decode_unscaled_launch((const uint8_t*)lhs, (f16*)workspace, (size_t)M * K, format_lhs, (hipStream_t)stream);
    X = (const f16*)workspace;
    xs = scale_lhs;
  }
  pta_weight w{format_rhs == PTA_F143 ? PTA_W_F143 : PTA_W_F152, tiled_rhs, scale_rhs, N, K, nullptr, PTA_ACT_NONE};
  // a decoded left-hand side lies on its own format's grid; an fp16 one is multiplied as it is (no x_scale)
  return linear_impl(X, xs, lhs_is_fp8 && format_lhs != PTA_F143 ? 2 : 0, 1, &w, nullptr, &Y, M, 0, fuse, stream);
}
