"""Thin torch-tensor front end of the C ABI (include/poptransformer_hip.h).

PyTorch is used for device memory and streams only: every function checks its operands on the
host, passes raw pointers to libpoptransformer_hip.so on torch's current stream and returns
torch tensors.  Nothing here computes on the CPU and nothing falls back to torch kernels.
"""
import ctypes

import torch

from . import _lib
from ._lib import Fusion, check

_i32 = torch.int32


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _need(t, dtype, name, dims=None):
    if not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dims is not None and t.dim() != dims:
        raise ValueError(f"The rank of {name} should be {dims}. But now it is {t.dim()}.")


class Norm:
    """A row normalisation to fuse in front of a GEMM: RMSNorm (bias None) or NormCE LayerNorm."""

    def __init__(self, weight, bias, eps):
        self.weight, self.bias, self.eps = weight, bias, float(eps)

    @property
    def kind(self):
        return _lib.NORM_RMS if self.bias is None else _lib.NORM_LAYER


def norm_fusable(M, K):
    """Whether the GEMM entry points can apply a fused norm for this shape."""
    return M <= 4 and M * (((K + 127) // 128) * 128 + 8) * 2 <= 40 * 1024


def _fusion(bias=None, residual=None, act=_lib.ACT_NONE, norm=None, mul=None, post_scale=0.0, workspace=None,
            out_grid=None, mix=None):
    """out_grid: (device int32 exponent, 'F143' | 'F152') - leave the result on that FP8 grid (half_to_fp8_grid).
    mix: (state [2, M, K] fp16, device int32 step) - the token shift done inside the Linears (pta_fusion.mix_state)."""
    if (bias is None and residual is None and act == _lib.ACT_NONE and norm is None and mul is None and not post_scale
            and workspace is None and out_grid is None and mix is None):
        return None
    if mix is not None:
        _need(mix[0], torch.float16, "mix state", 3)
        _need(mix[1], _i32, "step")
    if out_grid is not None:
        _need(out_grid[0], _i32, "fp8_scale")
    e = Fusion(_p(bias), _p(residual), act, _p(mul), float(post_scale), norm.kind if norm else _lib.NORM_NONE,
               _p(norm.weight) if norm else None, _p(norm.bias) if norm else None, norm.eps if norm else 0.0,
               _p(workspace), workspace.numel() * workspace.element_size() if workspace is not None else 0,
               _p(out_grid[0]) if out_grid is not None else None, _fmt(out_grid[1]) if out_grid is not None else 0,
               _p(mix[0]) if mix is not None else None, _p(mix[1]) if mix is not None else None)
    return ctypes.byref(e)


def linear_workspace(M, N, device):
    """Scratch that lets a single-weight `linear` of more than 16 rows split K across workgroups."""
    return torch.empty(_lib.load().pta_linear_workspace_bytes(M, N), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------ INT4 -----------------
def int4_to_half(packed, scale, axis=1):
    """ops.int4_to_half (reference: poptransformer/ops/customized.py:115-125)."""
    _need(packed, torch.int8, "input", 2)
    _need(scale, torch.float16, "scale", 1)
    n, m = packed.shape
    if axis == 1 and scale.shape[0] != n:
        raise ValueError(f"[Int4ToHalfOp] input.shape[0]({n}) should be equal to  scale.shape[0]({scale.shape[0]})")
    if axis == 0 and scale.shape[0] != m:
        raise ValueError(f"[Int4ToHalfOp] input.shape[1]({m}) should be equal to  scale.shape[0]({scale.shape[0]})")
    shape = (2 * m, n) if axis == 1 else (2 * n, m)
    out = torch.empty(shape if axis in (0, 1) else (1,), dtype=torch.float16, device=packed.device)
    check(_lib.load().pta_int4_to_half(_p(packed), _p(scale), _p(out), n, m, axis, _stream()))
    return out


class W4Weight:
    """A packed INT4 Linear weight re-tiled for the fused kernels, with its fp16 scales."""

    def __init__(self, packed, scale):
        _need(packed, torch.int8, "packed weight", 2)
        _need(scale, torch.float16, "scale", 1)
        self.N, half_k = packed.shape
        self.K = 2 * half_k
        if scale.shape[0] != self.N:
            raise ValueError(f"[Int4ToHalfOp] input.shape[0]({self.N}) should be equal to  scale.shape[0]({scale.shape[0]})")
        lib = _lib.load()
        nbytes = lib.pta_w4_tiled_bytes(self.N, self.K)
        self.tiled = torch.empty(nbytes, dtype=torch.uint8, device=packed.device)
        self.scale = scale
        check(lib.pta_w4_tile(_p(packed), _p(self.tiled), self.N, self.K, _stream()))

    @property
    def nbytes(self):
        return self.N * self.K // 2 + self.N * 2


def w4a16_gemm(x, w, bias=None, residual=None, act=_lib.ACT_NONE, out=None, norm=None, workspace=None):
    _need(x, torch.float16, "x", 2)
    M, K = x.shape
    if K != w.K:
        raise ValueError(f"matmul: contracting dimensions differ ({K} vs {w.K})")
    if out is None:
        out = torch.empty((M, w.N), dtype=torch.float16, device=x.device)
    check(_lib.load().pta_w4a16_gemm(_p(x), _p(w.tiled), _p(w.scale), _p(out), M, K, w.N,
                                     _fusion(bias, residual, act, norm, workspace=workspace), _stream()))
    return out


def w4a16_gemm_multi(x, weights, outs=None, norm=None):
    _need(x, torch.float16, "x", 2)
    M, K = x.shape
    n = len(weights)
    if outs is None:
        outs = [torch.empty((M, w.N), dtype=torch.float16, device=x.device) for w in weights]
    for w in weights:
        if w.K != K:
            raise ValueError(f"matmul: contracting dimensions differ ({K} vs {w.K})")
    VP = ctypes.c_void_p * n
    tiled = VP(*[w.tiled.data_ptr() for w in weights])
    scale = VP(*[w.scale.data_ptr() for w in weights])
    ys = VP(*[o.data_ptr() for o in outs])
    ns = (ctypes.c_int * n)(*[w.N for w in weights])
    check(_lib.load().pta_w4a16_gemm_multi(_p(x), n, tiled, scale, ys, ns, M, K, _fusion(norm=norm), _stream()))
    return outs


def w4a16_gemm_swiglu(x, w_gate, w_up, out=None, norm=None):
    _need(x, torch.float16, "x", 2)
    M, K = x.shape
    if w_gate.K != K or w_up.K != K or w_gate.N != w_up.N:
        raise ValueError("swiglu: gate/up weights must share their shape and match x")
    if out is None:
        out = torch.empty((M, w_gate.N), dtype=torch.float16, device=x.device)
    check(_lib.load().pta_w4a16_gemm_swiglu(_p(x), _p(w_gate.tiled), _p(w_gate.scale), _p(w_up.tiled),
                                            _p(w_up.scale), _p(out), M, K, w_gate.N, _fusion(norm=norm), _stream()))
    return out


# ------------------------------------------------------------------ FP16 -----------------
class F16Weight:
    """An fp16 Linear weight [N, K] (state-dict orientation) re-tiled for the fused kernel."""

    def __init__(self, w):
        _need(w, torch.float16, "weight", 2)
        self.N, self.K = w.shape
        lib = _lib.load()
        self.tiled = torch.empty(lib.pta_f16_tiled_bytes(self.N, self.K), dtype=torch.uint8, device=w.device)
        check(lib.pta_f16_tile(_p(w), _p(self.tiled), self.N, self.K, _stream()))

    @property
    def nbytes(self):
        return self.N * self.K * 2


def f16_gemm(x, w, bias=None, residual=None, act=_lib.ACT_NONE, out=None, norm=None):
    _need(x, torch.float16, "x", 2)
    M, K = x.shape
    if K != w.K:
        raise ValueError(f"matmul: contracting dimensions differ ({K} vs {w.K})")
    if out is None:
        out = torch.empty((M, w.N), dtype=torch.float16, device=x.device)
    check(_lib.load().pta_f16_gemm(_p(x), _p(w.tiled), _p(out), M, K, w.N, _fusion(bias, residual, act, norm), _stream()))
    return out


# ------------------------------------------------------------------ FP8 ------------------
def _fmt(name):
    if name not in _lib.FP8_FORMATS:
        raise ValueError(f"Unsupport fp8 meata data {name}, it must be F143 or F152")
    return _lib.FP8_FORMATS[name]


def half_to_fp8(x, scale, fp8_format="F143"):
    """ops.half_to_uint8 (reference: poptransformer/ops/customized.py:127-135)."""
    fmt = _fmt(fp8_format)
    _need(x, torch.float16, "x")
    _need(scale, _i32, "fp8_scale")
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    check(_lib.load().pta_half_to_fp8(_p(x), _p(out), _p(scale), x.numel(), fmt, _stream()))
    return out


def fp8_to_half(codes, scale, fp8_format="F143"):
    fmt = _fmt(fp8_format)
    _need(codes, torch.uint8, "codes")
    _need(scale, _i32, "fp8_scale")
    out = torch.empty(codes.shape, dtype=torch.float16, device=codes.device)
    check(_lib.load().pta_fp8_to_half(_p(codes), _p(out), _p(scale), codes.numel(), fmt, _stream()))
    return out


class F8Weight:
    """An FP8 Linear weight re-tiled for the fused kernel.  `w` is uint8 [N, K], or [K, N] with
    kn=True (the orientation the reference graph holds)."""

    def __init__(self, w, scale, fp8_format="F143", kn=False):
        _need(w, torch.uint8, "weight", 2)
        _need(scale, _i32, "weight scale")
        self.format = _fmt(fp8_format)
        self.N, self.K = (w.shape[1], w.shape[0]) if kn else w.shape
        self.scale = scale
        lib = _lib.load()
        self.tiled = torch.zeros(lib.pta_fp8_tiled_bytes(self.N, self.K), dtype=torch.uint8, device=w.device)
        check(lib.pta_fp8_tile(_p(w), _p(self.tiled), self.N, self.K, 1 if kn else 0, _stream()))

    @property
    def nbytes(self):
        return self.N * self.K


def fp8_gemm_workspace(M, K, device):
    return torch.empty(_lib.load().pta_fp8_gemm_workspace_bytes(M, K), dtype=torch.uint8, device=device)


def fp8_gemm(x, w, workspace, x_scale=None, x_format="F143", bias=None, residual=None, act=_lib.ACT_NONE, out=None,
             norm=None):
    """ops.fp8_matmul (reference: poptransformer/ops/customized.py:137-148): x fp16 or uint8 [M, K]."""
    if x.dtype not in (torch.float16, torch.uint8):
        raise ValueError(f"Invalid input data type of {x.dtype}, it must be FLOAT16 or UINT8")
    _need(x, x.dtype, "x", 2)
    M, K = x.shape
    if K != w.K:
        raise ValueError(f"matmul: contracting dimensions differ ({K} vs {w.K})")
    is8 = x.dtype == torch.uint8
    if is8 and x_scale is None:
        raise ValueError("an fp8 left-hand side needs its scale")
    if out is None:
        out = torch.empty((M, w.N), dtype=torch.float16, device=x.device)
    check(_lib.load().pta_fp8_gemm(_p(x), 1 if is8 else 0, _p(w.tiled), _p(out), M, K, w.N, _fmt(x_format) if is8 else 0,
                                   w.format, _p(x_scale), _p(w.scale), _p(workspace),
                                   _fusion(bias, residual, act, norm), _stream()))
    return out


def half_to_fp8_grid(x, scale, fp8_format="F143", out=None):
    """x rounded to the FP8 grid, returned as fp16 WITHOUT the scale (see pta_half_to_fp8_grid)."""
    fmt = _fmt(fp8_format)
    _need(x, torch.float16, "x")
    _need(scale, _i32, "fp8_scale")
    if out is None:
        out = torch.empty_like(x)
    check(_lib.load().pta_half_to_fp8_grid(_p(x), _p(out), _p(scale), x.numel(), fmt, _stream()))
    return out


# ------------------------------------------------------------------ general Linear -------
def _desc(w, x=None, act=_lib.ACT_NONE, mix=None):
    xp = x.data_ptr() if x is not None else None
    mp = mix.data_ptr() if mix is not None else None
    if isinstance(w, W4Weight):
        return _lib.Weight(_lib.W_INT4, w.tiled.data_ptr(), w.scale.data_ptr(), w.N, w.K, xp, act, mp)
    if isinstance(w, F16Weight):
        return _lib.Weight(_lib.W_F16, w.tiled.data_ptr(), None, w.N, w.K, xp, act, mp)
    if isinstance(w, F8Weight):
        return _lib.Weight(_lib.W_F143 if w.format == _lib.F143 else _lib.W_F152, w.tiled.data_ptr(), w.scale.data_ptr(),
                           w.N, w.K, xp, act, mp)
    raise TypeError(f"not a tiled weight: {type(w)}")


def linear(x, weights, outs, biases=None, x_scale=None, swiglu=False, bias=None, residual=None, act=_lib.ACT_NONE,
           norm=None, mul=None, post_scale=0.0, xs=None, acts=None, workspace=None, out_grid=None, mixes=None, mix=None):
    """pta_linear: up to four weights of one kind.  They share x, or each takes its own input from
    `xs`.  `biases` / `acts` are per-weight lists (or None); bias / residual / act / mul / post_scale
    apply to the single-weight form only.  mixes (per-weight mixing vectors) with mix = (state [2, M, K], step):
    the RWKV token shift inside the launch - weight i is fed norm(x) * mixes[i] + (1 - mixes[i]) * previous rows."""
    if xs is not None:
        x = xs[0]
    _need(x, torch.float16, "x", 2)
    M = x.shape[0]
    n = len(weights)
    if mixes is not None:
        for m_ in mixes:
            if m_ is not None:
                _need(m_, torch.float16, "mixing vector", 1)
    descs = (_lib.Weight * n)(*[_desc(w, xs[i] if xs is not None else None, acts[i] if acts is not None else _lib.ACT_NONE,
                                      mixes[i] if mixes is not None else None)
                                for i, w in enumerate(weights)])
    VP = ctypes.c_void_p * n
    ys = VP(*[o.data_ptr() for o in outs])
    bs = None
    if biases is not None and any(b is not None for b in biases):
        bs = VP(*[(b.data_ptr() if b is not None else None) for b in biases])
    for w in weights:
        if w.K != x.shape[1]:
            raise ValueError(f"matmul: contracting dimensions differ ({x.shape[1]} vs {w.K})")
    check(_lib.load().pta_linear(_p(x), _p(x_scale), n, descs, bs, ys, M, 1 if swiglu else 0,
                                 _fusion(bias, residual, act, norm, mul, post_scale, workspace, out_grid, mix), _stream()))
    return outs


def swiglu(gate, up, out=None):
    _need(gate, torch.float16, "gate")
    _need(up, torch.float16, "up")
    if out is None:
        out = torch.empty_like(up)
    check(_lib.load().pta_swiglu(_p(gate), _p(up), _p(out), up.numel(), _stream()))
    return out


# ------------------------------------------------------------------ norms ----------------
def rmsnorm(x, weight, eps, out=None):
    _need(x, torch.float16, "x")
    _need(weight, torch.float16, "weight", 1)
    cols = x.shape[-1]
    rows = x.numel() // cols
    if out is None:
        out = torch.empty_like(x)
    check(_lib.load().pta_rmsnorm(_p(x), _p(weight), _p(out), rows, cols, float(eps), _stream()))
    return out


def rmsnorm_fp8_grid(x, weight, eps, scale, fp8_format="F143", out=None):
    """half_to_fp8_grid(rmsnorm(x)) in one pass."""
    _need(x, torch.float16, "x")
    _need(weight, torch.float16, "weight", 1)
    _need(scale, _i32, "fp8_scale")
    cols = x.shape[-1]
    rows = x.numel() // cols
    if out is None:
        out = torch.empty_like(x)
    check(_lib.load().pta_rmsnorm_fp8_grid(_p(x), _p(weight), _p(out), _p(scale), _fmt(fp8_format), rows, cols, float(eps),
                                           _stream()))
    return out


def layer_norm_ce(x, gamma, beta, eps, out=None):
    if x.dtype != torch.float16:
        raise ValueError("[NormCE] only float16 is supported")
    _need(x, torch.float16, "x")
    _need(gamma, torch.float16, "gamma", 1)
    _need(beta, torch.float16, "beta", 1)
    cols = x.shape[-1]
    rows = x.numel() // cols
    if out is None:
        out = torch.empty_like(x)
    check(_lib.load().pta_layer_norm_ce(_p(x), _p(gamma), _p(beta), _p(out), rows, cols, float(eps), _stream()))
    return out


def softmax_ce(x, stable_mode=True):
    if x.dim() < 2:
        raise ValueError("[Softmax] rank of input should be >= 2")
    if x.dtype not in (torch.float16, torch.float32):
        raise ValueError("[Softmax] input type must be FLOAT16 or FLOAT")
    _need(x, x.dtype, "x")
    n = x.shape[-1]
    out = torch.empty_like(x)
    dt = _lib.F16 if x.dtype == torch.float16 else _lib.F32
    check(_lib.load().pta_softmax_ce(_p(x), _p(out), x.numel() // n, n, dt, 1 if stable_mode else 0, _stream()))
    return out


# ------------------------------------------------------------------ KV cache -------------
def _kv_dims(t, axis):
    outer = 1
    for s in t.shape[:axis]:
        outer *= s
    inner = 1
    for s in t.shape[axis + 1:]:
        inner *= s
    return outer, inner


def kv_cache_update(cache, clone, updater, step, sequence_axis):
    """Literal KVCache op on [.., max_len, ..] tensors; `cache` is updated in place and returned."""
    outer, inner = _kv_dims(cache, sequence_axis)
    _need(step, _i32, "step")
    check(_lib.load().pta_kv_cache_update(_p(cache), _p(clone), _p(updater), _p(step), outer,
                                          cache.shape[sequence_axis], updater.shape[sequence_axis], inner,
                                          cache.element_size(), _stream()))
    return cache


def kv_cache_append(ring, updater, step, outer, max_len, inner, max_bps=1):
    _need(step, _i32, "step")
    check(_lib.load().pta_kv_cache_append(_p(ring), _p(updater), _p(step), outer, max_len, inner,
                                          ring.element_size(), max_bps, _stream()))


def kv_cache_read(ring, out, step, outer, max_len, inner, max_bps=1):
    _need(step, _i32, "step")
    check(_lib.load().pta_kv_cache_read(_p(ring), _p(out), _p(step), outer, max_len, inner, ring.element_size(),
                                        max_bps, _stream()))
    return out


def kv_cache_pipeline_seq_last(caches, out, updater, step, outer, max_len, inner, max_bps):
    """KVCachePipeline with transpose = 1: `caches` [max_bps, outer, inner, max_len] updated in place, `out`
    [outer, max_len, inner] the op's output."""
    _need(step, _i32, "step")
    check(_lib.load().pta_kv_cache_pipeline_seq_last(_p(caches), _p(out), _p(updater), _p(step), outer, max_len, inner,
                                                     caches.element_size(), max_bps, _stream()))
    return out


def beam_search_step(logits, hyp_container, prob_container, step, workspace=None):
    """One call of the BeamSearch op; the containers are updated in place.  Returns (next_id, global_best_id)."""
    if logits.dim() != 3:
        raise ValueError(f"[Beam Search] The rank of logits should be 3. But now it is {logits.dim()}.")
    if hyp_container.dim() != 3 or prob_container.dim() != 2:
        raise ValueError("[Beam Search] hyp_container must have rank 3 and prob_container rank 2")
    B, beam, V = logits.shape
    if tuple(prob_container.shape) != (B, beam) or hyp_container.shape[0] != B or hyp_container.shape[2] != beam:
        raise ValueError("[Beam Search] batch or beam sizes of logits, hyp_container and prob_container differ")
    if logits.dtype not in (torch.float16, torch.float32) or prob_container.dtype != logits.dtype:
        raise ValueError("[Beam Search] logits and prob_container must both be float16 or float32")
    _need(hyp_container, _i32, "hyp_container")
    _need(step, _i32, "step")
    lib = _lib.load()
    if workspace is None:
        workspace = torch.empty(max(lib.pta_beam_search_workspace_bytes(B, beam), 256), dtype=torch.uint8, device=logits.device)
    next_id = torch.empty((B, beam), dtype=_i32, device=logits.device)
    best = torch.empty((B, beam), dtype=_i32, device=logits.device)
    logits = logits.contiguous()
    check(lib.pta_beam_search_step(_p(logits), _lib.F16 if logits.dtype == torch.float16 else _lib.F32,
                                   _p(hyp_container), _p(prob_container), _p(step), _p(next_id), _p(best), _p(workspace),
                                   B, beam, V, hyp_container.shape[1], _stream()))
    return next_id, best


# ------------------------------------------------------------------ attention ------------
def qkv_rope_append(q, k, v, q_out, kv_ring, step, inv_freq, B, Hq, Hkv, D, max_len, rope,
                    q_stride=None, k_stride=None, v_stride=None):
    q_stride = Hq * D if q_stride is None else q_stride
    k_stride = Hkv * D if k_stride is None else k_stride
    v_stride = Hkv * D if v_stride is None else v_stride
    check(_lib.load().pta_qkv_rope_append(_p(q), _p(k), _p(v), q_stride, k_stride, v_stride, _p(q_out), _p(kv_ring),
                                          _p(step), _p(inv_freq), B, Hq, Hkv, D, max_len, rope, _stream()))


def decode_attention_workspace(B, Hq, D, max_len, device):
    n = _lib.load().pta_decode_attention_workspace_bytes(B, Hq, D, max_len)
    return torch.empty(n, dtype=torch.uint8, device=device)


def decode_attention(q, kv_ring, step, workspace, out, B, Hq, Hkv, D, max_len, use_scale):
    check(_lib.load().pta_decode_attention(_p(q), _p(kv_ring), _p(step), _p(workspace), _p(out), B, Hq, Hkv, D,
                                           max_len, 1 if use_scale else 0, _stream()))
    return out


def _kv_ring_dtype(kv_ring, kv_scale):
    want = torch.float16 if kv_scale is None else torch.uint8
    if kv_ring.dtype != want:
        raise ValueError(f"kv_ring must be {want} ({'fp16' if kv_scale is None else 'FP8'} cache), got {kv_ring.dtype}")


def decode_attention_qkv(q, k, v, kv_ring, step, inv_freq, workspace, out, B, Hq, Hkv, D, max_len, rope, use_scale,
                         q_stride=None, k_stride=None, v_stride=None, kv_scale=None, out_grid=None):
    """qkv_rope_append + decode_attention in one pass (bit-identical to the two calls).  kv_scale (an int):
    kv_ring is a uint8 FP8 cache holding F143 bytes of value * 2^-kv_scale.  out_grid: (device int32 exponent,
    'F143' | 'F152') - the context vector is left on that FP8 grid (half_to_fp8_grid); fp16 caches only."""
    q_stride = Hq * D if q_stride is None else q_stride
    k_stride = Hkv * D if k_stride is None else k_stride
    v_stride = Hkv * D if v_stride is None else v_stride
    _kv_ring_dtype(kv_ring, kv_scale)
    if out_grid is not None:
        if kv_scale is not None:
            raise NotImplementedError("decode_attention_qkv: out_grid with an FP8 cache")
        _need(out_grid[0], _i32, "fp8_scale")
        check(_lib.load().pta_decode_attention_qkv_grid(_p(q), _p(k), _p(v), q_stride, k_stride, v_stride, _p(kv_ring),
                                                        _p(step), _p(inv_freq), _p(workspace), _p(out), B, Hq, Hkv, D,
                                                        max_len, rope, 1 if use_scale else 0, _p(out_grid[0]),
                                                        _fmt(out_grid[1]), _stream()))
        return out
    if kv_scale is not None:
        check(_lib.load().pta_decode_attention_qkv_f8(_p(q), _p(k), _p(v), q_stride, k_stride, v_stride, _p(kv_ring),
                                                      _p(step), _p(inv_freq), _p(workspace), _p(out), B, Hq, Hkv, D,
                                                      max_len, rope, 1 if use_scale else 0, int(kv_scale), _stream()))
        return out
    check(_lib.load().pta_decode_attention_qkv(_p(q), _p(k), _p(v), q_stride, k_stride, v_stride, _p(kv_ring), _p(step),
                                               _p(inv_freq), _p(workspace), _p(out), B, Hq, Hkv, D, max_len, rope,
                                               1 if use_scale else 0, _stream()))
    return out


def prompt_rope_append(q, k, v, q_out, kv_ring, step, inv_freq, B, rows, Hq, Hkv, D, max_len, rope,
                       q_stride=None, k_stride=None, v_stride=None, kv_scale=None):
    """qkv_rope_append over `rows` consecutive positions per sequence (row b*rows + r stands at step + r).
    kv_scale (an int): kv_ring is a uint8 FP8 cache."""
    _need(step, _i32, "step")
    q_stride = Hq * D if q_stride is None else q_stride
    k_stride = Hkv * D if k_stride is None else k_stride
    v_stride = Hkv * D if v_stride is None else v_stride
    _kv_ring_dtype(kv_ring, kv_scale)
    if kv_scale is not None:
        check(_lib.load().pta_prompt_rope_append_f8(_p(q), _p(k), _p(v), q_stride, k_stride, v_stride, _p(q_out), _p(kv_ring),
                                                    _p(step), _p(inv_freq), B, rows, Hq, Hkv, D, max_len, rope,
                                                    int(kv_scale), _stream()))
        return
    check(_lib.load().pta_prompt_rope_append(_p(q), _p(k), _p(v), q_stride, k_stride, v_stride, _p(q_out), _p(kv_ring),
                                             _p(step), _p(inv_freq), B, rows, Hq, Hkv, D, max_len, rope, _stream()))


def prompt_attention(q, kv_ring, step, workspace, out, B, rows, Hq, Hkv, D, max_len, use_scale, kv_scale=None):
    """decode_attention over `rows` consecutive positions per sequence; row r attends to positions 0..step+r.
    workspace: decode_attention_workspace(B * rows, ...).  kv_scale (an int): kv_ring is a uint8 FP8 cache."""
    _need(step, _i32, "step")
    need = _lib.load().pta_decode_attention_workspace_bytes(B * rows, Hq, D, max_len)
    if workspace.numel() * workspace.element_size() < need:
        raise ValueError(f"prompt_attention: the workspace holds {workspace.numel() * workspace.element_size()} bytes, {need} needed")
    _kv_ring_dtype(kv_ring, kv_scale)
    if kv_scale is not None:
        check(_lib.load().pta_prompt_attention_f8(_p(q), _p(kv_ring), _p(step), _p(workspace), _p(out), B, rows, Hq, Hkv, D,
                                                  max_len, 1 if use_scale else 0, int(kv_scale), _stream()))
        return out
    check(_lib.load().pta_prompt_attention(_p(q), _p(kv_ring), _p(step), _p(workspace), _p(out), B, rows, Hq, Hkv, D,
                                           max_len, 1 if use_scale else 0, _stream()))
    return out


# ------------------------------------------------------------------ selection ------------
def argmax(logits, ids=None, values=None):
    _need(logits, torch.float16, "logits")
    n = logits.shape[-1]
    rows = logits.numel() // n
    if ids is None:
        ids = torch.empty(rows, dtype=_i32, device=logits.device)
    check(_lib.load().pta_argmax(_p(logits), _p(ids), _p(values), rows, n, _stream()))
    return ids


def topk(logits, k, ids=None, values=None):
    """The k largest entries of every row of the last axis, descending, equal values by ascending index."""
    _need(logits, torch.float16, "logits")
    n = logits.shape[-1]
    rows = logits.numel() // n
    if not 1 <= k <= n:
        raise ValueError(f"topk: k must be in [1, {n}], got {k}")
    if ids is None:
        ids = torch.empty((rows, k), dtype=_i32, device=logits.device)
    if values is None:
        values = torch.empty((rows, k), dtype=torch.float16, device=logits.device)
    check(_lib.load().pta_topk(_p(logits), _p(ids), _p(values), rows, n, k, _stream()))
    return values, ids


def take_column(candidates, pick, out=None):
    """out[r] = candidates[r, pick[0]] (pick: device int32)."""
    _need(candidates, _i32, "candidates", 2)
    _need(pick, _i32, "pick")
    rows, k = candidates.shape
    if out is None:
        out = torch.empty(rows, dtype=_i32, device=candidates.device)
    check(_lib.load().pta_take_column(_p(candidates), _p(pick), _p(out), rows, k, _stream()))
    return out


def embedding(table, ids, out=None, pos_table=None, pos=None, ids_index=None):
    """Rows of `table`.  ids int32 [rows] or, with ids_index (device int32 scalar), a container
    [rows, L] of which column *ids_index is used."""
    _need(table, torch.float16, "table", 2)
    _need(ids, _i32, "ids")
    if ids_index is None:
        rows, stride = ids.numel(), 1
    else:
        rows, stride = ids.shape
    vocab, cols = table.shape
    if out is None:
        out = torch.empty((rows, cols), dtype=torch.float16, device=table.device)
    check(_lib.load().pta_embedding(_p(table), _p(ids), stride, _p(ids_index), _p(pos_table), _p(pos), _p(out), rows,
                                    cols, vocab, _stream()))
    return out


def step_update(container, mask, stop_mask, step, next_ids, ids_out, keep_going, pad_id, eos_id, early_stop):
    B, max_len = container.shape
    check(_lib.load().pta_step_update(_p(container), _p(mask), _p(stop_mask), _p(step), _p(next_ids), _p(ids_out),
                                      _p(keep_going), B, max_len, int(pad_id), int(eos_id), 1 if early_stop else 0,
                                      _stream()))


# ------------------------------------------------------------------ RWKV -----------------
def layer_norm_ce_mix(x, gamma, beta, eps, prev, ws, outs, out=None):
    """LayerNorm (NormCE) and the token-shift mixes of its result in one launch; prev is overwritten with the
    normalised rows, which `out` also receives when given."""
    _need(x, torch.float16, "x", 2)
    _need(prev, torch.float16, "prev", 2)
    _need(gamma, torch.float16, "gamma", 1)
    _need(beta, torch.float16, "beta", 1)
    rows, cols = x.shape
    if tuple(prev.shape) != (rows, cols) or len(ws) != len(outs) or not 1 <= len(ws) <= 3:
        raise ValueError("layer_norm_ce_mix: prev must have x's shape, and one to three mixing vectors an output each")
    for t in list(ws) + list(outs):
        _need(t, torch.float16, "mixing vector / output")
    w = list(ws) + [None] * (3 - len(ws))
    o = list(outs) + [None] * (3 - len(outs))
    check(_lib.load().pta_layer_norm_ce_mix(_p(x), _p(gamma), _p(beta), _p(out), _p(prev), _p(w[0]), _p(w[1]), _p(w[2]),
                                            _p(o[0]), _p(o[1]), _p(o[2]), rows, cols, float(eps), _stream()))
    return outs


def rwkv_mix(x, prev, ws, outs):
    """Token-shift mixes for 1..3 mixing vectors; prev is overwritten with x."""
    rows, cols = x.shape
    w = list(ws) + [None] * (3 - len(ws))
    o = list(outs) + [None] * (3 - len(outs))
    check(_lib.load().pta_rwkv_mix(_p(x), _p(prev), _p(w[0]), _p(w[1]), _p(w[2]), _p(o[0]), _p(o[1]), _p(o[2]), rows, cols,
                                   _stream()))
    return outs


def rwkv_wkv(k, v, r, time_decay, time_first, num, den, max_state, y):
    rows, cols = k.shape
    check(_lib.load().pta_rwkv_wkv(_p(k), _p(v), _p(r), _p(time_decay), _p(time_first), _p(num), _p(den), _p(max_state),
                                   _p(y), rows, cols, _stream()))
    return y


class DecodeStep:
    """One whole loop iteration of an INT4 Llama-2-shaped decoder in a single persistent launch
    (pta_llama_decode_step).  Holds the device copies of the layer descriptors and the workspace;
    raises NotImplementedError for shapes the kernel does not cover."""

    def __init__(self, layers, embed, final_norm, head, inv_freq, batch, hidden, n_head, head_dim, ffn, vocab, max_len,
                 eps, pad_id, eos_id, early_stop, state, kv_scale=None):
        lib = _lib.load()
        self.kv_scale = kv_scale            # not None: the layers' KV rings hold F143 bytes (pta_llama_decode_step_f8)
        dev = embed.device
        arr = (_lib.DecodeLayer * len(layers))()
        for dst, src in zip(arr, layers):
            for name, t in src.items():
                setattr(dst, name, t.data_ptr())
        self.layers = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8).to(dev)
        self._keep = (layers, embed, final_norm, head, inv_freq, state)
        self.model = _lib.DecodeModel(self.layers.data_ptr(), len(layers), embed.data_ptr(), final_norm.data_ptr(),
                                      head.data_ptr(), inv_freq.data_ptr(), batch, hidden, n_head, head_dim, ffn, vocab,
                                      max_len, eps, pad_id, eos_id, 1 if early_stop else 0)
        nbytes = lib.pta_decode_step_workspace_bytes(ctypes.byref(self.model))
        if nbytes == 0:
            raise NotImplementedError(f"decode step kernel: unsupported shape (batch {batch}, head size {head_dim}, "
                                      f"hidden {hidden}, ffn {ffn}, vocabulary {vocab})")
        self.workspace = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        self.state = _lib.DecodeState(**{k: v.data_ptr() for k, v in state.items()})

    def launch(self):
        if self.kv_scale is not None:
            check(_lib.load().pta_llama_decode_step_f8(ctypes.byref(self.model), ctypes.byref(self.state), int(self.kv_scale),
                                                       _p(self.workspace), _stream()))
            return
        check(_lib.load().pta_llama_decode_step(ctypes.byref(self.model), ctypes.byref(self.state), _p(self.workspace),
                                                _stream()))

    def launch_static(self, clear_failure=False):
        """The same iteration through the entry point that allocates nothing: its workspace is the array built
        into the library, not `self.workspace` (pta_llama_decode_step_static)."""
        if self.kv_scale is not None:
            raise NotImplementedError("the entry point without a workspace keeps fp16 KV rings")
        check(_lib.load().pta_llama_decode_step_static(ctypes.byref(self.model), ctypes.byref(self.state),
                                                       1 if clear_failure else 0, _stream()))

    def clear_failure(self):
        """Re-arms a workspace whose failure word a launch has set (the word is sticky: until it is cleared every
        launch returns at once)."""
        torch.cuda.synchronize()
        self.workspace.view(torch.int32)[1] = 0

    def failed(self):
        flag = ctypes.c_int(0)
        check(_lib.load().pta_decode_step_failed(_p(self.workspace), ctypes.byref(flag), _stream()))
        return bool(flag.value)
