"""CPU restatement (numpy) of the PopTransformer decode-step operators.

TEST INFRASTRUCTURE ONLY.  This module is the parity checker for the HIP library: it may be
imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``, and by nothing else.  It is never a fallback for the GPU path.

Every function cites the reference file:line it follows (paths relative to the PopTransformer
source tree).  The reference holds no tests, golden vectors or fixtures, and neither its Python
package (needs popart / poprt / hydra) nor its C++ (needs the Poplar SDK) can run without an
IPU software stack, so each function is pinned by what the mathematics fixes instead: truth
tables, closed forms, brute force on tiny inputs and library routines (see ``tests/``).

Functions whose exact numerics live in a third-party dependency of the reference that is not
part of its tree are PARITY UNPINNED; they implement the documented format and say so:
  * ``f8_encode`` / ``f8_decode``  (poprt 1.1.0 ``convert_float_to_uint8``; Poplar SDK 3.2
    ``popops::cast`` to QUARTER).  Inside each format's range they are checked against torch's
    fnuz casts; that values beyond the range saturate at the largest finite code is an
    assumption that nothing checks
  * ``gelu`` (PopART ``aiGraphcore.gelu``), ``swish`` (``aiGraphcore.swish``)
  * accumulation order of every MatMul (poplin), tie-breaking of ``popnn::topK``
"""
import math

import numpy as np

f16 = np.float16
f32 = np.float32


# --------------------------------------------------------------------------------------
# A1  Int4ToHalf
# --------------------------------------------------------------------------------------
def nibble_hi(b):
    """hi = int8(b) >> 4, arithmetic (custom_ops/int4_to_half_codelets.cpp:34)."""
    return np.asarray(b, dtype=np.int8) >> 4


def nibble_lo(b):
    """lo = int8(b << 4) >> 4 (custom_ops/int4_to_half_codelets.cpp:33)."""
    b = np.asarray(b, dtype=np.int8)
    return (b.view(np.uint8) << 4).astype(np.uint8).view(np.int8) >> 4


def int4_table():
    """The 256x2 lookup table of custom_ops/int4_to_half_custom_op.cpp:139-149:
    table[2i] = high nibble, table[2i+1] = low nibble of byte value i."""
    idx = np.arange(256, dtype=np.uint8).view(np.int8)
    return np.stack([nibble_hi(idx), nibble_lo(idx)], axis=1).astype(np.float32)


def int4_to_half(packed, scale, axis=1):
    """Int4ToHalf (poptransformer/ops/customized.py:115-125).

    packed int8 [n, m], scale fp16.
    axis=1 (custom_ops/int4_to_half_custom_op.cpp:280-380): per byte the LUT vertex emits
    [hi, lo] (int4_to_half_codelets.cpp:58-65); the result is reshaped to [n, 2m], transposed
    to [2m, n] and multiplied by scale[n] in fp16 (:362-378).
    axis=0 (:168-278): highData and lowData are [n, m], each already multiplied by scale[m]
    in fp16 (codelets:30-35), interleaved by rows into [2n, m] (:262-264).
    Shape guards follow Int4ToHalfOp::setup (:65-98).
    """
    packed = np.asarray(packed)
    scale = np.asarray(scale)
    if packed.ndim != 2:
        raise ValueError(f"[Int4ToHalfOp] The rank of input should be 2. But now it is {packed.ndim}.")
    if scale.ndim != 1:
        raise ValueError(f"[Int4ToHalfOp] The rank of scale should be 1. But now it is {scale.ndim}.")
    if packed.dtype != np.int8 or scale.dtype != f16:
        raise ValueError("[Int4ToHalfOp] input must be int8 and scale float16")
    n, m = packed.shape
    hi = nibble_hi(packed).astype(f16)
    lo = nibble_lo(packed).astype(f16)
    if axis == 1:
        if scale.shape[0] != n:
            raise ValueError(f"[Int4ToHalfOp] input.shape[0]({n}) should be equal to  scale.shape[0]({scale.shape[0]})")
        q = np.stack([hi, lo], axis=2).reshape(n, 2 * m)       # [n, 2m]: hi first
        return (q.T * scale[None, :]).astype(f16)               # [2m, n], one fp16 multiply
    if axis == 0:
        if scale.shape[0] != m:
            raise ValueError(f"[Int4ToHalfOp] input.shape[1]({m}) should be equal to  scale.shape[0]({scale.shape[0]})")
        h = (hi * scale[None, :]).astype(f16)
        l = (lo * scale[None, :]).astype(f16)
        return np.stack([h, l], axis=1).reshape(2 * n, m)
    raise ValueError(f"[Int4ToHalfOp] 'axis' should be 0 or 1. But now it is {axis}.")


def pack_int4(q):
    """Inverse of the nibble extraction: q int [n, 2m] in [-8, 7] -> int8 [n, m], element 2j in the
    high nibble (test helper; the reference only loads pre-packed checkpoints)."""
    q = np.asarray(q).astype(np.int16)
    assert q.min() >= -8 and q.max() <= 7 and q.shape[-1] % 2 == 0
    hi = (q[..., 0::2] & 0xF).astype(np.uint8)
    lo = (q[..., 1::2] & 0xF).astype(np.uint8)
    return ((hi << 4) | lo).astype(np.uint8).view(np.int8)


# --------------------------------------------------------------------------------------
# A3  MatMul
# --------------------------------------------------------------------------------------
def matmul(x, w):
    """ops.matmul (poptransformer/ops/popart.py:55-67): fp16 x fp16 -> fp16 with fp32 partials
    (the PopART default); numpy broadcasting over leading axes.  fp32 inputs stay fp32."""
    x = np.asarray(x)
    w = np.asarray(w)
    out = np.matmul(x.astype(f32), w.astype(f32))
    if x.dtype == f16 and w.dtype == f16:
        return out.astype(f16)
    return out


def w4a16_matmul(x, packed, scale):
    """prepare_int4_matmul + matmul_int4 (utils/param_handler/precision_strategy.py:56-60,74-75):
    W = Int4ToHalf(packed, scale, axis=1), then ops.matmul."""
    return matmul(x, int4_to_half(packed, scale, axis=1))


# --------------------------------------------------------------------------------------
# A7/A8  KV cache
# --------------------------------------------------------------------------------------
class KVCache:
    """KVCacheOpx::grow (custom_ops/kv_cache.cpp:94-187): a persistent tensor with the sequence
    axis extended to max_len.  Each call: clone = zeros if step == 0 else cache (:118-125);
    cache = concat(input, clone[0 : max_len - step_len]) along the sequence axis (:127-132);
    the op's output is the cache.  With fp8 (:102-104, :183-185) the input is first cast to F143 bytes
    with the constant metadata scale 1 (CastToUint8, :43-53), the persistent tensor holds bytes, and the
    output is the whole cache cast back to fp16 (CastUint8ToFP16, :56-74)."""
    FP8_SCALE = 1

    def __init__(self, max_len, sequence_axis=1, step_len=1, fp8=False):
        self.max_len, self.axis, self.step_len, self.fp8 = max_len, sequence_axis, step_len, fp8
        self.cache = None

    def __call__(self, step, updater):
        updater = np.asarray(updater)
        if updater.shape[self.axis] != self.step_len:
            raise ValueError("updater sequence length != step_len")
        if self.fp8:
            updater = f8_encode(updater, "F143", self.FP8_SCALE)
        if self.cache is None:
            shape = list(updater.shape)
            shape[self.axis] = self.max_len
            self.cache = np.zeros(shape, updater.dtype)   # contents are undefined before step 0
        clone = np.zeros_like(self.cache) if int(step) == 0 else self.cache.copy()
        keep = np.take(clone, range(0, self.max_len - self.step_len), axis=self.axis)
        self.cache = np.concatenate([updater, keep], axis=self.axis)
        if self.fp8:
            return f8_decode(self.cache, "F143", self.FP8_SCALE, f16)
        return self.cache


class KVCachePipeline:
    """KVCachePipelineOpx::grow (custom_ops/kv_cache_pipeline.cpp:374-451) with codelets
    custom_ops/kv_cache_codelet.cpp:18-131: max_bps independent caches; bpsIdx = step % max_bps
    (codelet:27-35); every cache zeroed when step == 0 (:46-64); only cache bpsIdx shifts in the
    new rows and is returned (pipeline.cpp:422-439).  The sequence axis must be rank - 2
    (custom_ops/kv_cache_pipeline.hpp:80-88).
    transpose (pipeline.cpp:397-401,445-449; codelet:170-212): the op swaps the last two axes of its input, keeps
    the persistent caches with the sequence as the LAST axis, shifts cache bpsIdx by one element along it in place
    (new element at index 0; step_len must be 1, pipeline.cpp:410) and swaps the axes of its output back: the
    output equals that of transpose = 0, the stored layout (`stored()`) differs."""

    def __init__(self, max_len, max_bps, step_len=1, transpose=False):
        if transpose and step_len != 1:
            raise ValueError("transpose = 1 takes one new row per call")
        self.max_len, self.max_bps, self.step_len, self.transpose = max_len, max_bps, step_len, transpose
        self.caches = None

    def stored(self):
        """The persistent tensors as the op holds them: [.., D, max_len] each when transpose, else [.., max_len, D]."""
        return [c.copy() for c in self.caches]

    def __call__(self, step, updater):
        updater = np.asarray(updater)
        if self.transpose:
            updater = np.swapaxes(updater, -1, -2)            # pipeline.cpp:397-401: the sequence becomes the last axis
            axis = updater.ndim - 1
        else:
            axis = updater.ndim - 2
        if self.caches is None:
            shape = list(updater.shape)
            shape[axis] = self.max_len
            self.caches = [np.zeros(shape, updater.dtype) for _ in range(self.max_bps)]
        if int(step) == 0:
            self.caches = [np.zeros_like(c) for c in self.caches]
        i = int(step) % self.max_bps
        keep = np.take(self.caches[i], range(0, self.max_len - self.step_len), axis=axis)
        self.caches[i] = np.concatenate([updater, keep], axis=axis)
        return np.swapaxes(self.caches[i], -1, -2) if self.transpose else self.caches[i]


# --------------------------------------------------------------------------------------
# A9  SoftmaxV3
# --------------------------------------------------------------------------------------
def softmax_ce(x, dim=-1, stable_mode=True):
    """getSoftmax (custom_ops/softmax.cpp:41-83).  Last axis only (softmax.hpp:71-91).
    [x -= max(x)] in the input type; e = exp(x) in the input type; S = sum(e) accumulated and
    kept in fp32 (:66-72); r = 1/S in fp32 (:73), cast to fp16 when the input is fp16 (:75-78);
    y = e * r in the input type (:81)."""
    x = np.asarray(x)
    if x.ndim < 2:
        raise ValueError("[Softmax] rank of input should be >= 2")
    if dim not in (-1, x.ndim - 1):
        raise ValueError("[Softmax] axis must be the last axis")
    dt = x.dtype
    if dt not in (f16, f32):
        raise ValueError("[Softmax] input type must be FLOAT16 or FLOAT")
    if stable_mode:
        x = (x - x.max(axis=-1, keepdims=True)).astype(dt)
    with np.errstate(over="ignore"):
        e = np.exp(x.astype(f32)).astype(dt)
    s = e.astype(f32).sum(axis=-1, keepdims=True, dtype=f32)
    with np.errstate(divide="ignore"):
        r = (f32(1.0) / s).astype(dt)
    return (e * r).astype(dt)


# --------------------------------------------------------------------------------------
# A11  NormCE LayerNorm
# --------------------------------------------------------------------------------------
def layer_norm_ce(x, gamma, beta, eps, batch_size, sequence_length, input_size):
    """ops.layer_norm_ce (poptransformer/ops/customized.py:69-102) -> NormCE.

    rows == 1: calSmallBatchNorm (custom_ops/NormCE.cpp:122-200) reduces mean and mean of squares
    in fp32 and GetInPlaceNorm (custom_ops/NormCECodelets.cpp:78-110) computes
    var = power - mean*mean + eps (fp32), rstd16 = fp16(rsqrt(var)), mean16 = fp16(mean).
    rows > 1: normInfKernel (custom_ops/NormCE.S:243-423; C form NormCECodelets.cpp:181-211):
    sum and sum of squares in fp32 (f16v8sqacc), avg = sum/N, mean16 = fp16(avg),
    var = max(sq/N - fp32(mean16)^2, 0) + eps, rstd16 = fp16(1/sqrt(var)).
    Both: y = (((x - mean16) * rstd16) * gamma) + beta, each an fp16 operation.
    Guards: the Python asserts (:81-82) and NormCEOutplaceOpx::grow (NormCE.cpp:541-577).
    """
    x = np.asarray(x)
    assert input_size & 1 == 0
    assert input_size < 8192
    if x.dtype != f16:
        raise ValueError("[NormCE] only float16 is supported")
    if input_size % 4 != 0:
        raise ValueError("[NormCE] the normalised size must be a multiple of 4")
    rows = int(np.prod([batch_size, sequence_length, input_size]) // input_size)
    shape = x.shape
    xr = x.reshape(rows, input_size)
    xf = xr.astype(f32)
    inv_n = f32(1.0 / input_size)
    s = xf.sum(axis=1, dtype=f32)
    sq = (xf * xf).sum(axis=1, dtype=f32)
    mean = (s * inv_n).astype(f32)
    power = (sq * inv_n).astype(f32)
    mean16 = mean.astype(f16)
    if rows == 1:
        var = (power - mean * mean + f32(eps)).astype(f32)
    else:
        m = mean16.astype(f32)
        var = (np.maximum(power - m * m, f32(0.0)) + f32(eps)).astype(f32)
    rstd16 = (f32(1.0) / np.sqrt(var, dtype=f32)).astype(f16)
    g = np.asarray(gamma, f16)[None, :]
    b = np.asarray(beta, f16)[None, :]
    y = (xr - mean16[:, None]).astype(f16)
    y = (y * rstd16[:, None]).astype(f16)
    y = (y * g).astype(f16)
    y = (y + b).astype(f16)
    return y.reshape(shape)


# --------------------------------------------------------------------------------------
# A12  RMSNorm
# --------------------------------------------------------------------------------------
def rms_norm(x, weight, eps):
    """BaseRMSLayerNorm.__call__ (poptransformer/layers/rms_layer_norm.py:26-36): cast to fp32,
    square, reducemean over the last axis, + eps, sqrt, reciprocal (all fp32), cast to fp16,
    x * variance (fp16), * weight (fp16)."""
    x = np.asarray(x, f16)
    v = x.astype(f32)
    v = (v * v).astype(f32)
    v = v.mean(axis=-1, keepdims=True, dtype=f32)
    v = (v + f32(eps)).astype(f32)
    v = np.sqrt(v, dtype=f32)
    v = (f32(1.0) / v).astype(f32)
    v = v.astype(f16)
    y = (x * v).astype(f16)
    return (y * np.asarray(weight, f16)).astype(f16)


# --------------------------------------------------------------------------------------
# A13  next-token selection
# --------------------------------------------------------------------------------------
def topk1(logits, axis=-1):
    """ops.topk(k=1) (poptransformer/ops/popart.py:135-137; layers/lm_head.py:55-56): values and
    indices of the maximum, keepdims; equal values resolve to the lowest index (ONNX TopK)."""
    logits = np.asarray(logits)
    idx = np.argmax(logits, axis=axis)            # numpy returns the first maximum
    idx = np.expand_dims(idx, axis)
    return np.take_along_axis(logits, idx, axis), idx.astype(np.int32)


# --------------------------------------------------------------------------------------
# activations (PARITY UNPINNED: PopART/poplibs implementations, textbook definitions used)
# --------------------------------------------------------------------------------------
def gelu(x):
    """aiGraphcore.gelu (poptransformer/ops/popart.py:142): tanh form, evaluated in fp32 from the
    fp16 input and rounded once.  PopART exposes the erf form as a separate op (geluerf)."""
    x = np.asarray(x)
    v = x.astype(f32)
    u = f32(0.7978845608028654) * (v + f32(0.044715) * v * v * v)
    return (f32(0.5) * v * (f32(1.0) + np.tanh(u))).astype(x.dtype)


def swish(x):
    """aiGraphcore.swish (poptransformer/ops/popart.py:218): x * sigmoid(x), fp32 then one rounding."""
    x = np.asarray(x)
    v = x.astype(f32)
    with np.errstate(over="ignore"):
        return (v / (f32(1.0) + np.exp(-v))).astype(x.dtype)


def sigmoid(x):
    """aiOnnx.sigmoid (poptransformer/ops/popart.py:209)."""
    x = np.asarray(x)
    with np.errstate(over="ignore"):
        return (f32(1.0) / (f32(1.0) + np.exp(-x.astype(f32)))).astype(x.dtype)


# --------------------------------------------------------------------------------------
# BeamSearch (custom_ops/beam_search_custom_op.cpp)
# --------------------------------------------------------------------------------------
def _topk_desc(x, k):
    """Values and indices of the k largest entries along the last axis, largest first, equal values in
    ascending order of index (popnn::topK with sorted = true; its tie order is not pinned by the reference tree)."""
    order = np.argsort(-x.astype(np.float64), axis=-1, kind="stable")[..., :k]
    return np.take_along_axis(x, order, axis=-1), order.astype(np.int32)


def beam_search_step(logits, hyp_container, prob_container, step, beam_size):
    """BeamSearchOpx::grow (custom_ops/beam_search_custom_op.cpp:333-478), one call of the op.
    logits [B, beam, V] (fp16 or fp32: the scores that add along a hypothesis), hyp_container int32
    [B, max_len, beam], prob_container [B, beam] of the logits' dtype, step int.  Returns (next_id [B, beam],
    global_best_id [B, beam], hyp_container, prob_container); the containers are new arrays.
    Shape guards: BeamSearchOp::setup (:103-177).
      every step: per beam the `beam` best scores and ids over the vocabulary (:347-354);
      step == 0 (:371-385): next_id = global_best_id = the ids of beam 0; hyp_container[:, 0] = next_id;
        prob_container = the scores of beam 0;
      step != 0 (:387-466): candidate (i, j) = prob_container[i] + score j of beam i, added in the containers'
        dtype (:400-401); row `step` of the beam-by-beam expanded hypotheses takes the candidate ids (:403-417;
        a step beyond the container writes nothing); the `beam` best candidates over the beam * beam (:424-432)
        give global_best_id (flat index i * beam + j), next_id (their ids, :438-446), every row of hyp_container
        re-gathered from the parent beam i (:452-463) and prob_container (:465-466)."""
    logits = np.asarray(logits)
    hyp = np.asarray(hyp_container)
    prob = np.asarray(prob_container)
    if logits.ndim != 3:
        raise ValueError(f"[Beam Search] The rank of logits should be 3. But now it is {logits.ndim}.")
    B, nb, V = logits.shape
    if beam_size > V:
        raise ValueError("[Beam Search] The parameter 'beam_size' should not be greater than the vocab_size")
    if hyp.ndim != 3 or prob.ndim != 2:
        raise ValueError("[Beam Search] hyp_container must have rank 3 and prob_container rank 2")
    if hyp.shape[0] != B or prob.shape[0] != B or nb != beam_size or hyp.shape[2] != beam_size or prob.shape[1] != beam_size:
        raise ValueError("[Beam Search] batch or beam sizes of logits, hyp_container and prob_container differ")
    dt = prob.dtype
    best_v, best_i = _topk_desc(logits, beam_size)                      # [B, beam, beam]
    if int(step) == 0:
        next_id = best_i[:, 0, :].copy()
        out_h = hyp.copy()
        out_h[:, 0, :] = next_id
        return next_id, next_id.copy(), out_h, best_v[:, 0, :].astype(dt)
    cand = (best_v.astype(dt) + prob[:, :, None]).astype(dt).reshape(B, beam_size * beam_size)
    ids = best_i.reshape(B, beam_size * beam_size)
    temp = np.repeat(hyp, beam_size, axis=2)                            # [B, max_len, beam * beam]: entry i * beam + j = hyp[.., i]
    if 0 <= int(step) < hyp.shape[1]:
        temp[:, int(step), :] = ids
    g_v, g_i = _topk_desc(cand, beam_size)                              # [B, beam]
    next_id = np.take_along_axis(ids, g_i, axis=1)
    out_h = np.take_along_axis(temp, np.broadcast_to(g_i[:, None, :], (B, hyp.shape[1], beam_size)), axis=2)
    return next_id.astype(np.int32), g_i.astype(np.int32), out_h.astype(np.int32), g_v.astype(dt)


# --------------------------------------------------------------------------------------
# A14  loop bookkeeping
# --------------------------------------------------------------------------------------
def initial_loop_state(input_ids, max_length):
    """build_default_inputs + build_model_graph_inputs (poptransformer/models/base_model.py:241-269):
    container = the padded prompt; step = 0; mask = [0, -10000, ...] fp16; stop_mask = 0."""
    input_ids = np.asarray(input_ids, np.int32)
    b = input_ids.shape[0]
    assert input_ids.shape[1] == max_length
    mask = np.full((b, max_length), -10000, f16)
    mask[:, 0] = 0
    return {"container": input_ids.copy(), "step": 0, "mask": mask, "stop_mask": np.zeros(b, np.int32)}


def step_containers(state, next_ids, pad_id):
    """HFDecBaseModel.step_containers (poptransformer/models/base_model.py:313-335).  The last
    iteration addresses index max_length, which lies outside the containers; such an update
    changes nothing here."""
    container, mask = state["container"], state["mask"]
    max_len = container.shape[1]
    next_ids = np.asarray(next_ids, np.int32).reshape(-1)
    next_step = state["step"] + 1
    if next_step < max_len:
        mask[:, next_step] = 0
        slot = container[:, next_step]
        id_to_update = np.where(slot == pad_id, next_ids, slot).astype(np.int32)
        container[:, next_step] = id_to_update
    else:
        id_to_update = next_ids
    state["step"] = next_step
    return id_to_update


def step_loop_cond(state, id_to_update, eos_id, early_stop, batch_size):
    """HFDecBaseModel.step_loop_cond (poptransformer/models/base_model.py:337-355): the stop mask
    accumulates (id == eos); with early_stop the loop continues while the PREVIOUS stop mask
    has fewer than batch_size entries set."""
    prev = state["stop_mask"]
    state["stop_mask"] = prev | (np.asarray(id_to_update) == eos_id).astype(np.int32)
    return bool(prev.sum() < batch_size) if early_stop else True


# --------------------------------------------------------------------------------------
# A10  rotary embeddings and attention, one new position (sequence_length == 1)
# --------------------------------------------------------------------------------------
def llama_sincos(step, head_dim):
    """Attention.fixed_pos_embedding (poptransformer/models/llama2/attention.py:28-38): inv_freq is
    an fp16 constant, step is cast to fp16, the angles are an fp16 MatMul, sin/cos are fp16."""
    inv_freq = np.array([1.0 / (10000 ** (i / head_dim)) for i in range(0, head_dim, 2)]).astype(f16)
    ind = np.array([[step]], np.int32).astype(f16)
    ang = matmul(ind, inv_freq.reshape(1, -1))
    return np.sin(ang.astype(f32)).astype(f16), np.cos(ang.astype(f32)).astype(f16)


def llama_rope(x, sin, cos):
    """apply_rotary_pos_emb + rotate_half (poptransformer/models/llama2/attention.py:40-56) on
    x [B, H, 1, D]: sin/cos duplicated to D; rot = concat(-x[D/2:], x[:D/2]);
    y = x*cos + rot*sin, each an fp16 op."""
    d = x.shape[-1]
    s = np.concatenate([sin, sin], axis=1).reshape(1, 1, 1, d)
    c = np.concatenate([cos, cos], axis=1).reshape(1, 1, 1, d)
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    rot = np.concatenate([(x2 * f16(-1)).astype(f16), x1], axis=-1)
    return ((x * c).astype(f16) + (rot * s).astype(f16)).astype(f16)


def glm2_sincos(step, rotary_dim):
    """Attention.fixed_pos_embedding (poptransformer/models/chatglm2/attention.py:77-96) with
    dim = rotary_dim // 2: inv_freq fp32, position cast to fp32, fp32 MatMul, duplicated, cast
    to fp16, then cos/sin in fp16.  Returns cos, sin of shape [dim]."""
    dim = rotary_dim // 2
    inv_freq = np.array([1.0 / (10000 ** (i / dim)) for i in range(0, dim, 2)]).astype(f32)
    freqs = (f32(step) * inv_freq).astype(f32)
    emb = np.concatenate([freqs, freqs]).astype(f16)
    return np.cos(emb.astype(f32)).astype(f16), np.sin(emb.astype(f32)).astype(f16)


def glm2_rope(x, cos, sin):
    """rotary_embedding + apply_rotary_pos_emb (poptransformer/models/chatglm2/attention.py:98-164)
    on x [B, 1, H, D]: only the first D/2 features rotate.  They are de-interleaved
    ([.., D/4, 2] -> transpose -> [.., 2, D/4] flattened), rotated with the rotate-half rule
    (split D/4 | D/4), and re-interleaved."""
    d = x.shape[-1]
    rd = d // 2
    x1, x2 = x[..., :rd], x[..., rd:]
    lead = x1.shape[:-1]
    t = x1.reshape(*lead, rd // 2, 2)
    t = np.swapaxes(t, -1, -2).reshape(*lead, rd)
    a, b = t[..., : rd // 2], t[..., rd // 2:]
    rot = np.concatenate([(b * f16(-1)).astype(f16), a], axis=-1)
    t = ((t * cos).astype(f16) + (rot * sin).astype(f16)).astype(f16)
    t = t.reshape(*lead, 2, rd // 2)
    t = np.swapaxes(t, -1, -2).reshape(*lead, rd)
    return np.concatenate([t, x2], axis=-1)


def attention_scores_to_context(q, k_t, v, mask, scale, softmax_dtype, stable_mode=False):
    """The matmul / scale / mask / softmax / matmul chain shared by the three attention layers.
    q [B,H,1,D], k_t [B,H,D,L], v [B,H,L,D], mask broadcastable [B,1,1,L] fp16.
      Llama2   (models/llama2/attention.py:97-113): scale fp16(1/sqrt(D)), softmax in fp32
      ChatGLM2 (models/chatglm2/attention.py:277-302): scale fp16(1/sqrt(D)), softmax in fp16
      GPT-2    (models/gpt2/attention.py:68-84): no scale in the graph, softmax in fp16."""
    w = matmul(q, k_t)
    if scale is not None:
        w = (w * f16(scale)).astype(f16)
    w = (w + mask).astype(f16)
    if softmax_dtype == f32:
        w = softmax_ce(w.astype(f32), -1, stable_mode).astype(f16)
    else:
        w = softmax_ce(w, -1, stable_mode)
    return matmul(w, v)


# --------------------------------------------------------------------------------------
# A4/A5/A6  FP8 (Graphcore F143 / F152).  PARITY UNPINNED: the encode/decode routines live in
# poprt (`convert_float_to_uint8`, requirements.txt:7) and in the Poplar SDK (`popops::cast` to
# QUARTER), neither of which is part of the reference tree.  The formats implemented here are
# the published ones ("8-bit Numerical Formats for Deep Neural Networks", Graphcore 2022):
#   F143: 1 sign, 4 exponent, 3 mantissa bits, bias 8, subnormals, no infinities, NaN = 0x80,
#         largest magnitude 240;  F152: 1-5-2, bias 16, NaN = 0x80, largest magnitude 57344
# (the `float8_e4m3fnuz` / `float8_e5m2fnuz` encodings).  A QuarterMetadata scale s means
# real value = decode(byte) * 2**s.  Encoding rounds to nearest even and saturates.
# --------------------------------------------------------------------------------------
_F8 = {"F143": (4, 3, 8), "F152": (5, 2, 16)}


def f8_table(fmt):
    """All 256 decoded values of a format as float32 (NaN at 0x80)."""
    if fmt not in _F8:
        raise ValueError(f"Unsupport fp8 meata data {fmt}, it must be F143 or F152")
    eb, mb, bias = _F8[fmt]
    out = np.zeros(256, np.float64)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> mb) & ((1 << eb) - 1)
        m = code & ((1 << mb) - 1)
        if code == 0x80:
            out[code] = np.nan
        elif e == 0:
            out[code] = s * 2.0 ** (1 - bias) * (m / (1 << mb))
        else:
            out[code] = s * 2.0 ** (e - bias) * (1 + m / (1 << mb))
    return out.astype(f32)


def f8_decode(codes, fmt="F143", scale=0, dtype=f16):
    """popops::cast QUARTER -> HALF with QuarterMetadata(fmt, scale)
    (custom_ops/matmul_fp8.cpp:904-930, custom_ops/kv_cache.cpp:56-74)."""
    t = f8_table(fmt).astype(np.float64) * 2.0 ** int(scale)
    with np.errstate(over="ignore"):
        return t[np.asarray(codes, np.uint8)].astype(dtype)


def f8_encode(x, fmt="F143", scale=0):
    """CastToUint8 (poptransformer/ops/customized.py:127-135, custom_ops/cast_to_uint8.cpp:107-127)
    and the host-side `convert_float_to_uint8(w, fmt, scale)` of
    utils/param_handler/precision_strategy.py:44-51: byte whose decoded value * 2**scale is
    nearest to x (ties to the even mantissa), saturating at the largest magnitude; NaN -> 0x80."""
    if fmt not in _F8:
        raise ValueError(f"Unsupport fp8 meata data {fmt}, it must be F143 or F152")
    x = np.asarray(x)
    v = x.astype(np.float64) * 2.0 ** (-int(scale))
    pos = f8_table(fmt)[:128].astype(np.float64)            # codes 0x00..0x7F ascend with the value
    mag = np.abs(v)
    hi = np.searchsorted(pos, mag, side="left").clip(1, 127)
    lo = hi - 1
    d_lo, d_hi = mag - pos[lo], pos[hi] - mag
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo)
    code = np.where(mag >= pos[127], 127, code)              # saturate
    code = np.where(mag <= 0, 0, code).astype(np.uint8)
    out = np.where((v < 0) & (code != 0), code | 0x80, code).astype(np.uint8)   # no negative zero
    return np.where(np.isnan(v), np.uint8(0x80), out).astype(np.uint8)


def fp8_matmul(lhs, rhs, scale_lhs, scale_rhs, fmt_lhs="F143", fmt_rhs="F143"):
    """FP8MatMul (poptransformer/ops/customized.py:137-148; custom_ops/matmul_fp8.cpp:177-250, 885-1003).
    rhs must be uint8; lhs is uint8 (both operands QUARTER, fp32 partials, HALF output) or
    float16 (rhs cast to HALF first, then an fp16 MatMul).  Scales are int32 tensors of which
    element 0 is read (:890-891)."""
    lhs, rhs = np.asarray(lhs), np.asarray(rhs)
    if lhs.dtype not in (f16, np.uint8):
        raise ValueError(f"Invalid input data type of {lhs.dtype}, it must be FLOAT16 or UINT8")
    if rhs.dtype != np.uint8:
        raise ValueError(f"Invalid weight data type of {rhs.dtype}, it must be UINT8")
    sl, sr = int(np.asarray(scale_lhs).reshape(-1)[0]), int(np.asarray(scale_rhs).reshape(-1)[0])
    if lhs.shape[-1] != rhs.shape[-2]:
        raise ValueError("contracting dimensions differ")
    if lhs.dtype == np.uint8:
        a = f8_decode(lhs, fmt_lhs, sl, np.float64)
        b = f8_decode(rhs, fmt_rhs, sr, np.float64)
        with np.errstate(over="ignore"):
            return np.matmul(a, b).astype(f32).astype(f16)
    return matmul(lhs, f8_decode(rhs, fmt_rhs, sr, f16))
