"""Pins of the numpy oracle: every operator restatement is checked against something the
reference's own text or the mathematics fixes (truth tables, closed forms, brute force on tiny
inputs, library routines), chosen so that a plausible mistake - a swapped nibble, a transposed
operand, a shifted index, a missing rounding - fails at least one check."""
import numpy as np
import pytest
import scipy.special
import torch

from oracle import ops as O

f16, f32 = np.float16, np.float32


# ---------------------------------------------------------------- A1 Int4ToHalf
def test_nibbles_exhaustive_truth_table():
    # the LUT loop of custom_ops/int4_to_half_custom_op.cpp:141-149, restated with C semantics:
    # high = float(char(idx) >> 4); low = float(char(idx << 4) >> 4)
    tab = O.int4_table()
    for i in range(256):
        c = i - 256 if i >= 128 else i                     # char(idx)
        hi = c >> 4                                          # arithmetic shift (python ints floor)
        lo8 = (i << 4) & 0xFF
        lo8 = lo8 - 256 if lo8 >= 128 else lo8
        lo = lo8 >> 4
        assert tab[i, 0] == hi and tab[i, 1] == lo
        assert -8 <= hi <= 7 and -8 <= lo <= 7
        assert ((hi & 0xF) << 4 | (lo & 0xF)) == i          # the two nibbles rebuild the byte


def test_pack_unpack_roundtrip():
    rng = np.random.default_rng(0)
    q = rng.integers(-8, 8, size=(5, 12))
    p = O.pack_int4(q)
    w = O.int4_to_half(p, np.ones(5, f16), axis=1)          # [12, 5]
    assert np.array_equal(w.T.astype(np.int64), q)


def test_int4_axis1_layout_brute_force():
    # n=3 rows (output channels), m=2 bytes: out[2j+h, r] = nibble_h(P[r, j]) * scale[r]
    P = np.array([[0x12, 0xF8], [0x7F, 0x80], [0xA5, 0x3C]], dtype=np.uint8).view(np.int8)
    s = np.array([1.0, 0.5, 2.0], f16)
    out = O.int4_to_half(P, s, axis=1)
    assert out.shape == (4, 3)
    expect = np.zeros((4, 3))
    for r in range(3):
        for j in range(2):
            b = int(P.view(np.uint8)[r, j])
            hi = (b >> 4) - 16 if (b >> 4) >= 8 else (b >> 4)
            lo = (b & 15) - 16 if (b & 15) >= 8 else (b & 15)
            expect[2 * j, r] = hi * float(s[r])
            expect[2 * j + 1, r] = lo * float(s[r])
    assert np.array_equal(out.astype(np.float64), expect)


def test_int4_axis0_layout_brute_force():
    P = np.array([[0x12, 0xF8], [0x7F, 0x80], [0xA5, 0x3C]], dtype=np.uint8).view(np.int8)
    s = np.array([1.0, 0.5], f16)
    out = O.int4_to_half(P, s, axis=0)                      # [2n, m] rows 2i = high, 2i+1 = low
    assert out.shape == (6, 2)
    for i in range(3):
        for c in range(2):
            assert out[2 * i, c] == f16(O.nibble_hi(P[i, c])) * s[c]
            assert out[2 * i + 1, c] == f16(O.nibble_lo(P[i, c])) * s[c]


def test_int4_scale_multiply_is_one_fp16_rounding():
    # 7 * s needs up to 14 significant bits: the product must be rounded ONCE to fp16 (RNE)
    rng = np.random.default_rng(1)
    s = rng.uniform(0.005, 0.02, 64).astype(f16)
    P = np.full((64, 1), 0x79, np.uint8).view(np.int8)      # hi = 7, lo = -7
    out = O.int4_to_half(P, s, axis=1)
    exact = 7.0 * s.astype(np.float64)
    assert np.array_equal(out[0], exact.astype(f16))
    assert np.array_equal(out[1], (-exact).astype(f16))
    assert np.any(out[0].astype(np.float64) != exact)       # the rounding is really exercised


def test_int4_guards():
    P = np.zeros((4, 4), np.int8)
    with pytest.raises(ValueError):
        O.int4_to_half(P, np.ones(4, f16), axis=2)
    with pytest.raises(ValueError):
        O.int4_to_half(P, np.ones(5, f16), axis=1)
    with pytest.raises(ValueError):
        O.int4_to_half(P[0], np.ones(4, f16), axis=1)
    with pytest.raises(ValueError):
        O.int4_to_half(P, np.ones((4, 1), f16), axis=1)


def test_w4a16_matmul_against_float64():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((3, 64)).astype(f16)
    q = rng.integers(-8, 8, size=(10, 64))
    s = rng.uniform(0.005, 0.02, 10).astype(f16)
    y = O.w4a16_matmul(x, O.pack_int4(q), s)
    w = (q.T.astype(f16) * s[None, :]).astype(f16)          # independent construction of W[k, n]
    ref = x.astype(np.float64) @ w.astype(np.float64)
    assert y.dtype == f16 and y.shape == (3, 10)
    assert np.abs(y.astype(np.float64) - ref).max() <= 2.0 ** -10 * np.abs(ref).max()


# ---------------------------------------------------------------- A7 / A8 KV cache
def _shift_register_reference(max_len, steps, shape, axis, rng, dtype):
    """concat(new, old[:-1]) as the reference itself restates the op in pure graph ops
    (poptransformer/models/chatglm/attention.py:44-56), with the zeroing at step 0."""
    cache = None
    for step in range(steps):
        new = rng.standard_normal(shape).astype(dtype)
        if step == 0 or cache is None:
            s = list(shape)
            s[axis] = max_len
            cache = np.zeros(s, dtype)
        idx = [slice(None)] * len(shape)
        idx[axis] = slice(0, max_len - 1)
        cache = np.concatenate([new, cache[tuple(idx)]], axis=axis)
        yield step, new, cache


@pytest.mark.parametrize("axis,shape", [(1, (2, 1, 3)), (3, (2, 1, 2, 1, 4))])
def test_kv_cache_brute_force_including_overflow(axis, shape):
    max_len = 4
    op = O.KVCache(max_len, axis, 1)
    rng = np.random.default_rng(3)
    news = []
    for step, new, ref in _shift_register_reference(max_len, max_len + 3, shape, axis, rng, f16):
        out = op(step, new)
        news.append(new)
        assert np.array_equal(out, ref)
        # closed form: row i of the output is the update of step - i, zero before step 0
        for i in range(max_len):
            row = np.take(out, [i], axis=axis)
            assert np.array_equal(row, news[step - i] if step - i >= 0 else np.zeros_like(new))
    out = op(0, news[0])                                    # step 0 clears the history
    assert np.count_nonzero(np.take(out, range(1, max_len), axis=axis)) == 0


def test_kv_cache_step_len_two():
    op = O.KVCache(6, 1, 2)
    a = np.arange(4, dtype=f32).reshape(1, 2, 2)
    b = a + 10
    op(0, a)
    out = op(1, b)
    assert np.array_equal(out[0, :2], b[0]) and np.array_equal(out[0, 2:4], a[0]) and not out[0, 4:].any()


def test_kv_cache_fp8_is_the_fp16_cache_on_the_f143_grid():
    """fp8 = true: every row of the output is the row the fp16 cache holds, cast to F143 with scale 1 and back
    (the cast is elementwise, so it commutes with the shift); values beyond 240 * 2 saturate at 480, values on
    the grid come back unchanged, and the rows before step 0 read as zero."""
    rng = np.random.default_rng(5)
    plain, cast = O.KVCache(4, 1, 1), O.KVCache(4, 1, 1, fp8=True)
    for step in range(7):
        new = (rng.standard_normal((2, 1, 8)) * 300).astype(f16)
        new[0, 0, :3] = [1000.0, -1000.0, 0.40625]             # saturating, saturating, on the grid (13 * 2^-5)
        ref = O.f8_decode(O.f8_encode(plain(step, new), "F143", 1), "F143", 1, f16)
        out = cast(step, new)
        assert out.dtype == f16 and np.array_equal(out, ref)
        assert out[0, 0, 0] == 480 and out[0, 0, 1] == -480 and out[0, 0, 2] == np.float16(0.40625)
    assert not cast(0, new)[:, 1:].any()


def test_kv_cache_pipeline_slots():
    op = O.KVCachePipeline(max_len=3, max_bps=2)
    seen = {0: [], 1: []}
    rng = np.random.default_rng(4)
    for step in range(9):
        new = rng.standard_normal((2, 1, 4)).astype(f16)
        out = op(step, new)
        slot = step % 2                                      # kv_cache_codelet.cpp:27-35
        seen[slot].insert(0, new)
        for i in range(3):
            want = seen[slot][i] if i < len(seen[slot]) else np.zeros_like(new)
            assert np.array_equal(out[:, i:i + 1], want)
    op(0, new)                                               # step 0 clears every slot
    assert not op.caches[1].any()


# ---------------------------------------------------------------- A9 softmax
@pytest.mark.parametrize("dtype,tol", [(f32, 1e-6), (f16, 2e-3)])
def test_softmax_matches_scipy_and_modes_agree(dtype, tol):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((4, 3, 50)) * 2).astype(dtype)
    ref = scipy.special.softmax(x.astype(np.float64), axis=-1)
    for stable in (False, True):
        y = O.softmax_ce(x, -1, stable)
        assert y.dtype == dtype
        assert np.abs(y.astype(np.float64) - ref).max() <= tol
        assert np.abs(y.astype(np.float64).sum(-1) - 1).max() <= 50 * tol


def test_softmax_mask_rows_are_exact_zero_and_unstable_overflows_like_fp16():
    x = np.array([[1.0, 2.0, -10000.0, -9998.0]], f16)
    y = O.softmax_ce(x, -1, False)
    assert y[0, 2] == 0 and y[0, 3] == 0
    big = np.array([[12.0, 0.0]], f16)                      # exp(12) > 65504: the non-stable form overflows
    assert not np.isfinite(O.softmax_ce(big, -1, False).astype(np.float32)).all() or O.softmax_ce(big, -1, False)[0, 0] == 0
    assert np.isfinite(O.softmax_ce(big, -1, True)).all()


def test_softmax_guards():
    with pytest.raises(ValueError):
        O.softmax_ce(np.zeros(4, f16))
    with pytest.raises(ValueError):
        O.softmax_ce(np.zeros((2, 4), f16), dim=0)


# ---------------------------------------------------------------- A11 / A12 norms
@pytest.mark.parametrize("rows", [1, 5])
def test_layer_norm_ce_against_torch(rows):
    rng = np.random.default_rng(6)
    n = 256
    x = (rng.standard_normal((rows, 1, n)) * 1.5 + 0.2).astype(f16)
    g = rng.uniform(0.5, 1.5, n).astype(f16)
    b = rng.standard_normal(n).astype(f16)
    y = O.layer_norm_ce(x, g, b, 1e-5, rows, 1, n)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x.astype(f32)), (n,), torch.from_numpy(g.astype(f32)),
                                         torch.from_numpy(b.astype(f32)), 1e-5).numpy()
    # four fp16 roundings in the output chain: a few ulp of the largest |gamma * normalised x|
    assert np.abs(y.astype(f32) - ref).max() <= 4 * 2.0 ** -10 * np.abs(ref).max()


def test_layer_norm_ce_invariants_and_guards():
    rng = np.random.default_rng(7)
    n = 512
    x = (rng.standard_normal((3, 1, n)) * 3 + 1).astype(f16)
    y = O.layer_norm_ce(x, np.ones(n, f16), np.zeros(n, f16), 1e-5, 3, 1, n).astype(np.float64)
    assert np.abs(y.mean(-1)).max() < 5e-3 and np.abs(y.var(-1) - 1).max() < 1e-2
    with pytest.raises(AssertionError):
        O.layer_norm_ce(np.zeros((1, 1, 8192), f16), np.ones(8192, f16), np.zeros(8192, f16), 1e-5, 1, 1, 8192)
    with pytest.raises(ValueError):
        O.layer_norm_ce(np.zeros((1, 1, 8), f32), np.ones(8, f16), np.zeros(8, f16), 1e-5, 1, 1, 8)


def test_layer_norm_variants_differ_only_in_variance_handling():
    # a constant row: var = 0.  rows > 1 clamps at 0 (+eps); rows == 1 uses the fp32 mean and no clamp
    n = 64
    x = np.full((2, 1, n), 0.1, f16)
    y2 = O.layer_norm_ce(x, np.ones(n, f16), np.zeros(n, f16), 1e-5, 2, 1, n)
    assert np.isfinite(y2).all()
    m16 = f16(np.float32(x[0, 0].astype(f32).sum() / n))
    assert np.all(y2 == (f16(x[0, 0, 0] - m16) * f16(1 / np.sqrt(np.float32(1e-5)))).astype(f16))


def test_rms_norm_against_hf_llama():
    from transformers.models.llama.modeling_llama import LlamaRMSNorm
    rng = np.random.default_rng(8)
    n = 128
    x = rng.standard_normal((2, 1, n)).astype(f16)
    w = rng.uniform(0.5, 1.5, n).astype(f16)
    mod = LlamaRMSNorm(n, eps=1e-5)
    with torch.no_grad():
        mod.weight.copy_(torch.from_numpy(w.astype(f32)))
        ref = mod(torch.from_numpy(x.astype(f32))).numpy()
    y = O.rms_norm(x, w, 1e-5)
    assert y.dtype == f16
    assert np.abs(y.astype(f32) - ref).max() <= 3 * 2.0 ** -10 * np.abs(ref).max()


# ---------------------------------------------------------------- A13 selection
def test_topk1_lowest_index_on_ties():
    x = np.array([[[1.0, 5.0, 5.0, -2.0]], [[7.0, 7.0, 7.0, 7.0]]], f16)
    v, i = O.topk1(x, axis=2)
    assert i.shape == (2, 1, 1) and i.dtype == np.int32
    assert i[0, 0, 0] == 1 and i[1, 0, 0] == 0 and v[0, 0, 0] == 5.0


# ---------------------------------------------------------------- A14 loop bookkeeping
def _loop_brute_force(ids, next_fn, pad, eos, early_stop, max_loop):
    """Independent scalar restatement of base_model.py:313-355, one sequence at a time."""
    B, L = ids.shape
    cont = ids.copy()
    mask = np.full((B, L), -10000.0)
    mask[:, 0] = 0
    stop = [0] * B
    step = 0
    for _ in range(max_loop):
        nxt = next_fn(step)
        prev_stop = list(stop)
        for b in range(B):
            ns = step + 1
            tok = nxt[b]
            if ns < L:
                mask[b, ns] = 0
                if cont[b, ns] != pad:
                    tok = cont[b, ns]
                cont[b, ns] = tok
            if tok == eos:
                stop[b] = 1
        step += 1
        if early_stop and sum(prev_stop) >= B:
            break
    return cont, mask, np.array(stop), step


@pytest.mark.parametrize("early_stop", [False, True])
def test_loop_bookkeeping(early_stop):
    rng = np.random.default_rng(9)
    B, L, pad, eos = 3, 10, 0, 2
    ids = np.zeros((B, L), np.int32)
    ids[0, :3] = [4, 5, 6]
    ids[1, :1] = [7]
    ids[2, :5] = [3, 3, 2, 3, 3]
    seq = [rng.integers(1, 5, size=B).astype(np.int32) for _ in range(L)]
    state = O.initial_loop_state(ids, L)
    steps = 0
    for _ in range(L):
        upd = O.step_containers(state, seq[state["step"]], pad)
        steps += 1
        if not O.step_loop_cond(state, upd, eos, early_stop, B):
            break
    cont, mask, stop, step = _loop_brute_force(ids, lambda s: seq[s], pad, eos, early_stop, L)
    assert np.array_equal(state["container"], cont)
    assert np.array_equal(state["mask"].astype(np.float64), mask)
    assert np.array_equal(state["stop_mask"], stop)
    assert state["step"] == step


# ---------------------------------------------------------------- A10 rotary embeddings
def test_llama_rope_against_hf():
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    rng = np.random.default_rng(10)
    D, step = 64, 37
    q = rng.standard_normal((2, 3, 1, D)).astype(f16)
    sin, cos = O.llama_sincos(step, D)
    got = O.llama_rope(q, sin, cos).astype(f32)
    inv = 1.0 / (10000 ** (np.arange(0, D, 2) / D))
    ang = step * inv
    c = torch.from_numpy(np.concatenate([np.cos(ang), np.cos(ang)]).astype(f32)).reshape(1, 1, D)
    s = torch.from_numpy(np.concatenate([np.sin(ang), np.sin(ang)]).astype(f32)).reshape(1, 1, D)
    qt = torch.from_numpy(q.astype(f32))
    ref, _ = apply_rotary_pos_emb(qt, qt, c, s)
    # fp16 angle: step * inv_freq rounded to fp16 (|error| <= 2^-11 * 37) bounds the deviation
    assert np.abs(got - ref.numpy()).max() <= 37 * 2.0 ** -10 * 4 + 4e-3


def test_glm2_rope_is_interleaved_pair_rotation():
    rng = np.random.default_rng(11)
    D, step = 128, 9
    x = rng.standard_normal((1, 1, 2, D)).astype(f16)
    cos, sin = O.glm2_sincos(step, D)
    got = O.glm2_rope(x, cos, sin).astype(np.float64)
    ref = x.astype(np.float64).copy()
    for j in range(D // 4):                                  # pairs (2j, 2j+1) of the first D/2 features
        th = step * 10000.0 ** (-2 * j / (D // 2))
        a, b = x[..., 2 * j].astype(np.float64), x[..., 2 * j + 1].astype(np.float64)
        ref[..., 2 * j] = a * np.cos(th) - b * np.sin(th)
        ref[..., 2 * j + 1] = b * np.cos(th) + a * np.sin(th)
    assert np.abs(got - ref).max() <= 2e-2                   # fp16 angle + fp16 products
    assert np.array_equal(got[..., D // 2:], x[..., D // 2:].astype(np.float64))


def test_activations():
    x = np.linspace(-6, 6, 101).astype(f16)
    assert np.abs(O.gelu(x).astype(f32) - torch.nn.functional.gelu(torch.from_numpy(x.astype(f32)), approximate="tanh").numpy()).max() < 3e-3
    assert np.abs(O.swish(x).astype(f32) - torch.nn.functional.silu(torch.from_numpy(x.astype(f32))).numpy()).max() < 3e-3


# ---------------------------------------------------------------- FP8 (format assumption, see oracle/ops.py)
@pytest.mark.parametrize("fmt,tdt", [("F143", torch.float8_e4m3fnuz), ("F152", torch.float8_e5m2fnuz)])
def test_f8_tables_match_fnuz_formats(fmt, tdt):
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(tdt).to(torch.float32).numpy()
    tab = O.f8_table(fmt)
    assert np.isnan(tab[0x80]) and np.isnan(ref[0x80])
    ok = np.arange(256) != 0x80
    assert np.array_equal(tab[ok], ref[ok])
    assert np.nanmax(tab) == (240.0 if fmt == "F143" else 57344.0)


@pytest.mark.parametrize("fmt,tdt", [("F143", torch.float8_e4m3fnuz), ("F152", torch.float8_e5m2fnuz)])
def test_f8_encode_matches_fnuz_cast_and_roundtrips(fmt, tdt):
    rng = np.random.default_rng(12)
    mx = 240.0 if fmt == "F143" else 57344.0
    x = np.concatenate([rng.standard_normal(4000) * 0.05, rng.uniform(-mx, mx, 4000), [0.0, -0.0, mx, -mx]]).astype(f16)
    got = O.f8_encode(x, fmt, 0)
    ref = torch.from_numpy(x.astype(f32)).to(tdt).view(torch.uint8).numpy()
    assert np.array_equal(got, ref)
    # every representable value encodes to its own code
    codes = np.array([c for c in range(256) if c not in (0x80,)], np.uint8)
    assert np.array_equal(O.f8_encode(O.f8_decode(codes, fmt, 0, np.float32), fmt, 0), codes)
    # Beyond the largest finite value nothing here is a pin: torch's fnuz cast gives NaN there, the oracle
    # saturates (its header and the fixture generator record that as an assumption about the Graphcore cast).
    # scale: encode(x, s) stores x * 2^-s
    assert np.array_equal(O.f8_encode(x, fmt, -1), O.f8_encode((x.astype(f32) * 2), fmt, 0))


def test_fp8_matmul_modes():
    rng = np.random.default_rng(13)
    x = rng.standard_normal((3, 32)).astype(f16)
    w = (rng.standard_normal((32, 8)) * 0.05).astype(f32)
    w8 = O.f8_encode(w, "F143", -1)
    s = np.array([-1], np.int32)
    wd = O.f8_decode(w8, "F143", -1, np.float64)
    assert np.abs(wd - w).max() <= 2.0 ** -11 + np.abs(w).max() * 2.0 ** -4   # 3 mantissa bits
    y16 = O.fp8_matmul(x, w8, s, s)
    assert np.abs(y16.astype(np.float64) - x.astype(np.float64) @ wd).max() <= 2e-3
    x8 = O.f8_encode(x, "F143", -1)
    y8 = O.fp8_matmul(x8, w8, s, s)
    xd = O.f8_decode(x8, "F143", -1, np.float64)
    assert np.abs(y8.astype(np.float64) - xd @ wd).max() <= 2e-3
    with pytest.raises(ValueError):
        O.fp8_matmul(x.astype(f32), w8, s, s)
    with pytest.raises(ValueError):
        O.f8_encode(x, "F999", 0)


# ---------------------------------------------------------------- BeamSearch, KVCachePipeline transpose
def _beam_brute_force(logits, hyps, scores, beam):
    """Textbook beam step on explicit hypotheses: every (hypothesis, token) extension scored by
    score + logit, the `beam` best kept (ties: lower hypothesis, then lower token).  No top-k per beam, no flat
    candidate index, no container: an independent formulation of what the op computes for one sequence."""
    ext = []
    for i, (h, s) in enumerate(zip(hyps, scores)):
        for v in range(logits.shape[1]):
            ext.append((-(float(s) + float(logits[i, v])), i, v, h + [v]))
    ext.sort(key=lambda e: (e[0], e[1], e[2]))
    best = ext[:beam]
    return [e[3] for e in best], [-e[0] for e in best], [e[1] for e in best], [e[2] for e in best]


@pytest.mark.parametrize("beam,V", [(2, 7), (3, 11), (4, 6)])
def test_beam_search_step_equals_brute_force(beam, V):
    """fp32 scores drawn from a grid whose sums are exact and distinct, so the op's two-stage selection (top-k
    per beam, then top-k of beam * beam) must keep exactly the brute-force best extensions: tokens, parent
    hypotheses, scores and the whole hypothesis container, over several steps and two sequences."""
    rng = np.random.default_rng(beam * 100 + V)
    B, L, steps = 2, 6, 5
    hyp = np.full((B, L, beam), -7, np.int32)
    prob = np.zeros((B, beam), f32)
    explicit = [None] * B
    for step in range(steps):
        # distinct values k / 1024 per sequence: sums of up to six of them stay exact in fp32
        logits = np.stack([rng.permutation(beam * V * 40)[:beam * V].reshape(beam, V) for _ in range(B)]).astype(f32) / 1024
        nxt, gbest, hyp, prob = O.beam_search_step(logits, hyp, prob, step, beam)
        for b in range(B):
            if step == 0:
                order = np.argsort(-logits[b, 0], kind="stable")[:beam]
                explicit[b] = ([[int(v)] for v in order], [float(logits[b, 0, v]) for v in order])
                assert np.array_equal(nxt[b], order) and np.array_equal(gbest[b], order)
            else:
                hyps, scores, parents, toks = _beam_brute_force(logits[b], *explicit[b], beam)
                explicit[b] = (hyps, scores)
                assert np.array_equal(nxt[b], toks)
                assert np.array_equal(gbest[b] // beam, parents)
                # the flat index names the parent and the rank of the token among the parent's candidates
                for r in range(beam):
                    rank = int(np.argsort(-logits[b, parents[r]], kind="stable").tolist().index(toks[r]))
                    assert gbest[b, r] == parents[r] * beam + rank
            assert np.array_equal(prob[b], np.array(explicit[b][1], f32))
            assert np.array_equal(hyp[b, :step + 1].T, np.array(explicit[b][0], np.int32))
            assert (hyp[b, step + 1:] == -7).all()          # rows beyond the step are only permuted


def test_beam_search_step_guards_dtype_and_ties():
    logits = np.zeros((1, 2, 5), f16)
    with pytest.raises(ValueError):
        O.beam_search_step(logits[0], np.zeros((1, 4, 2), np.int32), np.zeros((1, 2), f16), 0, 2)
    with pytest.raises(ValueError):
        O.beam_search_step(logits, np.zeros((1, 4, 3), np.int32), np.zeros((1, 2), f16), 0, 2)
    with pytest.raises(ValueError):
        O.beam_search_step(logits, np.zeros((1, 4, 2), np.int32), np.zeros((1, 2), f16), 0, 6)
    # equal scores come in ascending order of index, and the sum is rounded in the containers' type
    nxt, gbest, hyp, prob = O.beam_search_step(logits, np.zeros((1, 4, 2), np.int32), np.zeros((1, 2), f16), 0, 2)
    assert nxt.tolist() == [[0, 1]] and prob.dtype == f16
    big = np.full((1, 2, 5), 2048.0, f16)
    big[0, :, 1] = 1.0
    _, gbest, _, prob = O.beam_search_step(big, hyp, np.array([[1.0, 0.0]], f16), 1, 2)
    assert prob.tolist() == [[2048.0, 2048.0]] and gbest.tolist() == [[0, 1]]       # fp16(2048 + 1) = 2048: a tie
    # a step beyond the container writes no row
    _, _, h2, _ = O.beam_search_step(big, hyp, np.array([[1.0, 0.0]], f16), 9, 2)
    assert np.array_equal(np.sort(h2, axis=2), np.sort(hyp[:, :, [0, 0]], axis=2))


def test_kv_cache_pipeline_transposed_storage():
    """transpose = 1: the output is that of transpose = 0, the stored registers are its transposes, and one call
    moves every stored element one place along the last axis - the element loop of the codelet
    (custom_ops/kv_cache_codelet.cpp:180-211) written out for a single feature row."""
    rng = np.random.default_rng(31)
    max_len, max_bps = 6, 2
    plain, seq_last = O.KVCachePipeline(max_len, max_bps), O.KVCachePipeline(max_len, max_bps, transpose=True)
    row = np.zeros(max_len, f16)                          # feature 3 of outer index (1, 0) in register 1
    for step in list(range(9)) + [0, 1, 2]:               # a second generation restarts at step 0
        upd = rng.standard_normal((2, 2, 1, 4)).astype(f16)
        a, b = plain(step, upd), seq_last(step, upd)
        assert np.array_equal(a, b)
        for p, q in zip(plain.stored(), seq_last.stored()):
            assert q.shape == (2, 2, 4, max_len) and np.array_equal(np.swapaxes(p, -1, -2), q)
        if step == 0:
            row[:] = 0
        if step % max_bps == 1:
            for j in range(max_len - 1, 0, -1):
                row[j] = row[j - 1]
            row[0] = upd[1, 0, 0, 3]
        assert np.array_equal(seq_last.stored()[1][1, 0, 3], row)
    with pytest.raises(ValueError):
        O.KVCachePipeline(4, 2, step_len=2, transpose=True)
