"""Whole-model parity of the other benchmark configurations at their own widths (two layers each, so that the
oracle finishes in a minute or two): ChatGLM2 at the 6B width (hidden 4096, 32 query / 2 KV heads of 128, ffn 13696,
vocabulary 65024, batch 8, KV length 4096, a context that crosses 512), RWKV-4 at the 7B width (4096 / 16384 /
vocabulary 65536, batch 1 and 32), GPT-2 small at its full size (12 layers, 768, 12 x 64, vocabulary 50257 - no
multiple of 16 -, prompt 16, 32 new tokens, KV length 128).  Logits within 1e-2 at every step, ids equal wherever
the oracle's two best logits are clearly apart (random N(0, 0.02) weights make near ties frequent: at one, either
candidate is a correct greedy choice and the decoder is given the oracle's token to stay comparable).

The oracle is used with its Linears prepared once (`_Dense`: the fp16 -> fp32 / F143 -> float conversion of a weight
done at set-up instead of per call) and, for ChatGLM2, with the attention taken over the valid cache rows only and
without materialising the KV heads per query head; both are checked here against the oracle's own code paths."""
import copy

import numpy as np
import pytest
import torch

from oracle import models as OM
from oracle import ops as O

pytestmark = pytest.mark.gpu
f16, f32 = np.float16, np.float32


class _Dense:
    """An oracle Linear with the conversion of its weight hoisted out of the call.  fp16 weights (also unpacked INT4):
    O.matmul's fp32 product.  F143 weights with fp16 activations ('fp8_weight'): O.fp8_matmul's second branch, the
    weight cast to fp16 first.  F143 weights and activations ('fp8'): its first branch, a float64 product of the
    decoded operands."""

    def __init__(self, lin, act_fp8=None):
        self.b = lin.b
        if isinstance(lin, OM._LinearFP8):
            self.scale, self.act_fp8 = int(lin.scale[0]), lin.act_fp8 if act_fp8 is None else act_fp8
            # the oracle's decode of all 256 codes (to float64, or to fp16 as O.fp8_matmul does for fp16 activations),
            # then one gather
            table = O.f8_decode(np.arange(256, dtype=np.uint8), "F143", self.scale, np.float64 if self.act_fp8 else f16)
            self.w = (table if self.act_fp8 else table.astype(f32))[lin.w8]
        else:
            assert lin.w.dtype == f16
            self.scale, self.act_fp8 = None, False
            self.w = lin.w.astype(f32)

    def __call__(self, x):
        assert x.dtype == f16
        if self.act_fp8:
            a = O.f8_decode(O.f8_encode(x, "F143", self.scale), "F143", self.scale, np.float64)
            with np.errstate(over="ignore"):
                y = np.matmul(a, self.w).astype(f32).astype(f16)
        else:
            y = np.matmul(x.astype(f32), self.w).astype(f16)
        return (y + self.b).astype(f16) if self.b is not None else y


def _check_dense(lin, rows, seed):
    x = np.random.default_rng(seed).standard_normal((rows, lin.w8.shape[0] if isinstance(lin, OM._LinearFP8) else lin.w.shape[0])).astype(f16)
    assert np.array_equal(_Dense(lin)(x), lin(x)), "the prepared Linear differs from the oracle's"


def _follow(dec, oracle, ids, L, steps, pad, eos, tol, gap=3e-3, start=0, within_tol=False):
    """`steps` loop iterations on both sides, the oracle's written out with its own pieces (run_decode_loop,
    oracle/models.py) so that the loop may begin at iteration `start` over caches the caller has filled.  Every
    iteration: logits within `tol` (max relative error), ids equal wherever the oracle's two best logits are more than
    `gap` of the largest logit apart; at a nearer tie the decoder's token must be one of the two candidates and its
    container entry is set to the oracle's.  within_tol (FP8 activations, where the logits themselves are only held to
    `tol`): the candidates are instead all tokens the oracle scores within 2 * tol of its best.  Returns the number of
    such ties."""
    B = ids.shape[0]
    state = O.initial_loop_state(ids, L)
    state["step"] = start
    state["mask"][:, :start + 1] = 0
    dec.reset(ids)
    dec.step.fill_(start)
    if start:
        dec.mask[:, :start + 1] = 0
    worst, ties = 0.0, 0
    for it in range(steps):
        step = state["step"]
        ref_ids, ref_logits = oracle.step(state["container"][:, min(step, L - 1)].reshape(B, 1), step, state["mask"])
        O.step_loop_cond(state, O.step_containers(state, ref_ids, pad), eos, False, B)
        dec.step_fn()
        torch.cuda.synchronize()
        got = dec.logits.cpu().numpy().astype(np.float64)
        ref = ref_logits.astype(np.float64)
        worst = max(worst, np.abs(got - ref).max() / np.abs(ref).max())
        got_ids = dec.next_ids.cpu().numpy()
        top2 = np.sort(ref, axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > (2 * tol if within_tol else gap) * np.abs(ref).max()
        assert np.array_equal(got_ids[clear], ref_ids[clear]), f"token ids differ at step {step} without a near tie"
        for b in np.nonzero(got_ids != ref_ids)[0]:
            ties += 1
            if within_tol:
                assert ref[b, got_ids[b]] >= ref[b].max() - 2 * tol * np.abs(ref).max(), f"step {step}: the decoder's token is no near-best candidate"
            else:
                assert got_ids[b] in np.argsort(ref[b])[-2:], f"step {step}: the decoder's token is not one of the two tied candidates"
            if step + 1 < L and ids[b, step + 1] == pad:
                dec.container[b, step + 1] = int(ref_ids[b])
    assert worst <= tol, f"logits max rel err {worst}"
    assert np.array_equal(dec.container.cpu().numpy(), state["container"])
    assert int(dec.step.item()) == state["step"]
    return ties


def _prompt(rng, B, L, n, vocab, pad):
    ids = np.full((B, L), pad, np.int32)
    ids[:, :n] = rng.integers(3, vocab, size=(B, n))
    return ids


# ---------------------------------------------------------------------------------------------- ChatGLM2, 6B width
GLM2_6B_WIDTH = dict(padded_vocab_size=65024, hidden_size=4096, layernorm_epsilon=1e-5, multi_query_group_num=2,
                     num_attention_heads=32, ffn_hidden_size=13696, num_layers=2, kv_channels=128)


class _GLM2Valid(OM.ChatGLM2Oracle):
    """ChatGLM2Oracle with the attention chain applied to the valid cache rows only (a masked row's probability is
    exp(-10000 + s) = 0 exactly in fp16, and zeros change neither the sum nor the weighted sum) and with a KV head's
    rows shared by its query heads through broadcasting instead of a copy per query head."""

    def _attention_from_projections(self, lay, q, mixed, step, mask4):
        B, H, G, D = self.B, self.H, self.G, self.D
        k, v = mixed[..., : G * D], mixed[..., G * D:]
        q, k, v = q.reshape(B, 1, H, D), k.reshape(B, 1, G, D), v.reshape(B, 1, G, D)
        cos, sin = O.glm2_sincos(step, D)
        q, k = O.glm2_rope(q, cos, sin), O.glm2_rope(k, cos, sin)
        kv = np.concatenate([k, v], axis=0).reshape(2, B, 1, G, D).transpose(0, 1, 3, 2, 4)
        past = lay["cache"](step, kv)                                 # [2, B, G, L, D], newest row first
        n = min(int(step) + 1, self.L)
        qg = q.transpose(0, 2, 1, 3).reshape(B, G, H // G, 1, D)
        a = O.attention_scores_to_context(qg, past[0][:, :, None, :n].transpose(0, 1, 2, 4, 3), past[1][:, :, None, :n],
                                          mask4[:, :, None, :, :n], 1 / np.sqrt(D), f16, False)
        return lay["dense"](a.reshape(B, H, 1, D).transpose(0, 2, 1, 3).reshape(B, 1, H * D))


def test_the_prepared_chatglm2_oracle_is_the_oracle():
    """_GLM2Valid and _Dense against ChatGLM2Oracle itself on a small model, over a ring that fills up."""
    cfg = dict(padded_vocab_size=384, hidden_size=256, layernorm_epsilon=1e-5, multi_query_group_num=2,
               num_attention_heads=4, ffn_hidden_size=352, num_layers=2, kv_channels=64)
    B, L, steps, pad, eos = 2, 24, 20, 0, 2
    sd = OM.make_chatglm2_state_dict(cfg, seed=5)
    ids = _prompt(np.random.default_rng(1), B, L, 9, 384, pad)
    for precision in ("fp16", "fp8_weight", "fp8"):
        a, b = OM.ChatGLM2Oracle(sd, cfg, L, B, precision), _GLM2Valid(sd, cfg, L, B, precision)
        for lay in b.layers:
            for key in ("query", "key_value", "dense", "gate", "up", "down"):
                _check_dense(lay[key], 3, 7)
                lay[key] = _Dense(lay[key])
        b.head = _Dense(b.head)
        ta, tb = [], []
        ca, _ = OM.run_decode_loop(a, ids, L, steps, pad, eos, trace=ta)
        cb, _ = OM.run_decode_loop(b, ids, L, steps, pad, eos, trace=tb)
        assert np.array_equal(ca, cb)
        for (ia, la), (ib, lb) in zip(ta, tb):
            # the order of the sums over cache rows differs (valid rows only): fp16 results may differ in the last bit
            assert np.abs(la.astype(f32) - lb.astype(f32)).max() <= 2e-3 * np.abs(la.astype(f32)).max()


def _blockwise(fn, block=1 << 18, threads=8):
    """An elementwise oracle function applied block by block (cache-sized pieces, a few threads): the same values,
    several times faster on matrices of hundreds of millions of elements."""
    from concurrent.futures import ThreadPoolExecutor

    def run(x, *args):
        x = np.ascontiguousarray(x)
        flat = x.reshape(-1)
        if flat.size <= block:
            return fn(x, *args)
        pieces = [flat[i:i + block] for i in range(0, flat.size, block)]
        with ThreadPoolExecutor(threads) as ex:
            out = list(ex.map(lambda piece: fn(piece, *args), pieces))
        return np.concatenate(out).reshape(x.shape)
    return run


@pytest.fixture(scope="module")
def glm2_wide():
    """The state dict, and the oracle's Linears under the two FP8 precisions (the same F143 bytes: they are encoded
    once, by the oracle's own f8_encode applied block by block)."""
    sd = OM.make_chatglm2_state_dict(GLM2_6B_WIDTH, seed=41)
    x = np.random.default_rng(0).standard_normal((3, 1 << 19)).astype(f32)
    assert np.array_equal(_blockwise(O.f8_encode)(x, "F143", -1), O.f8_encode(x, "F143", -1))
    plain = O.f8_encode
    O.f8_encode = _blockwise(plain)
    try:
        f8 = OM.ChatGLM2Oracle(sd, GLM2_6B_WIDTH, 8, 1, "fp8_weight")
    finally:
        O.f8_encode = plain
    return sd, f8


def _glm2_oracle(wide, L, B, precision):
    sd, f8 = wide
    if precision == "fp16":
        o = _GLM2Valid(sd, GLM2_6B_WIDTH, L, B, precision)
    else:
        o = copy.copy(f8)
        o.__class__ = _GLM2Valid
        o.L, o.B = L, B
        o.layers = [dict(lay, cache=O.KVCache(L, 3, 1)) for lay in f8.layers]
    act = None if precision == "fp16" else precision == "fp8"
    for lay in o.layers:
        for key in ("query", "key_value", "dense", "gate", "up", "down"):
            lay[key] = _Dense(lay[key], act)
    o.head = _Dense(o.head, act)
    return o


@pytest.mark.timeout(900)
@pytest.mark.parametrize("precision,start,new,tol", [("fp16", 500, 24, 1e-2), ("fp8_weight", 0, 24, 1e-2), ("fp8", 500, 24, 1e-1)])
def test_chatglm2_at_the_6b_width_matches_oracle(glm2_wide, precision, start, new, tol):
    """The kernels the ChatGLM2 profile names, as a model: the FP8 / fp16 GEMVs over 13696 and 65024 channels at 8
    rows, the split decode attention with 16 query heads per KV head in a ring of 4096.  Two of the cases begin at
    iteration 500 over caches holding 500 random rows per layer (the same rows on both sides), so that the context
    grows across 512 - where the attention's splits take over rows from each other - within 24 iterations.  With FP8
    activations a one-ulp fp16 difference can flip a 3-bit rounding, so whole-model logits are held to 1e-1 there
    (test_chatglm2_fp8_stages_on_the_decoders_inputs holds every stage of every block to 1e-2 on identical inputs)."""
    from poptransformer_amd.engine import fused, loader
    B, L, pad, eos = 8, 4096, 0, 2
    G, D = GLM2_6B_WIDTH["multi_query_group_num"], GLM2_6B_WIDTH["kv_channels"]
    print(f"case: ChatGLM2 at the 6B width, {precision}, batch {B}, iterations {start}..{start + new - 1}", flush=True)
    sd = glm2_wide[0]
    oracle = _glm2_oracle(glm2_wide, L, B, precision)
    dec = fused.FusedDecoder(loader.chatglm2_spec(GLM2_6B_WIDTH, L, B, pad, eos), loader.chatglm2_weights(sd, GLM2_6B_WIDTH, precision))
    rng = np.random.default_rng(43)
    ids = _prompt(rng, B, L, start + 8, GLM2_6B_WIDTH["padded_vocab_size"], pad)
    for lay, ring in zip(oracle.layers, dec.rings):
        rows = (rng.standard_normal((2, B, G, start, D)) * 0.5).astype(f16)      # position p of the sequence in rows[..., p, :]
        lay["cache"].cache = np.zeros((2, B, G, L, D), f16)
        lay["cache"].cache[:, :, :, :start] = rows[:, :, :, ::-1]                # the oracle's register holds the newest row first
        ring.view(2, B, G, L, D)[:, :, :, :start] = torch.from_numpy(rows).cuda()   # the ring holds position p in row p
    ties = _follow(dec, oracle, ids, L, new, pad, eos, tol, start=start, within_tol=precision == "fp8")
    assert ties <= (new * B if precision == "fp8" else 40)


@pytest.mark.timeout(600)
def test_chatglm2_fp8_prompt_passes_at_the_6b_width(glm2_wide):
    """The prompt of the FP8 model in passes of 1024 and 8 rows at the 6B width: the projections of the 1024-row pass
    run on the FP8 matrix instruction's many-row kernel (row blocks of 128 for the gate / up pair, of 64 for the
    others), the loop's on the 8-row kernels that the tests above hold against the oracle.  The first block's KV rows
    come from identical inputs on both sides (embedding, norm, cast, query | key_value, rotary): equal to fp16
    rounding.  Behind them a flipped 3-bit rounding of an activation can build up (see the docstrings above): all
    blocks' rows are held to 1e-1, as at the small shape."""
    from poptransformer_amd.engine import fused, loader
    B, L, pad, eos, plen = 8, 256, 0, 2, 130
    sd = glm2_wide[0]
    print(f"case: ChatGLM2 fp8 at the 6B width, batch {B}, prompt of {plen} in passes against the loop", flush=True)
    make = lambda: fused.FusedDecoder(loader.chatglm2_spec(GLM2_6B_WIDTH, L, B, pad, eos), loader.chatglm2_weights(sd, GLM2_6B_WIDTH, "fp8"))
    ids = _prompt(np.random.default_rng(47), B, L, plen, GLM2_6B_WIDTH["padded_vocab_size"], pad)
    loop = make()
    loop.reset(ids)
    loop.run_steps(plen - 1)
    torch.cuda.synchronize()
    dec = make()
    dec.reset(ids)
    n = dec.consume_prompt()
    assert n == plen - 1 and int(dec.step.item()) == int(loop.step.item())
    assert torch.equal(dec.mask, loop.mask)
    for li, (a, b) in enumerate(zip(dec.rings, loop.rings)):
        a, b = a[:, :n].float(), b[:, :n].float()
        err = ((a - b).abs().max() / b.abs().max()).item()
        assert err <= (2e-3 if li == 0 else 1e-1), f"KV rows of block {li} differ from the loop's by {err}"


def _stages_on_the_decoders_inputs(dec, oracle, ids, L, steps, tol):
    """Every stage of every block of every iteration on identical inputs, the decoder's own: its residual stream
    entering a block goes through the oracle's norm and query / key_value Linears (compared with the decoder's); the
    decoder's projections go through the oracle's rotary embedding, cache, attention and output Linear (compared with
    the decoder's stream after the attention half); that stream goes through the oracle's MLP half (compared with the
    stream entering the next block).  Between two such points lie at most two casts of activations to FP8, so a wrong
    kernel shows up at its own stage while a flipped 3-bit rounding cannot build up: at block level it does - a
    difference of half a percent in the stream flips the rounding of one normalised feature in twenty, each by an
    eighth of its value, which is several percent on the next Linear's output.  Returns the worst error per stage."""
    B, d = ids.shape[0], oracle.d
    seen = []
    dec.probe = lambda name, li, t: seen.append((name, li, [u.clone() for u in t] if isinstance(t, (list, tuple)) else t.clone()))
    dec.reset(ids)
    mask = np.full((B, L), -10000, f16)
    mask[:, 0] = 0
    worst = {"projections": 0.0, "after_attention": 0.0, "block_out": 0.0}

    def held(name, got, ref, where):
        err = np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() / np.abs(ref.astype(np.float64)).max()
        worst[name] = max(worst[name], err)
        assert err <= tol, f"{where}, {name}: max rel err {err}"

    for step in range(steps):
        seen.clear()
        dec.step_fn()
        torch.cuda.synchronize()
        got = {(name, li): ([u.cpu().numpy() for u in t] if isinstance(t, list) else t.cpu().numpy()) for name, li, t in seen}
        mask4 = mask[:, None, None, :]
        for li, lay in enumerate(oracle.layers):
            where = f"iteration {step}, block {li}"
            x0 = got["block_in", li].reshape(B, 1, d)
            q, kv = (u.reshape(B, 1, -1) for u in got["projections", li])
            t = O.rms_norm(x0, lay["ln1"], oracle.eps)
            held("projections", np.concatenate([q, kv], axis=-1), np.concatenate([lay["query"](t), lay["key_value"](t)], axis=-1), where)
            x_mid = got["after_attention", li].reshape(B, 1, d)
            held("after_attention", x_mid, (x0 + oracle._attention_from_projections(lay, q, kv, step, mask4)).astype(f16), where)
            held("block_out", got["block_in", li + 1].reshape(B, 1, d), oracle.mlp_half(lay, x_mid), where)
        if step + 1 < L:
            mask[:, step + 1] = 0
    dec.probe = None
    return worst


@pytest.mark.timeout(900)
@pytest.mark.parametrize("width", ["small", "6b"])
def test_chatglm2_fp8_stages_on_the_decoders_inputs(glm2_wide, width):
    """precision 'fp8' (F143 weights and activations), where whole-model logits are only held to 1e-1: every stage of
    every block on the decoder's own inputs, to 1e-2 at the 6B width over 12 iterations and to 2e-2 at a small shape
    over 32 (one flipped rounding of a context feature is 1 % of the attention half's output among 256 features)."""
    from poptransformer_amd.engine import fused, loader
    pad, eos = 0, 2
    if width == "small":
        cfg = dict(padded_vocab_size=384, hidden_size=256, layernorm_epsilon=1e-5, multi_query_group_num=2,
                   num_attention_heads=4, ffn_hidden_size=352, num_layers=2, kv_channels=64)
        B, L, steps = 2, 48, 32
        sd = OM.make_chatglm2_state_dict(cfg, seed=4)
        oracle = OM.ChatGLM2Oracle(sd, cfg, L, B, "fp8")
    else:
        cfg, B, L, steps = GLM2_6B_WIDTH, 8, 4096, 12
        sd = glm2_wide[0]
        oracle = _glm2_oracle(glm2_wide, L, B, "fp8")
    print(f"case: ChatGLM2 fp8, stages on the decoder's inputs, {width} shape", flush=True)
    dec = fused.FusedDecoder(loader.chatglm2_spec(cfg, L, B, pad, eos), loader.chatglm2_weights(sd, cfg, "fp8"))
    ids = _prompt(np.random.default_rng(12), B, L, steps + 2, cfg["padded_vocab_size"], pad)
    worst = _stages_on_the_decoders_inputs(dec, oracle, ids, L, steps, 2e-2 if width == "small" else 1e-2)
    print("worst errors per stage:", {k: f"{v:.2e}" for k, v in worst.items()}, flush=True)


# ---------------------------------------------------------------------------------------------- RWKV-4, 7B width
RWKV_7B_WIDTH = dict(hidden_size=4096, intermediate_size=16384, attention_hidden_size=4096, layer_norm_epsilon=1e-5,
                     vocab_size=65536, num_hidden_layers=2, rescale_every=6)


@pytest.fixture(scope="module")
def rwkv_wide():
    """(state dict, oracle of batch 1 with its Linears prepared and its states untouched: the tests take copies
    with states of their own batch size)."""
    sd = OM.make_rwkv_state_dict(RWKV_7B_WIDTH, seed=51, int4=True)
    oracle = OM.RWKVOracle(sd, RWKV_7B_WIDTH, 40, 1)
    _check_dense(oracle.layers[0]["att_key"], 2, 3)
    for lay in oracle.layers:
        for key in [k for k, v in lay.items() if isinstance(v, OM._Linear)]:
            lay[key] = _Dense(lay[key])
    oracle.head = _Dense(oracle.head)
    return sd, oracle


@pytest.mark.timeout(900)
@pytest.mark.parametrize("B", [1, 32])
def test_rwkv_at_the_7b_width_matches_oracle(rwkv_wide, B):
    """INT4 projections of 4096 x 4096, 4096 x 16384, 16384 x 4096 and the 65536-channel head at 1 and 32 rows, the
    mixes and the WKV recurrence over 4096 channels: 8 prompt positions and 24 generated tokens."""
    from poptransformer_amd.engine import loader, rwkv
    L, pad, eos, plen = 40, 0, 65535, 8
    steps = plen - 1 + 24
    print(f"case: RWKV-4 at the 7B width, batch {B}, {steps} iterations", flush=True)
    sd, template = rwkv_wide
    oracle = copy.copy(template)
    oracle.B = B
    # the initial states of a batch of one, repeated per sequence
    oracle.layers = [dict(lay, state=[np.repeat(s0, B, axis=0) for s0 in lay["state"]]) for lay in template.layers]
    dec = rwkv.RWKVDecoder(loader.rwkv_spec(RWKV_7B_WIDTH, L, B, pad, eos), loader.rwkv_weights(sd, RWKV_7B_WIDTH))
    ids = _prompt(np.random.default_rng(53 + B), B, L, plen, 65000, pad)
    ties = _follow(dec, oracle, ids, L, steps, pad, eos, 1e-2)
    assert ties <= 2 * B + 8


# ---------------------------------------------------------------------------------------------- GPT-2 small, full size
GPT2_SMALL = dict(vocab_size=50257, n_embd=768, layer_norm_epsilon=1e-5, n_head=12, n_layer=12, n_positions=1024)


@pytest.mark.timeout(600)
def test_gpt2_small_at_its_own_shape_matches_oracle():
    """The plumbing configuration itself: 12 layers, 768 features, 12 heads of 64, vocabulary 50257 (the tied head's
    last channel block is ragged), batch 1, prompt 16, 32 new tokens, KV length 128."""
    from poptransformer_amd.engine import fused, loader
    B, L, pad, eos, plen, new = 1, 128, 50256, 50255, 16, 32
    steps = plen - 1 + new
    print("case: GPT-2 small, 12 layers, 47 iterations", flush=True)
    sd = OM.make_gpt2_state_dict(GPT2_SMALL, seed=61)
    oracle = OM.GPT2Oracle(sd, GPT2_SMALL, L, B)
    dec = fused.FusedDecoder(loader.gpt2_spec(GPT2_SMALL, L, B, pad, eos), loader.gpt2_weights(sd, GPT2_SMALL))
    ids = _prompt(np.random.default_rng(62), B, L, plen, 50000, pad)
    ties = _follow(dec, oracle, ids, L, steps, pad, eos, 1e-2)
    assert ties <= 8
    # the weights bench.py draws for this configuration are the same kind of checkpoint
    from poptransformer_amd.engine import synthetic
    mine = synthetic.gpt2_synthetic_state_dict(dict(GPT2_SMALL, n_layer=1), seed=0)
    ref = OM.make_gpt2_state_dict(dict(GPT2_SMALL, n_layer=1), seed=0)
    assert mine.keys() == ref.keys() and all(mine[k].shape == ref[k].shape and mine[k].dtype == ref[k].dtype for k in ref)
