"""The persistent decode step (one launch per loop iteration) against the numpy oracle and against
the per-operator path of the same engine."""
import numpy as np
import pytest
import torch

from oracle import models as OM
from tests.test_gpu_models import LLAMA_TINY, _prompt, _compare

pytestmark = pytest.mark.gpu


def _decoders(B, L, pad, eos, seed, early_stop=False, fp8_cache=False):
    from poptransformer_amd.engine import fused, loader
    sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=seed, int4=True)
    spec = loader.llama2_spec(LLAMA_TINY, L, B, pad, eos, fp8_cache=fp8_cache)
    spec.early_stop = early_stop
    w = loader.llama2_weights(sd, LLAMA_TINY)
    return sd, fused.FusedDecoder(spec, w), fused.FusedDecoder(spec, w).enable_persistent()


@pytest.mark.parametrize("B", [1, 3, 5, 8, 16])
def test_persistent_step_matches_oracle(B):
    """Greedy ids identical over the first 32 steps, fp16 logits within 1e-2 (max relative error)."""
    L, steps, pad, eos = 48, 32, 0, 2
    print("case: persistent step vs oracle, batch", B, flush=True)
    sd, _, dec = _decoders(B, L, pad, eos, seed=1)
    oracle = OM.Llama2Oracle(sd, LLAMA_TINY, L, B)
    ids = _prompt(np.random.default_rng(7), B, L, 8, LLAMA_TINY["vocab_size"], pad)
    _compare(dec, oracle, ids, L, steps, pad, eos)
    assert not dec.persistent.failed()


@pytest.mark.parametrize("B", [1, 3, 6, 16])
def test_persistent_step_with_fp8_kv_cache(B):
    """KV rings of F143 bytes (pta_llama_decode_step_f8).  Up to 4 sequences against the oracle (KVCache with
    fp8 = true): greedy ids identical over the first 32 steps, logits within 3e-2 (measured up to 1.8e-2: this kernel's
    INT4 projections agree with the oracle's to the last fp16 bit or differ in it, and where such a k or v element
    lies at an FP8 rounding boundary its byte - three mantissa bits - comes out one step away; the per-operator path,
    whose projections round as the oracle's do, is held to 1e-2 in test_llama2_fp8_kv_cache_matches_oracle).  Every
    batch size step by step against the per-operator path of the same cache format, fed the same tokens: logits
    within 3e-2 of their largest magnitude, ids equal wherever the reference's best two candidates are further
    apart than that; after 40 steps at least 99 % of the first layer's ring bytes are equal (measured 99.5 %) and at
    least 85 % of every later layer's (their inputs already differ by what those bytes changed: measured 92-94 %),
    and nothing is written past the steps taken."""
    L, steps, pad, eos = 48, 32, 0, 2
    print("case: persistent step with FP8 KV cache, batch", B, flush=True)
    sd, ref, dec = _decoders(B, L, pad, eos, seed=1, fp8_cache=True)
    ids = _prompt(np.random.default_rng(7), B, L, 12, LLAMA_TINY["vocab_size"], pad)
    if B <= 4:
        _compare(dec, OM.Llama2Oracle(sd, LLAMA_TINY, L, B, fp8_cache=True), ids, L, steps, pad, eos, tol=3e-2)
    ref.reset(ids)
    dec.reset(ids)
    for it in range(40):
        ref.step_fn()
        dec.step_fn()
        torch.cuda.synchronize()
        a = ref.logits.float().cpu().numpy()
        b = dec.logits.float().cpu().numpy()
        scale, tol = np.abs(a).max(), 3e-2
        assert np.abs(a - b).max() <= tol * scale, f"logits differ at step {it}"
        top2 = np.sort(a, axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 2 * tol * scale
        assert np.array_equal(ref.next_ids.cpu().numpy()[clear], dec.next_ids.cpu().numpy()[clear]), f"ids differ at step {it}"
        dec.container.copy_(ref.container)          # after a near tie: follow the reference's choice
    assert not dec.persistent.failed()
    for li, (ra, rb) in enumerate(zip(ref.rings, dec.rings)):
        a, b = ra[:, :40].cpu().numpy(), rb[:, :40].cpu().numpy()
        assert a.dtype == np.uint8 and (a == b).mean() >= (0.99 if li == 0 else 0.85), f"layer {li}"
        assert torch.equal(ra[:, 41:], rb[:, 41:])          # nothing written past the steps taken


@pytest.mark.parametrize("B", [6, 16])
def test_persistent_step_with_fp8_kv_cache_over_a_long_context(B):
    """The FP8 rings up to a context of 200 rows, step by step against the per-operator path of the same cache
    format, fed the same tokens (tolerances as in test_persistent_step_with_fp8_kv_cache): at 16 sequences the
    attention visits its cache rows in rounds of 32 with a window of four rounds requested ahead, so from 128 rows
    on every visit uses registers that an earlier round has been through."""
    L, pad, eos = 200, 0, 2
    print("case: persistent step with FP8 KV cache over a long context, batch", B, flush=True)
    _, ref, dec = _decoders(B, L, pad, eos, seed=3, fp8_cache=True)
    ids = _prompt(np.random.default_rng(13), B, L, 6, LLAMA_TINY["vocab_size"], pad)
    ref.reset(ids)
    dec.reset(ids)
    for it in range(L - 2):
        ref.step_fn()
        dec.step_fn()
        torch.cuda.synchronize()
        a = ref.logits.float().cpu().numpy()
        b = dec.logits.float().cpu().numpy()
        scale, tol = np.abs(a).max(), 3e-2
        assert np.abs(a - b).max() <= tol * scale, f"logits differ at step {it}"
        top2 = np.sort(a, axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 2 * tol * scale
        assert np.array_equal(ref.next_ids.cpu().numpy()[clear], dec.next_ids.cpu().numpy()[clear]), f"ids differ at step {it}"
        dec.container.copy_(ref.container)          # after a near tie: follow the reference's choice
    assert not dec.persistent.failed()
    a, b = ref.rings[0].cpu().numpy(), dec.rings[0].cpu().numpy()
    assert (a == b).mean() >= 0.99


@pytest.mark.parametrize("B", [1, 4, 7, 16])
def test_persistent_step_follows_the_per_operator_path(B):
    """Step by step over a long generation: logits agree to 2e-3 of their largest magnitude (the two
    paths merge attention partial sums in different orders) and the selected ids are equal wherever
    the per-operator logits separate the best two candidates by more than that; the comparison ends
    at the first step where a near tie sends the two generations apart (with more than 4 sequences, where
    near ties are frequent, the persistent decoder is then given the reference's token and goes on)."""
    L, pad, eos = 200, 0, 2
    print("case: persistent step vs per-operator path, batch", B, flush=True)
    _, ref, dec = _decoders(B, L, pad, eos, seed=5)
    ids = _prompt(np.random.default_rng(11), B, L, 5, LLAMA_TINY["vocab_size"], pad)
    ref.reset(ids)
    dec.reset(ids)
    compared = 0
    for it in range(L - 1):
        ref.step_fn()
        dec.step_fn()
        torch.cuda.synchronize()
        a = ref.logits.float().cpu().numpy()
        b = dec.logits.float().cpu().numpy()
        scale = np.abs(a).max()
        # beyond 4 sequences the per-operator path runs other kernels (exact INT4 decode, other summation orders)
        tol = 2e-3 if B <= 4 else 4e-3
        assert np.abs(a - b).max() <= tol * scale, f"logits differ at step {it}"
        top2 = np.sort(a, axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 2 * tol * scale
        ia, ib = ref.next_ids.cpu().numpy(), dec.next_ids.cpu().numpy()
        assert np.array_equal(ia[clear], ib[clear]), f"ids differ at step {it} without a near tie"
        compared += 1
        if not np.array_equal(ref.container.cpu().numpy(), dec.container.cpu().numpy()):
            if B <= 4:
                break
            dec.container.copy_(ref.container)      # a near tie (asserted above): follow the reference's choice
    assert compared >= 32
    assert not dec.persistent.failed()


def test_prompt_in_passes_then_persistent_steps():
    """The prompt taken in passes (one launch per operator, several positions at once), then the loop as
    persistent launches replayed from a graph: container and step equal the oracle's loop."""
    B, L, steps, pad, eos = 2, 64, 48, 0, 2
    print("case: prompt passes, then persistent steps", flush=True)
    sd, _, dec = _decoders(B, L, pad, eos, seed=1)
    ids = _prompt(np.random.default_rng(13), B, L, 21, LLAMA_TINY["vocab_size"], pad)
    ids[ids == eos] = eos + 1                # no end token inside the prompt: the passes take all of it
    ref_container, ref_step = OM.run_decode_loop(OM.Llama2Oracle(sd, LLAMA_TINY, L, B), ids, L, steps, pad, eos)
    dec.capture()
    for _ in range(2):                       # the second generation replays the passes' graph as well
        dec.reset(ids)
        n = dec.consume_prompt(rows_per_pass=8)
        assert n == 20
        dec.run_steps(steps - n)
        torch.cuda.synchronize()
        assert not dec.persistent.failed()
        assert np.array_equal(dec.container.cpu().numpy(), ref_container) and int(dec.step.item()) == ref_step


def test_persistent_step_graph_replay_equals_eager():
    B, L, pad, eos = 2, 64, 0, 2
    print("case: persistent step, graph replay vs eager", flush=True)
    _, _, eager = _decoders(B, L, pad, eos, seed=3)
    ids = _prompt(np.random.default_rng(9), B, L, 5, LLAMA_TINY["vocab_size"], pad)
    c_eager, s_eager = eager.run(ids, L)
    _, _, graphed = _decoders(B, L, pad, eos, seed=3)
    graphed.capture()
    for _ in range(2):                      # the second run checks that replays start from a clean state
        c_graph, s_graph = graphed.run(ids, L)
        assert np.array_equal(c_graph, c_eager) and s_graph == s_eager


def test_persistent_step_stops_with_the_loop_condition():
    """Early stop: once every sequence has produced eos the loop condition is false and further
    launches change nothing (models/base_model.py:313-355)."""
    B, L, pad = 1, 48, 0
    print("case: persistent step, early stop", flush=True)
    sd, ref, _ = _decoders(B, L, pad, eos=-1, seed=4)
    ids = _prompt(np.random.default_rng(5), B, L, 4, LLAMA_TINY["vocab_size"], pad)
    c, _ = ref.run(ids, 12)
    eos = int(c[0, 8])                       # a token the model will produce
    _, ref2, dec = _decoders(B, L, pad, eos, seed=4, early_stop=True)
    c_ref, s_ref = ref2.run(ids, L)
    c_dec, s_dec = dec.run(ids, L)
    assert s_ref < L and s_dec == s_ref and np.array_equal(c_dec, c_ref)
    before = dec.container.clone()
    dec.step_fn()
    torch.cuda.synchronize()
    assert torch.equal(before, dec.container) and int(dec.step.item()) == s_dec


def test_persistent_step_reports_failure_and_leaves_the_state():
    """The error word of the workspace is sticky: with it set (here from the host, standing in for
    a workgroup that gave up waiting) a launch must not touch the loop state and run() must raise."""
    B, L, pad, eos = 1, 32, 0, 2
    print("case: persistent step, sticky failure word", flush=True)
    _, _, dec = _decoders(B, L, pad, eos, seed=2)
    ids = _prompt(np.random.default_rng(3), B, L, 4, LLAMA_TINY["vocab_size"], pad)
    dec.reset(ids)
    dec.step_fn()
    torch.cuda.synchronize()
    assert int(dec.step.item()) == 1 and not dec.persistent.failed()
    dec.persistent.workspace.view(torch.int32)[1] = 1
    dec.step_fn()
    torch.cuda.synchronize()
    assert int(dec.step.item()) == 1 and dec.persistent.failed()
    with pytest.raises(RuntimeError):
        dec.run(ids, 4)


def test_persistent_step_rejects_unsupported_models():
    from poptransformer_amd.engine import fused, loader
    from tests.test_gpu_models import GPT2_TINY
    sd = OM.make_gpt2_state_dict(GPT2_TINY, seed=2)
    dec = fused.FusedDecoder(loader.gpt2_spec(GPT2_TINY, 40, 1, 999, 998), loader.gpt2_weights(sd, GPT2_TINY))
    with pytest.raises(NotImplementedError):
        dec.enable_persistent()
    sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=1, int4=True)
    spec = loader.llama2_spec(LLAMA_TINY, 48, 17, 0, 2)          # batch 17 > 16
    with pytest.raises(NotImplementedError):
        fused.FusedDecoder(spec, loader.llama2_weights(sd, LLAMA_TINY)).enable_persistent()
