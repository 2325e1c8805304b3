"""Whole-model parity of the fused decode loop against the numpy oracle: greedy token ids over
the first 32 steps identical, fp16 logits within 1e-2 (max relative error)."""
import numpy as np
import pytest
import torch

from oracle import models as OM

pytestmark = pytest.mark.gpu

LLAMA_TINY = dict(vocab_size=512, hidden_size=256, rms_norm_eps=1e-5, num_attention_heads=2,
                  intermediate_size=688, num_hidden_layers=2)
GPT2_TINY = dict(vocab_size=1000, n_embd=128, layer_norm_epsilon=1e-5, n_head=2, n_layer=2, n_positions=64)


def _prompt(rng, B, L, plen, vocab, pad):
    ids = np.full((B, L), pad, np.int32)
    ids[:, :plen] = rng.integers(1, vocab, size=(B, plen))
    ids[ids == pad] = pad + 1 if pad + 1 < vocab else 1
    ids[:, plen:] = pad
    return ids


def _compare(dec, oracle, ids, L, steps, pad, eos, tol=1e-2):
    trace = []
    ref_container, ref_step = OM.run_decode_loop(oracle, ids, L, steps, pad, eos, trace=trace)
    dec.reset(ids)
    worst = 0.0
    for it in range(steps):
        dec.step_fn()
        torch.cuda.synchronize()
        got = dec.logits.cpu().numpy().astype(np.float64)
        ref = trace[it][1].astype(np.float64)
        worst = max(worst, np.abs(got - ref).max() / np.abs(ref).max())
        assert np.array_equal(dec.next_ids.cpu().numpy(), trace[it][0]), f"token ids differ at step {it}"
    assert worst <= tol, f"logits max rel err {worst}"
    assert np.array_equal(dec.container.cpu().numpy(), ref_container)
    assert int(dec.step.item()) == ref_step
    return worst


@pytest.mark.parametrize("B", [1, 3])
def test_llama2_int4_decode_matches_oracle(B):
    from poptransformer_amd.engine import fused, loader
    L, steps, pad, eos = 48, 32, 0, 2
    sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=1, int4=True)
    oracle = OM.Llama2Oracle(sd, LLAMA_TINY, L, B)
    dec = fused.FusedDecoder(loader.llama2_spec(LLAMA_TINY, L, B, pad, eos), loader.llama2_weights(sd, LLAMA_TINY))
    ids = _prompt(np.random.default_rng(7), B, L, 8, LLAMA_TINY["vocab_size"], pad)
    _compare(dec, oracle, ids, L, steps, pad, eos)


@pytest.mark.parametrize("B", [1, 2])
def test_gpt2_fp16_decode_matches_oracle(B):
    from poptransformer_amd.engine import fused, loader
    L, steps, pad, eos = 40, 32, 999, 998
    sd = OM.make_gpt2_state_dict(GPT2_TINY, seed=2)
    oracle = OM.GPT2Oracle(sd, GPT2_TINY, L, B)
    dec = fused.FusedDecoder(loader.gpt2_spec(GPT2_TINY, L, B, pad, eos), loader.gpt2_weights(sd, GPT2_TINY))
    ids = _prompt(np.random.default_rng(8), B, L, 6, 900, pad)
    _compare(dec, oracle, ids, L, steps, pad, eos)


GLM2_TINY = dict(padded_vocab_size=384, hidden_size=256, layernorm_epsilon=1e-5, multi_query_group_num=2,
                 num_attention_heads=4, ffn_hidden_size=352, num_layers=2, kv_channels=64)


@pytest.mark.parametrize("precision", ["fp16", "fp8_weight", "fp8"])
def test_chatglm2_decode_matches_oracle(precision):
    from poptransformer_amd.engine import fused, loader
    B, L, steps, pad, eos = 2, 48, 32, 0, 2
    sd = OM.make_chatglm2_state_dict(GLM2_TINY, seed=4)
    # exponents near the format maximum for half of the Linears, the reference's -1 for the rest
    scales = {k[:-7]: OM.fp8_weight_scale(v) for k, v in sd.items() if k.endswith("dense.weight") or "h_to_4h_1" in k}
    oracle = OM.ChatGLM2Oracle(sd, GLM2_TINY, L, B, precision, scales)
    dec = fused.FusedDecoder(loader.chatglm2_spec(GLM2_TINY, L, B, pad, eos),
                             loader.chatglm2_weights(sd, GLM2_TINY, precision, scales))
    ids = _prompt(np.random.default_rng(10), B, L, 7, GLM2_TINY["padded_vocab_size"], pad)
    # With FP8 activations (3 mantissa bits) a one-ulp fp16 difference in an activation - which two
    # correct fp32-accumulating MatMuls already produce - can flip its FP8 rounding, a 6 % step in that
    # element: whole-model logits agree to a few percent, not to 1e-2.  The operator itself is held to
    # 1e-2 on identical inputs in test_gpu_kernels.py::test_fp8_gemm_both_modes; tokens must still match.
    _compare(dec, oracle, ids, L, steps, pad, eos, tol=1e-1 if precision == "fp8" else 1e-2)


RWKV_TINY = dict(hidden_size=256, intermediate_size=512, attention_hidden_size=256, layer_norm_epsilon=1e-5,
                 vocab_size=500, num_hidden_layers=4, rescale_every=2)


@pytest.mark.parametrize("B,int4", [(1, True), (3, True), (2, False), (20, True)])
def test_rwkv_decode_matches_oracle(B, int4):
    from poptransformer_amd.engine import loader, rwkv
    L, steps, pad, eos = 48, 32, 0, 499
    sd = OM.make_rwkv_state_dict(RWKV_TINY, seed=6, int4=int4)
    oracle = OM.RWKVOracle(sd, RWKV_TINY, L, B)
    dec = rwkv.RWKVDecoder(loader.rwkv_spec(RWKV_TINY, L, B, pad, eos), loader.rwkv_weights(sd, RWKV_TINY))
    ids = _prompt(np.random.default_rng(11), B, L, 9, 490, pad)
    _compare(dec, oracle, ids, L, steps, pad, eos)
    # a second generation starts from fresh states
    dec.capture()
    c, st = dec.run(ids, steps)
    ref_c, ref_s = OM.run_decode_loop(OM.RWKVOracle(sd, RWKV_TINY, L, B), ids, L, steps, pad, eos)
    assert np.array_equal(c, ref_c) and st == ref_s


def test_llama2_graph_replay_equals_eager():
    from poptransformer_amd.engine import fused, loader
    B, L, pad, eos = 2, 40, 0, 2
    sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=3, int4=True)
    ids = _prompt(np.random.default_rng(9), B, L, 5, LLAMA_TINY["vocab_size"], pad)
    spec = loader.llama2_spec(LLAMA_TINY, L, B, pad, eos)
    w = loader.llama2_weights(sd, LLAMA_TINY)
    eager = fused.FusedDecoder(spec, w)
    c_eager, s_eager = eager.run(ids, L)
    graphed = fused.FusedDecoder(spec, w)
    graphed.capture()
    for _ in range(2):                      # the second run checks that replays start from a clean state
        c_graph, s_graph = graphed.run(ids, L)
        assert np.array_equal(c_graph, c_eager) and s_graph == s_eager


def test_llama2_checkpoint_from_disk(tmp_path):
    """fp16 Hugging Face-style checkpoint on disk (sharded safetensors) -> quantised to the INT4 layout ->
    decoder: the tokens are those of the oracle on the same quantised weights."""
    from poptransformer_amd.engine import fused, loader
    from poptransformer_amd.utils import checkpoint
    B, L, steps, pad, eos = 2, 48, 32, 0, 2
    checkpoint.save_state_dict(OM.make_llama2_state_dict(LLAMA_TINY, seed=31, int4=False), str(tmp_path),
                               max_shard_bytes=256 * 1024)
    sd = checkpoint.quantize_state_dict_int4(checkpoint.load_state_dict(str(tmp_path)))
    assert sd["model.layers.0.mlp.down_proj.weight"].dtype == np.int8 and "lm_head.weight_scale" not in sd
    ids = _prompt(np.random.default_rng(17), B, L, 5, LLAMA_TINY["vocab_size"], pad)
    dec = fused.FusedDecoder(loader.llama2_spec(LLAMA_TINY, L, B, pad, eos), loader.llama2_weights(sd, LLAMA_TINY))
    _compare(dec, OM.Llama2Oracle(sd, LLAMA_TINY, L, B), ids, L, steps, pad, eos)


def test_llama2_top_k_sampling_draws_from_the_top_k():
    """topk > 1 (layers/lm_head.py:52-53): every generated token is one of the k best of that step's logits, all
    rows of the batch use the same draw, and over many steps every rank is drawn (the reference's generator and
    its stream are not reproduced: which rank is drawn at a step is not comparable)."""
    from poptransformer_amd.engine import fused, loader
    B, L, k, pad, eos = 2, 64, 4, 0, -1
    sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=1, int4=True)
    spec = loader.llama2_spec(LLAMA_TINY, L, B, pad, eos)
    spec.topk = k
    dec = fused.FusedDecoder(spec, loader.llama2_weights(sd, LLAMA_TINY))
    ids = _prompt(np.random.default_rng(3), B, L, 4, LLAMA_TINY["vocab_size"], pad)
    torch.manual_seed(0)
    dec.capture()
    dec.reset(ids)
    ranks = []
    for it in range(L - 2):
        dec.run_steps(1)
        torch.cuda.synchronize()
        logits = dec.logits.cpu().numpy().astype(np.float32)
        order = np.argsort(-logits, axis=1, kind="stable")[:, :k]
        nxt = dec.next_ids.cpu().numpy()
        r = [int(np.where(order[b] == nxt[b])[0][0]) for b in range(B)]     # raises if not among the top k
        assert len(set(r)) == 1
        ranks.append(r[0])
    assert set(ranks) == set(range(k))
    assert max(np.bincount(ranks)) < 0.6 * len(ranks)


LLAMA_WIDE = dict(vocab_size=640, hidden_size=1024, rms_norm_eps=1e-5, num_attention_heads=8,
                  intermediate_size=1408, num_hidden_layers=2)


@pytest.mark.parametrize("B", [6, 16])
def test_llama2_int4_decode_batch_up_to_16(B):
    """Hidden size 1024 and 5..16 sequences: the projections run on the kernel that shares activation fragments
    between channel blocks, with the norm as a kernel of its own and with the norm inside the GEMM."""
    from poptransformer_amd.engine import fused, loader
    L, steps, pad, eos = 40, 32, 0, 2
    sd = OM.make_llama2_state_dict(LLAMA_WIDE, seed=5, int4=True)
    ids = _prompt(np.random.default_rng(9), B, L, 6, LLAMA_WIDE["vocab_size"], pad)
    for fuse in (False, True):
        dec = fused.FusedDecoder(loader.llama2_spec(LLAMA_WIDE, L, B, pad, eos), loader.llama2_weights(sd, LLAMA_WIDE))
        dec.fuse_norm = fuse
        _compare(dec, OM.Llama2Oracle(sd, LLAMA_WIDE, L, B), ids, L, steps, pad, eos)


def test_llama2_int4_decode_more_than_16_sequences():
    """24 sequences on the per-operator path: the projections run on the kernels that stage the activation rows in
    LDS, and the engine brings the scratch that lets the attention output and the MLP down projection split K."""
    from poptransformer_amd.engine import fused, loader
    B, L, steps, pad, eos = 24, 40, 32, 0, 2
    sd = OM.make_llama2_state_dict(LLAMA_WIDE, seed=5, int4=True)
    ids = _prompt(np.random.default_rng(10), B, L, 6, LLAMA_WIDE["vocab_size"], pad)
    dec = fused.FusedDecoder(loader.llama2_spec(LLAMA_WIDE, L, B, pad, eos), loader.llama2_weights(sd, LLAMA_WIDE))
    assert dec._lin_ws is not None
    # 24 rows x 32 steps of a random model meet exact ties of the two best logits (one does at step 5): logits are
    # held to 1e-2 at every step, ids wherever the oracle's best two are further apart than the error allows, and the
    # decoder is given the oracle's token when a tie was broken the other way
    trace = []
    ref_container, ref_step = OM.run_decode_loop(OM.Llama2Oracle(sd, LLAMA_WIDE, L, B), ids, L, steps, pad, eos, trace=trace)
    dec.reset(ids)
    for it in range(steps):
        dec.step_fn()
        torch.cuda.synchronize()
        got, ref = dec.logits.cpu().numpy().astype(np.float64), trace[it][1].astype(np.float64)
        scale = np.abs(ref).max()
        assert np.abs(got - ref).max() <= 1e-2 * scale, f"logits differ at step {it}"
        top2 = np.sort(ref, axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 2e-2 * scale
        gi, ri = dec.next_ids.cpu().numpy(), trace[it][0]
        assert np.array_equal(gi[clear], ri[clear]), f"token ids differ at step {it} without a near tie"
        if not np.array_equal(gi, ri):
            pos = int(dec.step.item())
            col = dec.container[:, pos].cpu().numpy()
            col[gi != ri] = np.where(col[gi != ri] == gi[gi != ri], ri[gi != ri], col[gi != ri])
            dec.container[:, pos] = torch.from_numpy(col).to(dec.container.device)
    assert int(dec.step.item()) == ref_step


def _equal_up_to_a_near_tie(got, ref, trace, tol=2e-3):
    """Token ids per sequence equal the oracle's up to the first difference, which must sit where the oracle's two
    best logits lie within `tol` (four fp16 steps below 1.0; exact ties occur in these tiny random models) and be
    one of those two.  Returns whether any sequence parted there."""
    parted = False
    for b in range(ref.shape[0]):
        diff = np.nonzero(got[b] != ref[b])[0]
        if diff.size == 0:
            continue
        p_ = int(diff[0])                                  # chosen by loop iteration p_ - 1
        lg = trace[p_ - 1][1].reshape(ref.shape[0], -1)[b].astype(np.float32)
        best = np.argsort(lg)[-2:]
        assert lg[best[1]] - lg[best[0]] <= tol, f"sequence {b}, position {p_}: tokens differ without a near tie"
        assert got[b, p_] in best, f"sequence {b}, position {p_}: token {got[b, p_]} is not one of the two best"
        parted = True
    return parted


def _prompt_then_loop(dec, ids, steps, rows_per_pass=None):
    dec.reset(ids)
    n = dec.consume_prompt(rows_per_pass=rows_per_pass)
    dec.run_steps(steps - n)
    torch.cuda.synchronize()
    return n


@pytest.mark.parametrize("family,B,plen,rows_per_pass", [("llama2", 1, 41, None), ("llama2", 3, 30, 7), ("gpt2", 2, 25, None),
                                                          ("chatglm2", 2, 29, 16), ("chatglm2_fp8_weight", 2, 29, None),
                                                          ("chatglm2_fp8", 2, 29, None)])
def test_prompt_in_passes_equals_the_loop(family, B, plen, rows_per_pass):
    """The prompt taken several positions per pass (consume_prompt), then the loop: the container, the step and
    the tokens are those of the oracle's position-by-position loop (up to a tie of the oracle's own two best logits),
    and the KV rings hold what the loop leaves there to fp16 rounding.  Prompts of different lengths: the passes stop at the shortest."""
    from poptransformer_amd.engine import fused, loader
    L, steps, pad, eos = 64, 56, 0, 2
    if family == "llama2":
        sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=1, int4=True)
        oracle = OM.Llama2Oracle(sd, LLAMA_TINY, L, B)
        make = lambda: fused.FusedDecoder(loader.llama2_spec(LLAMA_TINY, L, B, pad, eos), loader.llama2_weights(sd, LLAMA_TINY))
        vocab = LLAMA_TINY["vocab_size"]
    elif family == "gpt2":
        pad, eos = 999, 998
        sd = OM.make_gpt2_state_dict(GPT2_TINY, seed=2)
        oracle = OM.GPT2Oracle(sd, GPT2_TINY, L, B)
        make = lambda: fused.FusedDecoder(loader.gpt2_spec(GPT2_TINY, L, B, pad, eos), loader.gpt2_weights(sd, GPT2_TINY))
        vocab = 900
    else:
        precision = family[9:] or "fp16"
        sd = OM.make_chatglm2_state_dict(GLM2_TINY, seed=4)
        scales = {k[:-7]: OM.fp8_weight_scale(v) for k, v in sd.items() if k.endswith("dense.weight") or "h_to_4h_1" in k}
        oracle = OM.ChatGLM2Oracle(sd, GLM2_TINY, L, B, precision, scales)
        make = lambda: fused.FusedDecoder(loader.chatglm2_spec(GLM2_TINY, L, B, pad, eos),
                                          loader.chatglm2_weights(sd, GLM2_TINY, precision, scales))
        vocab = GLM2_TINY["padded_vocab_size"]
    ids = _prompt(np.random.default_rng(21), B, L, plen, vocab, pad)
    if B > 1:
        ids[B - 1, plen - 4:] = pad                                  # one shorter prompt
    trace = []
    ref_container, ref_step = OM.run_decode_loop(oracle, ids, L, steps, pad, eos, trace=trace)
    loop = make()
    c_loop, s_loop = loop.run(ids, steps)
    dec = make()
    n = _prompt_then_loop(dec, ids, steps, rows_per_pass)
    assert n == (plen - 1 if B == 1 else plen - 5)
    assert int(dec.step.item()) == ref_step == s_loop
    assert torch.equal(dec.mask, loop.mask) and torch.equal(dec.stop_mask, loop.stop_mask)
    if family.endswith("fp8"):
        # FP8 activations (3 mantissa bits): a one-ulp fp16 difference between the many-row and the one-row
        # GEMM flips an FP8 rounding now and then, a 6 % step in that element, and these tiny random models
        # then pick other tokens later on.  Checked here: the prompt's part of the KV rings, to that step.
        for a, b in zip(dec.rings, loop.rings):
            a, b = a[:, :n].float(), b[:, :n].float()
            assert ((a - b).abs().max() / b.abs().max()).item() <= 1e-1
        return
    assert np.array_equal(c_loop, ref_container)
    # the passes round the context vectors in another order than the loop: where the oracle's two best logits tie
    # (ChatGLM2 here: exactly, at one late position), either token may come out; the rings are compared up to there
    first_c = dec.container.cpu().numpy()
    parted = _equal_up_to_a_near_tie(first_c, ref_container, trace)
    upto = n if parted else L
    for a, b in zip(dec.rings, loop.rings):
        a, b = a[:, :upto].float(), b[:, :upto].float()
        err = (a - b).abs().max().item() / b.abs().max().item()
        assert err <= 1e-2, f"KV ring differs from the loop's by {err}"
    # a second generation on the same decoder, graph-captured loop after the passes
    dec.capture()
    _prompt_then_loop(dec, ids, steps, rows_per_pass)
    assert np.array_equal(dec.container.cpu().numpy(), first_c)
    _equal_up_to_a_near_tie(dec.container.cpu().numpy(), ref_container, trace)


def test_prompt_passes_stop_before_an_end_token_and_check_their_arguments():
    from poptransformer_amd.engine import fused, loader
    B, L, pad, eos = 2, 48, 0, 2
    sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=1, int4=True)
    dec = fused.FusedDecoder(loader.llama2_spec(LLAMA_TINY, L, B, pad, eos, early_stop=True), loader.llama2_weights(sd, LLAMA_TINY))
    ids = _prompt(np.random.default_rng(3), B, L, 20, LLAMA_TINY["vocab_size"], pad)
    ids[ids == eos] = eos + 1
    ids[1, 9] = eos                                   # an end token inside the second prompt
    dec.reset(ids)
    assert dec.prompt_positions() == 8                # iterations 0..7 read positions 1..8: no end token yet
    with pytest.raises(ValueError):
        dec.consume_prompt(9)
    with pytest.raises(ValueError):
        dec.consume_prompt(4, rows_per_pass=1030)     # 2060 rows
    assert dec.consume_prompt(8) == 8
    with pytest.raises(RuntimeError):
        dec.consume_prompt(1)                         # only directly after reset
    oracle = OM.Llama2Oracle(sd, LLAMA_TINY, L, B)
    ref_container, ref_step = OM.run_decode_loop(oracle, ids, L, 40, pad, eos, early_stop=True)
    dec.run_steps(32)
    torch.cuda.synchronize()
    assert np.array_equal(dec.container.cpu().numpy(), ref_container)


@pytest.mark.parametrize("B", [1, 3])
def test_llama2_fp8_kv_cache_matches_oracle(B):
    """INT4 Llama 2 with the KV cache held as F143 bytes: tokens identical to the oracle whose KVCache op casts
    its input to FP8 and its output back (fp8 = true), logits within 1e-2; the prompt taken in passes gives the
    same tokens; the cache takes half the bytes."""
    from poptransformer_amd.engine import fused, loader
    L, steps, pad, eos = 48, 32, 0, 2
    sd = OM.make_llama2_state_dict(LLAMA_TINY, seed=1, int4=True)
    spec = loader.llama2_spec(LLAMA_TINY, L, B, pad, eos, fp8_cache=True)
    dec = fused.FusedDecoder(spec, loader.llama2_weights(sd, LLAMA_TINY))
    assert dec.rings[0].dtype == torch.uint8
    ids = _prompt(np.random.default_rng(7), B, L, 12, LLAMA_TINY["vocab_size"], pad)
    _compare(dec, OM.Llama2Oracle(sd, LLAMA_TINY, L, B, fp8_cache=True), ids, L, steps, pad, eos)
    reference = dec.container.cpu().numpy().copy()
    _prompt_then_loop(dec, ids, steps)
    assert np.array_equal(dec.container.cpu().numpy(), reference)

