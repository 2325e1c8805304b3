"""From a recorded graph to something that runs: `Session.compile` ends here.

Every graph can run op by op (engine/interpreter.py).  A graph that is one of the decoder loops
this package knows - GPT-2, Llama 2, ChatGLM2, RWKV as the models build them through the operator
API - is additionally mapped onto the fused executor for its family: the family is read off the
state-dict keys the layers registered as initializer names, the shapes off a one-iteration probe of
the interpreter, and the weights off the initializers.  The fused executor is then VALIDATED: it
must generate the same token ids as the interpreter on a probe prompt (for a sampling graph: the same top-k candidates), otherwise
the graph stays on the interpreter - or, for a strict session, compilation fails.  An INT4 Llama-2
graph at batch <= 16 is further mapped onto the one-launch-per-iteration persistent step, validated
the same way, and prompts are taken in passes over several positions.
"""
import dataclasses
import logging

import numpy as np
import torch

from .. import kernels as K
from ..popart import NP_OF
from . import fused, rwkv
from .fused import BlockWeights, DecoderSpec, LinearWeights, ModelWeights
from .interpreter import InterpretedProgram

log = logging.getLogger("poptransformer")

PROBE_STEPS = 6


# ----------------------------------------------------------------------------------- graph facts
def _find_loop(graph):
    loops = [n for n in graph.nodes if n.op == "aiOnnx.loop"]
    if len(loops) != 1:
        return None
    return loops[0]


def _const_value(graph, tid):
    g = graph
    while g is not None:
        for n in g.nodes:
            if n.op == "aiOnnx.constant" and n.outputs[0] == tid:
                return np.asarray(n.attrs["value"])
        g = g.parent
    return None


def _named_const(body, name):
    for n in body.nodes:
        if n.op == "aiOnnx.constant" and n.attrs.get("name") == name:
            return np.asarray(n.attrs["value"])
    return None


class GraphFacts:
    def __init__(self, graph):
        self.graph = graph
        self.loop = _find_loop(graph)
        if self.loop is None:
            raise ValueError("no single Loop in the main graph")
        self.body = self.loop.subgraph
        self.max_loop = int(_const_value(graph, self.loop.inputs[0]))
        ids = [t for t, i in graph.input_info.items() if t in self.loop.inputs]
        if len(ids) != 1:
            raise ValueError("expected exactly one host-fed loop input (the id container)")
        self.ids_name = ids[0]
        self.batch, self.max_len = graph.input_info[ids[0]].shape()
        pad, eos = _named_const(self.body, "pad_id"), _named_const(self.body, "eos_id")
        if pad is None or eos is None:
            raise ValueError("pad_id / eos_id constants not found in the loop body")
        self.pad_id, self.eos_id = int(pad), int(eos)
        cond = self.body.outputs[0]
        self.early_stop = _const_value(self.body, cond) is None
        self.init = graph.root.initializers
        self.ops = {}
        for n in self.body.nodes:
            self.ops[n.op] = self.ops.get(n.op, 0) + 1

    def has(self, key):
        return key in self.init

    def count_layers(self, fmt):
        n = 0
        while fmt.format(n) in self.init:
            n += 1
        return n


# ----------------------------------------------------------------------------------- weights
def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _need(facts, key):
    """An initializer the family's graph must hold; a graph without it is not that family's graph."""
    if key not in facts.init:
        raise ValueError(f"initializer {key} is missing")
    return facts.init[key]


def _linear(facts, ctx, bias, precision):
    """A Linear as the layer bound it (layers/linear.py + utils/param_handler.py): fp16 [in, out];
    packed INT4 int8 [out, in/2] with `<key>_scale` fp16 [out]; F143 bytes [in, out] with an int32
    `<key>_scale` exponent."""
    key = f"{ctx}.weight"
    w = _need(facts, key)
    b = _dev(_need(facts, f"{ctx}.bias").astype(np.float16)) if bias else None
    scale = facts.init.get(key + "_scale")
    if w.dtype == np.int8:
        if scale is None:
            raise ValueError(f"{key} is packed INT4 but has no scale")
        return LinearWeights(K.W4Weight(_dev(w), _dev(scale.astype(np.float16))), b)
    if w.dtype == np.uint8:
        exponent = int(scale.reshape(-1)[0])
        return LinearWeights(K.F8Weight(_dev(w), _dev(scale.astype(np.int32).reshape(-1)), "F143", kn=True), b,
                             act_fp8=precision == "fp8", scale_value=exponent)
    if w.dtype != np.float16:
        raise ValueError(f"{key}: fused executors take fp16, INT4 or FP8 weights, not {w.dtype}")
    return LinearWeights(K.F16Weight(_dev(np.ascontiguousarray(w.T))), b)


def _vec(facts, key):
    return _dev(_need(facts, key).astype(np.float16).reshape(-1))


def _precision(facts, probe_ops):
    if "custom.CastToUint8WithoutShapeInfer" in probe_ops:
        return "fp8"
    if "custom.FP8MatMulWithoutShapeInfer" in probe_ops:
        return "fp8_weight"
    return "fp16"


def _eps_from_rmsnorm(facts):
    v = _named_const(facts.body, "variance_epsilon")
    if v is None:
        raise ValueError("RMSNorm epsilon not found")
    return float(v)


def _eps_from_normce(facts):
    for n in facts.body.nodes:
        if n.op == "custom.NormCE":
            return float(n.attrs["epsilon"])
    raise ValueError("NormCE epsilon not found")


# ----------------------------------------------------------------------------------- families
def _build_transformer(facts, shapes, family, topk=1, fp8_cache=False):
    kv = shapes["custom.KVCache"][0][1]              # updater [2, B, Hkv, 1, D]
    sm = shapes["custom.SoftmaxV3"][0][0]            # scores  [B, Hq, 1, L]
    Hkv, D, Hq = kv[2], kv[4], sm[1]
    prec = _precision(facts, facts.ops)
    if family == "llama2":
        n_layer = facts.count_layers("model.layers.{}.input_layernorm.weight")
        blocks = []
        for i in range(n_layer):
            p = f"model.layers.{i}."
            blocks.append(BlockWeights(
                norm1=(_vec(facts, p + "input_layernorm.weight"), None),
                norm2=(_vec(facts, p + "post_attention_layernorm.weight"), None),
                qkv=[_linear(facts, p + "self_attn." + n, False, prec) for n in ("q_proj", "k_proj", "v_proj")],
                out=_linear(facts, p + "self_attn.o_proj", False, prec),
                mlp_in=[_linear(facts, p + "mlp." + n, False, prec) for n in ("gate_proj", "up_proj")],
                mlp_out=_linear(facts, p + "mlp.down_proj", False, prec)))
        embed = _need(facts, "model.embed_tokens.weight")
        inv = np.array([1.0 / (10000 ** (i / D)) for i in range(0, D, 2)]).astype(np.float16)
        w = ModelWeights(_dev(embed.astype(np.float16)), None, blocks, (_vec(facts, "model.norm.weight"), None),
                         _linear(facts, "lm_head", False, prec), _dev(inv))
        eps = _eps_from_rmsnorm(facts)
    elif family == "chatglm2":
        n_layer = facts.count_layers("transformer.encoder.layers.{}.input_layernorm.weight")
        blocks = []
        for i in range(n_layer):
            p = f"transformer.encoder.layers.{i}."
            has_bias = facts.has(p + "self_attention.query.bias")
            blocks.append(BlockWeights(
                norm1=(_vec(facts, p + "input_layernorm.weight"), None),
                norm2=(_vec(facts, p + "post_attention_layernorm.weight"), None),
                qkv=[_linear(facts, p + "self_attention.query", has_bias, prec),
                     _linear(facts, p + "self_attention.key_value", has_bias, prec)],
                out=_linear(facts, p + "self_attention.dense", False, prec),
                mlp_in=[_linear(facts, p + "mlp.dense_h_to_4h_1", False, prec), _linear(facts, p + "mlp.dense_h_to_4h_2", False, prec)],
                mlp_out=_linear(facts, p + "mlp.dense_4h_to_h", False, prec)))
        embed = _need(facts, "transformer.embedding.word_embeddings.weight")
        rot = D // 2
        inv = np.array([1.0 / (10000 ** (i / rot)) for i in range(0, rot, 2)]).astype(np.float32)
        w = ModelWeights(_dev(embed.astype(np.float16)), None, blocks,
                         (_vec(facts, "transformer.encoder.final_layernorm.weight"), None),
                         _linear(facts, "transformer.output_layer", False, prec), _dev(inv))
        eps = _eps_from_rmsnorm(facts)
    else:  # gpt2
        n_layer = facts.count_layers("transformer.h.{}.ln_1.weight")
        blocks = []
        for i in range(n_layer):
            p = f"transformer.h.{i}."
            blocks.append(BlockWeights(
                norm1=(_vec(facts, p + "ln_1.weight"), _vec(facts, p + "ln_1.bias")),
                norm2=(_vec(facts, p + "ln_2.weight"), _vec(facts, p + "ln_2.bias")),
                qkv=[_linear(facts, p + "attn.c_attn", True, prec)],
                out=_linear(facts, p + "attn.c_proj", True, prec),
                mlp_in=[_linear(facts, p + "mlp.c_fc", True, prec)],
                mlp_out=_linear(facts, p + "mlp.c_proj", True, prec)))
        wte = _dev(_need(facts, "transformer.wte.weight").astype(np.float16))
        w = ModelWeights(wte, _dev(_need(facts, "transformer.wpe.weight").astype(np.float16)), blocks,
                         (_vec(facts, "transformer.ln_f.weight"), _vec(facts, "transformer.ln_f.bias")),
                         LinearWeights(K.F16Weight(wte)), None)
        eps = _eps_from_normce(facts)
    if n_layer == 0 or facts.ops.get("custom.KVCache", 0) != n_layer:
        raise ValueError("layer count does not match the KV caches in the graph")
    d_model = w.embed.shape[1]
    spec = DecoderSpec(family, n_layer, d_model, Hq, Hkv, D, w.head.N, facts.max_len, facts.batch, eps, facts.pad_id,
                       facts.eos_id, facts.early_stop, topk=topk, fp8_cache=fp8_cache)
    return spec, w


def _build_rwkv(facts, shapes, topk=1):
    from .rwkv import RWKVBlockWeights, RWKVDecoder, RWKVSpec, RWKVWeights
    n_layer = facts.count_layers("rwkv.blocks.{}.ln1.weight")
    prec = _precision(facts, facts.ops)
    if prec != "fp16":
        raise ValueError("the fused RWKV executor takes fp16 or INT4 weights")

    def ln(key):
        return (_vec(facts, key + ".weight"), _vec(facts, key + ".bias"))

    blocks = []
    for i in range(n_layer):
        p = f"rwkv.blocks.{i}."
        blocks.append(RWKVBlockWeights(
            pre_ln=ln(p + "pre_ln") if facts.has(p + "pre_ln.weight") else None, ln1=ln(p + "ln1"), ln2=ln(p + "ln2"),
            att_key=_linear(facts, p + "attention.key", False, prec), att_value=_linear(facts, p + "attention.value", False, prec),
            att_receptance=_linear(facts, p + "attention.receptance", False, prec),
            att_output=_linear(facts, p + "attention.output", False, prec),
            time_decay=_vec(facts, p + "attention.time_decay"), time_first=_vec(facts, p + "attention.time_first"),
            att_mix=[_vec(facts, p + f"attention.time_mix_{n}") for n in ("key", "value", "receptance")],
            ffn_key=_linear(facts, p + "feed_forward.key", False, prec),
            ffn_receptance=_linear(facts, p + "feed_forward.receptance", False, prec),
            ffn_value=_linear(facts, p + "feed_forward.value", False, prec),
            ffn_mix=[_vec(facts, p + f"feed_forward.time_mix_{n}") for n in ("key", "receptance")]))
    w = RWKVWeights(_dev(_need(facts, "rwkv.embeddings.weight").astype(np.float16)), blocks, ln("rwkv.ln_out"),
                    _linear(facts, "head", False, prec))
    d = w.embed.shape[1]
    # every `rescale_every` blocks the hidden state is halved by a Div node
    n_div = sum(1 for n in facts.body.nodes if n.op == "aiOnnx.div" and _const_value(facts.body, n.inputs[1]) is not None
                and float(_const_value(facts.body, n.inputs[1])) == 2.0)
    rescale = n_layer // n_div if n_div else 0
    spec = RWKVSpec(n_layer, d, blocks[0].att_key.N, blocks[0].ffn_key.N, w.head.N, facts.max_len, facts.batch,
                    _eps_from_normce(facts), rescale, facts.pad_id, facts.eos_id, facts.early_stop, topk=topk)
    return RWKVDecoder(spec, w)


def _family(facts):
    if facts.has("model.layers.0.self_attn.q_proj.weight"):
        return "llama2"
    if facts.has("transformer.encoder.layers.0.self_attention.query.weight"):
        return "chatglm2"
    if facts.has("transformer.h.0.attn.c_attn.weight"):
        return "gpt2"
    if facts.has("rwkv.blocks.0.attention.key.weight"):
        return "rwkv"
    return None


# ----------------------------------------------------------------------------------- programs
class FusedProgram:
    fallback_reason = None

    def __init__(self, decoder, facts, anchors, batches_per_step, kind, prompt_passes=False):
        self.decoder, self.facts, self.anchors, self.bps, self.kind = decoder, facts, list(anchors), batches_per_step, kind
        self.prompt_passes = prompt_passes

    def _run_once(self, ids):
        container, step = self.decoder.run(ids, self.facts.max_loop, prompt_passes=self.prompt_passes)
        out = {}
        if len(self.anchors) > 0:
            out[self.anchors[0]] = container
        if len(self.anchors) > 1:
            out[self.anchors[1]] = np.array(step, np.int32)
        return out

    def run(self, feeds):
        ids = np.asarray(feeds[self.facts.ids_name], np.int32)
        B, L = self.facts.batch, self.facts.max_len
        if self.bps == 1:
            return self._run_once(ids.reshape(B, L))
        outs = [self._run_once(ids.reshape(self.bps, B, L)[i]) for i in range(self.bps)]
        return {a: np.stack([o[a] for o in outs]) for a in self.anchors}

    def anchor_arrays(self):
        lead = [self.bps] if self.bps > 1 else []
        shapes = [([self.facts.batch, self.facts.max_len], np.int32), ([], np.int32)]
        return {a: np.zeros(lead + s, t) for a, (s, t) in zip(self.anchors, shapes)}


def _probe_ids(facts, seed, n=3):
    rng = np.random.default_rng(seed)
    vocab_guess = 64
    for key, arr in facts.init.items():
        if arr.ndim == 2 and ("embed" in key or "wte" in key):
            vocab_guess = arr.shape[0]
            break
    ids = np.full((facts.batch, facts.max_len), facts.pad_id, np.int32)
    n = min(n, facts.max_len)
    p = rng.integers(0, vocab_guess, size=(facts.batch, n))
    p[p == facts.pad_id] = (facts.pad_id + 1) % vocab_guess
    p[p == facts.eos_id] = (facts.eos_id + 1) % vocab_guess if facts.eos_id >= 0 else p[p == facts.eos_id]
    ids[:, :n] = p
    return ids


def _sampling_k(facts):
    """k of LMHead's selection, read off the loop body: 1 for the top-1 graph, k for ops.random_sample
    (aiOnnx.topk with k > 1 whose pick is the argmax of aiOnnx.randomnormal draws, ops/popart.py:25-29)."""
    ks = []
    for n in facts.body.nodes:
        if n.op == "aiOnnx.topk":
            k = _const_value(facts.body, n.inputs[1])
            if k is None:
                raise ValueError("aiOnnx.topk with a k that is not a constant")
            ks.append(int(np.asarray(k).reshape(-1)[0]))
    random = facts.ops.get("aiOnnx.randomnormal", 0)
    if not random:
        if ks != [1]:
            raise ValueError(f"expected one top-1 selection in the loop body, found topk with k = {ks}")
        return 1
    if random != 1 or len(ks) != 1 or ks[0] < 2:
        raise ValueError(f"random draws in the loop body that are not one ops.random_sample (topk k = {ks})")
    return ks[0]


def _fp8_cache_of(facts, requested):
    """Whether the KV caches hold F143 bytes: the session option, or the `fp8` attribute of the graph's KVCache
    nodes (the reference's ops.kv_cache always records False, ops/customized.py:32)."""
    flags = {bool(n.attrs.get("fp8")) for n in facts.body.nodes if n.op == "custom.KVCache"}
    if len(flags) > 1:
        raise ValueError("KVCache nodes with and without fp8 storage in one graph")
    return bool(requested) or (flags == {True})


def _validate_greedy(decoder, prog, facts, steps, prompt_passes, what, seeds=(0, 1)):
    """The fused executors' arithmetic is not bit for bit the graph's (projections that the graph runs one by one
    share a launch with another summation order; the one-launch iteration applies an INT4 scale to the fp32 sum,
    the graph to every weight), so greedy tokens alone are comparable only up to the first near tie of two logits -
    and with a vocabulary of tens of thousands, or activations cast to FP8, a near tie comes within a few tokens.
    The check is therefore made on the logits.  A probe whose tokens all equal the graph's is accepted as it is.
    Otherwise the graph's logits of every iteration (the inputs of its top-1 selection) are recorded for each probe
    of a fixed list, and the executor is run iteration by iteration beside them, its container following the
    graph's tokens: every iteration's logits must agree within 2 % of the iteration's largest magnitude (10 % where
    the graph casts activations to FP8: one code of an activation is an eighth of its value), and the selected token
    must be the graph's wherever the graph's two best logits are further apart than twice that tolerance.  With
    prompt_passes the probe's leading positions go through the passes first, so those are part of what is checked."""
    interp = prog.interp
    ids = _probe_ids(facts, seeds[0], n=3)
    want = prog._run_once({facts.ids_name: ids})[prog.interp_outputs[0]]
    got, _ = decoder.run(ids, steps, prompt_passes=prompt_passes)
    if np.array_equal(got, want):
        return
    tol = 0.1 if any("CastToUint8" in n.op for n in facts.body.nodes) else 0.02
    for seed in seeds:
        ids = _probe_ids(facts, seed, n=3)
        interp.input_trace = {"aiOnnx.topk": []}
        try:
            want = np.asarray(prog._run_once({facts.ids_name: ids})[prog.interp_outputs[0]]).reshape(facts.batch, -1)
            logits = [np.asarray(i[0], np.float32).reshape(facts.batch, -1) for i in interp.input_trace["aiOnnx.topk"]]
        finally:
            interp.input_trace = None
        decoder.reset(ids)
        done = 0
        if prompt_passes:
            n = min(decoder.prompt_positions(), len(logits))
            if n > 0:
                done = decoder.consume_prompt(n)
        for t in range(done, len(logits)):
            decoder.run_steps(1)                    # the captured graph where there is one
            torch.cuda.synchronize()
            ref = logits[t]
            got = decoder.logits.float().cpu().numpy().reshape(facts.batch, -1)
            scale = float(np.abs(ref).max())
            err = float(np.abs(got - ref).max()) / scale if scale > 0 else float(np.abs(got).max())
            if not err <= tol:
                raise ValueError(f"{what}: logits differ from the graph's at probe iteration {t} (seed {seed}): "
                                 f"{err:.3g} of the largest magnitude, allowed {tol}")
            if t + 1 < want.shape[1]:
                # the token chosen at iteration t lands in column t + 1 where the prompt left that column free
                free = ids[:, t + 1] == facts.pad_id
                top2 = np.sort(ref, axis=1)[:, -2:]
                clear = free & (top2[:, 1] - top2[:, 0] > 2 * tol * scale)
                mine = decoder.next_ids.cpu().numpy().reshape(-1)
                if not np.array_equal(mine[clear], want[clear, t + 1]):
                    raise ValueError(f"{what}: a token differs from the graph's at probe iteration {t} (seed {seed}) "
                                     f"where no other logit comes near the largest")
                rows = np.nonzero(free & (mine != want[:, t + 1]))[0]
                for b in rows:                      # a near tie decided the other way: follow the graph
                    decoder.container[int(b), t + 1] = int(want[b, t + 1])
        if getattr(decoder, "persistent", None) is not None and decoder.persistent.failed():
            raise RuntimeError(f"{what}: a launch of the persistent decode step gave up during the probe")


def _validate_sampling(decoder, prog, facts, ids, steps, k):
    """A sampling graph draws from its own generator, so tokens are not comparable; the candidates are.  The probe
    holds a token at every position it reaches (nothing that is drawn feeds back), and the top-k ids of every
    iteration must equal those of the interpreter, in order."""
    interp = prog.interp
    interp.value_trace = {"aiOnnx.topk": []}
    try:
        prog._run_once({facts.ids_name: ids})
        want = [np.asarray(o[1]).reshape(facts.batch, k) for o in interp.value_trace["aiOnnx.topk"]]
    finally:
        interp.value_trace = None
    if len(want) != steps:
        raise ValueError("the probe did not run the expected number of iterations")
    decoder.reset(ids)
    for it in range(steps):
        decoder.step_fn()
        torch.cuda.synchronize()
        if not np.array_equal(decoder.select.ids.cpu().numpy(), want[it]):
            raise ValueError(f"the fused executor's top-{k} candidates differ from the graph's at probe iteration {it}")


def compile_graph(graph, anchors, batches_per_step=1, allow_fused=True, strict=False, fp8_cache=False,
                  persistent=True, prompt_passes=True):
    """Returns an executor with `run(feeds) -> {anchor: array}` and `anchor_arrays()`; its `kind` attribute says
    which one it is: 'interpreter', 'fused:<family>' (one launch per operator, replayed from a HIP graph) or
    'fused:llama2:persistent' (one launch per loop iteration).  A graph the fused executors do not cover stays on
    the interpreter, with the reason in `fallback_reason`; with `strict` that is an error instead.
    persistent: use the one-launch iteration where the model allows it (INT4 Llama 2, batch <= 16, top-1; it needs
    the whole device for itself while it runs).  prompt_passes: the leading iterations that only read the prompt
    run as passes over several positions.  fp8_cache: KV caches hold F143 bytes (KVCache with fp8 = true)."""
    from .. import _lib
    _lib.load()                                   # no HIP library, no executor: there is no CPU path
    prog = InterpretedProgram(graph, anchors, batches_per_step)
    if not allow_fused:
        if strict:
            raise ValueError("strict: the session asks for a fused executor but allow_fused is off")
        return prog
    interp = prog.interp
    try:
        facts = GraphFacts(graph)
        family = _family(facts)
        if family is None:
            raise ValueError("no known model family among the initializer names")
        if len(anchors) > 2 or list(anchors) != list(graph.outputs)[:len(anchors)]:
            raise ValueError("anchors other than the loop outputs")
        prog.interp_outputs = list(graph.outputs)
        k = _sampling_k(facts)
        use_fp8_cache = _fp8_cache_of(facts, fp8_cache)
        if use_fp8_cache and family == "rwkv":
            raise ValueError("fp8_cache: a recurrent model has no KV cache")
        steps = min(PROBE_STEPS, facts.max_loop)
        # one-iteration probe: operand shapes of the native operators
        interp.shape_trace = {}
        interp.max_trips = 1
        ids = _probe_ids(facts, 0, n=3 if k == 1 else steps + 1)
        prog._run_once({facts.ids_name: ids})
        shapes, interp.shape_trace = interp.shape_trace, None
        if family == "rwkv":
            decoder = _build_rwkv(facts, shapes, k)
        else:
            spec, weights = _build_transformer(facts, shapes, family, k, use_fp8_cache)
            decoder = fused.FusedDecoder(spec, weights)
        passes = prompt_passes and hasattr(decoder, "consume_prompt")
        interp.max_trips = steps
        if k > 1:
            _validate_sampling(decoder, prog, facts, ids, steps, k)
            decoder.capture()
            kind = f"fused:{family}"
        elif use_fp8_cache and not any(n.attrs.get("fp8") for n in facts.body.nodes if n.op == "custom.KVCache"):
            # the option changes what the graph computes (its caches are fp16): nothing to compare the tokens with;
            # the executor is checked against the graph with fp16 caches first, then switched
            plain = fused.FusedDecoder(dataclasses.replace(spec, fp8_cache=False), weights)
            _validate_greedy(plain, prog, facts, steps, passes, "the fused executor")
            decoder.capture()
            kind = f"fused:{family}"
            if persistent and hasattr(decoder, "enable_persistent"):
                # the persistent step likewise: checked with fp16 caches, used with FP8 ones
                try:
                    plain.enable_persistent()
                    plain.capture()
                    _validate_greedy(plain, prog, facts, steps, passes, "the persistent decode step")
                    decoder.enable_persistent()
                    decoder.capture()
                    kind += ":persistent"
                except NotImplementedError as e:
                    prog.persistent_reason = str(e)
                except (ValueError, RuntimeError) as e:
                    if strict:
                        raise
                    log.warning("the persistent decode step is not used: %s", e)
                    prog.persistent_reason = str(e)
                    decoder.persistent = None
                    decoder.capture()
            del plain
        else:
            # validation: identical ids over a few iterations (up to a near tie), eager and replayed
            _validate_greedy(decoder, prog, facts, steps, passes, "the fused executor")
            decoder.capture()
            _validate_greedy(decoder, prog, facts, steps, passes, "the captured HIP graph")
            kind = f"fused:{family}"
            if persistent and hasattr(decoder, "enable_persistent"):
                try:
                    decoder.enable_persistent()
                except NotImplementedError as e:
                    prog.persistent_reason = str(e)
                else:
                    decoder.capture()
                    try:
                        _validate_greedy(decoder, prog, facts, steps, passes, "the persistent decode step")
                        kind += ":persistent"
                    except (ValueError, RuntimeError) as e:
                        if strict:
                            raise
                        log.warning("the persistent decode step is not used: %s", e)
                        prog.persistent_reason = str(e)
                        decoder.persistent = None
                        decoder.capture()
        interp.max_trips = None
        out = FusedProgram(decoder, facts, anchors, batches_per_step, kind, passes)
        out.persistent_reason = getattr(prog, "persistent_reason", None)
        return out
    except (ValueError, NotImplementedError) as e:
        # the expected ways a graph is outside what the fused executors cover; anything else is a bug and propagates
        interp.max_trips = None
        interp.shape_trace = None
        interp.value_trace = None
        if strict:
            raise
        log.warning("graph stays on the op-by-op interpreter: %s", e)
        prog.fallback_reason = str(e)
        return prog
