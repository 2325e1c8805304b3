"""From a recorded graph to something that runs: `Session.compile` ends here.

Every graph can run op by op (engine/interpreter.py).  A graph that is one of the decoder loops
this package knows - GPT-2, Llama 2, ChatGLM2, RWKV as the models build them through the operator
API - is additionally mapped onto the fused executor for its family: the family is read off the
state-dict keys the layers registered as initializer names, the shapes off a one-iteration probe of
the interpreter, and the weights off the initializers.  The fused executor is then VALIDATED: it
must generate the same token ids as the interpreter on a probe prompt, otherwise the graph stays
on the interpreter.  A fused executor therefore never changes what a graph computes; it only
changes how fast.
"""
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


def _linear(facts, ctx, bias, precision):
    """A Linear as the layer bound it (layers/linear.py + utils/param_handler.py): fp16 [in, out];
    packed INT4 int8 [out, in/2] with `<key>_scale` fp16 [out]; F143 bytes [in, out] with an int32
    `<key>_scale` exponent."""
    key = f"{ctx}.weight"
    w = facts.init[key]
    b = _dev(facts.init[f"{ctx}.bias"].astype(np.float16)) if bias else None
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
    return _dev(facts.init[key].astype(np.float16).reshape(-1))


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
def _build_transformer(facts, shapes, family):
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
        embed = facts.init["model.embed_tokens.weight"]
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
        embed = facts.init["transformer.embedding.word_embeddings.weight"]
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
        wte = _dev(facts.init["transformer.wte.weight"].astype(np.float16))
        w = ModelWeights(wte, _dev(facts.init["transformer.wpe.weight"].astype(np.float16)), blocks,
                         (_vec(facts, "transformer.ln_f.weight"), _vec(facts, "transformer.ln_f.bias")),
                         LinearWeights(K.F16Weight(wte)), None)
        eps = _eps_from_normce(facts)
    if n_layer == 0 or facts.ops.get("custom.KVCache", 0) != n_layer:
        raise ValueError("layer count does not match the KV caches in the graph")
    d_model = w.embed.shape[1]
    spec = DecoderSpec(family, n_layer, d_model, Hq, Hkv, D, w.head.N, facts.max_len, facts.batch, eps, facts.pad_id,
                       facts.eos_id, facts.early_stop)
    return fused.FusedDecoder(spec, w)


def _build_rwkv(facts, shapes):
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
    w = RWKVWeights(_dev(facts.init["rwkv.embeddings.weight"].astype(np.float16)), blocks, ln("rwkv.ln_out"),
                    _linear(facts, "head", False, prec))
    d = w.embed.shape[1]
    # every `rescale_every` blocks the hidden state is halved by a Div node
    n_div = sum(1 for n in facts.body.nodes if n.op == "aiOnnx.div" and _const_value(facts.body, n.inputs[1]) is not None
                and float(_const_value(facts.body, n.inputs[1])) == 2.0)
    rescale = n_layer // n_div if n_div else 0
    spec = RWKVSpec(n_layer, d, blocks[0].att_key.N, blocks[0].ffn_key.N, w.head.N, facts.max_len, facts.batch,
                    _eps_from_normce(facts), rescale, facts.pad_id, facts.eos_id, facts.early_stop)
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
    def __init__(self, decoder, facts, anchors, batches_per_step, kind):
        self.decoder, self.facts, self.anchors, self.bps, self.kind = decoder, facts, list(anchors), batches_per_step, kind

    def _run_once(self, ids):
        container, step = self.decoder.run(ids, self.facts.max_loop)
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


def _probe_ids(facts, seed):
    rng = np.random.default_rng(seed)
    vocab_guess = 64
    for key, arr in facts.init.items():
        if arr.ndim == 2 and ("embed" in key or "wte" in key):
            vocab_guess = arr.shape[0]
            break
    ids = np.full((facts.batch, facts.max_len), facts.pad_id, np.int32)
    n = min(3, facts.max_len)
    p = rng.integers(0, vocab_guess, size=(facts.batch, n))
    p[p == facts.pad_id] = (facts.pad_id + 1) % vocab_guess
    p[p == facts.eos_id] = (facts.eos_id + 1) % vocab_guess if facts.eos_id >= 0 else p[p == facts.eos_id]
    ids[:, :n] = p
    return ids


def compile_graph(graph, anchors, batches_per_step=1, allow_fused=True):
    """Returns an executor with `run(feeds) -> {anchor: array}` and `anchor_arrays()`; its `kind`
    attribute says which one it is ('interpreter' or 'fused:<family>')."""
    from .. import _lib
    _lib.load()                                   # no HIP library, no executor: there is no CPU path
    prog = InterpretedProgram(graph, anchors, batches_per_step)
    if not allow_fused:
        return prog
    try:
        facts = GraphFacts(graph)
        family = _family(facts)
        if family is None:
            raise ValueError("no known model family among the initializer names")
        if len(anchors) > 2 or list(anchors) != list(graph.outputs)[:len(anchors)]:
            raise ValueError("anchors other than the loop outputs")
        # one-iteration probe: operand shapes of the native operators, and the reference output
        interp = prog.interp
        interp.shape_trace = {}
        interp.max_trips = 1
        ids = _probe_ids(facts, 0)
        prog._run_once({facts.ids_name: ids})
        shapes, interp.shape_trace = interp.shape_trace, None
        decoder = _build_rwkv(facts, shapes) if family == "rwkv" else _build_transformer(facts, shapes, family)
        # validation: identical ids after a few iterations, eager and replayed
        steps = min(PROBE_STEPS, facts.max_loop)
        interp.max_trips = steps
        want = prog._run_once({facts.ids_name: ids})[graph.outputs[0]]
        got, _ = decoder.run(ids, steps)
        if not np.array_equal(got, want):
            raise ValueError("the fused executor does not reproduce the graph's tokens on the probe")
        decoder.capture()
        got, _ = decoder.run(ids, steps)
        if not np.array_equal(got, want):
            raise ValueError("the captured HIP graph does not reproduce the graph's tokens on the probe")
        interp.max_trips = None
        return FusedProgram(decoder, facts, anchors, batches_per_step, f"fused:{family}")
    except Exception as e:  # noqa: BLE001 - any failure keeps the graph on the interpreter
        prog.interp.max_trips = None
        prog.interp.shape_trace = None
        log.warning("graph stays on the op-by-op interpreter: %s", e)
        prog.fallback_reason = str(e)
        return prog
