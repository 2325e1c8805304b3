"""Host-side behaviour of the operator API (no GPU): what the ops record, the registry and scope
semantics, layer weight binding per precision, and the guards the reference raises while a graph
is being built."""
import numpy as np
import pytest

from oracle import models as OM
from oracle import ops as O


@pytest.fixture()
def fresh():
    from poptransformer_amd.utils import REGISTRY, register_global_args
    REGISTRY.reset()
    register_global_args({"batch_size": 2, "precision": "fp16"})
    return REGISTRY


def test_registry_semantics(fresh):
    R = fresh
    with pytest.raises(KeyError):
        R.register("main_graph", None)            # duplicate key (registry.py:22-25)
    with pytest.raises(KeyError):
        R.get("nope")
    R.register("x", 1)
    R.update("x", 2)
    assert R.get("x") == 2


def test_options_scope_restores(fresh):
    from poptransformer_amd.utils import OptionsScope
    assert fresh.get("partialtype") is None
    with OptionsScope(amp=0.4, partialtype="half"):
        assert fresh.get("partialtype") == "half" and fresh.get("amp") == 0.4
        with OptionsScope(partialtype="float"):
            assert fresh.get("partialtype") == "float"
        assert fresh.get("partialtype") == "half"
    assert fresh.get("partialtype") is None and fresh.get("amp") is None


def test_ops_record_reference_custom_ops(fresh):
    from poptransformer_amd import ops, popart
    g = fresh.get("main_graph")
    x = g.addInputTensor(popart.TensorInfo("FLOAT16", [2, 1, 8]), "x")
    step = g.addInputTensor(popart.TensorInfo("INT32", []), "step")
    out = ops.kv_cache(g, step, x, 16, 1, 1)
    n = g.nodes[-1]
    assert n.op == "custom.KVCache" and n.inputs == [step, x] and n.outputs == [out]
    assert n.attrs == {"max_len": 16, "step_len": 1, "sequence_axis": 1, "fp8": False}   # customized.py:28-33
    ops.softmax_ce(g, x, -1, stable_mode=False)
    assert g.nodes[-1].op == "custom.SoftmaxV3" and g.nodes[-1].attrs == {"axis": -1, "stable_mode": False}
    w = g.addInitializedInputTensor(np.ones(8, np.float16), "w")
    ops.layer_norm_ce(g, x, w, w, 1e-5, 2, 1, 8)
    a = g.nodes[-1].attrs
    assert g.nodes[-1].op == "custom.NormCE" and a["num_groups"] == 2 and a["epsilon"] == 1e-5 and a["stable_algo"] is False
    with pytest.raises(AssertionError):
        ops.layer_norm_ce(g, x, w, w, 1e-5, 2, 1, 8192)          # customized.py:81-82
    ops.int4_to_half(g, x, w, x)
    assert g.nodes[-1].attrs == {"axis": 1, "remap": 1}
    # the two registered ops the reference has no Python wrapper for: attribute names of their OpCreators
    ops.kv_cache_pipeline(g, step, x, 16, 3, transpose=1)
    n = g.nodes[-1]
    assert n.op == "custom.KVCachePipeline" and n.inputs == [step, x]
    assert {k: n.attrs[k] for k in ("max_len", "max_bps", "step_len", "sequence_axis", "fp8", "transpose")} == \
        {"max_len": 16, "max_bps": 3, "step_len": 1, "sequence_axis": -2, "fp8": False, "transpose": 1}
    outs = ops.beam_search(g, x, x, x, step, 4)
    n = g.nodes[-1]
    assert n.op == "custom.BeamSearch" and len(outs) == 4 and n.outputs == outs and n.attrs == {"beam_size": 4}
    ops.half_to_uint8(g, x, w)
    assert g.nodes[-1].op == "custom.CastToUint8WithoutShapeInfer" and g.nodes[-1].attrs == {"fp8Format": "F143"}
    ops.fp8_matmul(g, x, x, w, w)
    assert g.nodes[-1].attrs == {"fp8FormatLHS": "F143", "fp8FormatRHS": "F143"}
    with pytest.raises(ValueError):
        ops.softmax(g, x, -1, stable_mode=True)                   # popart.py:129-132
    v, i = ops.topk(g, x, 2, 1)
    assert (v, i) == ("Topk:0", "Topk:1")
    parts = ops.split(g, x, 2, 2, [4, 4])
    assert len(parts) == 2


def test_loop_records_body_and_tensor_names(fresh):
    from poptransformer_amd.models.llama2 import LLAMA2DecModel
    cfg = dict(vocab_size=64, hidden_size=32, rms_norm_eps=1e-5, num_attention_heads=2, intermediate_size=48, num_hidden_layers=2)
    fresh.update("precision", "int4")
    from poptransformer_amd.utils import TensorType
    fresh.update("tensor_type", TensorType("int4"))
    sd = OM.make_llama2_state_dict(cfg, seed=1, int4=True)
    m = LLAMA2DecModel(hf_config=cfg, state_dict=sd, pad_token_id=0, eos_token_id=2, max_length=16)
    m.build_graph()
    g = m.graph
    assert g.getOutputTensorIds() == ["Loop:0", "Loop:1"]            # the anchors the reference reads
    loop = [n for n in g.nodes if n.op == "aiOnnx.loop"][0]
    body = loop.subgraph
    assert body.inputs[:2] == ["max_loop", "cond"] and len(body.outputs) == 5
    ops_in_body = [n.op for n in body.nodes]
    assert ops_in_body.count("custom.KVCache") == 2 and ops_in_body.count("custom.Int4ToHalf") == 14
    assert ops_in_body.count("custom.SoftmaxV3") == 2 and ops_in_body.count("aiOnnx.topk") == 1
    # INT4 binding: packed weight back in [out, in/2], scale registered next to it (precision_strategy.py:24-42)
    key = "model.layers.0.self_attn.q_proj.weight"
    assert g.initializers[key].dtype == np.int8 and g.initializers[key].shape == (32, 16)
    assert g.initializers[key + "_scale"].dtype == np.float16 and key + "_scale" in g.getInputTensorIds()
    assert g.initializers["lm_head.weight"].dtype == np.float16 and g.initializers["lm_head.weight"].shape == (32, 64)
    assert sorted(m.initializers) == sorted(g.initializers)


def test_fp8_weight_binding_uses_f143_with_exponent_minus_one(fresh):
    from poptransformer_amd.layers import Linear
    from poptransformer_amd.utils import TensorType
    fresh.update("precision", "fp8")
    fresh.update("tensor_type", TensorType("fp8"))
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((6, 8)) * 0.05).astype(np.float16)
    fresh.update("state_dict", {"l.weight": w})
    lin = Linear(None, "l", 8, 6, use_bias=False)
    g = fresh.get("main_graph")
    got = g.initializers[lin.weight_id]
    assert got.dtype == np.uint8 and got.shape == (8, 6)
    assert np.array_equal(g.initializers["l.weight_scale"], np.array([-1], np.int32))       # precision_strategy.py:46
    assert np.array_equal(got, O.f8_encode(w.T.astype(np.float32), "F143", -1))


def test_host_fp8_encoder_equals_oracle():
    from poptransformer_amd.engine.host_codecs import f8_encode_host
    rng = np.random.default_rng(1)
    for fmt, mx in (("F143", 240.0), ("F152", 57344.0)):
        x = np.concatenate([rng.standard_normal(5000) * 0.05, rng.uniform(-mx, mx, 5000), [0, -0.0, np.inf, -np.inf, np.nan, 1e-9]])
        for s in (0, -1, 4):
            assert np.array_equal(f8_encode_host(x, fmt, s), O.f8_encode(x, fmt, s))
    with pytest.raises(ValueError):
        f8_encode_host(x, "F999", 0)


def test_layer_guards(fresh):
    from poptransformer_amd.layers import MLP, LayerNorm, Linear
    from poptransformer_amd import popart
    with pytest.raises(ValueError):
        MLP("m", "mlp", 8, 16, "tanhh")                            # layers/mlp.py:27-28
    ln = LayerNorm("m", "ln", 8, 1e-5)
    g = fresh.get("main_graph")
    x = g.addInputTensor(popart.TensorInfo("FLOAT16", [2, 1, 8]), "x")
    with pytest.raises(ValueError):
        ln(g, x, 1, "batch")                                       # layers/layer_norm.py:39-40
    fresh.update("model_type", "tp")
    with pytest.raises(ValueError):
        Linear("m", "l", 8, 8)                                     # no tensor-parallel variant on one GPU
    fresh.update("model_type", "shard")
    fresh.update("state_dict", {"m.l.weight": np.zeros((4, 8), np.float16)})
    with pytest.raises(AssertionError):
        Linear("m", "l", 8, 8, use_bias=False)                    # shape check of base_layer.py:121-125


def test_gpt2_state_dict_processing_matches_reference_rewrite(fresh):
    """Conv1D weights [in, out] -> [out, in], query third pre-scaled (gpt2/model.py:154-166)."""
    from poptransformer_amd.models.gpt2 import GPT2DecModel
    cfg = dict(vocab_size=50, n_embd=16, layer_norm_epsilon=1e-5, n_head=2, n_layer=1, n_positions=8)
    processed = OM.make_gpt2_state_dict(cfg, seed=3)
    hf_like = dict(processed)
    d = 16
    for k in list(hf_like):
        if k.endswith(("attn.c_attn.weight", "attn.c_proj.weight", "mlp.c_fc.weight", "mlp.c_proj.weight")):
            w = hf_like[k].astype(np.float32).T.copy()
            if k.endswith("c_attn.weight"):
                w[:, :d] /= np.float32(1 / 8 ** 0.5)
            hf_like[k] = w.astype(np.float16)
    m = GPT2DecModel(hf_config=cfg, state_dict=hf_like, pad_token_id=49, eos_token_id=48, max_length=8)
    got = m.state_dict["transformer.h.0.attn.c_attn.weight"].astype(np.float32)
    ref = processed["transformer.h.0.attn.c_attn.weight"].astype(np.float32)
    assert got.shape == ref.shape and np.abs(got - ref).max() <= 2e-4
    assert m.state_dict["transformer.h.0.mlp.c_fc.weight"].shape == (64, 16)
