"""CPU restatement (numpy) of the PopTransformer decode loop for whole models.

TEST INFRASTRUCTURE ONLY (see oracle/ops.py): imported by tests/, by __graft_entry__.smoke()
and by the cpu_baseline leg of bench.py.  Each model walks the reference graph op by op with the
operator restatements of oracle/ops.py; state-dict keys and shapes are the reference's.
"""
import numpy as np

from . import ops as O

f16, f32 = np.float16, np.float32


# --------------------------------------------------------------------------------------
# synthetic checkpoints
# --------------------------------------------------------------------------------------
def quantize_int4(w):
    """Symmetric per-output-channel INT4 quantisation of w [out, in]: scale = max|w| / 7 (fp16),
    q = clip(round(w / scale), -8, 7), packed two per byte with feature 2j in the high nibble.
    The reference has no quantiser (it loads ChatGLM-int4 style checkpoints:
    `weight int8[out, in/2]`, `weight_scale fp16[out]`,
    poptransformer/utils/param_handler/precision_strategy.py:24-42); this only produces
    checkpoints of that layout for the synthetic configurations."""
    w = np.asarray(w, f32)
    scale = (np.abs(w).max(axis=1) / 7.0).astype(f16)
    scale = np.maximum(scale, np.finfo(f16).tiny).astype(f16)
    q = np.clip(np.rint(w / scale.astype(f32)[:, None]), -8, 7).astype(np.int8)
    return O.pack_int4(q), scale


def _normal(rng, shape, std=0.02):
    return (rng.standard_normal(shape, dtype=f32) * std).astype(f16)


def make_llama2_state_dict(cfg, seed=0, int4=True):
    """Random-init Llama-2-shaped checkpoint: weights N(0, 0.02), RMSNorm weights 1, Linear
    weights quantised to packed INT4 when `int4`, embeddings and lm_head fp16.  Keys and shapes:
    poptransformer/models/llama2/model.py:31-36,64-85,119-132, attention.py:58-62, mlp.py:15-18."""
    rng = np.random.Generator(np.random.PCG64(seed))
    d, f, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    sd = {"model.embed_tokens.weight": _normal(rng, (v, d))}

    def linear(key, out_f, in_f):
        w = _normal(rng, (out_f, in_f))
        if int4:
            sd[key + ".weight"], sd[key + ".weight_scale"] = quantize_int4(w)
        else:
            sd[key + ".weight"] = w

    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        sd[p + "input_layernorm.weight"] = np.ones(d, f16)
        for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
            linear(p + "self_attn." + n, d, d)
        sd[p + "post_attention_layernorm.weight"] = np.ones(d, f16)
        linear(p + "mlp.gate_proj", f, d)
        linear(p + "mlp.up_proj", f, d)
        linear(p + "mlp.down_proj", d, f)
    sd["model.norm.weight"] = np.ones(d, f16)
    sd["lm_head.weight"] = _normal(rng, (v, d))
    return sd


def make_gpt2_state_dict(cfg, seed=0):
    """Random-init GPT-2-shaped checkpoint as the reference holds it AFTER
    GPT2DecModel.process_hf_model_state_dict (poptransformer/models/gpt2/model.py:154-166): Linear
    weights in [out, in] orientation and the query third of c_attn pre-multiplied by
    1/sqrt(head_dim).  N(0, 0.02) weights, zero biases, LayerNorm gamma 1 / beta 0.
    Keys: models/gpt2/model.py:32-37,64-84, attention.py:33-35, embedding.py:27-29, layers/mlp.py:30-32."""
    rng = np.random.Generator(np.random.PCG64(seed))
    d, v, npos = cfg["n_embd"], cfg["vocab_size"], cfg["n_positions"]
    hd = d // cfg["n_head"]
    sd = {"transformer.wte.weight": _normal(rng, (v, d)), "transformer.wpe.weight": _normal(rng, (npos, d))}
    for i in range(cfg["n_layer"]):
        p = f"transformer.h.{i}."
        for ln in ("ln_1", "ln_2"):
            sd[p + ln + ".weight"] = np.ones(d, f16)
            sd[p + ln + ".bias"] = np.zeros(d, f16)
        w = (rng.standard_normal((3 * d, d), dtype=f32) * 0.02)
        w[:d] *= np.float32(1 / hd ** 0.5)
        sd[p + "attn.c_attn.weight"] = w.astype(f16)
        sd[p + "attn.c_attn.bias"] = np.zeros(3 * d, f16)
        sd[p + "attn.c_proj.weight"] = _normal(rng, (d, d))
        sd[p + "attn.c_proj.bias"] = np.zeros(d, f16)
        sd[p + "mlp.c_fc.weight"] = _normal(rng, (4 * d, d))
        sd[p + "mlp.c_fc.bias"] = np.zeros(4 * d, f16)
        sd[p + "mlp.c_proj.weight"] = _normal(rng, (d, 4 * d))
        sd[p + "mlp.c_proj.bias"] = np.zeros(d, f16)
    sd["transformer.ln_f.weight"] = np.ones(d, f16)
    sd["transformer.ln_f.bias"] = np.zeros(d, f16)
    return sd


# --------------------------------------------------------------------------------------
# shared pieces
# --------------------------------------------------------------------------------------
class _Linear:
    """BaseLinear (poptransformer/layers/linear.py:19-46) + ParamHandler.matmul
    (utils/param_handler/param_handler.py:57-61): `<ctx>.weight` is [out, in], stored transposed;
    an int8 weight is a packed INT4 matrix [out, in/2] with `<ctx>.weight_scale`
    (utils/param_handler/precision_strategy.py:24-42,56-60)."""

    def __init__(self, sd, ctx, use_bias):
        w = sd[ctx + ".weight"]
        if w.dtype == np.int8:
            self.w = O.int4_to_half(w, sd[ctx + ".weight_scale"], axis=1)   # [in, out] fp16
        else:
            self.w = np.ascontiguousarray(w.T)
        self.b = sd[ctx + ".bias"] if use_bias else None

    def __call__(self, x):
        y = O.matmul(x, self.w)
        return (y + self.b).astype(f16) if self.b is not None else y


def run_decode_loop(model, input_ids, max_length, max_loop, pad_id, eos_id, early_stop=False, trace=None):
    """HFDecBaseModel.build_graph / build_post_model_graph (poptransformer/models/base_model.py:271-311):
    a Loop of max_loop iterations over {container, step, mask, stop_mask}; returns the container
    and the final step like the anchors 'Loop:0' and 'Loop:1'."""
    state = O.initial_loop_state(input_ids, max_length)
    b = state["container"].shape[0]
    for _ in range(max_loop):
        step = state["step"]
        ids = state["container"][:, min(step, max_length - 1)].reshape(b, 1)
        next_ids, logits = model.step(ids, step, state["mask"])
        if trace is not None:
            trace.append((next_ids.copy(), logits.copy()))
        upd = O.step_containers(state, next_ids, pad_id)
        if not O.step_loop_cond(state, upd, eos_id, early_stop, b):
            break
    return state["container"], state["step"]


# --------------------------------------------------------------------------------------
# Llama 2
# --------------------------------------------------------------------------------------
class Llama2Oracle:
    """LLAMA2DecModel.build_model_graph (poptransformer/models/llama2/model.py:162-197) for
    sequence_length == 1: embedding gather, per block RMSNorm -> attention -> add -> RMSNorm ->
    SwiGLU MLP -> add (model.py:38-46), final RMSNorm, LMHead top-1 (layers/lm_head.py:47-57).
    fp8_cache: the `fp8_cache` argument of models/llama2/attention.py:18-24 taken to mean what the KVCache
    op does with fp8 = true (custom_ops/kv_cache.cpp:102-104,183-185); the reference's Python never sets
    the attribute (ops/customized.py:32 passes False)."""

    def __init__(self, sd, cfg, max_length, batch_size, fp8_cache=False):
        self.cfg, self.L, self.B = cfg, max_length, batch_size
        self.d, self.H = cfg["hidden_size"], cfg["num_attention_heads"]
        self.D = self.d // self.H
        self.eps = cfg["rms_norm_eps"]
        self.embed = sd["model.embed_tokens.weight"]
        self.layers = []
        for i in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{i}."
            self.layers.append({
                "ln1": sd[p + "input_layernorm.weight"], "ln2": sd[p + "post_attention_layernorm.weight"],
                "q": _Linear(sd, p + "self_attn.q_proj", False), "k": _Linear(sd, p + "self_attn.k_proj", False),
                "v": _Linear(sd, p + "self_attn.v_proj", False), "o": _Linear(sd, p + "self_attn.o_proj", False),
                "gate": _Linear(sd, p + "mlp.gate_proj", False), "up": _Linear(sd, p + "mlp.up_proj", False),
                "down": _Linear(sd, p + "mlp.down_proj", False),
                "cache": O.KVCache(max_length, 3, 1, fp8=fp8_cache),
            })
        self.norm = sd["model.norm.weight"]
        self.head = _Linear(sd, "lm_head", False)

    def _attention(self, lay, x, step, mask4):
        """Attention.forward_qkv / forward_attention / forward_output
        (poptransformer/models/llama2/attention.py:64-114)."""
        B, H, D = self.B, self.H, self.D
        q, k, v = lay["q"](x), lay["k"](x), lay["v"](x)
        q = q.reshape(B, 1, H, D).transpose(0, 2, 1, 3)
        k = k.reshape(B, 1, H, D).transpose(0, 2, 1, 3)
        v = v.reshape(B, 1, H, D).transpose(0, 2, 1, 3)
        sin, cos = O.llama_sincos(step, D)
        q, k = O.llama_rope(q, sin, cos), O.llama_rope(k, sin, cos)
        kv = np.concatenate([k, v], axis=0).reshape(2, B, H, 1, D)
        past = lay["cache"](step, kv)
        kt = past[0].transpose(0, 1, 3, 2)
        a = O.attention_scores_to_context(q, kt, past[1], mask4, 1 / np.sqrt(D), f32, stable_mode=False)
        a = a.transpose(0, 2, 1, 3).reshape(B, 1, H * D)
        return lay["o"](a)

    def step(self, ids, step, mask):
        B = self.B
        x = self.embed[ids.reshape(B, 1)]                        # [B, 1, d] gather
        mask4 = mask[:, None, None, :]
        for lay in self.layers:
            t = O.rms_norm(x, lay["ln1"], self.eps)
            t = self._attention(lay, t, step, mask4)
            x = (x + t).astype(f16)
            t = O.rms_norm(x, lay["ln2"], self.eps)
            t2 = t.reshape(-1, self.d)                          # ShardMLP (models/llama2/mlp.py:20-28)
            g = O.swish(lay["gate"](t2))
            u = (lay["up"](t2) * g).astype(f16)
            t = lay["down"](u).reshape(B, -1, self.d)
            x = (x + t).astype(f16)
        x = O.rms_norm(x, self.norm, self.eps)
        logits = self.head(x)                                    # [B, 1, V]
        _, idx = O.topk1(logits, axis=2)
        return idx.reshape(B), logits.reshape(B, -1)


# --------------------------------------------------------------------------------------
# GPT-2
# --------------------------------------------------------------------------------------
class GPT2Oracle:
    """GPT2DecModel.build_model_graph (poptransformer/models/gpt2/model.py:168-201), blocks
    (model.py:39-46), embedding wte[id] + wpe[step] (models/gpt2/embedding.py:31-36), LayerNorm via
    NormCE, head tied to wte (model.py:144-151, layers/lm_head.py:47-57)."""

    def __init__(self, sd, cfg, max_length, batch_size):
        self.cfg, self.L, self.B = cfg, max_length, batch_size
        self.d, self.H = cfg["n_embd"], cfg["n_head"]
        self.D = self.d // self.H
        self.eps = cfg["layer_norm_epsilon"]
        self.wte, self.wpe = sd["transformer.wte.weight"], sd["transformer.wpe.weight"]
        self.layers = []
        for i in range(cfg["n_layer"]):
            p = f"transformer.h.{i}."
            self.layers.append({
                "ln1": (sd[p + "ln_1.weight"], sd[p + "ln_1.bias"]), "ln2": (sd[p + "ln_2.weight"], sd[p + "ln_2.bias"]),
                "c_attn": _Linear(sd, p + "attn.c_attn", True), "c_proj": _Linear(sd, p + "attn.c_proj", True),
                "c_fc": _Linear(sd, p + "mlp.c_fc", True), "mlp_proj": _Linear(sd, p + "mlp.c_proj", True),
                "cache": O.KVCache(max_length, 3, 1),
            })
        self.ln_f = (sd["transformer.ln_f.weight"], sd["transformer.ln_f.bias"])
        self.head_w = np.ascontiguousarray(self.wte.T)            # ops.transpose(wte, [1, 0])

    def _ln(self, x, wb):
        return O.layer_norm_ce(x, wb[0], wb[1], self.eps, self.B, 1, self.d)

    def _attention(self, lay, x, step, mask4):
        """BaseAttention (poptransformer/models/gpt2/attention.py:37-90)."""
        B, H, D, d = self.B, self.H, self.D, self.d
        qkv = lay["c_attn"](x)                                     # [B, 1, 3d]
        q, kv = qkv[..., :d], qkv[..., d:]
        q = q.reshape(B, 1, H, D).transpose(0, 2, 1, 3)
        kv = kv.reshape(B, 1, 2, H, D).transpose(2, 0, 3, 1, 4)    # [2, B, H, 1, D]
        past = lay["cache"](step, kv)
        a = O.attention_scores_to_context(q, past[0].transpose(0, 1, 3, 2), past[1], mask4, None, f16, False)
        a = a.transpose(0, 2, 1, 3).reshape(B, 1, d)
        return lay["c_proj"](a)

    def step(self, ids, step, mask):
        B = self.B
        x = (self.wte[ids.reshape(B, 1)] + self.wpe[np.full((B, 1), step)]).astype(f16)
        mask4 = mask[:, None, None, :]
        for lay in self.layers:
            t = self._ln(x, lay["ln1"])
            t = self._attention(lay, t, step, mask4)
            x = (x + t).astype(f16)
            t = self._ln(x, lay["ln2"])
            t = t.reshape(-1, self.d)                              # BaseMLP (layers/mlp.py:34-41)
            t = lay["mlp_proj"](O.gelu(lay["c_fc"](t))).reshape(B, -1, self.d)
            x = (x + t).astype(f16)
        x = self._ln(x, self.ln_f)
        logits = O.matmul(x, self.head_w)
        _, idx = O.topk1(logits, axis=2)
        return idx.reshape(B), logits.reshape(B, -1)


# --------------------------------------------------------------------------------------
# ChatGLM2
# --------------------------------------------------------------------------------------
def make_chatglm2_state_dict(cfg, seed=0):
    """Random-init ChatGLM2-shaped checkpoint in the form the reference holds it after
    ChatGLM2DecModel.prepare_state_dict (poptransformer/models/chatglm2/model.py:256-274):
    `query_key_value` split into `query` / `key_value`, `dense_h_to_4h` into `_1` (gate) / `_2` (up).
    fp16 throughout: FP8 conversion happens when the Linear layers bind their weights
    (utils/param_handler/precision_strategy.py:44-51)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    d, f, v = cfg["hidden_size"], cfg["ffn_hidden_size"], cfg["padded_vocab_size"]
    kv = 2 * cfg["multi_query_group_num"] * cfg["kv_channels"]
    sd = {"transformer.embedding.word_embeddings.weight": _normal(rng, (v, d))}
    for i in range(cfg["num_layers"]):
        p = f"transformer.encoder.layers.{i}."
        sd[p + "input_layernorm.weight"] = np.ones(d, f16)
        sd[p + "self_attention.query.weight"] = _normal(rng, (d, d))
        sd[p + "self_attention.query.bias"] = _normal(rng, (d,))
        sd[p + "self_attention.key_value.weight"] = _normal(rng, (kv, d))
        sd[p + "self_attention.key_value.bias"] = _normal(rng, (kv,))
        sd[p + "self_attention.dense.weight"] = _normal(rng, (d, d))
        sd[p + "post_attention_layernorm.weight"] = np.ones(d, f16)
        sd[p + "mlp.dense_h_to_4h_1.weight"] = _normal(rng, (f, d))
        sd[p + "mlp.dense_h_to_4h_2.weight"] = _normal(rng, (f, d))
        sd[p + "mlp.dense_4h_to_h.weight"] = _normal(rng, (d, f))
    sd["transformer.encoder.final_layernorm.weight"] = np.ones(d, f16)
    sd["transformer.output_layer.weight"] = _normal(rng, (v, d))
    return sd


def fp8_weight_scale(w, fmt="F143"):
    """Power-of-two exponent s such that max|w| * 2^-s lands in (max/2, max] of the format: the
    "per-tensor scale bias chosen so max|w| maps near format max" of the FP8 benchmark
    configuration.  (The reference itself always uses -1, precision_strategy.py:46.)"""
    mx = 240.0 if fmt == "F143" else 57344.0
    m = float(np.abs(np.asarray(w, f32)).max())
    return int(np.ceil(np.log2(m / mx))) if m > 0 else 0


class _LinearFP8:
    """Linear under precision 'fp8' / 'fp8_weight' (utils/param_handler/precision_strategy.py:44-51,
    62-69,77-81): the [in, out] weight is converted to F143 bytes with exponent `scale`; with 'fp8'
    the activations are cast with the same scale tensor before the FP8 MatMul."""

    def __init__(self, sd, ctx, use_bias, precision, scale=-1):
        w = np.asarray(sd[ctx + ".weight"], f32).T               # [in, out]
        self.scale = np.array([scale], np.int32)
        self.w8 = O.f8_encode(w, "F143", scale)
        self.b = sd[ctx + ".bias"] if use_bias else None
        self.act_fp8 = precision == "fp8"

    def __call__(self, x):
        if self.act_fp8:
            x = O.f8_encode(x, "F143", int(self.scale[0]))
        y = O.fp8_matmul(x, self.w8, self.scale, self.scale, "F143", "F143")
        return (y + self.b).astype(f16) if self.b is not None else y


class ChatGLM2Oracle:
    """ChatGLM2DecModel.build_model_graph (poptransformer/models/chatglm2/model.py:296-341): embedding,
    blocks RMSNorm -> multi-query attention -> add -> RMSNorm -> SwiGLU MLP -> add (model.py:95-117),
    final RMSNorm, LMHead top-1.  precision: 'fp16', 'fp8' or 'fp8_weight'; `scales` maps a Linear
    context to its FP8 exponent (default -1 as in the reference)."""

    def __init__(self, sd, cfg, max_length, batch_size, precision="fp16", scales=None):
        self.cfg, self.L, self.B = cfg, max_length, batch_size
        self.d, self.H, self.G = cfg["hidden_size"], cfg["num_attention_heads"], cfg["multi_query_group_num"]
        self.D = self.d // self.H
        self.eps = cfg["layernorm_epsilon"]
        scales = scales or {}

        def lin(ctx, bias):
            if precision in ("fp8", "fp8_weight"):
                return _LinearFP8(sd, ctx, bias, precision, scales.get(ctx, -1))
            return _Linear(sd, ctx, bias)

        self.embed = sd["transformer.embedding.word_embeddings.weight"]
        self.layers = []
        for i in range(cfg["num_layers"]):
            p = f"transformer.encoder.layers.{i}."
            self.layers.append({
                "ln1": sd[p + "input_layernorm.weight"], "ln2": sd[p + "post_attention_layernorm.weight"],
                "query": lin(p + "self_attention.query", True), "key_value": lin(p + "self_attention.key_value", True),
                "dense": lin(p + "self_attention.dense", False),
                "gate": lin(p + "mlp.dense_h_to_4h_1", False), "up": lin(p + "mlp.dense_h_to_4h_2", False),
                "down": lin(p + "mlp.dense_4h_to_h", False), "cache": O.KVCache(max_length, 3, 1)})
        self.norm = sd["transformer.encoder.final_layernorm.weight"]
        self.head = lin("transformer.output_layer", False)

    def _attention(self, lay, x, step, mask4):
        """MultiQueryAttention.forward_qkv / forward_attention / forward_output
        (poptransformer/models/chatglm2/attention.py:166-302)."""
        return self._attention_from_projections(lay, lay["query"](x), lay["key_value"](x), step, mask4)

    def _attention_from_projections(self, lay, q, mixed, step, mask4):
        """The same from the outputs of the query and key_value Linears on."""
        B, H, G, D = self.B, self.H, self.G, self.D
        k, v = mixed[..., : G * D], mixed[..., G * D:]
        q = q.reshape(B, 1, H, D)
        k = k.reshape(B, 1, G, D)
        v = v.reshape(B, 1, G, D)
        cos, sin = O.glm2_sincos(step, D)
        q, k = O.glm2_rope(q, cos, sin), O.glm2_rope(k, cos, sin)
        q = q.transpose(0, 2, 1, 3)
        kv = np.concatenate([k, v], axis=0).reshape(2, B, 1, G, D).transpose(0, 1, 3, 2, 4)
        past = lay["cache"](step, kv)
        kk = np.repeat(past[0][:, :, None], H // G, axis=2).reshape(B, H, self.L, D)
        vv = np.repeat(past[1][:, :, None], H // G, axis=2).reshape(B, H, self.L, D)
        a = O.attention_scores_to_context(q, kk.transpose(0, 1, 3, 2), vv, mask4, 1 / np.sqrt(D), f16, False)
        a = a.transpose(0, 2, 1, 3).reshape(B, 1, H * D)
        return lay["dense"](a)

    def mlp_half(self, lay, x):
        """The second half of a GLMBlock: x + MLP(RMSNorm(x)) (models/chatglm2/model.py:110-117, mlp.py:51-59)."""
        t = O.rms_norm(x, lay["ln2"], self.eps).reshape(-1, self.d)
        g = O.swish(lay["gate"](t))
        u = (lay["up"](t) * g).astype(f16)
        return (x + lay["down"](u).reshape(self.B, -1, self.d)).astype(f16)

    def block(self, lay, x, step, mask4):
        """One GLMBlock (poptransformer/models/chatglm2/model.py:95-117) on the residual stream x [B, 1, d]."""
        t = O.rms_norm(x, lay["ln1"], self.eps)
        t = self._attention(lay, t, step, mask4)
        return self.mlp_half(lay, (x + t).astype(f16))

    def step(self, ids, step, mask):
        B = self.B
        x = self.embed[ids.reshape(B, 1)]
        mask4 = mask[:, None, None, :]
        for lay in self.layers:
            x = self.block(lay, x, step, mask4)
        x = O.rms_norm(x, self.norm, self.eps)
        logits = self.head(x)
        _, idx = O.topk1(logits, axis=2)
        return idx.reshape(B), logits.reshape(B, -1)


# --------------------------------------------------------------------------------------
# RWKV-4
# --------------------------------------------------------------------------------------
def make_rwkv_state_dict(cfg, seed=0, int4=True):
    """Random-init RWKV-4-shaped checkpoint in the form the reference holds it after
    RWKVDecodeModel.process_hf_model_state_dict (poptransformer/models/rwkv/model.py:150-155):
    `attention.output.weight` and `feed_forward.value.weight` of block i divided by
    2^(i // rescale_every).  Weights N(0, 0.02), time_decay U(-8, -1), time_first U(-1, 1),
    time_mix_* U(0, 1), LayerNorm gamma 1 / beta 0; Linear weights packed INT4 when `int4`.
    Keys: models/rwkv/model.py:34-42,81-94,129-148, attention.py:29-57, ffn.py:27-38, embedding.py:26-27."""
    rng = np.random.Generator(np.random.PCG64(seed))
    d, f, a, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["attention_hidden_size"], cfg["vocab_size"]
    sd = {"rwkv.embeddings.weight": _normal(rng, (v, d))}

    def linear(key, out_f, in_f, div=1.0):
        w = (rng.standard_normal((out_f, in_f), dtype=f32) * 0.02 / div).astype(f16)
        if int4:
            sd[key + ".weight"], sd[key + ".weight_scale"] = quantize_int4(w)
        else:
            sd[key + ".weight"] = w

    def ln(key):
        sd[key + ".weight"], sd[key + ".bias"] = np.ones(d, f16), np.zeros(d, f16)

    for i in range(cfg["num_hidden_layers"]):
        p = f"rwkv.blocks.{i}."
        div = 2.0 ** (i // cfg["rescale_every"]) if cfg["rescale_every"] > 0 else 1.0
        if i == 0:
            ln(p + "pre_ln")
        ln(p + "ln1")
        ln(p + "ln2")
        linear(p + "attention.key", a, d)
        linear(p + "attention.value", a, d)
        linear(p + "attention.receptance", a, d)
        linear(p + "attention.output", d, a, div)
        sd[p + "attention.time_decay"] = rng.uniform(-8, -1, d).astype(f16)
        sd[p + "attention.time_first"] = rng.uniform(-1, 1, d).astype(f16)
        for n in ("key", "value", "receptance"):
            sd[p + f"attention.time_mix_{n}"] = rng.uniform(0, 1, (1, 1, d)).astype(f16)
        linear(p + "feed_forward.key", f, d)
        linear(p + "feed_forward.receptance", d, d)
        linear(p + "feed_forward.value", d, f, div)
        for n in ("key", "receptance"):
            sd[p + f"feed_forward.time_mix_{n}"] = rng.uniform(0, 1, (1, 1, d)).astype(f16)
    ln("rwkv.ln_out")
    sd["head.weight"] = _normal(rng, (v, d))
    return sd


def _gate(a, w, b):
    """BaseRWKVAttention.gate (poptransformer/models/rwkv/attention.py:59-64): fp16 ops."""
    y1 = (a * w).astype(f16)
    y2 = (f16(1) - w).astype(f16)
    y2 = (y2 * b).astype(f16)
    return (y1 + y2).astype(f16)


class RWKVOracle:
    """RWKVDecodeModel.build_model_graph (poptransformer/models/rwkv/model.py:189-213), RWKVModel.__call__
    (:96-119), RWKVBlock (:44-53), BaseRWKVAttention (attention.py:66-105), BaseRWKVFeedforward
    (ffn.py:47-59).  States per block (model.py:157-187): two fp16 token-shift rows and the fp32
    numerator / denominator / maximum (-1e30).  The WKV arithmetic runs in fp32 as the reference does
    under precision 'fp16' (attention.py:78-82); the same is assumed for INT4 Linear weights, where
    the reference's `== 'fp16'` guard would leave fp16 operands next to fp32 states."""

    def __init__(self, sd, cfg, max_length, batch_size):
        self.cfg, self.L, self.B = cfg, max_length, batch_size
        self.d = cfg["hidden_size"]
        self.eps = cfg["layer_norm_epsilon"]
        self.rescale = cfg["rescale_every"]
        self.embed = sd["rwkv.embeddings.weight"]
        self.layers = []
        B, d = batch_size, self.d
        for i in range(cfg["num_hidden_layers"]):
            p = f"rwkv.blocks.{i}."
            lay = {n: (sd[p + n + ".weight"], sd[p + n + ".bias"]) for n in ("ln1", "ln2")}
            if i == 0:
                lay["pre_ln"] = (sd[p + "pre_ln.weight"], sd[p + "pre_ln.bias"])
            for n in ("key", "value", "receptance", "output"):
                lay["att_" + n] = _Linear(sd, p + "attention." + n, False)
            for n in ("key", "receptance", "value"):
                lay["ffn_" + n] = _Linear(sd, p + "feed_forward." + n, False)
            lay["time_decay"] = sd[p + "attention.time_decay"]
            lay["time_first"] = sd[p + "attention.time_first"]
            for n in ("key", "value", "receptance"):
                lay["att_mix_" + n] = sd[p + f"attention.time_mix_{n}"]
            for n in ("key", "receptance"):
                lay["ffn_mix_" + n] = sd[p + f"feed_forward.time_mix_{n}"]
            lay["state"] = [np.zeros((B, 1, d), f16), np.zeros((B, 1, d), f16), np.zeros((B, 1, d), f32),
                            np.zeros((B, 1, d), f32), np.full((B, 1, d), -1e30, f32)]
            self.layers.append(lay)
        self.ln_out = (sd["rwkv.ln_out.weight"], sd["rwkv.ln_out.bias"])
        self.head = _Linear(sd, "head", False)

    def _ln(self, x, wb):
        return O.layer_norm_ce(x, wb[0], wb[1], self.eps, self.B, 1, self.d)

    def _attention(self, lay, hidden):
        st = lay["state"]
        num, den, mx = st[2], st[3], st[4]
        key = _gate(hidden, lay["att_mix_key"], st[1])
        value = _gate(hidden, lay["att_mix_value"], st[1])
        rec = _gate(hidden, lay["att_mix_receptance"], st[1])
        st[1] = hidden
        key, value = lay["att_key"](key), lay["att_value"](value)
        rec = O.sigmoid(lay["att_receptance"](rec))
        td, k, v, tf = lay["time_decay"].astype(f32), key.astype(f32), value.astype(f32), lay["time_first"].astype(f32)
        t1 = (k + tf).astype(f32)
        m_out = np.where(mx > t1, mx, t1)
        with np.errstate(under="ignore"):
            e1, e2 = np.exp(mx - m_out, dtype=f32), np.exp(t1 - m_out, dtype=f32)
            out = ((e1 * num + e2 * v) / (e1 * den + e2)).astype(f32)
            t2 = (mx - np.exp(td, dtype=f32)).astype(f32)
            m_st = np.where(t2 > k, t2, k)
            e1, e2 = np.exp(t2 - m_st, dtype=f32), np.exp(k - m_st, dtype=f32)
        st[2] = (e1 * num + e2 * v).astype(f32)
        st[3] = (e1 * den + e2).astype(f32)
        st[4] = m_st.astype(f32)
        out = (rec * out.astype(f16)).astype(f16)
        return lay["att_output"](out)

    def _ffn(self, lay, hidden):
        st = lay["state"]
        key = _gate(hidden, lay["ffn_mix_key"], st[0])
        rec = _gate(hidden, lay["ffn_mix_receptance"], st[0])
        st[0] = hidden
        key = lay["ffn_key"](key)
        key = np.maximum(key, f16(0))
        key = (key * key).astype(f16)
        value = lay["ffn_value"](key)
        rec = O.sigmoid(lay["ffn_receptance"](rec))
        return (rec * value).astype(f16)

    def step(self, ids, step, mask=None):
        B = self.B
        hidden = self.embed[ids.reshape(B, 1)]
        for i, lay in enumerate(self.layers):
            if i == 0:
                hidden = self._ln(hidden, lay["pre_ln"])
            hidden = (hidden + self._attention(lay, self._ln(hidden, lay["ln1"]))).astype(f16)
            hidden = (hidden + self._ffn(lay, self._ln(hidden, lay["ln2"]))).astype(f16)
            if self.rescale > 0 and (i + 1) % self.rescale == 0:
                hidden = (hidden / f16(2)).astype(f16)
        hidden = self._ln(hidden, self.ln_out)
        logits = self.head(hidden)
        _, idx = O.topk1(logits, axis=2)
        return idx.reshape(B), logits.reshape(B, -1)
