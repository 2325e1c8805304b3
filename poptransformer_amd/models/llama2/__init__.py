"""Llama 2 decoder (reference: poptransformer/models/llama2/{model,attention,mlp,embedding}.py)."""
import math

import numpy as np

from ... import ops
from ...layers import BaseLayer, Embedding, Linear, LMHead, RMSLayerNorm
from ..base_model import HFDecBaseModel


class Attention(BaseLayer):
    """Separate q/k/v/o projections without bias, rotary embedding from `step`, KV cache on axis 3,
    fp32 softmax (reference: llama2/attention.py:19-114)."""
    softmax_fn_map = {"aionnx": ops.softmax, "ce": ops.softmax_ce}

    def __init__(self, context, name, input_size, num_head, cache_max_length, fp8_cache=False):
        super().__init__(context, name)
        self.input_size, self.num_head, self.cache_max_length = input_size, num_head, cache_max_length
        self.head_size = input_size // num_head
        self.fp8_cache = fp8_cache
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        d = self.input_size
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = (
            Linear(self.context, n, d, d, use_bias=False) for n in ("q_proj", "k_proj", "v_proj", "o_proj"))

    def fixed_pos_embedding(self, graph, step, head_dim):
        """sin/cos of step * inv_freq, everything in the activation type (attention.py:28-38)."""
        inv_freq = np.array([1.0 / (10000 ** (i / head_dim)) for i in range(0, head_dim, 2)]).astype(self.np_float_type)
        inv_freq = ops.reshape(graph, ops.constant(graph, inv_freq, "inv_freq"), [1, -1])
        pos = ops.cast(graph, ops.reshape(graph, step, [-1, 1]), self.popart_float_type)
        angle = ops.matmul(graph, pos, inv_freq)
        return graph.aiOnnx.sin([angle]), graph.aiOnnx.cos([angle])

    def rotate_half(self, graph, x, n_head, head_dim, batch_size=1):
        lo, hi = ops.split(graph, x, 2, 3, [head_dim // 2, head_dim // 2], "split_rotate_every_two")
        hi = ops.mul(graph, hi, ops.constant(graph, np.array([-1]).astype(self.np_float_type)))
        return ops.reshape(graph, ops.concat(graph, hi, lo, 3), [batch_size, n_head, 1, head_dim])

    def apply_rotary_pos_emb(self, graph, q, k, sincos, n_head, head_dim, batch_size=1):
        sin = ops.reshape(graph, ops.concat(graph, sincos[0], sincos[0], 1), [1, 1, 1, -1])
        cos = ops.reshape(graph, ops.concat(graph, sincos[1], sincos[1], 1), [1, 1, 1, -1])

        def rotate(t):
            return ops.add(graph, ops.mul(graph, t, cos), ops.mul(graph, self.rotate_half(graph, t, n_head, head_dim, batch_size), sin))
        return rotate(q), rotate(k)

    def forward_qkv(self, graph, x, step):
        B, S, H, D = self.batch_size, self.sequence_length, self.num_head, self.head_size

        def heads(t):
            return ops.transpose(graph, ops.reshape(graph, t, [B, S, H, D]), [0, 2, 1, 3])
        q, k, v = heads(self.q_proj(graph, x)), heads(self.k_proj(graph, x)), heads(self.v_proj(graph, x))
        q, k = self.apply_rotary_pos_emb(graph, q, k, self.fixed_pos_embedding(graph, step, D), H, D, B)
        kv = ops.reshape(graph, ops.concat(graph, k, v, 0), [2, B, H, S, D])
        with graph.nameScope("attn_past_update"):
            past = ops.kv_cache(graph, step, kv, self.cache_max_length, 3, S)
            past_k, past_v = ops.split(graph, past, 2, axis=0, splits=[1, 1], name="split_past")
            past_k = ops.transpose(graph, ops.squeeze(graph, past_k, [0]), [0, 1, 3, 2])
            past_v = ops.squeeze(graph, past_v, [0])
        return q, past_k, past_v

    def forward_attention(self, graph, q, k, attention_mask, softmax_type):
        w = ops.matmul(graph, q, k)
        w = ops.mul(graph, w, ops.constant(graph, np.array([1 / math.sqrt(self.head_size)]).astype(self.np_float_type)))
        w = ops.cast(graph, ops.add(graph, w, attention_mask), "FLOAT")
        fn = self.softmax_fn_map.get(softmax_type)
        if fn is None:
            raise ValueError(f"Invalid softmax_fn {softmax_type}, options: {self.softmax_fn_map.keys()}")
        return ops.cast(graph, fn(graph, w, -1, stable_mode=self.sequence_length != 1), self.popart_float_type)

    def forward_output(self, graph, score, v):
        a = ops.transpose(graph, ops.matmul(graph, score, v), [0, 2, 1, 3])
        return self.o_proj(graph, ops.reshape(graph, a, [self.batch_size, self.sequence_length, -1]))

    def __call__(self, graph, x, step, attention_mask, sequence_length, softmax_type="ce"):
        with graph.nameScope(self.context):
            self.sequence_length = sequence_length
            q, k, v = self.forward_qkv(graph, x, step)
            return self.forward_output(graph, self.forward_attention(graph, q, k, attention_mask, softmax_type), v)


class MLP(BaseLayer):
    """down(up(x) * swish(gate(x))) (reference: llama2/mlp.py:12-28)."""
    act_fn_map = {"gelu": ops.gelu, "swish": ops.swish}

    def __init__(self, context, name, input_size, hidden_size, act_fn):
        super().__init__(context, name)
        self.input_size, self.hidden_size = input_size, hidden_size
        self.act_fn = self.act_fn_map.get(act_fn)
        if self.act_fn is None:
            raise ValueError(f"Invalid act_fn {act_fn}, options: {self.act_fn_map.keys()}")
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        self.gate_proj = Linear(self.context, "gate_proj", self.input_size, self.hidden_size, use_bias=False)
        self.up_proj = Linear(self.context, "up_proj", self.input_size, self.hidden_size, use_bias=False)
        self.down_proj = Linear(self.context, "down_proj", self.hidden_size, self.input_size, use_bias=False)

    def __call__(self, graph, x):
        x = ops.reshape(graph, x, [-1, self.input_size])
        gate = self.act_fn(graph, self.gate_proj(graph, x))
        y = self.down_proj(graph, ops.mul(graph, self.up_proj(graph, x), gate))
        return ops.reshape(graph, y, [self.batch_size, -1, self.input_size])


class TransformerBlock(BaseLayer):
    def __init__(self, context, name, input_size, eps, n_head, intermediate_size, max_length, fp8_cache=False):
        super().__init__(context, name)
        self.layer_norm1 = RMSLayerNorm(self.context, "input_layernorm", input_size, eps)
        self.attention = Attention(self.context, "self_attn", input_size, n_head, max_length, fp8_cache)
        self.layer_norm2 = RMSLayerNorm(self.context, "post_attention_layernorm", input_size, eps)
        self.mlp = MLP(self.context, "mlp", input_size, intermediate_size, "swish")

    def __call__(self, graph, x, sequence_length, step, attention_mask, norm_type="ce", softmax_type="ce", **kwargs):
        with graph.nameScope(self.context):
            x = ops.add(graph, x, self.attention(graph, self.layer_norm1(graph, x), step, attention_mask, sequence_length, softmax_type))
            return ops.add(graph, x, self.mlp(graph, self.layer_norm2(graph, x)))


class Transformer(BaseLayer):
    def __init__(self, context, name, vocab_size, embd_size, eps, n_head, intermediate_size, max_length, n_layer,
                 layer_per_ipu, fp8_cache=False):
        super().__init__(context, name)
        self.n_layer, self.layer_per_ipu = n_layer, layer_per_ipu
        self.embedding = Embedding(self.context, "embed_tokens", vocab_size, embd_size)
        self.blocks = [TransformerBlock(self.context, f"layers.{i}", embd_size, eps, n_head, intermediate_size, max_length,
                                        fp8_cache) for i in range(n_layer)]
        self.layer_norm = RMSLayerNorm(self.context, "norm", embd_size, eps)

    def __call__(self, graph, input_ids, position_ids, step, attention_mask, sequence_length, **kwargs):
        norm_type, softmax_type = kwargs.get("norm_type", "ce"), kwargs.get("softmax_type", "ce")
        with self.device_scope(graph, 0, 0):
            h = self.embedding(graph, input_ids, sequence_length)
        ends = np.cumsum(self.layer_per_ipu) if len(self.layer_per_ipu) else np.array([])
        stage = 0
        for i, block in enumerate(self.blocks):
            stage = int(sum(i >= ends))
            with self.device_scope(graph, stage, stage):
                h = block(graph, h, sequence_length, step, attention_mask, norm_type, softmax_type)
        with self.device_scope(graph, stage, stage):
            return self.layer_norm(graph, h)


class LLAMA2DecModel(HFDecBaseModel):
    """reference: llama2/model.py:112-230.  hf_config fields: vocab_size, hidden_size, rms_norm_eps,
    num_attention_heads, intermediate_size, num_hidden_layers."""

    def __init__(self, **kwargs):
        super().__init__(**kwargs)
        c = self.hf_config
        self.fp8_cache, self.topk = kwargs.get("fp8_cache", False), kwargs.get("topk", 1)
        self.outline_blocks = kwargs.get("outline_blocks", False)
        self.transformer = Transformer(None, "model", c.vocab_size, c.hidden_size, c.rms_norm_eps, c.num_attention_heads,
                                       c.intermediate_size, self.max_length, c.num_hidden_layers, self.layer_per_ipu,
                                       self.fp8_cache)
        self.lm_head = LMHead(None, "lm_head", self.topk, c.vocab_size, c.hidden_size)

    def build_model_graph(self, model_graph, model_graph_inputs, sequence_length=1):
        g = model_graph
        step = model_graph_inputs["step"]
        with self.device_scope(g, 0, 0):
            input_ids = ops.dynamic_slice(g, model_graph_inputs["input_ids_container"], step, axes=[1], sizes=[sequence_length])
            mask = ops.unsqueeze(g, model_graph_inputs["attention_mask"], [1, 2])
            position_ids = ops.unsqueeze(g, step, [0])
        hidden = self.transformer(g, input_ids, position_ids, step, mask, sequence_length=sequence_length,
                                  outline_blocks=self.outline_blocks)
        last = max(len(self.layer_per_ipu) - 1, 0)
        with self.device_scope(g, last, last):
            self.lm_head.set_virtual_id(last)
            next_ids = self.lm_head(g, hidden, sequence_length=sequence_length)
        return {"next_ids": next_ids, "stage_offset": len(self.layer_per_ipu)}
