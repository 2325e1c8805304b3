"""ChatGLM2 decoder (reference: poptransformer/models/chatglm2/{model,attention,mlp,emebdding}.py)."""
import math

import numpy as np

from ... import ops
from ...layers import BaseLayer, Embedding, Linear, LMHead, RMSLayerNorm
from ...utils import REGISTRY
from ..base_model import HFDecBaseModel


class MultiQueryAttention(BaseLayer):
    """`query` and `key_value` projections with bias, `multi_query_group_num` cache heads shared by
    groups of query heads, rotary embedding of interleaved pairs on the first half of each head,
    fp16 softmax (reference: chatglm2/attention.py:29-302)."""
    softmax_fn_map = {"aionnx": ops.softmax, "ce": ops.softmax_ce}

    def __init__(self, context, name, hidden_size, multi_query_group_num, num_attention_heads, cache_max_length,
                 layer_number, add_qkv_bias=True):
        super().__init__(context, name)
        self.hidden_size, self.groups, self.num_heads = hidden_size, multi_query_group_num, num_attention_heads
        self.head_size = hidden_size // num_attention_heads
        self.cache_max_length, self.layer_number = cache_max_length, layer_number
        self.input_length = 1
        self.rotary_dim = self.head_size
        self.norm_factor = math.sqrt(self.head_size)
        self.query = Linear(self.context, "query", hidden_size, hidden_size, use_bias=add_qkv_bias)
        self.key_value = Linear(self.context, "key_value", hidden_size, 2 * self.head_size * self.groups, use_bias=add_qkv_bias)
        self.dense = Linear(self.context, "dense", hidden_size, hidden_size, use_bias=False)

    def fixed_pos_embedding(self, graph, position_id, dim):
        """cos/sin of position * inv_freq: the angle is an fp32 product, cast to the activation type
        before cos/sin (attention.py:77-96)."""
        inv_freq = np.array([1.0 / (10000 ** (i / dim)) for i in range(0, dim, 2)]).astype(np.float32)
        inv_freq = ops.reshape(graph, ops.constant(graph, inv_freq, "inv_freq"), [1, -1])
        pos = ops.cast(graph, ops.reshape(graph, position_id, [-1, 1]), "FLOAT")
        freqs = ops.matmul(graph, pos, inv_freq)
        emb = ops.reshape(graph, ops.concat(graph, freqs, freqs, axis=-1), shape=[1, -1, 1, dim])
        emb = ops.cast(graph, emb, self.popart_float_type)
        return graph.aiOnnx.cos([emb]), graph.aiOnnx.sin([emb])

    def rotate_half(self, graph, x):
        quarter = self.rotary_dim // 4
        a, b = ops.split(graph, x, num_outputs=2, axis=-1, splits=[quarter, quarter], name="rope_split")
        b = ops.mul(graph, b, ops.constant(graph, np.array([-1]).astype(self.np_float_type)))
        return ops.concat(graph, b, a, axis=-1)

    def apply_rotary_pos_emb(self, graph, x, cos_sin, num_heads):
        """De-interleave the pairs, rotate-half, re-interleave (attention.py:110-132)."""
        cos, sin = cos_sin
        B, S = self.batch_size, self.input_length
        x = ops.reshape(graph, x, shape=[B, S, num_heads, -1, 2])
        x = ops.reshape(graph, ops.transpose(graph, x, perm=[0, 1, 2, 4, 3]), shape=[B, S, num_heads, -1])
        x = ops.add(graph, ops.mul(graph, x, cos), ops.mul(graph, self.rotate_half(graph, x), sin))
        x = ops.reshape(graph, x, shape=[B, S, num_heads, 2, -1])
        return ops.reshape(graph, ops.transpose(graph, x, perm=[0, 1, 2, 4, 3]), shape=[B, S, num_heads, -1])

    def rotary_embedding(self, graph, q, k, position_ids):
        half = self.rotary_dim // 2
        with graph.nameScope("build_rotary"):
            cos_sin = self.fixed_pos_embedding(graph, position_ids, dim=half)
            q1, q2 = ops.split(graph, q, num_outputs=2, axis=-1, splits=[half, half], name="rope_split_q")
            k1, k2 = ops.split(graph, k, num_outputs=2, axis=-1, splits=[half, half], name="rope_split_k")
        with graph.nameScope("apply_rotary"):
            q1 = self.apply_rotary_pos_emb(graph, q1, cos_sin, self.num_heads)
            k1 = self.apply_rotary_pos_emb(graph, k1, cos_sin, self.groups)
            return ops.concat(graph, q1, q2, axis=-1), ops.concat(graph, k1, k2, axis=-1)

    def forward_qkv(self, graph, x, step):
        B, S, H, G, D, L = self.batch_size, self.sequence_length, self.num_heads, self.groups, self.head_size, self.cache_max_length
        q = self.query(graph, x)
        k, v = ops.split(graph, self.key_value(graph, x), num_outputs=2, axis=-1, splits=[G * D, G * D])
        q = ops.reshape(graph, q, shape=[B, S, H, D])
        k = ops.reshape(graph, k, shape=[B, S, G, D])
        v = ops.reshape(graph, v, shape=[B, S, G, D])
        q, k = self.rotary_embedding(graph, q, k, position_ids=step)
        q = ops.transpose(graph, q, perm=[0, 2, 1, 3])
        kv = ops.reshape(graph, ops.concat(graph, k, v, 0), [2, B, S, G, D])
        kv = ops.transpose(graph, kv, perm=[0, 1, 3, 2, 4])
        with graph.nameScope("attn_past_update"):
            past = ops.kv_cache(graph, step, kv, L, 3, S)
            k, v = ops.split(graph, past, 2, axis=0, splits=[1, 1], name="split_past")

            def share(t):     # [B, G, L, D] -> [B, H, L, D]: each cache head serves H // G query heads
                t = ops.unsqueeze(graph, ops.squeeze(graph, t, [0]), [2])
                t = ops.expand(graph, t, [1, 1, H // G, 1, 1])
                return ops.reshape(graph, t, shape=[B, H, L, D])
            k, v = share(k), share(v)
            k = ops.transpose(graph, k, [0, 1, 3, 2])
        return q, k, v

    def forward_attention(self, graph, q, k, attention_mask, softmax_type):
        scores = ops.matmul(graph, q, k)
        scores = ops.mul(graph, scores, ops.constant(graph, np.array([1.0 / self.norm_factor]).astype(self.np_float_type)))
        scores = ops.add(graph, scores, attention_mask)
        fn = self.softmax_fn_map.get(softmax_type)
        if fn is None:
            raise ValueError(f"Invalid softmax_fn {softmax_type}, options: {self.softmax_fn_map.keys()}")
        return ops.cast(graph, fn(graph, scores, -1, stable_mode=self.sequence_length != 1), self.popart_float_type)

    def forward_output(self, graph, score, v):
        c = ops.transpose(graph, ops.matmul(graph, score, v), [0, 2, 1, 3])
        return self.dense(graph, ops.reshape(graph, c, [self.batch_size, self.sequence_length, -1]))

    def __call__(self, graph, x, step, attention_mask, sequence_length, softmax_type="ce"):
        with graph.nameScope(self.context):
            self.sequence_length = sequence_length
            q, k, v = self.forward_qkv(graph, x, step)
            return self.forward_output(graph, self.forward_attention(graph, q, k, attention_mask, softmax_type), v)


class MLP(BaseLayer):
    """4h_to_h(h_to_4h_2(x) * swish(h_to_4h_1(x))) (reference: chatglm2/mlp.py:20-59)."""

    def __init__(self, context, name, hidden_size, ffn_hidden_size):
        super().__init__(context, name)
        self.hidden_size = hidden_size
        self.gate_proj = Linear(self.context, "dense_h_to_4h_1", hidden_size, ffn_hidden_size, use_bias=False)
        self.up_proj = Linear(self.context, "dense_h_to_4h_2", hidden_size, ffn_hidden_size, use_bias=False)
        self.down_proj = Linear(self.context, "dense_4h_to_h", ffn_hidden_size, hidden_size, use_bias=False)

    def __call__(self, graph, x):
        x = ops.reshape(graph, x, [-1, self.hidden_size])
        gate = ops.swish(graph, self.gate_proj(graph, x))
        y = self.down_proj(graph, ops.mul(graph, self.up_proj(graph, x), gate))
        return ops.reshape(graph, y, [self.batch_size, -1, self.hidden_size])


class ChatGLM2Block(BaseLayer):
    def __init__(self, context, name, hidden_size, layernorm_epsilon, multi_query_group_num, num_attention_heads,
                 ffn_hidden_size, max_length, layer_number):
        super().__init__(context, name)
        self.layer_norm1 = RMSLayerNorm(self.context, "input_layernorm", hidden_size, layernorm_epsilon)
        self.attention = MultiQueryAttention(self.context, "self_attention", hidden_size, multi_query_group_num,
                                             num_attention_heads, max_length, layer_number)
        self.layer_norm2 = RMSLayerNorm(self.context, "post_attention_layernorm", hidden_size, layernorm_epsilon)
        self.mlp = MLP(self.context, "mlp", hidden_size, ffn_hidden_size)

    def __call__(self, graph, x, sequence_length, step, attention_mask, softmax_type="ce", **kwargs):
        # the reference asks for half-precision partials in both sub-layers (model.py:106-116)
        matmul_kwargs = {"amp": 0.4, "partialtype": "half"}
        with graph.nameScope(self.context):
            t = self.layer_norm1(graph, x)
            with self.option_scope(**matmul_kwargs):
                t = self.attention(graph, t, step, attention_mask, sequence_length, softmax_type)
            x = ops.add(graph, x, t)
            t = self.layer_norm2(graph, x)
            with self.option_scope(**matmul_kwargs):
                t = self.mlp(graph, t)
            return ops.add(graph, x, t)


class Transformer(BaseLayer):
    def __init__(self, context, name, padded_vocab_size, num_embedding_partitions, hidden_size, layernorm_epsilon,
                 multi_query_group_num, num_attention_heads, ffn_hidden_size, max_length, num_layers, layer_per_ipu):
        super().__init__(context, name)
        self.num_layers, self.layer_per_ipu = num_layers, layer_per_ipu
        self.embedding = Embedding(".".join([self.context, "embedding"]), "word_embeddings", padded_vocab_size, hidden_size)
        self.blocks = [ChatGLM2Block(".".join([self.context, "encoder"]), f"layers.{i}", hidden_size, layernorm_epsilon,
                                     multi_query_group_num, num_attention_heads, ffn_hidden_size, max_length, i)
                       for i in range(num_layers)]
        self.layer_norm = RMSLayerNorm(".".join([self.context, "encoder"]), "final_layernorm", hidden_size, layernorm_epsilon)

    def __call__(self, graph, input_ids, position_ids, step, attention_mask, sequence_length, **kwargs):
        softmax_type = kwargs.get("softmax_type", "ce")
        with self.device_scope(graph, 0, 0):
            h = self.embedding(graph, input_ids, sequence_length)
        for block in self.blocks:
            h = block(graph, h, sequence_length, step, attention_mask, softmax_type)
        return self.layer_norm(graph, h)


class ChatGLM2DecModel(HFDecBaseModel):
    """reference: chatglm2/model.py:211-359.  hf_config fields: padded_vocab_size, hidden_size,
    layernorm_epsilon, multi_query_group_num, num_attention_heads, ffn_hidden_size, num_layers, kv_channels.
    A state dict with the Hugging Face `query_key_value` / `dense_h_to_4h` tensors is split at load
    like the reference does (model.py:256-274); already split keys pass through."""

    def __init__(self, **kwargs):
        super().__init__(**kwargs)
        c = self.hf_config
        self.outline_blocks = kwargs.get("outline_blocks", False)
        self.num_embedding_partitions = kwargs.get("num_embedding_partitions", 1)
        self.transformer = Transformer(None, "transformer", c.padded_vocab_size, self.num_embedding_partitions, c.hidden_size,
                                       c.layernorm_epsilon, c.multi_query_group_num, c.num_attention_heads,
                                       c.ffn_hidden_size, self.max_length, c.num_layers, self.layer_per_ipu)
        self.lm_head = LMHead(None, "transformer.output_layer", 1, c.padded_vocab_size, c.hidden_size)

    def process_hf_model_state_dict(self):
        c = self.hf_config
        for key in list(self.state_dict):
            if "query_key_value" in key:
                w = np.asarray(self.state_dict.pop(key))
                self.state_dict[key.replace("query_key_value", "query")] = w[: c.hidden_size]
                self.state_dict[key.replace("query_key_value", "key_value")] = w[c.hidden_size:]
            elif "dense_h_to_4h" in key and not key.split("dense_h_to_4h")[1].startswith("_"):
                w = np.asarray(self.state_dict.pop(key))
                half = w.shape[0] // 2
                self.state_dict[key.replace("dense_h_to_4h", "dense_h_to_4h_1")] = w[:half]
                self.state_dict[key.replace("dense_h_to_4h", "dense_h_to_4h_2")] = w[half:]
        REGISTRY.update("query_size", c.hidden_size)
        REGISTRY.update("key_value_size", c.multi_query_group_num * c.kv_channels)

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
        return {"next_ids": next_ids, "stage_offset": self.transformer.num_layers + 1}
