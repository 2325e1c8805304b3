"""GPT-2 decoder (reference: poptransformer/models/gpt2/{model,attention,embedding}.py)."""
import numpy as np

from ... import ops
from ...layers import MLP, BaseLayer, Embedding, LayerNorm, Linear, LMHead
from ..base_model import HFDecBaseModel


class Attention(BaseLayer):
    """Fused c_attn projection with bias, no rotary embedding, scores without an in-graph 1/sqrt(D)
    (the query weights are pre-scaled at load), fp16 softmax (reference: gpt2/attention.py:19-90)."""
    softmax_fn_map = {"aionnx": ops.softmax, "ce": ops.softmax_ce}

    def __init__(self, context, name, input_size, num_head, cache_max_length):
        super().__init__(context, name)
        self.input_size, self.num_head, self.cache_max_length = input_size, num_head, cache_max_length
        self.head_size = input_size // num_head
        self.c_attn = Linear(self.context, "c_attn", input_size, input_size * 3)
        self.c_proj = Linear(self.context, "c_proj", input_size, input_size)

    def forward_qkv(self, graph, x, step):
        B, S, H, D, d = self.batch_size, self.sequence_length, self.num_head, self.head_size, self.input_size
        q, kv = ops.split(graph, self.c_attn(graph, x), num_outputs=2, axis=2, splits=[d, 2 * d])
        q = ops.transpose(graph, ops.reshape(graph, q, [B, S, H, D]), [0, 2, 1, 3])
        kv = ops.transpose(graph, ops.reshape(graph, kv, [B, S, 2, H, D]), [2, 0, 3, 1, 4])
        past = ops.remap_tensor(graph, ops.kv_cache(graph, step, kv, self.cache_max_length, 3, S))
        if S != 1 and S < self.cache_max_length:
            past = ops.static_slice(graph, past, [0], [S], [3])
        k, v = ops.split(graph, past, 2, axis=0, splits=[1, 1], name="split_past")
        return q, ops.squeeze(graph, k, [0]), ops.squeeze(graph, v, [0])

    def forward_attention(self, graph, q, k, attention_mask, softmax_type):
        score = ops.matmul(graph, q, ops.transpose(graph, k, [0, 1, 3, 2]))
        if self.sequence_length != 1:
            score = ops.remap_tensor(graph, score, fwd_after_matmul=True)
        fn = self.softmax_fn_map.get(softmax_type)
        if fn is None:
            raise ValueError(f"Invalid softmax_fn {softmax_type}, options: {self.softmax_fn_map.keys()}")
        return fn(graph, ops.add(graph, score, attention_mask), -1, stable_mode=self.sequence_length != 1)

    def forward_output(self, graph, score, v):
        a = ops.transpose(graph, ops.matmul(graph, score, v), [0, 2, 1, 3])
        return self.c_proj(graph, ops.reshape(graph, a, [self.batch_size, self.sequence_length, self.input_size]))

    def __call__(self, graph, x, step, attention_mask, sequence_length, softmax_type="ce"):
        with graph.nameScope(self.context):
            self.sequence_length = sequence_length
            q, k, v = self.forward_qkv(graph, x, step)
            return self.forward_output(graph, self.forward_attention(graph, q, k, attention_mask, softmax_type), v)


class TransformerEmbedding(BaseLayer):
    """wte[id] + wpe[position] (reference: gpt2/embedding.py:19-36)."""

    def __init__(self, context, name, vocab_size, embd_size, max_position):
        super().__init__(context, name)
        self.wte = Embedding(self.context, "wte", vocab_size, embd_size)
        self.wpe = Embedding(self.context, "wpe", max_position, embd_size)

    def __call__(self, graph, input_ids, position_ids, sequence_length):
        with graph.nameScope(self.context):
            e = ops.add(graph, self.wte(graph, input_ids, sequence_length), self.wpe(graph, position_ids, sequence_length))
        return ops.remap_tensor(graph, e)


class TransformerBlock(BaseLayer):
    def __init__(self, context, name, input_size, eps, n_head, max_length):
        super().__init__(context, name)
        self.layer_norm1 = LayerNorm(self.context, "ln_1", input_size, eps)
        self.attention = Attention(self.context, "attn", input_size, n_head, max_length)
        self.layer_norm2 = LayerNorm(self.context, "ln_2", input_size, eps)
        self.mlp = MLP(self.context, "mlp", input_size, input_size * 4, "gelu")

    def __call__(self, graph, x, sequence_length, step, attention_mask, norm_type="ce", softmax_type="ce", **kwargs):
        with graph.nameScope(self.context):
            t = self.layer_norm1(graph, x, sequence_length, norm_type)
            x = ops.add(graph, x, self.attention(graph, t, step, attention_mask, sequence_length, softmax_type))
            return ops.add(graph, x, self.mlp(graph, self.layer_norm2(graph, x, sequence_length, norm_type)))


class Transformer(BaseLayer):
    def __init__(self, context, name, vocab_size, embd_size, eps, n_head, max_length, n_layer, layer_per_ipu, max_position):
        super().__init__(context, name)
        self.n_layer, self.layer_per_ipu = n_layer, layer_per_ipu
        self.embedding = TransformerEmbedding(self.context, None, vocab_size, embd_size, max_position)
        self.blocks = [TransformerBlock(self.context, f"h.{i}", embd_size, eps, n_head, max_length) for i in range(n_layer)]
        self.layer_norm = LayerNorm(self.context, "ln_f", embd_size, eps)

    def __call__(self, graph, input_ids, position_ids, step, attention_mask, sequence_length, **kwargs):
        norm_type, softmax_type = kwargs.get("norm_type", "ce"), kwargs.get("softmax_type", "ce")
        with self.device_scope(graph, 0, 0):
            h = self.embedding(graph, input_ids, position_ids, sequence_length)
        ends = np.cumsum(self.layer_per_ipu) if len(self.layer_per_ipu) else np.array([])
        stage = 0
        for i, block in enumerate(self.blocks):
            stage = int(sum(i >= ends))
            with self.device_scope(graph, stage, stage):
                h = block(graph, h, sequence_length, step, attention_mask, norm_type, softmax_type)
        with self.device_scope(graph, stage, stage):
            return self.layer_norm(graph, h, sequence_length, norm_type), stage


class GPT2DecModel(HFDecBaseModel):
    """reference: gpt2/model.py:123-229.  hf_config fields: vocab_size, n_embd, layer_norm_epsilon, n_head,
    n_layer, n_positions.  The state dict is expected as Hugging Face holds it (Conv1D weights [in, out],
    unscaled queries) unless `state_dict_is_processed`; process_hf_model_state_dict applies the
    reference's rewrite (model.py:154-166): transpose to [out, in] and pre-multiply the query third
    of c_attn by 1/sqrt(head_dim)."""

    def __init__(self, **kwargs):
        self.state_dict_is_processed = kwargs.get("state_dict_is_processed", False)
        super().__init__(**kwargs)
        c = self.hf_config
        self.topk = kwargs.get("topk", 1)
        self.outline_blocks = kwargs.get("outline_blocks", True)
        self.transformer = Transformer(None, "transformer", c.vocab_size, c.n_embd, c.layer_norm_epsilon, c.n_head,
                                       self.max_length, c.n_layer, self.layer_per_ipu, c.n_positions)
        self.lm_head = LMHead(None, "lm_head", self.topk, c.vocab_size, c.n_embd,
                              tie_weight=self.transformer.embedding.wte.weight_id)
        self.lm_head.set_virtual_id(0)

    def process_hf_model_state_dict(self):
        if self.state_dict_is_processed or not self.state_dict:
            return
        c = self.hf_config
        d = c.n_embd
        scale = np.float32(1 / (d // c.n_head) ** 0.5)
        for key in list(self.state_dict):
            w = np.asarray(self.state_dict[key])
            if key.endswith("attn.c_attn.weight"):
                w = w.astype(np.float32).copy()
                w[:, :d] *= scale
                self.state_dict[key] = np.ascontiguousarray(w.T).astype(np.float16 if self.precision != "fp32" else np.float32)
            elif key.endswith("attn.c_attn.bias"):
                w = w.astype(np.float32).copy()
                w[:d] *= scale
                self.state_dict[key] = w.astype(np.float16 if self.precision != "fp32" else np.float32)
            elif key.endswith(("attn.c_proj.weight", "mlp.c_fc.weight", "mlp.c_proj.weight")):
                self.state_dict[key] = np.ascontiguousarray(w.T)

    def build_model_graph(self, model_graph, model_graph_inputs, sequence_length=1):
        g = model_graph
        step = model_graph_inputs["step"]
        with self.device_scope(g, 0, 0):
            input_ids = ops.dynamic_slice(g, model_graph_inputs["input_ids_container"], step, axes=[1], sizes=[sequence_length])
            mask = ops.unsqueeze(g, model_graph_inputs["attention_mask"], [1, 2])
            position_ids = ops.unsqueeze(g, step, [0])
        hidden, stage = self.transformer(g, input_ids, position_ids, step, mask, sequence_length=sequence_length,
                                         outline_blocks=self.outline_blocks)
        with self.device_scope(g, pipeline_stage_id=stage):
            next_ids = self.lm_head(g, hidden, sequence_length=sequence_length)
        return {"next_ids": next_ids, "stage_offset": stage}
