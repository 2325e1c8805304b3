"""RWKV-4 decoder (reference: poptransformer/models/rwkv/{model,attention,ffn,embedding}.py)."""
import numpy as np

from ... import ops
from ...layers import BaseLayer, Embedding, LayerNorm, Linear, LMHead
from ..base_model import HFDecBaseModel


def _token_shift(layer, graph, x, w, prev):
    """x * w + (1 - w) * prev in the activation type (reference: `gate`, rwkv/attention.py:59-64)."""
    one = ops.constant(graph, np.array(1).astype(layer.np_float_type))
    return ops.add(graph, ops.mul(graph, x, w), ops.mul(graph, ops.sub(graph, one, w), prev))


class RWKVAttention(BaseLayer):
    """Time mixing with the numerically stable WKV recurrence (reference: rwkv/attention.py:21-105)."""

    def __init__(self, context, name, hidden_size, attention_hidden_size, layer_id):
        super().__init__(context, name)
        self.hidden_size, self.attention_hidden_size, self.layer_id = hidden_size, attention_hidden_size, layer_id
        self.key_linear = Linear(self.context, "key", hidden_size, attention_hidden_size, use_bias=False)
        self.receptance_linear = Linear(self.context, "receptance", hidden_size, attention_hidden_size, use_bias=False)
        self.value_linear = Linear(self.context, "value", hidden_size, attention_hidden_size, use_bias=False)
        self.output_linear = Linear(self.context, "output", attention_hidden_size, hidden_size, use_bias=False)
        self.time_decay = self._vector("time_decay", [hidden_size])
        self.time_first = self._vector("time_first", [hidden_size])
        self.time_mix_key = self._vector("time_mix_key", [1, 1, hidden_size])
        self.time_mix_value = self._vector("time_mix_value", [1, 1, hidden_size])
        self.time_mix_receptance = self._vector("time_mix_receptance", [1, 1, hidden_size])

    def _vector(self, name, shape):
        key = f"{self.context}.{name}"
        return self.add_initialized_input_tensor(self.get_param_from_state_dict(key, shape), key)

    def __call__(self, graph, hidden, layer_state):
        g = graph
        with g.nameScope("extract_key_value"):
            num, den, mx = layer_state[2:]
            key = self.key_linear(g, _token_shift(self, g, hidden, self.time_mix_key, layer_state[1]))
            value = self.value_linear(g, _token_shift(self, g, hidden, self.time_mix_value, layer_state[1]))
            rec = self.receptance_linear(g, _token_shift(self, g, hidden, self.time_mix_receptance, layer_state[1]))
            rec = ops.sigmoid(g, rec)
            layer_state[1] = hidden
        # The recurrence runs in fp32.  The reference casts under precision 'fp16' only
        # (attention.py:78-82,101); its states are fp32 in every precision (model.py:157-187), so the
        # INT4 / FP8 modes, whose activations are fp16 too, are given the same casts here.
        half = self.popart_float_type == "FLOAT16"
        time_decay, time_first = self.time_decay, self.time_first
        if half:
            time_decay, key, value, time_first = (ops.cast(g, t, "FLOAT") for t in (time_decay, key, value, time_first))
        with g.nameScope("rwkv_linear_attention"):
            t1 = ops.add(g, key, time_first)
            m = ops.maximum(g, mx, t1)
            e1, e2 = ops.exp(g, ops.sub(g, mx, m)), ops.exp(g, ops.sub(g, t1, m))
            out = ops.div(g, ops.add(g, ops.mul(g, e1, num), ops.mul(g, e2, value)), ops.add(g, ops.mul(g, e1, den), e2))
            t2 = ops.sub(g, mx, ops.exp(g, time_decay))
            m = ops.maximum(g, t2, key)
            e1, e2 = ops.exp(g, ops.sub(g, t2, m)), ops.exp(g, ops.sub(g, key, m))
            layer_state[2] = ops.add(g, ops.mul(g, e1, num), ops.mul(g, e2, value))
            layer_state[3] = ops.add(g, ops.mul(g, e1, den), e2)
            layer_state[4] = m
        if half:
            out = ops.cast(g, out, self.popart_float_type)
        return self.output_linear(g, ops.mul(g, rec, out)), layer_state


class RWKVFeedforward(BaseLayer):
    """Channel mixing (reference: rwkv/ffn.py:20-59)."""

    def __init__(self, context, name, hidden_size, intermediate_size, layer_id):
        super().__init__(context, name)
        self.key_linear = Linear(self.context, "key", hidden_size, intermediate_size, use_bias=False)
        self.receptance_linear = Linear(self.context, "receptance", hidden_size, hidden_size, use_bias=False)
        self.value_linear = Linear(self.context, "value", intermediate_size, hidden_size, use_bias=False)
        self.time_mix_key = self._vector("time_mix_key", [1, 1, hidden_size])
        self.time_mix_receptance = self._vector("time_mix_receptance", [1, 1, hidden_size])

    _vector = RWKVAttention._vector

    def __call__(self, graph, hidden, layer_state):
        prev = layer_state[0]
        key = _token_shift(self, graph, hidden, self.time_mix_key, prev)
        rec = _token_shift(self, graph, hidden, self.time_mix_receptance, prev)
        layer_state[0] = hidden
        key = ops.relu(graph, self.key_linear(graph, key))
        value = self.value_linear(graph, ops.mul(graph, key, key))
        rec = ops.sigmoid(graph, self.receptance_linear(graph, rec))
        return ops.mul(graph, rec, value), layer_state


class RWKVBlock(BaseLayer):
    def __init__(self, context, name, hidden_size, intermediate_size, attention_hidden_size, eps, layer_id):
        super().__init__(context, name)
        self.layer_id = layer_id
        if layer_id == 0:
            self.pre_ln = LayerNorm(self.context, "pre_ln", hidden_size, eps)
        self.ln1 = LayerNorm(self.context, "ln1", hidden_size, eps)
        self.ln2 = LayerNorm(self.context, "ln2", hidden_size, eps)
        self.attention = RWKVAttention(self.context, "attention", hidden_size, attention_hidden_size, layer_id)
        self.feed_forward = RWKVFeedforward(self.context, "feed_forward", hidden_size, intermediate_size, layer_id)

    def __call__(self, graph, hidden, layer_state, sequence_length, norm_type="group"):
        if self.layer_id == 0:
            hidden = self.pre_ln(graph, hidden, sequence_length, norm_type)
        att, layer_state = self.attention(graph, self.ln1(graph, hidden, sequence_length, norm_type), layer_state)
        hidden = ops.add(graph, hidden, att)
        ffn, layer_state = self.feed_forward(graph, self.ln2(graph, hidden, sequence_length, norm_type), layer_state)
        return ops.add(graph, hidden, ffn), layer_state


class RWKVModel(BaseLayer):
    def __init__(self, context, name, hidden_size, intermediate_size, attention_hidden_size, eps, vocab_size,
                 num_hidden_layers, rescale_every, layer_per_ipu):
        super().__init__(context, name)
        self.rescale_every, self.layer_per_ipu = rescale_every, layer_per_ipu
        self.embeddings = Embedding(".".join([self.context, "embeddings"]), None, vocab_size, hidden_size)
        self.blocks = [RWKVBlock(self.context, f"blocks.{i}", hidden_size, intermediate_size, attention_hidden_size, eps, i)
                       for i in range(num_hidden_layers)]
        self.ln_out = LayerNorm(self.context, "ln_out", hidden_size, eps)

    def __call__(self, graph, input_ids, states, sequence_length, norm_type="ce", **kwargs):
        hidden = self.embeddings(graph, input_ids, sequence_length)
        new_states = []
        for i, block in enumerate(self.blocks):
            hidden, st = block(graph, hidden, list(states[5 * i: 5 * i + 5]), sequence_length, norm_type)
            if self.rescale_every > 0 and (i + 1) % self.rescale_every == 0:
                hidden = ops.div(graph, hidden, ops.constant(graph, np.array(2, dtype=self.np_float_type), "2"))
            new_states.append(st)
        return self.ln_out(graph, hidden, sequence_length, norm_type=norm_type), new_states


class RWKVDecodeModel(HFDecBaseModel):
    """reference: rwkv/model.py:121-259.  hf_config fields: hidden_size, intermediate_size,
    attention_hidden_size, layer_norm_epsilon, vocab_size, num_hidden_layers, rescale_every.  The state
    dict is expected as Hugging Face holds it unless `state_dict_is_processed`;
    process_hf_model_state_dict divides `attention.output.weight` and `feed_forward.value.weight` of
    block i by 2^(i // rescale_every) (model.py:150-155)."""

    def __init__(self, **kwargs):
        self.state_dict_is_processed = kwargs.get("state_dict_is_processed", False)
        super().__init__(**kwargs)
        c = self.hf_config
        self.topk = kwargs.get("topk", 1)
        self.outline_blocks = kwargs.get("outline_blocks", True)
        self.cell = RWKVModel(None, "rwkv", c.hidden_size, c.intermediate_size, c.attention_hidden_size,
                              c.layer_norm_epsilon, c.vocab_size, c.num_hidden_layers, c.rescale_every, self.layer_per_ipu)
        self.head = LMHead(None, "head", self.topk, c.vocab_size, c.hidden_size)
        self.head.set_virtual_id(max(len(self.layer_per_ipu) - 1, 0))

    def process_hf_model_state_dict(self):
        c = self.hf_config
        if self.state_dict_is_processed or c.rescale_every <= 0:
            return
        for key in list(self.state_dict):
            if key.endswith("attention.output.weight") or key.endswith("feed_forward.value.weight"):
                w = np.asarray(self.state_dict[key])
                if w.dtype == np.int8:
                    raise ValueError(f"{key} is already quantised: rescale before quantising and pass state_dict_is_processed")
                block_id = int(key.split("blocks.")[1].split(".")[0])
                self.state_dict[key] = (w.astype(np.float32) / 2 ** (block_id // c.rescale_every)).astype(w.dtype)

    def build_model_graph_inputs(self, graph, inputs):
        """Loop state: step, stop mask and five state tensors per block - two token-shift rows in the
        activation type, numerator and denominator (fp32 zeros), running maximum (fp32, -1e30)."""
        c = self.hf_config
        B, d = self.batch_size, c.hidden_size
        with graph.nameScope("step"):
            inputs["step"] = ops.constant(self.graph, np.array(0).astype(np.int32), "init_step")
        with graph.nameScope("stop_mask"):
            inputs["stop_mask"] = ops.constant(self.graph, np.zeros((B,)).astype(np.int32), "stop_mask")
        with graph.nameScope("states"):
            for i in range(c.num_hidden_layers):
                for j in range(2):
                    inputs[f"state_{i}_{j}"] = ops.constant(self.graph, np.zeros((B, 1, d), dtype=self.np_float_type), f"layer{i}_{j}")
                for j in range(2, 4):
                    inputs[f"state_{i}_{j}"] = ops.constant(self.graph, np.zeros((B, 1, d), dtype=np.float32), f"layer{i}_{j}")
                inputs[f"state_{i}_4"] = ops.constant(self.graph, np.zeros((B, 1, d), dtype=np.float32) - 1e30, f"layer{i}_4")
        del inputs["position_ids"]
        del inputs["attention_mask"]
        return inputs

    def build_model_graph(self, model_graph, model_graph_inputs, sequence_length=1):
        g = model_graph
        step = model_graph_inputs["step"]
        states = [v for k, v in model_graph_inputs.items() if k.startswith("state_")]
        with self.device_scope(g, 0, 0):
            input_ids = ops.dynamic_slice(g, model_graph_inputs["input_ids_container"], step, axes=[1], sizes=[sequence_length])
            hidden, states = self.cell(graph=g, input_ids=input_ids, states=states, sequence_length=sequence_length,
                                       norm_type="ce", outline_blocks=self.outline_blocks)
        next_ids = self.head(g, hidden, sequence_length=sequence_length)
        outputs = {"next_ids": next_ids, "stage_offset": 1}
        for i, layer in enumerate(states):
            for j, t in enumerate(layer):
                outputs[f"states/layer_{i}_{j}"] = t
        return outputs

    def build_post_model_graph(self, model_graph, model_graph_inputs, model_outputs):
        with self.device_scope(model_graph, 0, pipeline_stage_id=model_outputs["stage_offset"]):
            container, step, _, new_ids = self.step_containers(
                model_graph, model_graph_inputs["input_ids_container"], model_graph_inputs["step"], None,
                model_outputs["next_ids"])
            stop_mask, keep_going = self.step_loop_cond(model_graph, new_ids, model_graph_inputs["stop_mask"])
        self.add_output_tensor(model_graph, [keep_going, container, step, stop_mask] +
                               [v for k, v in model_outputs.items() if k.startswith("states/")])
