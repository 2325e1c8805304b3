"""Model base classes: graph construction of the decode loop (reference:
poptransformer/models/base_model.py:25-355).

The reference obtains weights, config and tokenizer from the Hugging Face hub
(`from_pretrained`, base_model.py:199-223).  There is no network here: a model is given its
configuration (`hf_config`, a mapping or an object with the same attribute names), its state dict
(reference key names, numpy arrays) and the pad / eos token ids directly; a tokenizer is optional
and only used by build_input_dict / build_output_dict.
"""
from collections import OrderedDict
from types import SimpleNamespace

import numpy as np

from .. import ops, popart
from ..utils import REGISTRY, DeviceScope, OptionsScope


class BaseModel:
    def __init__(self, **kwargs):
        self.anchor_return_type = kwargs.get("anchor_return_type", "ALL")
        self.layer_per_ipu = kwargs.get("layer_per_ipu", [])

    graph = property(lambda self: REGISTRY.get("main_graph"))
    logger = property(lambda self: REGISTRY.get("logger"))
    tensor_type = property(lambda self: REGISTRY.get("tensor_type"))
    enable_pipeline = property(lambda self: REGISTRY.get("enable_pipeline"))
    batch_size = property(lambda self: REGISTRY.get("batch_size"))
    batch_per_step = property(lambda self: REGISTRY.get("batch_per_step"))
    model_type = property(lambda self: REGISTRY.get("model_type"))
    num_replicas = property(lambda self: REGISTRY.get("num_replicas"))
    popart_float_type = property(lambda self: REGISTRY.get("tensor_type").popart_float_type)
    np_float_type = property(lambda self: REGISTRY.get("tensor_type").np_float_type)
    precision = property(lambda self: REGISTRY.get("tensor_type").precision)

    @property
    def stage_num(self):
        return max(len(self.layer_per_ipu), 1)

    def device_scope(self, graph, virtual_graph_id=None, pipeline_stage_id=None, outline_attr=None):
        return DeviceScope(graph, virtual_graph_id, pipeline_stage_id, self.enable_pipeline, outline_attr)

    def option_scope(self, amp=None, partialtype=None, serial_factor=None, serial_mode=None):
        return OptionsScope(amp, partialtype, serial_factor, serial_mode)

    def register_state_dict(self):
        REGISTRY.update("state_dict", self.state_dict)

    @property
    def initializers(self):
        return [t for t in self.graph.getInputTensorIds() if self.graph.isInitializer(t)]

    @property
    def model_output(self):
        art = popart.AnchorReturnType(self.anchor_return_type)
        return {key: art for key in self.graph.getOutputTensorIds()}

    @property
    def model_proto(self):
        return self.graph.getModelProto()

    # graph plumbing (base_model.py:125-186)
    def add_input_tensor(self, graph, popart_dtype, shape, name):
        if self.model_type != "shard":
            raise ValueError(f"Invalid model_type: {self.model_type}")
        return graph.addInputTensor(popart.TensorInfo(popart_dtype, shape), debugContext=name)

    def add_input_tensor_from_parent_graph(self, graph, tensor_id):
        for t in ([tensor_id] if isinstance(tensor_id, str) else tensor_id):
            if not isinstance(t, str):
                raise ValueError(f"Invalid tensor_id: {t}")
            graph.addInputTensorFromParentGraph(t)

    def add_output_tensor(self, graph, output):
        for t in ([output] if isinstance(output, str) else output):
            graph.addOutputTensor(t)

    def create_sub_graph(self, graph, name, sub_graph_inputs, is_loop_graph=False):
        sub = graph.createSubgraphBuilder()
        sub.setGraphName(name)
        if is_loop_graph:
            self.add_input_tensor(sub, "INT32", [], "max_loop")
            self.add_input_tensor(sub, "BOOL", [], "cond")
        self.add_input_tensor_from_parent_graph(sub, sub_graph_inputs)
        return sub


class HFBaseModel(BaseModel):
    def __init__(self, **kwargs):
        super().__init__(**kwargs)
        cfg = kwargs.get("hf_config")
        if cfg is None:
            raise ValueError("hf_config is required (there is no hub to load it from)")
        self.hf_config = SimpleNamespace(**cfg) if isinstance(cfg, dict) else cfg
        self.hf_tokenizer = kwargs.get("hf_tokenizer", None)
        self.state_dict = dict(kwargs.get("state_dict") or {})
        self._pad_token_id = kwargs.get("pad_token_id", getattr(self.hf_config, "pad_token_id", None))
        self._eos_token_id = kwargs.get("eos_token_id", getattr(self.hf_config, "eos_token_id", None))
        self.prepare_state_dict()

    def process_hf_model_state_dict(self):
        """Hook for load-time weight rewrites (GPT-2 query pre-scale, RWKV rescale)."""

    def prepare_state_dict(self):
        self.process_hf_model_state_dict()
        self.register_state_dict()

    @property
    def pad_token_id(self):
        tok = self.hf_tokenizer
        if tok is not None and getattr(tok, "pad_token_id", None):
            return tok.pad_token_id
        if self._pad_token_id is None:
            raise ValueError("pad_token_id is required")
        return self._pad_token_id

    @property
    def eos_token_id(self):
        tok = self.hf_tokenizer
        if tok is not None and getattr(tok, "eos_token_id", None):
            return tok.eos_token_id
        if self._eos_token_id is None:
            raise ValueError("eos_token_id is required")
        return self._eos_token_id


class HFDecBaseModel(HFBaseModel):
    """One-stage decoder: a Loop of `max_loop` iterations whose body runs the model on the token at
    `step` and then updates the id container, the attention mask and the stop mask
    (base_model.py:226-355).  The prompt is consumed inside the same loop: a container slot that
    already holds a prompt token (anything but pad) wins over the generated id."""

    def __init__(self, **kwargs):
        super().__init__(**kwargs)
        self.early_stop = kwargs.get("early_stop", False)
        self.max_length = kwargs.get("max_length", 128)
        self.max_loop = kwargs.get("max_loop", None) or self.max_length

    def build_model_graph(self, model_graph, model_graph_inputs, sequence_length=1):
        raise NotImplementedError

    def build_default_inputs(self):
        B, L = self.batch_size, self.max_length
        inputs = OrderedDict()
        inputs["input_ids_container"] = self.add_input_tensor(self.graph, "INT32", [B, L], "input_ids")
        inputs["step"] = self.add_input_tensor(self.graph, "INT32", [], "step")
        inputs["attention_mask"] = self.add_input_tensor(self.graph, "INT32", [B, L], "attention_mask")
        inputs["position_ids"] = self.add_input_tensor(self.graph, "INT32", [B, L], "position_ids")
        inputs["stop_mask"] = self.add_input_tensor(self.graph, "INT32", [], "stop_mask")
        return inputs

    def build_model_graph_inputs(self, graph, inputs):
        """Initial loop state (base_model.py:255-269): mask 0 at position 0 and -10000 elsewhere,
        step 0, stop mask 0.  Only the id container is fed from the host."""
        with graph.nameScope("mask"):
            mask = np.full((self.batch_size, self.max_length), -10000, dtype=self.np_float_type)
            mask[:, 0] = 0
            inputs["attention_mask"] = ops.constant(graph, mask, "attention_mask")
        with graph.nameScope("step"):
            inputs["step"] = ops.constant(self.graph, np.array(0).astype(np.int32), "init_step")
        with graph.nameScope("stop_mask"):
            inputs["stop_mask"] = ops.constant(self.graph, np.zeros((self.batch_size,)).astype(np.int32), "stop_mask")
        del inputs["position_ids"]
        return inputs

    def build_graph(self):
        inputs = self.build_default_inputs()
        with self.graph.virtualGraph(0):
            inputs = self.build_model_graph_inputs(self.graph, inputs)
        body = self.create_sub_graph(self.graph, "model_graph", list(inputs.values()), True)
        outputs = self.build_model_graph(body, inputs, sequence_length=1)
        self.build_post_model_graph(body, inputs, outputs)
        with self.device_scope(self.graph, 0):
            anchors = ops.loop(self.graph, self.max_loop, list(inputs.values()), body)[:2]
        self.add_output_tensor(self.graph, anchors)

    def build_post_model_graph(self, model_graph, model_graph_inputs, model_outputs):
        with self.device_scope(model_graph, 0, pipeline_stage_id=model_outputs["stage_offset"]):
            container, step, mask, new_ids = self.step_containers(
                model_graph, model_graph_inputs["input_ids_container"], model_graph_inputs["step"],
                model_graph_inputs["attention_mask"], model_outputs["next_ids"])
            stop_mask, keep_going = self.step_loop_cond(model_graph, new_ids, model_graph_inputs["stop_mask"])
        self.add_output_tensor(model_graph, [keep_going, container, step, mask, stop_mask])

    def step_containers(self, graph, input_ids_container, step, attention_mask, next_ids):
        """base_model.py:313-335"""
        with graph.nameScope("step_containers"):
            next_step = ops.add(graph, step, ops.constant(graph, np.array(1).astype(np.int32), "1"))
            next_mask = None
            if attention_mask is not None:
                opened = ops.constant(graph, np.zeros((self.batch_size, 1), dtype=self.np_float_type), "attention_mask_add")
                next_mask = ops.dynamic_update(graph, attention_mask, next_step, opened, axes=[1], sizes=[1])
            slot = ops.dynamic_slice(graph, input_ids_container, next_step, axes=[1], sizes=[1])
            is_pad = ops.equal(graph, slot, ops.constant(graph, np.array(self.pad_token_id), "pad_id"))
            new_ids = ops.where(graph, is_pad, next_ids, slot)
            container = ops.dynamic_update(graph, input_ids_container, next_step, new_ids, axes=[1], sizes=[1])
        return container, next_step, next_mask, new_ids

    def step_loop_cond(self, graph, id_to_update, stop_mask):
        """base_model.py:337-355"""
        with graph.nameScope("step_loop_cond"):
            ids = ops.squeeze(graph, id_to_update, [1])
            hit = ops.cast(graph, ops.equal(graph, ids, ops.constant(graph, np.array(self.eos_token_id), "eos_id")), "INT32")
            next_stop = ops.bitwiseor(graph, stop_mask, hit)
            if self.early_stop:
                stopped = ops.reduce_sum(graph, stop_mask, axes=[0], keepdims=False)
                keep_going = ops.less(graph, stopped, ops.constant(graph, np.array(self.batch_size).astype(np.int32), "batch_size"))
            else:
                keep_going = ops.constant(graph, np.array(True).astype(np.bool_), "cond")
        return next_stop, keep_going

    # host-side I/O ---------------------------------------------------------------------------------
    def build_input_dict(self, **kwargs):
        """`input_ids` [B * batch_per_step, max_length], prompt then pad.  Token ids may be given
        directly (`input_ids`, a list of id lists) or as strings when a tokenizer is present."""
        rows = self.batch_size * self.batch_per_step
        if "input_ids" in kwargs:
            prompts = [list(p) for p in kwargs["input_ids"]]
        else:
            if self.hf_tokenizer is None:
                raise ValueError("a tokenizer is needed to encode input strings")
            prompts = [self.hf_tokenizer.encode(s, add_special_tokens=False) for s in kwargs.get("input_string_list", [])]
        prompts = (prompts + [prompts[0]] * rows)[:rows]
        ids = np.full((rows, self.max_length), self.pad_token_id, dtype=np.int32)
        for r, p in enumerate(prompts):
            ids[r, :min(len(p), self.max_length)] = p[: self.max_length]
        return {"input_ids": ids}

    def build_output_dict(self, anchor_arrays):
        output, decode_step = anchor_arrays["Loop:0"], anchor_arrays["Loop:1"]
        if output.ndim == 3:
            output, decode_step = output[0], decode_step[0]
        if self.hf_tokenizer is not None:
            text = self.hf_tokenizer.batch_decode(output, skip_special_tokens=True)
            return {"output": {str(i): v for i, v in enumerate(text)}, "decode_step": decode_step}
        return {"output": {str(i): v for i, v in enumerate(output)}, "decode_step": decode_step}
