"""Process-wide registry, precision descriptor and the scope helpers of the reference's
`poptransformer.utils` package (registry.py, tensor_type.py, device_scope.py, options_scope.py,
prepare.py, param_handler/)."""
import contextlib
import logging

import numpy as np

from .. import popart


class Registry:
    """Key/value store shared by models and layers (reference: utils/registry.py:17-46).
    `register` refuses a key that exists, `get` a key that does not."""

    def __init__(self):
        self._items = {}

    def register(self, key, value):
        if key in self._items:
            raise KeyError(f"Duplicate key: {key}")
        self._items[key] = value

    def update(self, key, value):
        self._items[key] = value

    def get(self, key):
        if key not in self._items:
            raise KeyError(f"key: {key} not found")
        return self._items[key]

    def __contains__(self, key):
        return key in self._items

    def reset(self):
        """Fresh main graph and defaults.  The reference creates them once at import, which allows one
        model per process (registry.py:40-46); tests build several, so the reset is explicit here."""
        self._items.clear()
        self._items.update({
            "main_graph": popart.Builder(opsets={"ai.onnx": 10, "ai.graphcore": 1}),
            "serial_factor": None, "serial_mode": None, "partialtype": None, "amp": None, "state_dict": {},
            "logger": logging.getLogger("poptransformer"),
        })


REGISTRY = Registry()
REGISTRY.reset()


class TensorType:
    """Activation dtype per precision (reference: utils/tensor_type.py:17-33): the INT4 and FP8 modes
    compute on fp16 activations."""
    all_precision = ["fp32", "fp16", "int4", "fp8", "fp8_weight"]

    def __init__(self, precision):
        assert precision in self.all_precision
        self.precision = precision

    @property
    def np_float_type(self):
        return np.float32 if self.precision == "fp32" else np.float16

    @property
    def popart_float_type(self):
        return "FLOAT" if self.precision == "fp32" else "FLOAT16"


class DeviceScope:
    """Placement scope (reference: utils/device_scope.py:17-37).  Enters the builder's virtual-graph /
    pipeline-stage / outline scopes, which record nothing on a single GPU."""

    def __init__(self, graph, virtual_graph_id=None, pipeline_stage_id=None, enable_pipeline=False, outline_attr=None):
        self.graph = graph
        self.virtual_graph_id, self.pipeline_stage_id = virtual_graph_id, pipeline_stage_id
        self.enable_pipeline, self.outline_attr = enable_pipeline, outline_attr

    def __enter__(self):
        self._stack = contextlib.ExitStack()
        if self.virtual_graph_id is not None:
            self._stack.enter_context(self.graph.virtualGraph(self.virtual_graph_id))
        if self.enable_pipeline and self.pipeline_stage_id is not None:
            self._stack.enter_context(self.graph.pipelineStage(self.pipeline_stage_id))
        if self.outline_attr is not None:
            self._stack.enter_context(self.graph.outlineAttributes(self.outline_attr))
        return self

    def __exit__(self, *exc):
        self._stack.close()
        return False


class OptionsScope:
    """Temporarily overrides the matmul options that `ops.matmul` reads from the registry
    (reference: utils/options_scope.py:17-59).  `partialtype` is the only one with a numeric meaning;
    the GPU kernels always accumulate in fp32, which the 1e-2 tolerance on fp16 results covers."""
    _keys = ("amp", "partialtype", "serial_factor", "serial_mode")

    def __init__(self, amp=None, partialtype=None, serial_factor=None, serial_mode=None):
        self._new = {"amp": amp, "partialtype": partialtype, "serial_factor": serial_factor, "serial_mode": serial_mode}

    def __enter__(self):
        self._old = {k: REGISTRY.get(k) for k in self._keys}
        for k, v in self._new.items():
            if v is not None:
                REGISTRY.update(k, v)
        return self

    def __exit__(self, *exc):
        for k, v in self._old.items():
            REGISTRY.update(k, v)
        return False


from .param_handler import ParamHandler  # noqa: E402
from .prepare import prepare_model_session, register_global_args  # noqa: E402

__all__ = ["REGISTRY", "Registry", "TensorType", "DeviceScope", "OptionsScope", "ParamHandler",
           "prepare_model_session", "register_global_args"]
