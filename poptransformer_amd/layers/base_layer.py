import numpy as np

from ..utils import REGISTRY, DeviceScope, OptionsScope


def require_single_device(cls_name):
    """The reference dispatches every layer on REGISTRY['model_type'] ('shard' | 'tp', e.g.
    layers/linear.py:71-90).  Only 'shard' (whole weights on one device) is available here."""
    model_type = REGISTRY.get("model_type")
    if model_type != "shard":
        raise ValueError(f"Invalid model_type {model_type}, options: ['shard'] ({cls_name} has no tensor-parallel variant on one GPU)")


class BaseLayer:
    """Common base of all layers (reference: layers/base_layer.py:20-128): the context string that
    prefixes state-dict keys, registry accessors, and the two weight helpers."""

    def __init__(self, context, name):
        self.context = ".".join([context, name]) if (context and name) else (context or name)
        self.name = name

    # registry views -----------------------------------------------------------------------------
    logger = property(lambda self: REGISTRY.get("logger"))
    model_type = property(lambda self: REGISTRY.get("model_type"))
    batch_per_step = property(lambda self: REGISTRY.get("batch_per_step"))
    batch_size = property(lambda self: REGISTRY.get("batch_size"))
    num_replicas = property(lambda self: REGISTRY.get("num_replicas"))
    main_graph = property(lambda self: REGISTRY.get("main_graph"))
    state_dict = property(lambda self: REGISTRY.get("state_dict"))
    enable_pipeline = property(lambda self: REGISTRY.get("enable_pipeline"))
    popart_float_type = property(lambda self: REGISTRY.get("tensor_type").popart_float_type)
    np_float_type = property(lambda self: REGISTRY.get("tensor_type").np_float_type)
    precision = property(lambda self: REGISTRY.get("tensor_type").precision)

    def option_scope(self, amp=None, partialtype=None, serial_factor=None, serial_mode=None):
        return OptionsScope(amp, partialtype, serial_factor, serial_mode)

    def device_scope(self, graph, virtual_graph_id=None, pipeline_stage_id=None, outline_attr=None):
        return DeviceScope(graph, virtual_graph_id, pipeline_stage_id, self.enable_pipeline, outline_attr)

    def __call__(self, graph, *args):
        raise NotImplementedError

    def collect_bind_layer_weights(self):
        raise NotImplementedError

    # weights ------------------------------------------------------------------------------------
    def add_initialized_input_tensor(self, weight_np, weight_key, **variable_setting):
        """Registers a weight on the main graph under its state-dict key (base_layer.py:103-109).
        Replica variable settings have no meaning on one device and are dropped."""
        return self.main_graph.addInitializedInputTensor(np.asarray(weight_np), debugContext=weight_key)

    def get_param_from_state_dict(self, weight_key, shape_list):
        """State-dict lookup (base_layer.py:111-128): a missing key falls back to unseeded N(0, 1)
        values of `shape_list`, a found one is shape-checked except under int4 / fp8 precision."""
        value = self.state_dict.get(weight_key, None)
        if value is None:
            self.logger.info(f"{weight_key} not found, using random tensor")
            assert shape_list, f"no shape provided for random initializing the tensor {weight_key}"
            return np.random.randn(*shape_list).astype(self.np_float_type)
        value = value.numpy() if hasattr(value, "numpy") else np.asarray(value)
        if shape_list and self.precision not in ("int4", "fp8", "fp8_weight"):
            assert tuple(value.shape) == tuple(shape_list), \
                f"{weight_key} shape {value.shape} not matched with provided {shape_list}"
        return value
