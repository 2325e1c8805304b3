"""Weight preparation and matmul hooks per precision (reference:
utils/param_handler/param_handler.py:19-83 and precision_strategy.py:24-119).  Only the `identity`
tensor-parallel strategy exists here (tensor_parallel_strategy.py:103-108): one GPU holds every
weight whole."""
import numpy as np

from . import REGISTRY


def _ops():
    from .. import ops
    return ops


def _main_inputs():
    return REGISTRY.get("main_graph").getInputTensorIds()


class _Strategy:
    name = None

    def weight(self, layer, w, key):
        return w

    def prepare(self, graph, x, weight):
        return x, weight

    def matmul(self, graph, x, weight):
        return _ops().matmul(graph, x, weight)


class _Float(_Strategy):
    pass


class _Int4(_Strategy):
    """An int8 Linear weight is a packed INT4 matrix.  The Linear layer has transposed the checkpoint
    tensor [out, in/2] to [in/2, out]; it is transposed back and its `<key>_scale` registered
    (precision_strategy.py:24-42).  fp16 weights (embeddings, lm_head) pass through."""

    def weight(self, layer, w, key):
        if w.dtype != np.int8:
            return w
        if w.ndim != 2:
            raise ValueError(f"weight_np can only have rank 2 or 3, but got {w.ndim}.")
        w = w.transpose(1, 0)
        scale_key = key + "_scale"
        scale = layer.get_param_from_state_dict(scale_key, shape_list=(w.shape[0],))
        layer.add_initialized_input_tensor(np.asarray(scale, np.float16), scale_key)
        return w

    def prepare(self, graph, x, weight):
        if weight + "_scale" in _main_inputs():
            weight = _ops().int4_to_half(graph, weight, weight + "_scale", x, axis=1)
        return x, weight


class _Fp8(_Strategy):
    """Every Linear weight becomes F143 bytes with exponent -1 and an int32 `<key>_scale`
    (precision_strategy.py:44-51); the state dict may override the exponent with `<key>_scale`."""
    cast_activations = True

    def weight(self, layer, w, key):
        from ..engine.host_codecs import f8_encode_host
        scale_key = key + "_scale"
        given = layer.state_dict.get(scale_key, None)
        exponent = int(np.asarray(given).reshape(-1)[0]) if given is not None else -1
        layer.add_initialized_input_tensor(np.array([exponent], np.int32), scale_key)
        return f8_encode_host(np.asarray(w, np.float32), "F143", exponent)

    def prepare(self, graph, x, weight):
        if self.cast_activations and weight + "_scale" in _main_inputs():
            x = _ops().half_to_uint8(graph, x, weight + "_scale")
        return x, weight

    def matmul(self, graph, x, weight):
        scale = weight + "_scale"
        if scale in _main_inputs():
            return _ops().fp8_matmul(graph, x, weight, scale, scale, "F143", "F143")
        return _ops().matmul(graph, x, weight)


class _Fp8Weight(_Fp8):
    cast_activations = False


PrecisionStrategyMap = {"fp16": _Float(), "fp32": _Float(), "int4": _Int4(), "fp8": _Fp8(), "fp8_weight": _Fp8Weight()}


class ParamHandler:
    def __init__(self, host_layer, tp_strategy_name="identity", **vs_setting):
        if tp_strategy_name not in (None, "identity"):
            raise ValueError(f"tensor-parallel strategy '{tp_strategy_name}' is not available: the model runs on one GPU")
        self.host_layer = host_layer
        self.strategy = PrecisionStrategyMap[self.precision]

    @property
    def precision(self):
        return REGISTRY.get("precision")

    @property
    def num_replicas(self):
        return REGISTRY.get("num_replicas")

    def process_linear_weight(self, weight_np, weight_key):
        return self.strategy.weight(self.host_layer, weight_np, weight_key)

    def process_linear_bias(self, bias):
        return bias

    def matmul(self, graph, x, weight):
        x, weight = self.strategy.prepare(graph, x, weight)
        return self.strategy.matmul(graph, x, weight)
