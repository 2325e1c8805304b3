import numpy as np

from .. import ops
from .base_layer import BaseLayer, require_single_device


class RMSLayerNorm(BaseLayer):
    """RMSNorm composed from elementwise graph ops (reference: layers/rms_layer_norm.py:20-36): the
    statistics in fp32, the inverse RMS cast back to the activation type, two multiplies."""

    def __init__(self, context, name, input_size, eps):
        require_single_device("RMSLayerNorm")
        super().__init__(context, name)
        self.input_size, self.eps = input_size, eps
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        key = f"{self.context}.weight"
        self.weight_id = self.add_initialized_input_tensor(self.get_param_from_state_dict(key, [self.input_size]), key)

    def __call__(self, graph, x):
        eps = ops.constant(graph, np.array(self.eps).astype(np.float32), "variance_epsilon")
        v = ops.cast(graph, x, "FLOAT")
        v = ops.reducemean(graph, ops.mul(graph, v, v))
        v = ops.reciprocal(graph, ops.sqrt(graph, ops.add(graph, v, eps)))
        v = ops.cast(graph, v, self.popart_float_type)
        return ops.mul(graph, ops.mul(graph, x, v), self.weight_id)
