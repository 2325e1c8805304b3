from .. import ops
from ..utils import ParamHandler
from .base_layer import BaseLayer, require_single_device


class Linear(BaseLayer):
    """y = x @ W^T (+ b) (reference: layers/linear.py:19-46).  `<context>.weight` is [out, in]; it is
    stored transposed and passed through the precision hook (INT4: packed [out, in/2] + scales;
    FP8: F143 bytes + exponent), `<context>.bias` is [out]."""

    def __init__(self, context, name, input_size, output_size, use_bias=True, **kwargs):
        require_single_device("Linear")
        super().__init__(context, name)
        self.input_size, self.output_size, self.use_bias, self.kwargs = input_size, output_size, use_bias, kwargs
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        self.param_handler = ParamHandler(host_layer=self)
        key = f"{self.context}.weight"
        w = self.get_param_from_state_dict(key, [self.output_size, self.input_size]).transpose(1, 0)
        self.weight_id = self.add_initialized_input_tensor(self.param_handler.process_linear_weight(w, key), key)
        if self.use_bias:
            key = f"{self.context}.bias"
            b = self.param_handler.process_linear_bias(self.get_param_from_state_dict(key, [self.output_size]))
            self.bias_id = self.add_initialized_input_tensor(b, key)

    def __call__(self, graph, x):
        with graph.nameScope(self.context):
            y = self.param_handler.matmul(graph, x, self.weight_id)
            return ops.add(graph, y, self.bias_id) if self.use_bias else y
