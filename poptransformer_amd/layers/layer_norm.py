from .. import ops
from .base_layer import BaseLayer, require_single_device


class LayerNorm(BaseLayer):
    """LayerNorm with weights `<context>.weight/.bias` (reference: layers/layer_norm.py:19-43);
    norm_type 'ce' is the NormCE operator, 'group' a one-group group normalisation."""
    norm_fn_map = {"group": ops.group_norm, "ce": ops.layer_norm_ce}

    def __init__(self, context, name, input_size, eps):
        require_single_device("LayerNorm")
        super().__init__(context, name)
        self.input_size, self.eps = input_size, eps
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        for attr, suffix in (("weight_id", "weight"), ("bias_id", "bias")):
            key = f"{self.context}.{suffix}"
            setattr(self, attr, self.add_initialized_input_tensor(self.get_param_from_state_dict(key, [self.input_size]), key))

    def __call__(self, graph, x, sequence_length, norm_type):
        with graph.nameScope(self.context):
            fn = self.norm_fn_map.get(norm_type)
            if fn is None:
                raise ValueError(f"Invalid norm_fn {norm_type}, options: {self.norm_fn_map.keys()}")
            return fn(graph, x, self.weight_id, self.bias_id, self.eps, self.batch_size, sequence_length, self.input_size)
