from .. import ops
from .base_layer import BaseLayer, require_single_device
from .linear import Linear


class MLP(BaseLayer):
    """c_proj(act(c_fc(x))) on rows flattened to [B*S, d] (reference: layers/mlp.py:19-41)."""
    act_fn_map = {"gelu": ops.gelu}

    def __init__(self, context, name, input_size, hidden_size, act_fn):
        require_single_device("MLP")
        super().__init__(context, name)
        self.input_size, self.hidden_size = input_size, hidden_size
        self.act_fn = self.act_fn_map.get(act_fn)
        if self.act_fn is None:
            raise ValueError(f"Invalid act_fn {act_fn}, options: {self.act_fn_map.keys()}")
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        self.c_fc = Linear(self.context, "c_fc", self.input_size, self.hidden_size)
        self.c_proj = Linear(self.context, "c_proj", self.hidden_size, self.input_size)

    def __call__(self, graph, x):
        with graph.nameScope(self.context):
            x = ops.reshape(graph, x, [-1, self.input_size])
            x = self.c_proj(graph, self.act_fn(graph, self.c_fc(graph, x)))
            return ops.reshape(graph, x, [self.batch_size, -1, self.input_size])
