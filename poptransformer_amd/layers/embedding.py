from .. import ops
from .base_layer import BaseLayer, require_single_device


class Embedding(BaseLayer):
    """Row gather from `<context>.weight` [vocab, embed] (reference: layers/embedding.py:21-36)."""

    def __init__(self, context, name, vocab_size, embed_size):
        require_single_device("Embedding")
        super().__init__(context, name)
        self.vocab_size, self.embed_size = vocab_size, embed_size
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        key = f"{self.context}.weight"
        self.weight_id = self.add_initialized_input_tensor(
            self.get_param_from_state_dict(key, [self.vocab_size, self.embed_size]), key)

    def __call__(self, graph, input_ids, sequence_length):
        with graph.nameScope(self.context):
            return ops.gather(graph, self.weight_id, input_ids)
