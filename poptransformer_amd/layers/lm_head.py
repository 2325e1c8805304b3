from .. import ops
from .base_layer import BaseLayer, require_single_device
from .linear import Linear


class LMHead(BaseLayer):
    """Vocabulary projection without bias followed by token selection (reference:
    layers/lm_head.py:22-57): top-1 indices when topk == 1, otherwise a random pick among the top k.
    With `tie_weight` the projection reuses an embedding table [vocab, embed], transposed in-graph."""

    def __init__(self, context, name, topk, vocab_size, embedding_size, tie_weight=None):
        require_single_device("LMHead")
        super().__init__(context, name)
        self.topk, self.vocab_size, self.embedding_size = topk, vocab_size, embedding_size
        self.virtual_id, self.use_tied_embedding, self.tie_weight = None, False, tie_weight
        self.collect_bind_layer_weights()

    def collect_bind_layer_weights(self):
        self.head = Linear(self.context, None, self.embedding_size, self.vocab_size, False)
        if self.tie_weight is not None:
            self.tie_embedding(self.tie_weight)

    def tie_embedding(self, weight_id):
        self.head.weight_id, self.use_tied_embedding = weight_id, True

    def set_virtual_id(self, virtual_id):
        self.virtual_id = virtual_id

    def __call__(self, graph, logits, sequence_length):
        with graph.virtualGraph(self.virtual_id):
            if self.use_tied_embedding:
                self.head.weight_id = ops.transpose(graph, self.head.weight_id, [1, 0])
            logits = self.head(graph, logits)
            if self.topk != 1:
                next_token = ops.random_sample(graph, logits, k=self.topk, dim=2)
            else:
                _, next_token = ops.topk(graph, logits, axis=2, k=1)
            return ops.squeeze(graph, next_token, [2])
