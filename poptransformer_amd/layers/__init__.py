"""Layer library with the class names, constructor signatures and weight keys of the reference's
`poptransformer/layers` package, single-device ('shard') variants only: the tensor-parallel
variants exist to split weights over IPU replicas and are not built for one GPU."""
from .base_layer import BaseLayer
from .linear import Linear
from .layer_norm import LayerNorm
from .rms_layer_norm import RMSLayerNorm
from .embedding import Embedding
from .mlp import MLP
from .lm_head import LMHead

__all__ = ["BaseLayer", "Linear", "LayerNorm", "RMSLayerNorm", "Embedding", "MLP", "LMHead"]
