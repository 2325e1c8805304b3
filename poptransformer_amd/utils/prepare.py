"""Bootstrap (reference: utils/prepare.py:21-45) without hydra: the configuration is a plain dict with
the same sections (`global_args`, `model`, `session`) and the classes are passed directly."""
import logging

from . import REGISTRY, TensorType


def register_global_args(global_args):
    """num_replicas, batch_size, batch_per_step, model_type, enable_pipeline, precision -> REGISTRY."""
    defaults = {"num_replicas": 1, "batch_size": 1, "batch_per_step": 1, "model_type": "shard",
                "enable_pipeline": False, "precision": "fp16"}
    defaults.update(global_args or {})
    for key, value in defaults.items():
        REGISTRY.update(key, value)
    REGISTRY.update("tensor_type", TensorType(defaults["precision"]))
    logger = logging.getLogger("poptransformer")
    REGISTRY.update("logger", logger)


def prepare_model_session(config, model_class, session_class=None):
    """config = {'global_args': {...}, 'model': {...}, 'session': {...}}.  Returns (session, model),
    compiled, like the reference."""
    from ..sessions import Session
    REGISTRY.reset()
    register_global_args(config.get("global_args"))
    logging.getLogger("poptransformer").setLevel(str(config.get("log_level", "warning")).upper())
    model = model_class(**config.get("model", {}))
    session = (session_class or Session)(**config.get("session", {}))
    model.build_graph()
    model.graph.saveInitializersExternally(model.initializers, "saved_initializer.onnx")
    session.compile(model)
    return session, model
