"""The operator API of PopTransformer: free functions `f(graph, tensor_id..., python scalars...)`
returning tensor ids, with the names, argument order and defaults of the reference's
`poptransformer/ops/popart.py` and `poptransformer/ops/customized.py` (file:line given per function).

Each function records one or a few nodes on `graph` (a `poptransformer_amd.popart.Builder`); what
the nodes compute is defined by `poptransformer_amd.engine.interpreter`.  The native operators
(`kv_cache`, `softmax_ce`, `layer_norm_ce`, `int4_to_half`, `half_to_uint8`, `fp8_matmul`) are
custom-op nodes with the reference's op names and attribute dictionaries; where the reference
`dlopen`s custom_ops.so at import (customized.py:17-18), the C-ABI library is loaded when the graph is
compiled.
"""
import numpy as np

from ..utils import REGISTRY

_DOMAIN = "ai.graphcore"


# ------------------------------------------------------------------------------ elementwise families
def _unary(opset, name):
    def fn(graph, x):
        return getattr(getattr(graph, opset), name)([x])
    return fn


def _binary(opset, name):
    def fn(graph, x, y):
        return getattr(getattr(graph, opset), name)([x, y])
    return fn


# popart.py:31-53,88-92,191-219: thin wrappers over aiOnnx / aiGraphcore
add, sub, mul, div = (_binary("aiOnnx", n) for n in ("add", "sub", "mul", "div"))
less, greater, equal = (_binary("aiOnnx", n) for n in ("less", "greater", "equal"))
bitwiseor, bitwiseand = _binary("aiGraphcore", "bitwiseor"), _binary("aiGraphcore", "bitwiseand")
tanh, relu, sigmoid, exp, sqrt, reciprocal, mean = (_unary("aiOnnx", n) for n in
                                                    ("tanh", "relu", "sigmoid", "exp", "sqrt", "reciprocal", "mean"))
gelu, swish = _unary("aiGraphcore", "gelu"), _unary("aiGraphcore", "swish")


def sum_op(graph, inputs):
    """popart.py:40-41"""
    return graph.aiOnnx.sum(inputs)


def reduce_sum(graph, x, axes, keepdims):
    """popart.py:43-44"""
    return graph.aiOnnx.reducesum([x], axes=axes, keepdims=keepdims)


def reducemean(graph, x):
    """popart.py:230-231: mean over the last axis, keepdims."""
    return graph.aiOnnx.reducemean([x], axes=[-1])


def maximum(graph, x, y):
    """popart.py:212-215: where(x > y, x, y)."""
    return where(graph, greater(graph, x, y), x, y)


def where(graph, cond, x1, x2):
    """popart.py:126-127"""
    return graph.aiOnnx.where([cond, x1, x2])


def clip(graph, x, clip_min=10, clip_max=100):
    """popart.py:154-156"""
    return graph.aiOnnx.clip([x], max=clip_max, min=clip_min)


# ------------------------------------------------------------------------------ matmul / conv
def matmul(graph, x, y):
    """popart.py:55-67.  The available-memory proportion, partials type and serialisation read from the
    registry are IPU planning hints; they are forwarded to the builder, which ignores them."""
    o = graph.aiOnnx.matmul([x, y])
    amp, partialtype = REGISTRY.get("amp"), REGISTRY.get("partialtype")
    serial_factor, serial_mode = REGISTRY.get("serial_factor"), REGISTRY.get("serial_mode")
    if amp is not None:
        graph.setAvailableMemoryProportion(o, amp)
    if partialtype is not None:
        graph.setPartialsType(o, partialtype)
    if serial_factor is not None:
        graph.setSerializeMatMul({o}, mode=serial_mode, factor=serial_factor)
    return o


def conv(graph, x, weight, bias, kernel_shape, strides, pads, dilations, group):
    """popart.py:183-198 (no decode model uses it)."""
    args = [x, weight] if bias is None else [x, weight, bias]
    return graph.aiOnnx.conv(args=args, kernel_shape=kernel_shape, strides=strides, pads=pads, dilations=dilations,
                             group=group)


# ------------------------------------------------------------------------------ constants and shapes
def constant(graph, tensor, tensor_name="constant"):
    """popart.py:69-70"""
    return graph.aiOnnx.constant(tensor, debugContext=tensor_name)


def reshape(graph, x, shape):
    """popart.py:106-108: the target shape travels as an int32 constant input."""
    return graph.aiOnnx.reshape([x, constant(graph, np.asarray(shape, dtype=np.int32))])


def transpose(graph, x, perm):
    """popart.py:103-104"""
    return graph.aiOnnx.transpose([x], perm=perm)


def unsqueeze(graph, x, dim_list):
    """popart.py:117-118"""
    return graph.aiOnnx.unsqueeze([x], dim_list)


def squeeze(graph, x, dim_list):
    """popart.py:120-121"""
    return graph.aiOnnx.squeeze([x], dim_list)


def expand(graph, x, shape_list):
    """popart.py:158-161"""
    return graph.aiOnnx.expand([x, constant(graph, np.array(shape_list, dtype=np.int32), "shape")])


def tile(graph, x, repeats):
    """popart.py:166-168"""
    return graph.aiOnnx.tile([x, constant(graph, np.array(repeats, dtype=np.int64), "repeats")], "tile")


def pad(graph, x, pad_list, mode="constant", constant_value=0.0):
    """popart.py:19-20"""
    return graph.aiOnnx.pad([x], pads=pad_list, mode=mode, value=constant_value)


def cast(graph, x, popart_float_type):
    """popart.py:114-115"""
    return graph.aiOnnx.cast([x], popart_float_type)


def concat(graph, x, y, axis):
    """popart.py:145-146"""
    return graph.aiOnnx.concat([x, y], axis=axis)


def concat_sequence(graph, inputs, axis):
    """popart.py:148-149"""
    return graph.aiOnnx.concat(inputs, axis=axis)


def split(graph, x, num_outputs, axis, splits, name="split"):
    """popart.py:100-101"""
    return graph.aiOnnx.split([x], num_outputs=num_outputs, axis=axis, split=splits, debugContext=name)


def static_slice(graph, x, starts, ends, axes):
    """popart.py:110-111"""
    return graph.aiGraphcore.slice([x], starts=starts, ends=ends, axes=axes)


def dynamic_slice(graph, x, index, axes, sizes):
    """popart.py:113-114"""
    return graph.aiGraphcore.dynamicslice([x, index], axes=axes, sizes=sizes)


def dynamic_update(graph, x, index, slice_tensor, axes, sizes):
    """popart.py:116-117"""
    return graph.aiGraphcore.dynamicupdate([x, index, slice_tensor], axes=axes, sizes=sizes)


def gather(graph, weight, input_ids):
    """popart.py:82-83"""
    return graph.aiOnnx.gather([weight, input_ids])


def grouped_gather(graph, weight, indexs, axis=0, group_size=1):
    """popart.py:85-86"""
    return graph.aiGraphcore.groupedgather([weight, indexs], axis=axis, group_size=group_size)


# ------------------------------------------------------------------------------ normalisation / softmax / selection
def _group_norm(graph, x, gamma, beta, eps):
    return graph.aiGraphcore.groupnormalization([x, gamma, beta], 1, eps)[0]


def group_norm(graph, x, gamma, beta, eps, batch_size, sequence_length, input_size):
    """popart.py:72-80: LayerNorm as a one-group group normalisation over [B*S, d]."""
    x = reshape(graph, x, [batch_size * sequence_length, input_size])
    x = _group_norm(graph, x, gamma, beta, eps)
    return reshape(graph, x, [batch_size, sequence_length, input_size])


def softmax(graph, x, dim, stable_mode=None):
    """popart.py:129-132"""
    if stable_mode:
        raise ValueError("set use unstable softmax in session, or use type ce ")
    return graph.aiOnnx.softmax([x], dim)


def log_softmax(graph, x, axis=-1):
    """popart.py:151-152"""
    return graph.aiOnnx.logsoftmax([x], axis)


def argmax(graph, x, axis, keepdims=True):
    """popart.py:134-135"""
    return graph.aiOnnx.argmax([x], axis=axis, keepdims=keepdims)


def topk(graph, x, axis, k):
    """popart.py:137-139: returns [values, indices]."""
    return graph.aiOnnx.topk([x, constant(graph, np.array(k).astype(np.int64), "k")], axis=axis)


def randomnormal(graph, shape, dtype, scale):
    """popart.py:22-23"""
    return graph.aiOnnx.randomnormal(shape=shape, dtype=dtype, scale=scale)


def random_sample(graph, logits, k, dim=1):
    """popart.py:25-29: one of the top-k ids, picked by the argmax of k normal draws."""
    _, next_token = topk(graph, logits, axis=dim, k=k)
    rand = argmax(graph, randomnormal(graph, [1, k], 1, 1), 1)
    return dynamic_slice(graph, next_token, rand, axes=[dim], sizes=[1])


def printtensor(graph, x, title):
    """popart.py:141-142"""
    return graph.aiGraphcore.printtensor([x], title=title)


# ------------------------------------------------------------------------------ control flow / collectives
def loop(graph, max_loop_num, loop_graph_input_list, loop_graph):
    """popart.py:170-178: ONNX Loop with trip count max_loop_num and an initial condition of True."""
    max_loop = constant(graph, np.array(max_loop_num).astype(np.int32), "max_loop")
    init_cond = constant(graph, np.array(True).astype(np.bool_), "cond")
    return graph.aiOnnx.loop([max_loop, init_cond] + loop_graph_input_list, len(loop_graph_input_list), loop_graph)


def call_sub_graph(graph, input_list, sub_graph):
    """popart.py:180-181"""
    return graph.aiGraphcore.call(input_list, 1, sub_graph)


def replicated_all_reduce(graph, x):
    """popart.py:183-184.  One replica: the reduction of a single contribution."""
    return graph.aiGraphcore.replicatedallreduce([x])


# ------------------------------------------------------------------------------ native operators
def _custom(graph, op_name, inputs, attributes):
    return graph.customOp(opName=op_name, domain=_DOMAIN, opVersion=1, inputs=inputs, attributes=attributes)[0]


def kv_cache(graph, step, updater, max_len, sequence_axis=1, step_len=1):
    """customized.py:21-35"""
    return _custom(graph, "KVCache", [step, updater],
                   {"max_len": max_len, "step_len": step_len, "sequence_axis": sequence_axis, "fp8": False})


def kv_cache_pipeline(graph, step, updater, max_len, max_bps, step_len=1, sequence_axis=-2, fp8=False, transpose=0):
    """The KVCachePipeline custom op (custom_ops/kv_cache_pipeline.hpp:104-145: attributes max_len, max_bps,
    step_len, sequence_axis, fp8, transpose).  The reference registers the op but has no Python wrapper for it;
    this one follows the wrapper of KVCache (customized.py:21-35)."""
    return _custom(graph, "KVCachePipeline", [step, updater],
                   {"max_len": max_len, "max_bps": max_bps, "step_len": step_len, "sequence_axis": sequence_axis,
                    "fp8": fp8, "transpose": transpose, "debug_str": "kv_cache_pipeline"})


def beam_search(graph, logits, hyp_container, prob_container, step, beam_size):
    """The BeamSearch custom op (custom_ops/beam_search_custom_op.cpp:53-214: inputs logits, hyp_container,
    prob_container, step; attribute beam_size; outputs next_id, global_best_id, hyp_container, prob_container).
    The reference registers the op but has no Python wrapper for it.  Returns the four output ids."""
    return graph.customOp(opName="BeamSearch", domain=_DOMAIN, opVersion=1,
                          inputs=[logits, hyp_container, prob_container, step],
                          attributes={"beam_size": beam_size}, numOutputs=4)


def remap_tensor(graph, x, fwd_after_matmul=0, name="remap"):
    """customized.py:38-54: an IPU tile-layout hint; the values are unchanged."""
    return _custom(graph, "Remap", [x], {"fwd_grain_size": 8, "bwd_grain_size": 8, "fwd_clone_layout": 0,
                                          "bwd_clone_layout": 0, "fwd_after_matmul": fwd_after_matmul,
                                          "bwd_after_matmul": 0, "debug_str": name})


def softmax_ce(graph, x, dim, stable_mode=True):
    """customized.py:57-65"""
    return _custom(graph, "SoftmaxV3", [x], {"axis": dim, "stable_mode": stable_mode})


def layer_norm_ce(graph, x, gamma, beta, eps, batch_size, sequence_length, input_size):
    """customized.py:69-70"""
    return _layer_norm_ce(graph, x, gamma, beta, batch_size, sequence_length, input_size, eps)


def _layer_norm_ce(graph, x, weight, bias, batch_size, sequence_length, input_size, epsilon, fwd_grain_size=-1,
                   bwd_grain_size=-1, fwd_after_matmul=0, bwd_after_matmul=0, stable_algo=False, name="layer_norm_ce"):
    """customized.py:73-102, including its asserts (even size, below 8192)."""
    with graph.nameScope(name):
        num_groups = int(np.prod([batch_size, sequence_length, input_size]) // input_size)
        assert input_size & 1 == 0
        assert input_size < 8192
        attrs = {"fwd_after_matmul": 1 if fwd_after_matmul else 0, "bwd_after_matmul": 1 if bwd_after_matmul else 0,
                 "fwd_grain_size": input_size if fwd_grain_size != -1 else fwd_grain_size,
                 "bwd_grain_size": input_size if bwd_grain_size != -1 else bwd_grain_size,
                 "epsilon": epsilon, "num_groups": num_groups, "stable_algo": stable_algo,
                 "debug_str": graph.getNameScope() + "op"}
        return _custom(graph, "NormCE", [x, weight, bias], attrs)


def replicated_allgather(graph, matmul_output):
    """customized.py:105-112 (tensor parallelism only)."""
    return _custom(graph, "ReplicatedAllGather", [matmul_output], {})


def int4_to_half(graph, x, scale, ref, axis=1, remap=1):
    """customized.py:115-125"""
    return _custom(graph, "Int4ToHalf", [x, scale, ref], {"axis": axis, "remap": remap})


def half_to_uint8(graph, x, fp8_scale, fp8_format="F143"):
    """customized.py:127-135"""
    return _custom(graph, "CastToUint8WithoutShapeInfer", [x, fp8_scale], {"fp8Format": fp8_format})


def fp8_matmul(graph, input_l, input_r, fp8_scale_lhs, fp8_scale_rhs, fp8_format_lhs="F143", fp8_format_rhs="F143"):
    """customized.py:137-148"""
    return _custom(graph, "FP8MatMulWithoutShapeInfer", [input_l, input_r, fp8_scale_lhs, fp8_scale_rhs],
                   {"fp8FormatLHS": fp8_format_lhs, "fp8FormatRHS": fp8_format_rhs})
