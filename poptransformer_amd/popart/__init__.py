"""Recorder with the surface of the `popart` module that PopTransformer uses.

The reference builds an ONNX graph through `popart.Builder` (REGISTRY['main_graph'],
poptransformer/utils/registry.py:41) and runs it with `popart.InferenceSession`
(poptransformer/sessions.py:35-49, 91-98).  This module keeps those names and call signatures but
only RECORDS: every `graph.aiOnnx.*`, `graph.aiGraphcore.*` and `graph.customOp(...)` call
appends a node to a small IR and returns fresh tensor ids (strings, as PopART does).  Execution
is the business of `poptransformer_amd.engine` (an op-by-op interpreter on the GPU, and the fused
executors it validates and then prefers).

Methods that only steer IPU placement, memory or compilation (virtual graphs, pipeline stages,
outlining, available-memory proportion, partials type, matmul serialisation, replication and
variable settings) are accepted and ignored: one GPU holds the whole graph.
"""
import contextlib
import logging

import numpy as np

__all__ = ["Builder", "TensorInfo", "InputSettings", "ReplicatedStreamMode", "AnchorReturnType", "DataFlow",
           "SessionOptions", "DeviceManager", "InferenceSession", "PyStepIO", "VirtualGraphMode", "getLogger",
           "VariableSettings", "CommGroup", "CommGroupType", "VariableRetrievalMode", "popart_exception"]

NP_OF = {"FLOAT16": np.float16, "FLOAT": np.float32, "INT32": np.int32, "INT64": np.int64, "INT8": np.int8,
         "UINT8": np.uint8, "BOOL": np.bool_, "UINT32": np.uint32}
NAME_OF = {np.dtype(v): k for k, v in NP_OF.items()}


class popart_exception(RuntimeError):
    """Graph-construction error (the reference raises popart::error from Op::setup)."""


class TensorInfo:
    def __init__(self, dtype, shape):
        if isinstance(dtype, np.ndarray):
            dtype, shape = NAME_OF[dtype.dtype], list(dtype.shape)
        if dtype not in NP_OF:
            raise popart_exception(f"unknown data type {dtype}")
        self.dtype, self._shape = dtype, [int(s) for s in shape]

    def shape(self):
        return list(self._shape)

    def data_type(self):
        return self.dtype

    def __repr__(self):
        return f"TensorInfo({self.dtype}, {self._shape})"


class _Enum:
    def __init__(self, name):
        self.name = name

    def __repr__(self):
        return self.name


class ReplicatedStreamMode:
    Broadcast, Replicate = _Enum("Broadcast"), _Enum("Replicate")


class VirtualGraphMode:
    Off, Manual, Auto = _Enum("Off"), _Enum("Manual"), _Enum("Auto")


class CommGroupType:
    All, Consecutive, Orthogonal, Ungrouped = _Enum("All"), _Enum("Consecutive"), _Enum("Orthogonal"), _Enum("None")


class VariableRetrievalMode:
    OnePerGroup, AllReduceReplicas, AllReplicas = _Enum("OnePerGroup"), _Enum("AllReduceReplicas"), _Enum("AllReplicas")


class CommGroup:
    def __init__(self, type=None, replicaGroupSize=0):
        self.type, self.replicaGroupSize = type, replicaGroupSize


class VariableSettings:
    def __init__(self, comm_group=None, retrieval_mode=None):
        self.comm_group, self.retrieval_mode = comm_group, retrieval_mode


class InputSettings:
    def __init__(self, mode=None):
        self.mode = mode


class AnchorReturnType:
    def __init__(self, kind="ALL"):
        self.kind = kind


class DataFlow:
    def __init__(self, batches_per_step, anchors):
        self.batches_per_step, self.anchors = batches_per_step, dict(anchors)


class SessionOptions:
    """Plain attribute bag: every option the reference sets (sessions.py:62-89) is an IPU compile knob."""

    def __init__(self):
        self.__dict__["_opts"] = {}

    def __setattr__(self, k, v):
        self._opts[k] = v

    def __getattr__(self, k):
        try:
            return self.__dict__["_opts"][k]
        except KeyError:
            raise AttributeError(k)


class DeviceInfo:
    def __init__(self, n):
        self.numIpus = n

    def __repr__(self):
        return "DeviceInfo(one MI355X)"


class DeviceManager:
    def acquireAvailableDevice(self, numIpus=1, **kwargs):
        """The reference asks for 2^ceil(log2(stages * replicas)) IPUs (sessions.py:57-58); here the
        whole graph lives on the one GPU, whatever number is asked for."""
        return DeviceInfo(numIpus)


def getLogger(name="popart"):
    class _L:
        def setLevel(self, level):
            logging.getLogger("poptransformer.popart").setLevel(level if level != "OFF" else "CRITICAL")
    return _L()


# ----------------------------------------------------------------------------------------- IR
class Node:
    __slots__ = ("op", "inputs", "outputs", "attrs", "scope", "subgraph")

    def __init__(self, op, inputs, outputs, attrs, scope, subgraph=None):
        self.op, self.inputs, self.outputs, self.attrs, self.scope, self.subgraph = op, list(inputs), list(outputs), attrs, scope, subgraph

    def __repr__(self):
        return f"{self.outputs} = {self.op}({self.inputs}, {self.attrs})"


# number of outputs for ops that do not return exactly one tensor
def _n_outputs(op, inputs, args, kwargs):
    if op == "aiOnnx.split":
        return kwargs.get("num_outputs", args[0] if args else 1), True
    if op == "aiOnnx.topk":
        return 2, True
    if op == "aiGraphcore.groupnormalization":
        return 3, True
    return 1, False


class _OpSet:
    def __init__(self, builder, prefix):
        self._b, self._prefix = builder, prefix

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        op = f"{self._prefix}.{name}"

        def record(*args, **kwargs):
            return self._b._record(op, args, kwargs)
        return record


class Builder:
    def __init__(self, modelProtoOrFilename=None, opsets=None, builderCore=None, parent=None):
        self.opsets = opsets or {"ai.onnx": 10, "ai.graphcore": 1}
        self.parent = parent
        self.root = parent.root if parent is not None else self
        self.name = "main" if parent is None else "subgraph"
        self.nodes = []
        self.inputs = []              # ids in declaration order (graph inputs and initializers)
        self.input_info = {}          # id -> TensorInfo (typed inputs)
        self.initializers = {}        # id -> numpy array
        self.outputs = []
        self.children = []
        self._scopes = []
        if parent is None:
            self._names = {}
        self.aiOnnx = _OpSet(self, "aiOnnx")
        self.aiGraphcore = _OpSet(self, "aiGraphcore")
        self.aiOnnxMl = _OpSet(self, "aiOnnxMl")

    # ---- naming --------------------------------------------------------------------------
    def _fresh(self, base):
        names = self.root._names
        scope = "/".join(self._scopes)
        full = f"{scope}/{base}" if scope else base
        n = names.get(full, 0)
        names[full] = n + 1
        return full if n == 0 else f"{full}/{n}"

    def getNameScope(self, name=""):
        s = "/".join(self._scopes)
        return (s + "/" if s else "") + name

    @contextlib.contextmanager
    def nameScope(self, name):
        self._scopes.append(str(name))
        try:
            yield self
        finally:
            self._scopes.pop()

    @contextlib.contextmanager
    def _noop_scope(self, *a, **k):
        yield self

    virtualGraph = pipelineStage = executionPhase = outlineAttributes = recomputeOutput = _noop_scope

    # ---- graph inputs / outputs ----------------------------------------------------------------
    def addInputTensor(self, tensorInfo, *args, **kwargs):
        name = kwargs.get("debugContext", None)
        for a in args:
            if isinstance(a, str):
                name = a
        if not isinstance(tensorInfo, TensorInfo):      # (dtype, shape) form
            tensorInfo = TensorInfo(tensorInfo, args[0])
        tid = self._fresh(name or "input")
        self.inputs.append(tid)
        self.input_info[tid] = tensorInfo
        return tid

    def addUntypedInputTensor(self, debugContext=""):
        tid = self._fresh(debugContext or "input")
        self.inputs.append(tid)
        return tid

    def addInitializedInputTensor(self, array, *args, **kwargs):
        name = kwargs.get("debugContext", None)
        for a in args:
            if isinstance(a, str):
                name = a
        arr = np.ascontiguousarray(np.asarray(array))
        if arr.dtype not in NAME_OF and arr.dtype != np.float64:
            raise popart_exception(f"unsupported initializer dtype {arr.dtype}")
        tid = self._fresh(name or "init_input")
        self.inputs.append(tid)
        self.initializers[tid] = arr
        return tid

    def addInputTensorFromParentGraph(self, tensor_id):
        if self.parent is None:
            raise popart_exception("addInputTensorFromParentGraph on the main graph")
        self.inputs.append(tensor_id)
        return tensor_id

    def addOutputTensor(self, tensor_id):
        self.outputs.append(tensor_id)

    def getInputTensorIds(self):
        return list(self.inputs)

    def getOutputTensorIds(self):
        return list(self.outputs)

    def isInitializer(self, tensor_id):
        return tensor_id in self.initializers

    def getValueTensorIds(self):
        return [o for n in self.nodes for o in n.outputs]

    # ---- sub-graphs ------------------------------------------------------------------------------
    def createSubgraphBuilder(self):
        child = Builder(opsets=self.opsets, parent=self)
        self.children.append(child)
        return child

    def setGraphName(self, name):
        self.name = name

    # ---- recording ---------------------------------------------------------------------------------
    def _record(self, op, args, kwargs):
        args = list(args)
        inputs = list(args.pop(0)) if args and isinstance(args[0], (list, tuple)) else []
        attrs = dict(kwargs)
        dbg = attrs.pop("debugContext", None) or attrs.pop("debugPrefix", None)
        subgraph = None
        short = op.split(".", 1)[1]
        if op == "aiOnnx.constant":
            value = np.asarray(args[0] if args else kwargs.get("value"))
            attrs = {"value": value}
            if args[1:] and isinstance(args[1], str):
                dbg = args[1]
            args = []
        elif op == "aiOnnx.loop":
            # loop(inputs, num_outputs, body)
            n_out, subgraph = args[0], args[1]
            attrs["num_outputs"] = n_out
            args = []
        elif op == "aiGraphcore.call":
            n_out, subgraph = args[0], args[1]
            attrs["num_outputs"] = n_out
            args = []
        elif args and isinstance(args[-1], str) and op not in ("aiOnnx.cast",):
            dbg = args.pop()
        attrs["args"] = args
        attrs["name"] = dbg
        if op in ("aiOnnx.loop", "aiGraphcore.call"):
            n, as_list = attrs["num_outputs"], True
        else:
            n, as_list = _n_outputs(op, inputs, args, kwargs)
        base = short[0].upper() + short[1:]
        outs = [self._fresh(f"{base}:{i}") for i in range(n)]
        self.nodes.append(Node(op, inputs, outs, attrs, "/".join(self._scopes), subgraph))
        return outs if as_list else outs[0]

    def customOp(self, opName, opVersion=1, domain="ai.graphcore", inputs=(), attributes=None, numOutputs=1, name=""):
        outs = [self._fresh(f"{opName}:{i}") for i in range(numOutputs)]
        self.nodes.append(Node(f"custom.{opName}", inputs, outs, dict(attributes or {}), "/".join(self._scopes)))
        return outs

    # ---- IPU-only knobs: accepted, ignored ----------------------------------------------------------
    def setAvailableMemoryProportion(self, *a, **k): pass
    def setPartialsType(self, *a, **k): pass
    def setSerializeMatMul(self, *a, **k): pass
    def setInplacePreferences(self, *a, **k): pass
    def excludePatterns(self, *a, **k): pass
    def addNodeAttribute(self, *a, **k): pass

    # ---- model export --------------------------------------------------------------------------------
    def getModelProto(self):
        """The reference hands an ONNX ModelProto string to InferenceSession (sessions.py:91-98); here
        the recorded graph object itself plays that part."""
        return self

    def saveInitializersExternally(self, ids, filename):
        """utils/prepare.py:40-43 moves every initializer out of the proto to keep it under 2 GB; the
        recorded graph has no such limit, so the initializers stay where they are."""
        self._external = (list(ids), filename)

    def saveModelProto(self, filename):
        raise NotImplementedError("the recorder holds no ONNX proto")


# ----------------------------------------------------------------------------------------- session
class PyStepIO:
    def __init__(self, inputs, outputs):
        self.inputs, self.outputs = dict(inputs), outputs


class InferenceSession:
    """popart.InferenceSession as poptransformer/sessions.py uses it: prepareDevice() compiles,
    weightsFromHost() uploads, initAnchorArrays() allocates the outputs, run(stepio) executes."""

    def __init__(self, fnModel, dataFlow, deviceInfo, userOptions=None, **kwargs):
        if not isinstance(fnModel, Builder):
            raise popart_exception("fnModel must be the proto returned by Builder.getModelProto()")
        self.graph, self.data_flow, self.device_info, self.options = fnModel, dataFlow, deviceInfo, userOptions
        self.executor = None
        self.anchors = None

    def prepareDevice(self, **kwargs):
        from ..engine import compiler
        self.executor = compiler.compile_graph(self.graph, list(self.data_flow.anchors), self.data_flow.batches_per_step,
                                               getattr(self, "allow_fused", True), **getattr(self, "executor_options", {}))

    def weightsFromHost(self):
        if self.executor is None:
            raise popart_exception("prepareDevice() must be called first")

    def initAnchorArrays(self):
        self.anchors = self.executor.anchor_arrays()
        return self.anchors

    def run(self, stepio):
        out = self.executor.run(stepio.inputs)
        for k, v in out.items():
            if k in stepio.outputs:
                np.copyto(stepio.outputs[k], v.reshape(stepio.outputs[k].shape))
