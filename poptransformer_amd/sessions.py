"""Session (reference: poptransformer/sessions.py:19-102): compile(model) then run(input_dict), results
in anchor_arrays.  Placement, outlining, replication, caching and profiling options of the reference
are accepted; on one GPU they have nothing to act on."""
import math

from . import popart
from .utils import REGISTRY


class Session:
    def __init__(self, **kwargs):
        self.execution_cache_name = kwargs.get("execution_cache_name", None)
        self.disable_outlining = kwargs.get("disable_outlining", False)
        self.unstable_softmax = kwargs.get("unstable_softmax", False)
        self.disable_matmul_multi_stage_reduce = kwargs.get("disable_matmul_multi_stage_reduce", False)
        self.constant_folding_of_multiple_consumers = kwargs.get("constant_folding_of_multiple_consumers", False)
        self.use_loop_candidate_creator = kwargs.get("use_loop_candidate_creator", True)
        self.profile_name = kwargs.get("profile_name", None)
        # executor choices of this build (the reference has one executor, PopART's):
        #   allow_fused   map a known decoder loop onto the fused executors (else: op by op)
        #   strict        fail compilation instead of falling back to the op-by-op interpreter
        #   persistent    one launch per loop iteration where the model allows it (INT4 Llama 2, batch <= 16); that
        #                 kernel occupies every compute unit while it runs: nothing else may run on the device beside it
        #   prompt_passes take the prompt's positions in passes of up to 1024 rows instead of one per iteration
        #   fp8_cache     KV caches hold F143 bytes, as the KVCache op does with fp8 = true (per operator and persistent)
        self.allow_fused = kwargs.get("allow_fused", True)
        self.executor_options = {k: kwargs[k] for k in ("strict", "persistent", "prompt_passes", "fp8_cache") if k in kwargs}
        self.enable_pipeline = REGISTRY.get("enable_pipeline")
        self.batch_per_step = REGISTRY.get("batch_per_step")

    logger = property(lambda self: REGISTRY.get("logger"))

    def compile(self, model):
        self.model = model
        self.data_flow = popart.DataFlow(self.batch_per_step, model.model_output)
        n = pow(2, math.ceil(math.log2(max(model.stage_num * model.num_replicas, 1))))
        self.device_info = popart.DeviceManager().acquireAvailableDevice(n)
        self.options = self._build_options()
        self.session = popart.InferenceSession(fnModel=model.model_proto, deviceInfo=self.device_info,
                                               dataFlow=self.data_flow, userOptions=self.options)
        self.session.allow_fused = self.allow_fused
        self.session.executor_options = self.executor_options
        self.session.prepareDevice()
        self.session.weightsFromHost()
        self._anchor_arrays = self.session.initAnchorArrays()

    def _build_options(self):
        o = popart.SessionOptions()
        o.enableOutlining = not self.disable_outlining
        o.enableNonStableSoftmax = self.unstable_softmax
        o.enableReplicatedGraphs = self.model.num_replicas != 1
        o.replicatedGraphCount = self.model.num_replicas
        o.enableConstantFoldingOfMultipleConsumers = self.constant_folding_of_multiple_consumers
        o.useLoopCandidateCreator = self.use_loop_candidate_creator
        o.enablePipelining = self.enable_pipeline
        if self.execution_cache_name:
            o.enableEngineCaching, o.cachePath = True, self.execution_cache_name
        return o

    def run(self, input_dict):
        self.session.run(popart.PyStepIO(input_dict, self.anchor_arrays))

    @property
    def anchor_arrays(self):
        return self._anchor_arrays

    @property
    def executor_kind(self):
        """'interpreter', 'fused:<family>' or 'fused:llama2:persistent'."""
        return self.session.executor.kind

    @property
    def fallback_reason(self):
        """Why the graph runs on the op-by-op interpreter although fused executors were allowed (else None)."""
        return getattr(self.session.executor, "fallback_reason", None)
