"""Op-by-op execution of a recorded graph on the GPU.

This is the unfused execution mode: every node recorded through `poptransformer_amd.ops` runs as its
own step over torch device tensors, with the reference's native operators (KVCache, SoftmaxV3,
NormCE, Int4ToHalf, CastToUint8, FP8MatMul) going through libpoptransformer_hip.so exactly as the
fused path does.  It defines what a graph means, serves graphs that the fused executors do not
recognise, and is the yardstick against which a fused executor is validated when a graph is compiled
(engine/compiler.py).  Node semantics follow the ONNX / PopART operators that
poptransformer/ops/popart.py and customized.py emit.
"""
import numpy as np
import torch

from .. import kernels as K
from ..popart import NP_OF, popart_exception

_TORCH_OF = {"FLOAT16": torch.float16, "FLOAT": torch.float32, "INT32": torch.int32, "INT64": torch.int64,
             "INT8": torch.int8, "UINT8": torch.uint8, "BOOL": torch.bool, "UINT32": torch.int64}


def _align(a, b):
    """ONNX wants equal element types; graphs written against PopART sometimes multiply by a
    one-element constant of another float type - it takes the other operand's type."""
    if a.dtype == b.dtype:
        return a, b
    if b.numel() == 1 and a.is_floating_point() and b.is_floating_point():
        return a, b.to(a.dtype)
    if a.numel() == 1 and a.is_floating_point() and b.is_floating_point():
        return a.to(b.dtype), b
    if not a.is_floating_point() and not b.is_floating_point():
        t = torch.promote_types(a.dtype, b.dtype)
        return a.to(t), b.to(t)
    raise popart_exception(f"operands of different element types: {a.dtype} and {b.dtype}")


class Interpreter:
    def __init__(self, graph, device="cuda"):
        self.graph, self.dev = graph, device
        self.weights = {}          # initializer id -> device tensor
        self.consts = {}           # node output id -> (host array, device tensor)
        self.state = {}            # per-node persistent state (KV caches)
        self._upload(graph)

    # ------------------------------------------------------------------ set-up
    def _upload(self, g):
        for tid, arr in g.initializers.items():
            a = arr.astype(np.float32) if arr.dtype == np.float64 else arr
            self.weights[tid] = torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)
        for n in g.nodes:
            if n.op == "aiOnnx.constant":
                v = np.asarray(n.attrs["value"])
                hv = v.astype(np.float32) if v.dtype == np.float64 else v
                self.consts[n.outputs[0]] = (v, torch.from_numpy(np.ascontiguousarray(hv)).to(self.dev))
        for c in g.children:
            self._upload(c)

    def reset(self):
        self.state.clear()

    # ------------------------------------------------------------------ execution
    def run_graph(self, g, env):
        for n in g.nodes:
            self._exec(n, env)

    def _get(self, env, tid):
        e = env
        while e is not None:
            if tid in e:
                return e[tid]
            e = e.get("__parent__")
        if tid in self.weights:
            return self.weights[tid]
        if tid in self.consts:
            return self.consts[tid][1]
        raise popart_exception(f"tensor '{tid}' has no value")

    def _host_const(self, tid):
        if tid in self.consts:
            return self.consts[tid][0]
        raise popart_exception(f"'{tid}' must be a constant (its value shapes the graph)")

    def _exec(self, n, env):
        op = n.op
        if op == "aiOnnx.constant":
            return
        ins = [self._get(env, t) for t in n.inputs] if op not in ("aiOnnx.reshape", "aiOnnx.expand", "aiOnnx.tile", "aiOnnx.topk") \
            else [self._get(env, n.inputs[0])]
        fn = getattr(self, "_" + op.replace(".", "_"), None)
        if fn is None:
            raise NotImplementedError(f"operator {op} is not implemented")
        if self.shape_trace is not None and op.startswith("custom."):
            self.shape_trace.setdefault(op, []).append([tuple(t.shape) for t in ins])
        if self.input_trace is not None and op in self.input_trace:
            self.input_trace[op].append([v.detach().cpu().numpy() if torch.is_tensor(v) else v for v in ins])
        out = fn(n, env, *ins)
        if self.value_trace is not None and op in self.value_trace:
            vals = out if isinstance(out, (list, tuple)) else [out]
            self.value_trace[op].append([v.detach().cpu().numpy() for v in vals])
        if isinstance(out, (list, tuple)):
            for t, v in zip(n.outputs, out):
                env[t] = v
        else:
            env[n.outputs[0]] = out

    # ------------------------------------------------------------------ arithmetic
    def _aiOnnx_add(self, n, env, a, b): a, b = _align(a, b); return a + b
    def _aiOnnx_sub(self, n, env, a, b): a, b = _align(a, b); return a - b
    def _aiOnnx_mul(self, n, env, a, b): a, b = _align(a, b); return a * b
    def _aiOnnx_div(self, n, env, a, b): a, b = _align(a, b); return a / b
    def _aiOnnx_less(self, n, env, a, b): a, b = _align(a, b); return a < b
    def _aiOnnx_greater(self, n, env, a, b): a, b = _align(a, b); return a > b
    def _aiOnnx_equal(self, n, env, a, b): a, b = _align(a, b); return a == b
    def _aiGraphcore_bitwiseor(self, n, env, a, b): a, b = _align(a, b); return a | b
    def _aiGraphcore_bitwiseand(self, n, env, a, b): a, b = _align(a, b); return a & b
    def _aiOnnx_tanh(self, n, env, x): return torch.tanh(x)
    def _aiOnnx_relu(self, n, env, x): return torch.relu(x)
    def _aiOnnx_sigmoid(self, n, env, x): return torch.sigmoid(x)
    def _aiOnnx_exp(self, n, env, x): return torch.exp(x)
    def _aiOnnx_sqrt(self, n, env, x): return torch.sqrt(x)
    def _aiOnnx_sin(self, n, env, x): return torch.sin(x)
    def _aiOnnx_cos(self, n, env, x): return torch.cos(x)
    def _aiOnnx_reciprocal(self, n, env, x): return torch.reciprocal(x)
    def _aiOnnx_mean(self, n, env, *xs): return xs[0] if len(xs) == 1 else torch.stack(xs).float().mean(0).to(xs[0].dtype)
    def _aiOnnx_sum(self, n, env, *xs):
        out = xs[0]
        for x in xs[1:]:
            out = out + x
        return out
    def _aiGraphcore_gelu(self, n, env, x): return torch.nn.functional.gelu(x, approximate="tanh")
    def _aiGraphcore_swish(self, n, env, x): return torch.nn.functional.silu(x)
    def _aiOnnx_where(self, n, env, c, a, b):
        a, b = _align(a, b)
        return torch.where(c.bool(), a, b)
    def _aiOnnx_clip(self, n, env, x): return torch.clamp(x, min=n.attrs.get("min"), max=n.attrs.get("max"))
    def _aiOnnx_reducesum(self, n, env, x):
        return x.sum(dim=tuple(n.attrs["axes"]), keepdim=bool(n.attrs.get("keepdims", 1)), dtype=x.dtype)
    def _aiOnnx_reducemean(self, n, env, x):
        return x.mean(dim=tuple(n.attrs["axes"]), keepdim=bool(n.attrs.get("keepdims", 1)))
    def _aiOnnx_matmul(self, n, env, a, b):
        if a.dtype != b.dtype:
            raise popart_exception(f"MatMul operands of different element types: {a.dtype} and {b.dtype}")
        return torch.matmul(a, b)
    def _aiOnnx_cast(self, n, env, x):
        to = n.attrs["args"][0] if n.attrs["args"] else n.attrs.get("to")
        return x.to(_TORCH_OF[to])

    # ------------------------------------------------------------------ shapes
    def _aiOnnx_reshape(self, n, env, x):
        return x.reshape([int(s) for s in self._host_const(n.inputs[1]).reshape(-1)])
    def _aiOnnx_transpose(self, n, env, x): return x.permute(*n.attrs["perm"])
    def _aiOnnx_unsqueeze(self, n, env, x):
        axes = n.attrs["args"][0] if n.attrs["args"] else n.attrs["axes"]
        for a in sorted(a if a >= 0 else a + x.dim() + len(axes) for a in axes):
            x = x.unsqueeze(a)
        return x
    def _aiOnnx_squeeze(self, n, env, x):
        axes = n.attrs["args"][0] if n.attrs["args"] else n.attrs["axes"]
        for a in sorted((a if a >= 0 else a + x.dim() for a in axes), reverse=True):
            x = x.squeeze(a)
        return x
    def _aiOnnx_expand(self, n, env, x):
        shape = [int(s) for s in self._host_const(n.inputs[1]).reshape(-1)]
        return x.expand(torch.broadcast_shapes(tuple(x.shape), tuple(shape)))
    def _aiOnnx_tile(self, n, env, x):
        return x.repeat(*[int(s) for s in self._host_const(n.inputs[1]).reshape(-1)])
    def _aiOnnx_concat(self, n, env, *xs): return torch.cat(xs, dim=n.attrs["axis"])
    def _aiOnnx_split(self, n, env, x):
        sizes = n.attrs.get("split")
        if not sizes:
            sizes = [x.shape[n.attrs["axis"]] // n.attrs["num_outputs"]] * n.attrs["num_outputs"]
        return list(torch.split(x, list(sizes), dim=n.attrs["axis"]))
    def _aiOnnx_pad(self, n, env, x):
        pads = n.attrs["pads"]
        r = x.dim()
        tp = []
        for d in reversed(range(r)):
            tp += [pads[d], pads[d + r]]
        return torch.nn.functional.pad(x, tp, mode=n.attrs.get("mode", "constant"), value=n.attrs.get("value", 0.0))
    def _aiGraphcore_slice(self, n, env, x):
        for s, e, a in zip(n.attrs["starts"], n.attrs["ends"], n.attrs["axes"]):
            x = x.narrow(a, s, min(e, x.shape[a]) - s)
        return x
    def _aiOnnx_gather(self, n, env, w, ids):
        axis = n.attrs.get("axis", 0)
        return torch.index_select(w, axis, ids.reshape(-1).long()).reshape(*w.shape[:axis], *ids.shape, *w.shape[axis + 1:])
    def _aiGraphcore_groupedgather(self, n, env, w, idx):
        g = n.attrs.get("group_size", 1)
        axis = n.attrs.get("axis", 0)
        wg = w.reshape(g, *w.shape[1:]) if w.shape[0] == g else w
        return torch.stack([torch.index_select(wg[i], axis - 1 if axis > 0 else 0, idx.reshape(g, -1)[i].long()) for i in range(g)])
    def _aiGraphcore_dynamicslice(self, n, env, x, index):
        """Window of `sizes[0]` entries starting at the device-side `index` along `axes[0]`; the start
        is never read on the host, so a step of the loop stays free of synchronisation."""
        (axis,), (size,) = n.attrs["axes"], n.attrs["sizes"]
        pos = index.reshape(-1)[:1].long() + torch.arange(size, device=x.device)
        return torch.index_select(x, axis, pos.clamp(0, x.shape[axis] - 1))
    def _aiGraphcore_dynamicupdate(self, n, env, x, index, upd):
        """x with the window at `index` replaced by `upd`; an index outside the tensor (the last loop
        iteration addresses max_length) replaces nothing."""
        (axis,), (size,) = n.attrs["axes"], n.attrs["sizes"]
        x, upd = _align(x, upd)
        out = x
        shape = [1] * x.dim()
        shape[axis] = x.shape[axis]
        ar = torch.arange(x.shape[axis], device=x.device).reshape(shape)
        for j in range(size):
            hit = ar == (index.reshape(-1)[:1].long() + j)
            out = torch.where(hit, upd.narrow(axis, j, 1), out)
        return out

    # ------------------------------------------------------------------ reductions / selection
    def _aiOnnx_softmax(self, n, env, x):
        axis = n.attrs["args"][0] if n.attrs["args"] else n.attrs.get("axis", -1)
        return torch.softmax(x, dim=axis)
    def _aiOnnx_logsoftmax(self, n, env, x):
        axis = n.attrs["args"][0] if n.attrs["args"] else n.attrs.get("axis", -1)
        return torch.log_softmax(x, dim=axis)
    def _aiOnnx_argmax(self, n, env, x):
        axis = n.attrs.get("axis", 0)
        if x.dtype == torch.float16 and axis in (-1, x.dim() - 1):
            idx = K.argmax(x.contiguous()).reshape(x.shape[:-1])
            return idx.unsqueeze(-1) if n.attrs.get("keepdims", True) else idx
        return torch.argmax(x, dim=axis, keepdim=bool(n.attrs.get("keepdims", True))).to(torch.int32)
    def _aiOnnx_topk(self, n, env, x):
        k = int(self._host_const(n.inputs[1]))
        axis = n.attrs.get("axis", -1)
        if k == 1 and x.dtype == torch.float16 and axis in (-1, x.dim() - 1):
            xc = x.contiguous()
            vals = torch.empty(xc.shape[:-1], dtype=torch.float16, device=x.device)
            idx = K.argmax(xc, values=vals).reshape(xc.shape[:-1])
            return [vals.unsqueeze(-1), idx.unsqueeze(-1)]
        if x.dtype == torch.float16 and axis in (-1, x.dim() - 1):
            xc = x.contiguous()
            vals, idx = K.topk(xc, k)
            return [vals.reshape(*xc.shape[:-1], k), idx.reshape(*xc.shape[:-1], k)]
        v, i = torch.topk(x, k, dim=axis)
        return [v, i.to(torch.int32)]
    def _aiOnnx_randomnormal(self, n, env):
        return torch.randn(n.attrs["shape"], device=self.dev) * n.attrs.get("scale", 1.0)
    def _aiGraphcore_groupnormalization(self, n, env, x, g, b):
        groups, eps = n.attrs["args"][0], n.attrs["args"][1]
        y = torch.nn.functional.group_norm(x.float(), groups, g.float(), b.float(), eps).to(x.dtype)
        return [y, y.new_zeros(1), y.new_zeros(1)]
    def _aiGraphcore_printtensor(self, n, env, x):
        print(n.attrs.get("title", ""), x)
        return x
    def _aiGraphcore_replicatedallreduce(self, n, env, x): return x

    # ------------------------------------------------------------------ control flow
    def _aiOnnx_loop(self, n, env, max_loop, cond, *carried):
        """ONNX Loop as ops.loop builds it: body inputs = [iteration bound, condition, carried...],
        body outputs = [condition, carried...]; the op returns the carried values."""
        body = n.subgraph
        names = body.inputs
        state = list(carried)
        trips = int(max_loop.item()) if torch.is_tensor(max_loop) else int(max_loop)
        if self.max_trips is not None:
            trips = min(trips, self.max_trips)
        keep = cond
        for it in range(trips):
            sub = {"__parent__": env, names[0]: max_loop, names[1]: keep}
            for name, v in zip(names[2:], state):
                sub[name] = v
            self.run_graph(body, sub)
            outs = [self._get(sub, t) for t in body.outputs]
            keep, state = outs[0], outs[1:]
            if self.loop_checks_condition and not bool(keep.item() if torch.is_tensor(keep) else keep):
                break
        return state
    loop_checks_condition = True
    max_trips = None            # cap on loop iterations (shape discovery, validation probes)
    shape_trace = None          # when a dict: operand shapes of the native operators, per op name
    value_trace = None          # when a dict {op name: []}: the outputs of every execution of those ops (host copies)
    input_trace = None          # the same for their inputs

    def _aiGraphcore_call(self, n, env, *ins):
        body = n.subgraph
        sub = {"__parent__": env}
        for name, v in zip(body.inputs, ins):
            sub[name] = v
        self.run_graph(body, sub)
        return [self._get(sub, t) for t in body.outputs]

    # ------------------------------------------------------------------ native operators
    def _custom_Remap(self, n, env, x): return x

    def _custom_KVCache(self, n, env, step, upd):
        a = n.attrs
        if a.get("fp8"):
            raise NotImplementedError("KVCache with fp8 storage")
        axis, max_len, step_len = a["sequence_axis"], a["max_len"], a["step_len"]
        if upd.shape[axis] != step_len:
            raise popart_exception(f"KVCache: updater has {upd.shape[axis]} rows along the sequence axis, step_len is {step_len}")
        if upd.dtype not in (torch.float16, torch.float32):
            raise popart_exception("KVCache: FLOAT16 or FLOAT expected")
        key = n.outputs[0]
        if key not in self.state:
            shape = list(upd.shape)
            shape[axis] = max_len
            self.state[key] = (torch.zeros(shape, dtype=upd.dtype, device=upd.device),
                               torch.zeros(shape, dtype=upd.dtype, device=upd.device))
        cache, clone = self.state[key]
        K.kv_cache_update(cache, clone, upd.contiguous(), step.reshape(()).to(torch.int32).contiguous(), axis)
        return cache

    def _custom_KVCachePipeline(self, n, env, step, upd):
        a = n.attrs
        if a.get("fp8"):
            raise NotImplementedError("KVCachePipeline with fp8 storage")
        max_len, max_bps, step_len = a["max_len"], a["max_bps"], a.get("step_len", 1)
        axis = a.get("sequence_axis", -2)
        axis = axis + upd.dim() if axis < 0 else axis
        if axis != upd.dim() - 2:
            raise popart_exception(f"[KVCachePipeline] Only support axis = {upd.dim() - 2}(or -2),but now it is {axis}.")
        if step_len != 1 or upd.shape[axis] != 1:
            raise NotImplementedError("KVCachePipeline: one new row per call (step_len = 1)")
        outer, inner = int(np.prod(upd.shape[:axis])), upd.shape[-1]
        st = step.reshape(()).to(torch.int32).contiguous()
        key = n.outputs[0]
        shape = list(upd.shape)
        shape[axis] = max_len
        out = torch.empty(shape, dtype=upd.dtype, device=upd.device)
        if a.get("transpose"):
            if key not in self.state:
                self.state[key] = torch.zeros((max_bps, outer, inner, max_len), dtype=upd.dtype, device=upd.device)
            return K.kv_cache_pipeline_seq_last(self.state[key], out, upd.contiguous(), st, outer, max_len, inner, max_bps)
        if key not in self.state:
            self.state[key] = torch.zeros((max_bps, outer, max_len, inner), dtype=upd.dtype, device=upd.device)
        # the ring addresses rows by step / max_bps: the calls must come with step = 0, 1, 2, ... as a loop issues them
        K.kv_cache_append(self.state[key], upd.contiguous(), st, outer, max_len, inner, max_bps)
        return K.kv_cache_read(self.state[key], out, st, outer, max_len, inner, max_bps)

    def _custom_BeamSearch(self, n, env, logits, hyp, prob, step):
        beam = int(n.attrs["beam_size"])
        if logits.dim() == 3 and logits.shape[1] != beam:
            raise popart_exception(f"[Beam Search] logits.shape[1]({logits.shape[1]}) should beequal to parameter "
                                   f"'beam_size'({beam}).")
        hyp, prob = hyp.to(torch.int32).contiguous().clone(), prob.contiguous().clone()
        next_id, best = K.beam_search_step(logits, hyp, prob, step.reshape(()).to(torch.int32).contiguous())
        return [next_id, best, hyp, prob]

    def _custom_SoftmaxV3(self, n, env, x):
        axis = n.attrs["axis"]
        if x.dim() < 2:
            raise popart_exception("[Softmax] rank of input should be >= 2")
        if axis not in (-1, x.dim() - 1):
            raise popart_exception("[Softmax] axis must be the last axis")
        return K.softmax_ce(x.contiguous(), bool(n.attrs["stable_mode"]))

    def _custom_NormCE(self, n, env, x, g, b):
        a = n.attrs
        if a.get("stable_algo"):
            raise popart_exception("[NormCE] stable_algo must be false")
        cols = x.shape[-1]
        if x.numel() // cols != a["num_groups"]:
            raise popart_exception("[NormCE] num_groups must equal the number of rows")
        if cols % 4 != 0:
            raise popart_exception("[NormCE] the normalised size must be a multiple of 4")
        return K.layer_norm_ce(x.contiguous(), g, b, a["epsilon"])

    def _custom_Int4ToHalf(self, n, env, x, scale, ref):
        return K.int4_to_half(x.contiguous(), scale, n.attrs.get("axis", 1))

    def _custom_CastToUint8WithoutShapeInfer(self, n, env, x, scale):
        return K.half_to_fp8(x.contiguous(), scale.reshape(-1).to(torch.int32), n.attrs.get("fp8Format", "F143"))

    def _custom_FP8MatMulWithoutShapeInfer(self, n, env, a, b, sa, sb):
        fa, fb = n.attrs.get("fp8FormatLHS", "F143"), n.attrs.get("fp8FormatRHS", "F143")
        if b.dtype != torch.uint8:
            raise popart_exception(f"Invalid weight data type of {b.dtype}, it must be UINT8")
        if a.dtype not in (torch.float16, torch.uint8):
            raise popart_exception(f"Invalid input data type of {a.dtype}, it must be FLOAT16 or UINT8")
        if a.shape[-1] != b.shape[-2]:
            raise popart_exception("FP8MatMul: contracting dimensions differ")
        bw = K.fp8_to_half(b.contiguous(), sb.reshape(-1).to(torch.int32), fb)
        if a.dtype == torch.uint8:
            aw = K.fp8_to_half(a.contiguous(), sa.reshape(-1).to(torch.int32), fa)
            return torch.matmul(aw.float(), bw.float()).half()
        return torch.matmul(a, bw)

    def _custom_ReplicatedAllGather(self, n, env, x): return x.reshape(-1)


class InterpretedProgram:
    """Executor over the interpreter with the interface the session expects."""

    def __init__(self, graph, anchors, batches_per_step=1):
        self.graph, self.anchors, self.bps = graph, list(anchors), batches_per_step
        self.interp = Interpreter(graph)
        self.kind = "interpreter"
        self.fallback_reason = None
        self._shapes = None

    def _run_once(self, feeds):
        self.interp.reset()
        env = {}
        for tid in self.graph.inputs:
            if tid in self.graph.initializers:
                continue
            if tid in feeds:
                info = self.graph.input_info.get(tid)
                arr = np.asarray(feeds[tid])
                if info is not None:
                    arr = arr.astype(NP_OF[info.dtype]).reshape(info.shape())
                env[tid] = torch.from_numpy(np.ascontiguousarray(arr)).to(self.interp.dev)
        self.interp.run_graph(self.graph, env)
        torch.cuda.synchronize()
        return {a: self.interp._get(env, a).cpu().numpy() for a in self.anchors}

    def run(self, feeds):
        if self.bps == 1:
            return self._run_once(feeds)
        outs = []
        for i in range(self.bps):
            outs.append(self._run_once({k: np.asarray(v).reshape(self.bps, -1)[i] for k, v in feeds.items()}))
        return {a: np.stack([o[a] for o in outs]) for a in self.anchors}

    def anchor_arrays(self):
        """Output buffers, shaped by a dry run on zero inputs when the shapes are not known yet."""
        if self._shapes is None:
            feeds = {t: np.zeros(i.shape(), NP_OF[i.dtype]) for t, i in self.graph.input_info.items()}
            self.interp.max_trips = 1
            try:
                self._shapes = {a: v for a, v in self._run_once(feeds).items()}
            finally:
                self.interp.max_trips = None
        lead = [self.bps] if self.bps > 1 else []
        return {a: np.zeros(lead + list(v.shape), v.dtype) for a, v in self._shapes.items()}
