"""Fused executor of the decode loop for decoder-only transformers.

The reference runs one PopART `Loop` whose body is the model graph followed by the container /
stop-mask bookkeeping (poptransformer/models/base_model.py:271-355), everything on the device.
Here the same loop body is a fixed sequence of HIP kernel launches over persistent device
buffers, recorded once into a HIP graph and replayed per token; `step`, the id container and
the stop mask live in device memory exactly as they are graph tensors in the reference, so a
replay needs no host data.

The executor is parameterised by a `DecoderSpec` (what a transformer block looks like) and by
prepared weights; sessions.py builds both from a recorded model graph.  Supported block
shapes: GPT-2 (models/gpt2), Llama 2 (models/llama2), ChatGLM2 (models/chatglm2).
"""
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np
import torch

from .. import _lib
from .. import kernels as K


@dataclass
class DecoderSpec:
    family: str                      # 'gpt2' | 'llama2' | 'chatglm2'
    n_layer: int
    d_model: int
    n_head: int
    n_kv_head: int
    head_dim: int
    vocab: int
    max_len: int
    batch: int
    eps: float
    pad_id: int = 0
    eos_id: int = -1
    early_stop: bool = False
    topk: int = 1                    # > 1: the next token is one of the top-k, drawn as ops.random_sample does
    fp8_cache: bool = False          # KV rings hold F143 bytes with metadata scale 1 (KVCacheOp with fp8 = true)

    @property
    def norm(self):
        return "ln" if self.family == "gpt2" else "rms"

    @property
    def rope(self):
        return {"gpt2": _lib.ROPE_NONE, "llama2": _lib.ROPE_LLAMA, "chatglm2": _lib.ROPE_GLM2}[self.family]

    @property
    def scale_scores(self):
        # GPT-2 folds 1/sqrt(D) into the query weights at load (models/gpt2/model.py:154-166)
        return self.family != "gpt2"


class LinearWeights:
    """One Linear: a tiled weight (INT4, FP16 or FP8), an optional fp16 bias and, for FP8 weights,
    whether the activations are cast to FP8 first (precision 'fp8') or stay fp16 ('fp8_weight')."""

    def __init__(self, weight, bias=None, act_fp8=False, scale_value=None):
        self.w, self.bias, self.act_fp8 = weight, bias, act_fp8
        self.N, self.K = weight.N, weight.K
        self.scale_value = scale_value            # host copy of the FP8 exponent (for grouping)

    @property
    def is_int4(self):
        return isinstance(self.w, K.W4Weight)

    @property
    def is_fp8(self):
        return isinstance(self.w, K.F8Weight)

    def group_key(self):
        """Linears with equal keys can share one launch (same weight kind; for FP8 also the same
        format, activation handling and exponent, since they share the cast activations)."""
        if self.is_fp8:
            return ("fp8", self.w.format, self.act_fp8, self.scale_value if self.act_fp8 else None)
        return ("int4",) if self.is_int4 else ("f16",)

    @property
    def nbytes(self):
        return self.w.nbytes + (self.bias.numel() * 2 if self.bias is not None else 0)


@dataclass
class BlockWeights:
    norm1: tuple                      # (gamma, beta or None)
    norm2: tuple
    qkv: List[LinearWeights]          # [q, k, v] or [fused qkv] or [q, kv]
    out: LinearWeights
    mlp_in: List[LinearWeights]       # [gate, up] (SwiGLU) or [fc] (GELU)
    mlp_out: LinearWeights


@dataclass
class ModelWeights:
    embed: torch.Tensor               # [V, d] fp16
    pos_embed: Optional[torch.Tensor]
    blocks: List[BlockWeights]
    final_norm: tuple
    head: LinearWeights
    inv_freq: Optional[torch.Tensor] = None

    def nbytes(self):
        n = self.head.nbytes
        for b in self.blocks:
            for lw in b.qkv + [b.out] + b.mlp_in + [b.mlp_out]:
                n += lw.nbytes
            for g in (b.norm1, b.norm2):
                n += sum(t.numel() * 2 for t in g if t is not None)
        n += sum(t.numel() * 2 for t in self.final_norm if t is not None)
        return n


class LayerOps:
    """The per-layer operators over `rows` activation rows: the row buffers and the calls that the decode
    iteration (rows = batch) and the prompt passes (rows = batch * positions) share."""

    def __init__(self, spec: DecoderSpec, weights: ModelWeights, device, rows):
        self.spec, self.w, self.dev, self._rows = spec, weights, device, rows
        s, f16 = spec, torch.float16

        def buf(*shape, dtype=f16):
            return torch.zeros(shape, dtype=dtype, device=device)

        self._buf = buf
        d, ffn = s.d_model, weights.blocks[0].mlp_out.K
        self.x, self.h, self.ctx = buf(rows, d), buf(rows, d), buf(rows, d)
        self.qkv = buf(rows, sum(lw.N for lw in weights.blocks[0].qkv))
        self.q_rot = buf(rows, s.n_head, s.head_dim)
        self.act = buf(rows, ffn)
        self.attn_ws = K.decode_attention_workspace(rows, s.n_head, s.head_dim, s.max_len, device)
        # The norm inside the GEMM: every workgroup normalises the rows it stages.  Up to 4 rows that is cheaper than
        # a launch of its own since the rows' sums over a wave are made by data-parallel moves (Llama 2 at the 7B
        # width, batch 1, one launch per operator: 1.687 -> 1.593 ms per step; with shuffles it cost 5 us per
        # launch and lost).  At batch 16 it costs 4 us per launch against a 4.4 us kernel, and two of the three
        # GEMMs that follow a norm each pay for it: separate there.  The kernels support up to 16 rows.
        self.fuse_norm = rows <= 4 and K.norm_fusable(rows, d)
        # fp16 staging of activations rounded to the FP8 grid, one buffer per input width
        self._fp8_buf = {k: buf(rows, k) for k in {d, ffn}}
        self._gate, self._up = buf(rows, ffn), buf(rows, ffn)
        self._on_grid = {}      # buffer address -> the FP8 grid (format, exponent) its values are on
        # scratch that lets a Linear of more than 16 rows with few output channels (attention output, MLP down) split K
        self._lin_ws = K.linear_workspace(rows, d, device) if rows > 16 else None

    def _norm(self, x, gb, out):
        if self.spec.norm == "rms":
            return K.rmsnorm(x, gb[0], self.spec.eps, out)
        return K.layer_norm_ce(x, gb[0], gb[1], self.spec.eps, out)

    def _normed(self, x, gb, consumers):
        """Input and fused-norm argument for the Linears `consumers` of norm(x): the norm runs inside the
        GEMM when the shape allows it, as a kernel of its own into self.h otherwise (always when a consumer
        casts its input to FP8 first: the cast needs the normalised values)."""
        if self.fuse_norm and not any(lw.is_fp8 and lw.act_fp8 for lw in consumers):
            return x, K.Norm(gb[0], gb[1], self.spec.eps)
        grid = self._common_grid(consumers)
        if grid is not None and self.spec.norm == "rms":
            # every consumer casts its input to the same FP8 grid: the norm leaves its rows on it
            buf = self._fp8_buf[x.shape[1]]
            K.rmsnorm_fp8_grid(x, gb[0], self.spec.eps, grid[0], grid[1], out=buf)
            self._on_grid[buf.data_ptr()] = self._grid_id(consumers[0])
            return buf, None
        self._norm(x, gb, self.h)
        return self.h, None

    @staticmethod
    def _grid_id(lw):
        """Identifies the FP8 grid an FP8 Linear casts its input to: format and exponent (by value when the
        loader recorded it, else by the tensor that holds it)."""
        key = lw.scale_value if lw.scale_value is not None else ("at", lw.w.scale.data_ptr())
        return (lw.w.format, key)

    @classmethod
    def _common_grid(cls, consumers):
        """(scale tensor, format name) when all `consumers` are FP8 Linears that cast their input to one and
        the same grid, else None."""
        if not consumers or not all(lw.is_fp8 and lw.act_fp8 for lw in consumers):
            return None
        if len({cls._grid_id(lw) for lw in consumers}) != 1:
            return None
        first = consumers[0].w
        return first.scale, ("F143" if first.format == _lib.F143 else "F152")

    def _lhs(self, x, lw, norm):
        """Left-hand side for a Linear: FP8 activations are rounded to the FP8 grid first
        (half_to_uint8 of precision_strategy.py:62-66), everything else passes through."""
        if not (lw.is_fp8 and lw.act_fp8):
            return x, None, norm
        if norm is not None:                      # the cast needs the normalised values
            raise NotImplementedError("fused norm is not combined with FP8 activations")
        if self._on_grid.get(x.data_ptr()) == self._grid_id(lw):
            return x, lw.w.scale, None            # its producer already left x on this Linear's grid
        buf = self._fp8_buf[x.shape[1]]
        self._on_grid.pop(buf.data_ptr(), None)
        K.half_to_fp8_grid(x, lw.w.scale, "F143" if lw.w.format == _lib.F143 else "F152", out=buf)
        return buf, lw.w.scale, None

    def _linear(self, x, lw, out, residual=None, act=_lib.ACT_NONE, norm=None):
        xin, xs, norm = self._lhs(x, lw, norm)
        self._on_grid.pop(out.data_ptr(), None)
        K.linear(xin, [lw.w], [out], x_scale=xs, bias=lw.bias, residual=residual, act=act, norm=norm,
                 workspace=self._lin_ws)
        return out

    def _linear_group(self, x, lws, outs, norm=None, swiglu=False, consumer=None):
        """Several Linears on the same input: one launch when they are alike, else one each.  `consumer`: the
        Linear that takes the SwiGLU result; when it casts its input to FP8 the pair's launch does that cast."""
        keys = {lw.group_key() for lw in lws}
        for o in outs:
            self._on_grid.pop(o.data_ptr(), None)
        if len(keys) == 1 and (not swiglu or all(lw.bias is None for lw in lws)):
            xin, xs, norm = self._lhs(x, lws[0], norm)
            grid = self._common_grid([consumer]) if swiglu and consumer is not None else None
            K.linear(xin, [lw.w for lw in lws], outs, biases=[lw.bias for lw in lws], x_scale=xs, swiglu=swiglu, norm=norm,
                     out_grid=grid)
            if grid is not None:
                self._on_grid[outs[0].data_ptr()] = self._grid_id(consumer)
            return
        if swiglu:                                 # unlike weights: two launches and the elementwise form
            self._linear(x, lws[0], self._gate, norm=norm)
            self._linear(x, lws[1], self._up, norm=norm)
            K.swiglu(self._gate, self._up, outs[0])
            return
        for lw, o in zip(lws, outs):
            self._linear(x, lw, o, norm=norm)

    def _prepare_qkv_views(self, blk):
        """Output buffers of the projections and the (pointer, row stride) views of q, k, v."""
        s = self.spec
        B, Hq, Hkv, D = self._rows, s.n_head, s.n_kv_head, s.head_dim
        f16 = torch.float16
        if len(blk.qkv) == 1:           # GPT-2: one row holds q | k | v
            row = (Hq + 2 * Hkv) * D
            self._qkv_bufs = [self.qkv]
            self._qkv_views = (self.qkv, self.qkv[:, Hq * D:], self.qkv[:, (Hq + Hkv) * D:], row, row, row)
        elif len(blk.qkv) == 3:         # Llama 2: separate q, k, v
            self._qkv_bufs = [torch.zeros((B, lw.N), dtype=f16, device=self.dev) for lw in blk.qkv]
            q, k, v = self._qkv_bufs
            self._qkv_views = (q, k, v, Hq * D, Hkv * D, Hkv * D)
        else:                           # ChatGLM2: query, and key_value holding k | v
            self._qkv_bufs = [torch.zeros((B, lw.N), dtype=f16, device=self.dev) for lw in blk.qkv]
            q, kv = self._qkv_bufs
            self._qkv_views = (q, kv, kv[:, Hkv * D:], Hq * D, 2 * Hkv * D, 2 * Hkv * D)


class NextToken:
    """LMHead's selection (layers/lm_head.py:52-56) over the logits of one iteration: top-1, or with topk > 1
    ops.random_sample (ops/popart.py:25-29): the top-k ids, then the column chosen by the argmax of k normal
    draws, one draw per iteration for the whole batch."""

    def __init__(self, batch, vocab, topk, device):
        if topk < 1 or topk > vocab:
            raise ValueError(f"topk = {topk} outside [1, vocabulary size {vocab}]")
        self.topk = topk
        if topk > 1:
            i32, f16 = torch.int32, torch.float16
            self.ids = torch.zeros((batch, topk), dtype=i32, device=device)
            self.vals = torch.zeros((batch, topk), dtype=f16, device=device)
            self.draws = torch.zeros((1, topk), dtype=f16, device=device)
            self.pick = torch.zeros((1,), dtype=i32, device=device)

    def __call__(self, logits, next_ids):
        if self.topk == 1:
            K.argmax(logits, next_ids)
            return
        K.topk(logits, self.topk, self.ids, self.vals)
        self.draws.normal_()
        K.argmax(self.draws, self.pick)
        K.take_column(self.ids, self.pick, next_ids)


class FusedDecoder(LayerOps):
    def __init__(self, spec: DecoderSpec, weights: ModelWeights, device="cuda"):
        super().__init__(spec, weights, device, spec.batch)
        s, buf = spec, self._buf
        B = s.batch
        i32 = torch.int32
        self.logits = buf(B, s.vocab)
        self.next_ids = buf(B, dtype=i32)
        self.select = NextToken(B, s.vocab, s.topk, device)
        self.container = buf(B, s.max_len, dtype=i32)
        self.mask = buf(B, s.max_len)
        self.stop_mask = buf(B, dtype=i32)
        self.step = torch.zeros((), dtype=i32, device=device)
        self.keep_going = torch.ones((), dtype=i32, device=device)
        # one ring per layer: keys then values, [2*B*Hkv, max_len, D]
        self.kv_scale = 1 if s.fp8_cache else None        # the constant of custom_ops/kv_cache.cpp:45
        self.rings = [buf(2 * B * s.n_kv_head, s.max_len, s.head_dim, dtype=torch.uint8 if s.fp8_cache else torch.float16)
                      for _ in range(s.n_layer)]
        self.graph = None
        self._stream = torch.cuda.Stream()
        self.persistent = None
        self.probe = None                # callable(name, block index, tensor or tensors): looks into eager iterations of the per-operator path

    def enable_persistent(self):
        """Run each loop iteration as one persistent launch (pta_llama_decode_step) instead of one
        launch per operator.  Raises NotImplementedError when the model is not an INT4 Llama-2
        shape the kernel covers; the per-operator path stays available through `persistent = None`."""
        s, w = self.spec, self.w
        if s.topk != 1:
            raise NotImplementedError("the persistent decode step selects greedily (topk = 1)")
        if s.family != "llama2" or s.n_kv_head != s.n_head:
            raise NotImplementedError("the persistent decode step covers Llama-2 blocks with as many KV heads as heads")
        lins = [lw for b in w.blocks for lw in b.qkv + [b.out] + b.mlp_in + [b.mlp_out]]
        if not all(lw.is_int4 and lw.bias is None for lw in lins):
            raise NotImplementedError("the persistent decode step needs bias-free INT4 Linears")
        if not isinstance(w.head.w, K.F16Weight) or w.head.bias is not None:
            raise NotImplementedError("the persistent decode step needs a bias-free fp16 lm_head")
        layers = []
        for b, ring in zip(w.blocks, self.rings):
            q, k, v = b.qkv
            g, u = b.mlp_in
            layers.append(dict(wq=q.w.tiled, wk=k.w.tiled, wv=v.w.tiled, wo=b.out.w.tiled, wg=g.w.tiled, wu=u.w.tiled,
                               wd=b.mlp_out.w.tiled, sq=q.w.scale, sk=k.w.scale, sv=v.w.scale, so=b.out.w.scale,
                               sg=g.w.scale, su=u.w.scale, sd=b.mlp_out.w.scale, norm1=b.norm1[0], norm2=b.norm2[0],
                               kv_ring=ring))
        state = dict(container=self.container, mask=self.mask, stop_mask=self.stop_mask, step=self.step,
                     keep_going=self.keep_going, next_ids=self.next_ids, logits=self.logits)
        self.persistent = K.DecodeStep(layers, w.embed, w.final_norm[0], w.head.w.tiled, w.inv_freq, s.batch, s.d_model,
                                       s.n_head, s.head_dim, w.blocks[0].mlp_out.K, s.vocab, s.max_len, s.eps, s.pad_id,
                                       s.eos_id, s.early_stop, state, kv_scale=self.kv_scale)
        return self

    def step_fn(self):
        if self.persistent is not None:
            self.persistent.launch()
            return
        s, w = self.spec, self.w
        B = s.batch
        K.embedding(w.embed, self.container, self.x, pos_table=w.pos_embed,
                    pos=self.step if w.pos_embed is not None else None, ids_index=self.step)
        for li, blk in enumerate(w.blocks):
            if not hasattr(self, "_qkv_views"):
                self._prepare_qkv_views(blk)
            probe = self.probe                           # diagnostics of eager iterations: callable(name, block, tensor(s))
            if probe is not None:
                probe("block_in", li, self.x)
            h, nrm = self._normed(self.x, blk.norm1, blk.qkv)
            self._linear_group(h, blk.qkv, self._qkv_bufs, nrm)
            if probe is not None:
                probe("projections", li, self._qkv_bufs)
            qp, kp, vp, qs, ks, vs = self._qkv_views
            # the output projection's cast of its input to FP8 is done by the attention where it stores the context
            grid = self._common_grid([blk.out]) if self.kv_scale is None else None
            self._on_grid.pop(self.ctx.data_ptr(), None)
            K.decode_attention_qkv(qp, kp, vp, self.rings[li], self.step, w.inv_freq, self.attn_ws, self.ctx, B,
                                   s.n_head, s.n_kv_head, s.head_dim, s.max_len, s.rope, s.scale_scores, qs, ks, vs,
                                   kv_scale=self.kv_scale, out_grid=grid)
            if grid is not None:
                self._on_grid[self.ctx.data_ptr()] = self._grid_id(blk.out)
            self._linear(self.ctx, blk.out, self.x, residual=self.x)
            if probe is not None:
                probe("after_attention", li, self.x)
            h, nrm = self._normed(self.x, blk.norm2, blk.mlp_in)
            if len(blk.mlp_in) == 2:
                self._linear_group(h, blk.mlp_in, [self.act, self.act], nrm, swiglu=True, consumer=blk.mlp_out)
            else:
                self._linear(h, blk.mlp_in[0], self.act, act=_lib.ACT_GELU_TANH, norm=nrm)
            self._linear(self.act, blk.mlp_out, self.x, residual=self.x)
        if self.probe is not None:                       # ... and the stream leaving the last block
            self.probe("block_in", len(w.blocks), self.x)
        h, nrm = self._normed(self.x, w.final_norm, [w.head])
        self._linear(h, w.head, self.logits, norm=nrm)
        self.select(self.logits, self.next_ids)
        K.step_update(self.container, self.mask, self.stop_mask, self.step, self.next_ids, None, self.keep_going,
                      s.pad_id, s.eos_id, s.early_stop)

    # ------------------------------------------------------------------ loop
    def reset(self, input_ids):
        """Initial loop state of build_model_graph_inputs (models/base_model.py:255-269)."""
        s = self.spec
        ids = torch.as_tensor(np.asarray(input_ids, np.int32))
        if tuple(ids.shape) != (s.batch, s.max_len):
            raise ValueError(f"input_ids must be [{s.batch}, {s.max_len}], got {tuple(ids.shape)}")
        self._host_ids = ids.numpy().copy()
        self.container.copy_(ids)
        self.mask.fill_(-10000.0)
        self.mask[:, 0] = 0
        self.stop_mask.zero_()
        self.step.zero_()
        self.keep_going.fill_(1)

    def prompt_positions(self):
        """How many leading loop iterations only read the prompt: their `next_ids` are dropped because the
        container already holds a token at the next position (models/base_model.py:313-318), and no
        sequence meets its end token there.  These are the positions `consume_prompt` may take at once."""
        s, ids = self.spec, self._host_ids
        n = s.max_len - 1
        for row in ids:
            later = row[1:]
            pads = np.nonzero(later == s.pad_id)[0]
            ends = np.nonzero(later == s.eos_id)[0]
            n = min(n, int(pads[0]) if len(pads) else s.max_len - 1, int(ends[0]) if len(ends) else s.max_len - 1)
        return max(n, 0)

    def consume_prompt(self, n=None, rows_per_pass=None):
        """Runs the first `n` loop iterations (default: `prompt_positions()`) as passes over up to
        `rows_per_pass` consecutive positions of every sequence at once instead of one position per iteration.
        Each weight matrix is then read once per pass instead of once per position.  The KV rings and the loop
        state end up as `n` iterations of the loop leave them; the logits of these positions are not computed
        (the loop would discard their tokens).  Call after `reset`.  Returns n."""
        from .prompt import PromptPass
        s = self.spec
        limit = self.prompt_positions()
        n = limit if n is None else int(n)
        if n < 0 or n > limit:
            raise ValueError(f"consume_prompt: n = {n} outside [0, {limit}] (the prompt's own positions before any end token)")
        if int(self.step.item()) != 0:
            raise RuntimeError("consume_prompt must follow reset()")
        if n == 0:
            return 0
        # by default passes of up to 1024 rows: from a few hundred rows on the projections run on the kernel whose
        # workgroups take 128-row panels, at 2-3 times the rate per row of the 64-row kernels
        R = max(1, min(n, 1024 // s.batch)) if rows_per_pass is None else int(rows_per_pass)
        if R < 1 or R * s.batch > 2048:
            raise ValueError(f"consume_prompt: rows_per_pass * batch must lie in [1, 2048], got {R} * {s.batch}")
        if not hasattr(self, "_prompt_passes"):
            self._prompt_passes = {}
        with torch.cuda.stream(self._stream):
            p0 = 0
            while p0 < n:
                rc = min(R, n - p0)
                if rc not in self._prompt_passes:
                    self._prompt_passes[rc] = PromptPass(self, rc)
                self._prompt_passes[rc].run(p0)
                p0 += rc
            # the state n iterations leave behind (pta_step_update n times): positions 0..n open, no stop
            self.mask[:, :n + 1] = 0
            self.step.fill_(n)
        self._stream.synchronize()
        return n

    def capture(self):
        """Record one loop iteration into a HIP graph (after an eager iteration has warmed up
        every code path).  The iteration depends on device state only, so it can be replayed."""
        self.reset(np.zeros((self.spec.batch, self.spec.max_len), np.int32))
        with torch.cuda.stream(self._stream):
            self.step_fn()
            torch.cuda.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=self._stream):
                self.step_fn()
        torch.cuda.synchronize()
        return self.graph

    def run_steps(self, n):
        if self.graph is None:
            for _ in range(n):
                self.step_fn()
        else:
            for _ in range(n):
                self.graph.replay()

    def run(self, input_ids, max_loop, check_every=16, prompt_passes=False):
        """The whole generation (one `session.run` of the reference, poptransformer/sessions.py:47-49).
        Returns (container, step) like the anchors 'Loop:0' and 'Loop:1'.  prompt_passes: the leading
        iterations that only read the prompt run as passes over several positions (consume_prompt)."""
        self.reset(input_ids)
        done = 0
        if prompt_passes:
            n = min(self.prompt_positions(), max_loop)
            if n > 0:
                done = self.consume_prompt(n)
        while done < max_loop:
            n = min(check_every, max_loop - done) if self.spec.early_stop else max_loop - done
            self.run_steps(n)
            done += n
            if self.spec.early_stop and int(self.keep_going.item()) == 0:
                break
        torch.cuda.synchronize()
        if self.persistent is not None and self.persistent.failed():
            raise RuntimeError("persistent decode step: a workgroup gave up waiting (the kernel needs every compute unit "
                               "of the device for itself while it runs); the loop state was not advanced past the failing "
                               "iteration.  The failure word is sticky: persistent.clear_failure() re-arms the decoder")
        return self.container.cpu().numpy(), int(self.step.item())
