"""Fused executor of the RWKV-4 decode loop (recurrent: per-block states instead of a KV cache).

Reference graph: poptransformer/models/rwkv/model.py:96-119 (blocks, rescaling), :157-187 (state
initialisation), :189-232 (loop body and carried states), attention.py:66-105, ffn.py:47-59.
One loop iteration is a fixed sequence of HIP kernels over persistent device buffers, recorded
into a HIP graph like the transformer executor (engine/fused.py).
"""
from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import torch

from .. import _lib
from .. import kernels as K
from .fused import LinearWeights, NextToken


@dataclass
class RWKVSpec:
    n_layer: int
    d_model: int
    attn_dim: int
    ffn: int
    vocab: int
    max_len: int
    batch: int
    eps: float
    rescale_every: int
    pad_id: int = 0
    eos_id: int = -1
    early_stop: bool = False
    topk: int = 1                    # > 1: ops.random_sample among the top-k (layers/lm_head.py:52-53)


@dataclass
class RWKVBlockWeights:
    pre_ln: Optional[tuple]
    ln1: tuple
    ln2: tuple
    att_key: LinearWeights
    att_value: LinearWeights
    att_receptance: LinearWeights
    att_output: LinearWeights
    time_decay: torch.Tensor
    time_first: torch.Tensor
    att_mix: List[torch.Tensor]          # key, value, receptance
    ffn_key: LinearWeights
    ffn_receptance: LinearWeights
    ffn_value: LinearWeights
    ffn_mix: List[torch.Tensor]          # key, receptance


@dataclass
class RWKVWeights:
    embed: torch.Tensor
    blocks: List[RWKVBlockWeights]
    ln_out: tuple
    head: LinearWeights

    def nbytes(self):
        n = self.head.nbytes
        for b in self.blocks:
            for lw in (b.att_key, b.att_value, b.att_receptance, b.att_output, b.ffn_key, b.ffn_receptance, b.ffn_value):
                n += lw.nbytes
        return n


class RWKVDecoder:
    def __init__(self, spec: RWKVSpec, weights: RWKVWeights, device="cuda"):
        self.spec, self.w, self.dev = spec, weights, device
        s = spec
        B, d, A, f = s.batch, s.d_model, s.attn_dim, s.ffn
        if A != d:
            raise NotImplementedError("attention_hidden_size must equal hidden_size (states are [B, hidden])")
        f16, i32, f32 = torch.float16, torch.int32, torch.float32

        def buf(*shape, dtype=f16):
            return torch.zeros(shape, dtype=dtype, device=device)

        self.x, self.x2, self.h = buf(B, d), buf(B, d), buf(B, d)
        self.mix = [buf(B, d) for _ in range(3)]
        self.k, self.v, self.r, self.y = buf(B, A), buf(B, A), buf(B, A), buf(B, A)
        self.fk, self.fr = buf(B, f), buf(B, d)
        self.logits = buf(B, s.vocab)
        self.next_ids = buf(B, dtype=i32)
        self.select = NextToken(B, s.vocab, s.topk, device)
        self.container = buf(B, s.max_len, dtype=i32)
        self.stop_mask = buf(B, dtype=i32)
        self.step = torch.zeros((), dtype=i32, device=device)
        self.keep_going = torch.ones((), dtype=i32, device=device)
        # states per block: token-shift rows for the FFN and the attention (fp16), numerator,
        # denominator and running maximum of the WKV recurrence (fp32)
        # (two copies of the token-shift rows, used in turn, where the shift runs inside the Linears: see step_fn)
        self.fuse_shift = K.norm_fusable(B, d)
        self.st_ffn = [buf(2, B, d) if self.fuse_shift else buf(B, d) for _ in range(s.n_layer)]
        self.st_att = [buf(2, B, d) if self.fuse_shift else buf(B, d) for _ in range(s.n_layer)]
        self.st_num = [buf(B, d, dtype=f32) for _ in range(s.n_layer)]
        self.st_den = [buf(B, d, dtype=f32) for _ in range(s.n_layer)]
        self.st_max = [buf(B, d, dtype=f32) for _ in range(s.n_layer)]
        self.graph = None
        self._stream = torch.cuda.Stream()
        # more than 16 rows: scratch that lets the two single-weight Linears of a layer (4096 channels: too few
        # channel blocks to fill the machine) split K across workgroups
        self._lin_ws = K.linear_workspace(B, d, device) if B > 16 else None

    @staticmethod
    def _group(xs, lws, outs, acts):
        if len({lw.group_key() for lw in lws}) == 1 and not lws[0].is_fp8:
            K.linear(None, [lw.w for lw in lws], outs, xs=xs, acts=acts)
        else:
            for x, lw, o, a in zip(xs, lws, outs, acts):
                K.linear(x, [lw.w], [o], act=a)

    def _shifted(self, x, ln, lws, mixes, state, outs, acts):
        """outs[i] = act_i(Linear_i(shift_i(LayerNorm(x)))) with the norm and the shifts inside the launch(es); every
        launch reads the state's copy of this step's parity and leaves the normalised rows in the other."""
        norm = K.Norm(ln[0], ln[1], self.spec.eps)
        if len({lw.group_key() for lw in lws}) == 1 and not lws[0].is_fp8:
            K.linear(x, [lw.w for lw in lws], outs, acts=acts, norm=norm, mixes=mixes, mix=(state, self.step))
        else:
            for lw, m_, o, a in zip(lws, mixes, outs, acts):
                K.linear(x, [lw.w], [o], act=a, norm=norm, mixes=[m_], mix=(state, self.step))

    def step_fn(self):
        s, w = self.spec, self.w
        K.embedding(w.embed, self.container, self.x, ids_index=self.step)
        x, spare = self.x, self.x2
        for i, blk in enumerate(w.blocks):
            if blk.pre_ln is not None:
                K.layer_norm_ce(x, blk.pre_ln[0], blk.pre_ln[1], s.eps, spare)
                x, spare = spare, x
            if self.fuse_shift:
                # up to 4 rows: LayerNorm and the token shift run where the Linears stage their input (two launches
                # fewer); the shift's rows of the previous token live in two copies that the steps use in turn
                self._shifted(x, blk.ln1, [blk.att_key, blk.att_value, blk.att_receptance], blk.att_mix, self.st_att[i],
                              [self.k, self.v, self.r], [_lib.ACT_NONE, _lib.ACT_NONE, _lib.ACT_SIGMOID])
            else:
                K.layer_norm_ce_mix(x, blk.ln1[0], blk.ln1[1], s.eps, self.st_att[i], blk.att_mix, self.mix)
                self._group(self.mix, [blk.att_key, blk.att_value, blk.att_receptance], [self.k, self.v, self.r],
                            [_lib.ACT_NONE, _lib.ACT_NONE, _lib.ACT_SIGMOID])
            K.rwkv_wkv(self.k, self.v, self.r, blk.time_decay, blk.time_first, self.st_num[i], self.st_den[i],
                       self.st_max[i], self.y)
            K.linear(self.y, [blk.att_output.w], [x], residual=x, workspace=self._lin_ws)
            if self.fuse_shift:
                self._shifted(x, blk.ln2, [blk.ffn_key, blk.ffn_receptance], blk.ffn_mix, self.st_ffn[i], [self.fk, self.fr],
                              [_lib.ACT_RELU_SQUARE, _lib.ACT_SIGMOID])
            else:
                K.layer_norm_ce_mix(x, blk.ln2[0], blk.ln2[1], s.eps, self.st_ffn[i], blk.ffn_mix, self.mix[:2])
                self._group(self.mix[:2], [blk.ffn_key, blk.ffn_receptance], [self.fk, self.fr],
                            [_lib.ACT_RELU_SQUARE, _lib.ACT_SIGMOID])
            halve = s.rescale_every > 0 and (i + 1) % s.rescale_every == 0
            K.linear(self.fk, [blk.ffn_value.w], [x], mul=self.fr, residual=x, post_scale=0.5 if halve else 0.0,
                     workspace=self._lin_ws)
        K.layer_norm_ce(x, w.ln_out[0], w.ln_out[1], s.eps, self.h)
        K.linear(self.h, [w.head.w], [self.logits])
        self.select(self.logits, self.next_ids)
        K.step_update(self.container, None, self.stop_mask, self.step, self.next_ids, None, self.keep_going,
                      s.pad_id, s.eos_id, s.early_stop)

    def reset(self, input_ids):
        s = self.spec
        ids = torch.as_tensor(np.asarray(input_ids, np.int32))
        if tuple(ids.shape) != (s.batch, s.max_len):
            raise ValueError(f"input_ids must be [{s.batch}, {s.max_len}], got {tuple(ids.shape)}")
        self.container.copy_(ids)
        self.stop_mask.zero_()
        self.step.zero_()
        self.keep_going.fill_(1)
        for t in self.st_ffn + self.st_att + self.st_num + self.st_den:
            t.zero_()
        for t in self.st_max:
            t.fill_(-1e30)

    def capture(self):
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
        for _ in range(n):
            if self.graph is None:
                self.step_fn()
            else:
                self.graph.replay()

    def run(self, input_ids, max_loop, check_every=16, prompt_passes=False):
        """prompt_passes is accepted for symmetry with the transformer executor; a recurrent model reads its
        prompt one position per iteration."""
        self.reset(input_ids)
        done = 0
        while done < max_loop:
            n = min(check_every, max_loop - done) if self.spec.early_stop else max_loop - done
            self.run_steps(n)
            done += n
            if self.spec.early_stop and int(self.keep_going.item()) == 0:
                break
        torch.cuda.synchronize()
        return self.container.cpu().numpy(), int(self.step.item())
