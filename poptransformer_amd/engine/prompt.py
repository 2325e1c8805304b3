"""The prompt in passes of several positions.

The reference's GPT-2, Llama-2 and ChatGLM2 loops take a prompt one position per iteration: the
container already holds the prompt's tokens, so the token an iteration selects is dropped and the
stored one is used (models/base_model.py:313-318).  Those iterations only fill the KV cache.  Its
two-stage ChatGLM model runs the same layer stack once over the whole prompt with sequence_length > 1
(models/chatglm/model.py:301-330, models/chatglm/attention.py:89-140) before the loop starts.

`PromptPass` is that first stage for the decoders here: R consecutive positions of every sequence
(B*R <= 2048 rows) go through each layer together - the projections as GEMMs over B*R rows, which read
each weight once per pass, the rotary embedding and cache append per row at its own position, and
causal attention of row r over positions 0..p0+r.  The final norm, the head and the token selection
are skipped: the loop would discard their result.  What it leaves in the KV rings is what R iterations
of the loop leave there, up to the rounding of a different summation order in the GEMMs.
"""
import torch

from .. import _lib
from .. import kernels as K
from .fused import LayerOps


class PromptPass(LayerOps):
    """Buffers for B*rows rows and one pass over the layers; shares weights and KV rings with the decoder `dec`."""

    def __init__(self, dec, rows):
        super().__init__(dec.spec, dec.w, dec.dev, dec.spec.batch * int(rows))
        self.dec, self.rows = dec, int(rows)
        s, i32 = self.spec, torch.int32
        self.first = torch.zeros((), dtype=i32, device=self.dev)       # position of row 0 of every sequence
        self._offsets = torch.arange(self.rows, dtype=i32, device=self.dev)
        self.graph = None
        # scratch for the K split of the projections with few output channels (attention output, MLP down)
        self._lin_ws = K.linear_workspace(self._rows, max(s.d_model, self.w.blocks[0].mlp_out.K), self.dev)

    def run(self, p0):
        """Positions p0 .. p0+rows-1 of every sequence (row b*rows + r is sequence b at p0 + r).  The pass
        depends on device state only (`first`, the container, the rings): the first call runs it eagerly,
        the second records it into a HIP graph, later calls replay that graph."""
        s = self.spec
        if p0 < 0 or p0 + self.rows > s.max_len:
            raise ValueError(f"prompt pass over positions {p0}..{p0 + self.rows - 1} leaves the cache (max_len {s.max_len})")
        self.first.fill_(p0)
        if self.graph is not None:
            self.graph.replay()
        elif not getattr(self, "_warm", False):
            self._layers()
            self._warm = True
        else:
            stream = torch.cuda.current_stream()
            stream.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=stream):
                self._layers()
            self.graph.replay()

    def _layers(self):
        s, w, dec = self.spec, self.w, self.dec
        B, R = s.batch, self.rows
        positions = self._offsets + self.first
        ids = dec.container.index_select(1, positions).reshape(-1)
        K.embedding(w.embed, ids, self.x)
        if w.pos_embed is not None:        # GPT-2: learned positions, one table row per position
            self.x.add_(w.pos_embed.index_select(0, positions).repeat(B, 1))
        for li, blk in enumerate(w.blocks):
            if not hasattr(self, "_qkv_views"):
                self._prepare_qkv_views(blk)
            h, nrm = self._normed(self.x, blk.norm1, blk.qkv)
            self._linear_group(h, blk.qkv, self._qkv_bufs, nrm)
            qp, kp, vp, qs, ks, vs = self._qkv_views
            K.prompt_rope_append(qp, kp, vp, self.q_rot, dec.rings[li], self.first, w.inv_freq, B, R, s.n_head,
                                 s.n_kv_head, s.head_dim, s.max_len, s.rope, qs, ks, vs, kv_scale=dec.kv_scale)
            K.prompt_attention(self.q_rot, dec.rings[li], self.first, self.attn_ws, self.ctx, B, R, s.n_head,
                               s.n_kv_head, s.head_dim, s.max_len, s.scale_scores, kv_scale=dec.kv_scale)
            self._linear(self.ctx, blk.out, self.x, residual=self.x)
            h, nrm = self._normed(self.x, blk.norm2, blk.mlp_in)
            if len(blk.mlp_in) == 2:
                self._linear_group(h, blk.mlp_in, [self.act, self.act], nrm, swiglu=True, consumer=blk.mlp_out)
            else:
                self._linear(h, blk.mlp_in[0], self.act, act=_lib.ACT_GELU_TANH, norm=nrm)
            self._linear(self.act, blk.mlp_out, self.x, residual=self.x)
