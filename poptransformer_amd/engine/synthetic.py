"""Random-init weights generated directly on the device, for benchmarks of full-size shapes.

Same distributions and checkpoint layout as the CPU generators the parity tests use (N(0, 0.02)
weights, symmetric per-output-channel INT4 with scale = max|w| / 7, unit norm weights), but
drawn with torch's device generator so that a 7B-parameter shape is ready in seconds.  This is
benchmark set-up, not part of the decode path.
"""
import numpy as np
import torch

from .. import kernels as K
from .fused import BlockWeights, LinearWeights, ModelWeights


def quantize_int4_device(w):
    """w fp16 [out, in] on the device -> (packed int8 [out, in/2], scale fp16 [out])."""
    wf = w.float()
    scale = (wf.abs().amax(dim=1) / 7.0).half().clamp_min(torch.finfo(torch.float16).tiny)
    q = torch.clamp(torch.round(wf / scale.float()[:, None]), -8, 7).to(torch.int16)
    hi = (q[:, 0::2] & 0xF).to(torch.uint8)
    lo = (q[:, 1::2] & 0xF).to(torch.uint8)
    return ((hi << 4) | lo).view(torch.int8).contiguous(), scale.contiguous()


def _linear_int4(gen, out_f, in_f, device):
    w = (torch.randn((out_f, in_f), generator=gen, device=device, dtype=torch.float32) * 0.02).half()
    packed, scale = quantize_int4_device(w)
    return LinearWeights(K.W4Weight(packed, scale))



def llama2_synthetic_weights(cfg, seed=0, device="cuda"):
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    d, f, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    hd = d // cfg["num_attention_heads"]
    ones = torch.ones(d, dtype=torch.float16, device=device)

    def f16w(rows, cols):
        return (torch.randn((rows, cols), generator=gen, device=device, dtype=torch.float32) * 0.02).half()

    embed = f16w(v, d)
    blocks = []
    for _ in range(cfg["num_hidden_layers"]):
        blocks.append(BlockWeights(
            norm1=(ones.clone(), None), norm2=(ones.clone(), None),
            qkv=[_linear_int4(gen, d, d, device) for _ in range(3)],
            out=_linear_int4(gen, d, d, device),
            mlp_in=[_linear_int4(gen, f, d, device) for _ in range(2)],
            mlp_out=_linear_int4(gen, d, f, device)))
    head = LinearWeights(K.F16Weight(f16w(v, d)))
    inv_freq = torch.from_numpy(np.array([1.0 / (10000 ** (i / hd)) for i in range(0, hd, 2)]).astype(np.float16)).to(device)
    torch.cuda.synchronize()
    return ModelWeights(embed=embed, pos_embed=None, blocks=blocks, final_norm=(ones.clone(), None), head=head,
                        inv_freq=inv_freq)
