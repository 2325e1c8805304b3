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


_F8_STD = 0.02


def _f8_model_exponent(std=_F8_STD):
    """Power-of-two exponent e with 8 std * 2^-e <= 240 (the largest F143 value; a normal sample of the model's size
    stays below 6.5 std): the one scale of the benchmark configuration, shared by every Linear as in the reference,
    which binds the constant -1 to every FP8 weight (utils/param_handler/precision_strategy.py:44-49; what
    loader.linear_from_state_dict does)."""
    return int(np.ceil(np.log2(8.0 * std / 240.0)))


def _linear_f143(gen, out_f, in_f, device, act_fp8, bias=False):
    from .loader import f143_encode_device
    w = (torch.randn((out_f, in_f), generator=gen, device=device, dtype=torch.float32) * _F8_STD).half()
    e = _f8_model_exponent()
    w8, sc = f143_encode_device(w, e)
    b = torch.zeros(out_f, dtype=torch.float16, device=device) if bias else None
    return LinearWeights(K.F8Weight(w8, sc, "F143"), b, act_fp8=act_fp8, scale_value=e)


def chatglm2_synthetic_weights(cfg, precision="fp8", seed=0, device="cuda"):
    """ChatGLM2-shaped weights, every Linear cast to F143 with the model's power-of-two scale
    (precision "fp8": activations are cast to F143 too; "fp8_weight": they stay fp16)."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    d, f, v = cfg["hidden_size"], cfg["ffn_hidden_size"], cfg["padded_vocab_size"]
    hd = d // cfg["num_attention_heads"]
    kv = 2 * cfg["multi_query_group_num"] * hd
    ones = torch.ones(d, dtype=torch.float16, device=device)
    act8 = precision == "fp8"
    blocks = []
    for _ in range(cfg["num_layers"]):
        blocks.append(BlockWeights(
            norm1=(ones.clone(), None), norm2=(ones.clone(), None),
            qkv=[_linear_f143(gen, d, d, device, act8, bias=True), _linear_f143(gen, kv, d, device, act8, bias=True)],
            out=_linear_f143(gen, d, d, device, act8),
            mlp_in=[_linear_f143(gen, f, d, device, act8) for _ in range(2)],
            mlp_out=_linear_f143(gen, d, f, device, act8)))
    embed = (torch.randn((v, d), generator=gen, device=device, dtype=torch.float32) * 0.02).half()
    rot = hd // 2
    inv_freq = torch.from_numpy(np.array([1.0 / (10000 ** (i / rot)) for i in range(0, rot, 2)]).astype(np.float32)).to(device)
    head = _linear_f143(gen, v, d, device, act8)
    torch.cuda.synchronize()
    return ModelWeights(embed=embed, pos_embed=None, blocks=blocks, final_norm=(ones.clone(), None), head=head,
                        inv_freq=inv_freq)


def rwkv_synthetic_weights(cfg, seed=0, device="cuda"):
    """RWKV-4-shaped weights: INT4 Linear weights, time_decay U(-8, -1), time_first U(-1, 1), time_mix U(0, 1)."""
    from .rwkv import RWKVBlockWeights, RWKVWeights
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    d, a, f, v = cfg["hidden_size"], cfg["attention_hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]

    def ln(n):
        return (torch.ones(n, dtype=torch.float16, device=device), torch.zeros(n, dtype=torch.float16, device=device))

    def uni(n, lo, hi):
        return (torch.rand(n, generator=gen, device=device) * (hi - lo) + lo).half()

    blocks = []
    for i in range(cfg["num_hidden_layers"]):
        blocks.append(RWKVBlockWeights(
            pre_ln=ln(d) if i == 0 else None, ln1=ln(d), ln2=ln(d),
            att_key=_linear_int4(gen, a, d, device), att_value=_linear_int4(gen, a, d, device),
            att_receptance=_linear_int4(gen, a, d, device), att_output=_linear_int4(gen, d, a, device),
            time_decay=uni(a, -8.0, -1.0), time_first=uni(a, -1.0, 1.0), att_mix=[uni(d, 0.0, 1.0) for _ in range(3)],
            ffn_key=_linear_int4(gen, f, d, device), ffn_receptance=_linear_int4(gen, d, d, device),
            ffn_value=_linear_int4(gen, d, f, device), ffn_mix=[uni(d, 0.0, 1.0) for _ in range(2)]))
    embed = (torch.randn((v, d), generator=gen, device=device, dtype=torch.float32) * 0.02).half()
    head = LinearWeights(K.F16Weight((torch.randn((v, d), generator=gen, device=device, dtype=torch.float32) * 0.02).half()))
    torch.cuda.synchronize()
    return RWKVWeights(embed=embed, blocks=blocks, ln_out=ln(d), head=head)


def gpt2_synthetic_state_dict(cfg, seed=0):
    """Random-init GPT-2-shaped checkpoint (numpy, on the host) as the reference holds it after
    GPT2DecModel.process_hf_model_state_dict (poptransformer/models/gpt2/model.py:154-166): Linear weights in
    [out, in] orientation, the query third of c_attn pre-multiplied by 1 / sqrt(head size); N(0, 0.02) weights,
    zero biases, LayerNorm gamma 1 / beta 0.  What `loader.gpt2_weights` reads."""
    rng = np.random.Generator(np.random.PCG64(seed))
    d, v, npos = cfg["n_embd"], cfg["vocab_size"], cfg["n_positions"]
    hd = d // cfg["n_head"]

    def normal(*shape):
        return (rng.standard_normal(shape, dtype=np.float32) * 0.02).astype(np.float16)

    sd = {"transformer.wte.weight": normal(v, d), "transformer.wpe.weight": normal(npos, d)}
    for i in range(cfg["n_layer"]):
        p = f"transformer.h.{i}."
        for ln in ("ln_1", "ln_2"):
            sd[p + ln + ".weight"] = np.ones(d, np.float16)
            sd[p + ln + ".bias"] = np.zeros(d, np.float16)
        w = rng.standard_normal((3 * d, d), dtype=np.float32) * 0.02
        w[:d] *= np.float32(1 / hd ** 0.5)
        sd[p + "attn.c_attn.weight"] = w.astype(np.float16)
        sd[p + "attn.c_attn.bias"] = np.zeros(3 * d, np.float16)
        sd[p + "attn.c_proj.weight"] = normal(d, d)
        sd[p + "attn.c_proj.bias"] = np.zeros(d, np.float16)
        sd[p + "mlp.c_fc.weight"] = normal(4 * d, d)
        sd[p + "mlp.c_fc.bias"] = np.zeros(4 * d, np.float16)
        sd[p + "mlp.c_proj.weight"] = normal(d, 4 * d)
        sd[p + "mlp.c_proj.bias"] = np.zeros(d, np.float16)
    sd["transformer.ln_f.weight"] = np.ones(d, np.float16)
    sd["transformer.ln_f.bias"] = np.zeros(d, np.float16)
    return sd
