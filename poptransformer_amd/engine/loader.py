"""State dict (numpy, reference key names) -> device weights of the fused executor.

Mirrors what the reference layers do when they bind their weights
(poptransformer/layers/linear.py:28-40 with utils/param_handler/precision_strategy.py:24-51):
an int8 `<ctx>.weight` is a packed INT4 matrix [out, in/2] with `<ctx>.weight_scale`; other
Linear weights are fp16 [out, in].  Weights are re-tiled on the device once, here.
"""
import numpy as np
import torch

from .. import kernels as K
from .fused import BlockWeights, DecoderSpec, LinearWeights, ModelWeights


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def f143_encode_device(w, scale):
    """fp32/fp16 device tensor -> F143 bytes with exponent `scale` (the bind-time conversion of
    utils/param_handler/precision_strategy.py:44-51), through the library's own encoder."""
    sc = torch.tensor([scale], dtype=torch.int32, device=w.device)
    return K.half_to_fp8(w.half().contiguous(), sc, "F143"), sc


def linear_from_state_dict(sd, ctx, use_bias, device="cuda", precision="fp16", fp8_scale=-1):
    w = sd[ctx + ".weight"]
    w = w if isinstance(w, np.ndarray) else np.asarray(w)
    bias = _dev(np.asarray(sd[ctx + ".bias"], np.float16), device) if use_bias else None
    if precision in ("fp8", "fp8_weight"):
        w8, sc = f143_encode_device(_dev(w.astype(np.float16), device), fp8_scale)
        return LinearWeights(K.F8Weight(w8, sc, "F143"), bias, act_fp8=precision == "fp8", scale_value=fp8_scale)
    if w.dtype == np.int8:
        scale = sd.get(ctx + ".weight_scale")
        if scale is None:
            raise KeyError(f"{ctx}.weight is packed INT4 but {ctx}.weight_scale is missing")
        tw = K.W4Weight(_dev(w, device), _dev(np.asarray(scale, np.float16), device))
    else:
        tw = K.F16Weight(_dev(w.astype(np.float16), device))
    return LinearWeights(tw, bias)


def llama2_weights(sd, cfg, device="cuda"):
    d = cfg["hidden_size"]
    hd = d // cfg["num_attention_heads"]
    blocks = []
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        blocks.append(BlockWeights(
            norm1=(_dev(sd[p + "input_layernorm.weight"], device), None),
            norm2=(_dev(sd[p + "post_attention_layernorm.weight"], device), None),
            qkv=[linear_from_state_dict(sd, p + "self_attn." + n, False, device) for n in ("q_proj", "k_proj", "v_proj")],
            out=linear_from_state_dict(sd, p + "self_attn.o_proj", False, device),
            mlp_in=[linear_from_state_dict(sd, p + "mlp." + n, False, device) for n in ("gate_proj", "up_proj")],
            mlp_out=linear_from_state_dict(sd, p + "mlp.down_proj", False, device)))
    inv_freq = np.array([1.0 / (10000 ** (i / hd)) for i in range(0, hd, 2)]).astype(np.float16)
    return ModelWeights(embed=_dev(sd["model.embed_tokens.weight"], device), pos_embed=None, blocks=blocks,
                        final_norm=(_dev(sd["model.norm.weight"], device), None),
                        head=linear_from_state_dict(sd, "lm_head", False, device), inv_freq=_dev(inv_freq, device))


def llama2_spec(cfg, max_len, batch, pad_id=0, eos_id=2, early_stop=False, fp8_cache=False):
    d, h = cfg["hidden_size"], cfg["num_attention_heads"]
    return DecoderSpec("llama2", cfg["num_hidden_layers"], d, h, h, d // h, cfg["vocab_size"], max_len, batch,
                       cfg["rms_norm_eps"], pad_id, eos_id, early_stop, fp8_cache=fp8_cache)


def gpt2_weights(sd, cfg, device="cuda"):
    blocks = []
    for i in range(cfg["n_layer"]):
        p = f"transformer.h.{i}."
        blocks.append(BlockWeights(
            norm1=(_dev(sd[p + "ln_1.weight"], device), _dev(sd[p + "ln_1.bias"], device)),
            norm2=(_dev(sd[p + "ln_2.weight"], device), _dev(sd[p + "ln_2.bias"], device)),
            qkv=[linear_from_state_dict(sd, p + "attn.c_attn", True, device)],
            out=linear_from_state_dict(sd, p + "attn.c_proj", True, device),
            mlp_in=[linear_from_state_dict(sd, p + "mlp.c_fc", True, device)],
            mlp_out=linear_from_state_dict(sd, p + "mlp.c_proj", True, device)))
    wte = _dev(sd["transformer.wte.weight"], device)
    return ModelWeights(embed=wte, pos_embed=_dev(sd["transformer.wpe.weight"], device), blocks=blocks,
                        final_norm=(_dev(sd["transformer.ln_f.weight"], device), _dev(sd["transformer.ln_f.bias"], device)),
                        head=LinearWeights(K.F16Weight(wte)), inv_freq=None)


def gpt2_spec(cfg, max_len, batch, pad_id=50257, eos_id=50256, early_stop=False):
    d, h = cfg["n_embd"], cfg["n_head"]
    return DecoderSpec("gpt2", cfg["n_layer"], d, h, h, d // h, cfg["vocab_size"], max_len, batch,
                       cfg["layer_norm_epsilon"], pad_id, eos_id, early_stop)


def chatglm2_weights(sd, cfg, precision="fp16", scales=None, device="cuda"):
    scales = scales or {}
    hd = cfg["hidden_size"] // cfg["num_attention_heads"]

    def lin(ctx, bias):
        return linear_from_state_dict(sd, ctx, bias, device, precision, scales.get(ctx, -1))

    blocks = []
    for i in range(cfg["num_layers"]):
        p = f"transformer.encoder.layers.{i}."
        blocks.append(BlockWeights(
            norm1=(_dev(sd[p + "input_layernorm.weight"], device), None),
            norm2=(_dev(sd[p + "post_attention_layernorm.weight"], device), None),
            qkv=[lin(p + "self_attention.query", True), lin(p + "self_attention.key_value", True)],
            out=lin(p + "self_attention.dense", False),
            mlp_in=[lin(p + "mlp.dense_h_to_4h_1", False), lin(p + "mlp.dense_h_to_4h_2", False)],
            mlp_out=lin(p + "mlp.dense_4h_to_h", False)))
    rot = hd // 2
    inv_freq = np.array([1.0 / (10000 ** (i / rot)) for i in range(0, rot, 2)]).astype(np.float32)
    return ModelWeights(embed=_dev(sd["transformer.embedding.word_embeddings.weight"], device), pos_embed=None,
                        blocks=blocks, final_norm=(_dev(sd["transformer.encoder.final_layernorm.weight"], device), None),
                        head=lin("transformer.output_layer", False), inv_freq=_dev(inv_freq, device))


def chatglm2_spec(cfg, max_len, batch, pad_id=0, eos_id=2, early_stop=False):
    d, h = cfg["hidden_size"], cfg["num_attention_heads"]
    return DecoderSpec("chatglm2", cfg["num_layers"], d, h, cfg["multi_query_group_num"], d // h,
                       cfg["padded_vocab_size"], max_len, batch, cfg["layernorm_epsilon"], pad_id, eos_id, early_stop)


def rwkv_weights(sd, cfg, device="cuda"):
    from .rwkv import RWKVBlockWeights, RWKVWeights

    def ln(key):
        return (_dev(sd[key + ".weight"], device), _dev(sd[key + ".bias"], device))

    def vec(key):
        return _dev(np.asarray(sd[key], np.float16).reshape(-1), device)

    blocks = []
    for i in range(cfg["num_hidden_layers"]):
        p = f"rwkv.blocks.{i}."
        blocks.append(RWKVBlockWeights(
            pre_ln=ln(p + "pre_ln") if i == 0 else None, ln1=ln(p + "ln1"), ln2=ln(p + "ln2"),
            att_key=linear_from_state_dict(sd, p + "attention.key", False, device),
            att_value=linear_from_state_dict(sd, p + "attention.value", False, device),
            att_receptance=linear_from_state_dict(sd, p + "attention.receptance", False, device),
            att_output=linear_from_state_dict(sd, p + "attention.output", False, device),
            time_decay=vec(p + "attention.time_decay"), time_first=vec(p + "attention.time_first"),
            att_mix=[vec(p + f"attention.time_mix_{n}") for n in ("key", "value", "receptance")],
            ffn_key=linear_from_state_dict(sd, p + "feed_forward.key", False, device),
            ffn_receptance=linear_from_state_dict(sd, p + "feed_forward.receptance", False, device),
            ffn_value=linear_from_state_dict(sd, p + "feed_forward.value", False, device),
            ffn_mix=[vec(p + f"feed_forward.time_mix_{n}") for n in ("key", "receptance")]))
    return RWKVWeights(embed=_dev(sd["rwkv.embeddings.weight"], device), blocks=blocks, ln_out=ln("rwkv.ln_out"),
                       head=linear_from_state_dict(sd, "head", False, device))


def rwkv_spec(cfg, max_len, batch, pad_id=0, eos_id=-1, early_stop=False):
    from .rwkv import RWKVSpec
    return RWKVSpec(cfg["num_hidden_layers"], cfg["hidden_size"], cfg["attention_hidden_size"], cfg["intermediate_size"],
                    cfg["vocab_size"], max_len, batch, cfg["layer_norm_epsilon"], cfg["rescale_every"], pad_id, eos_id,
                    early_stop)
