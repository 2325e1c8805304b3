#!/usr/bin/env python3
"""Writes the fixtures of this directory from sources that are independent of the oracle and of the kernels:
torch's float8 fnuz casts, scipy, torch.nn.functional and Hugging Face model classes built from local
configs (nothing is downloaded).  The FP8 fixtures hold values inside each format's range only: what the
Graphcore cast does beyond it (taken here to saturate at the largest finite value, where torch's fnuz cast
gives NaN) is an assumption that no fixture pins.  The reference repository holds no test vectors of its own; these stand in
for them.  Run from the repository root: `python tests/golden/make_vectors.py`.

Model weights are not stored: `seeded_state_dict` regenerates them from a numpy seed, in the key order of
the Hugging Face state dict, and the script loads exactly those values into the Hugging Face model before
it computes the expected logits.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

LLAMA_GOLDEN = dict(vocab_size=256, hidden_size=128, intermediate_size=352, num_hidden_layers=2, num_attention_heads=2,
                    rms_norm_eps=1e-5)


def seeded_state_dict(shapes, seed):
    """{key: fp16 array}: N(0, 0.05) for matrices, 1 + N(0, 0.1) for norm weights, in the order given."""
    rng = np.random.default_rng(seed)
    out = {}
    for key, shape in shapes:
        if "norm" in key:
            out[key] = (1.0 + 0.1 * rng.standard_normal(shape)).astype(np.float16)
        else:
            out[key] = (0.05 * rng.standard_normal(shape)).astype(np.float16)
    return out


def llama_shapes(cfg):
    d, f, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    shapes = [("model.embed_tokens.weight", (v, d))]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        shapes += [(p + "self_attn.q_proj.weight", (d, d)), (p + "self_attn.k_proj.weight", (d, d)),
                   (p + "self_attn.v_proj.weight", (d, d)), (p + "self_attn.o_proj.weight", (d, d)),
                   (p + "mlp.gate_proj.weight", (f, d)), (p + "mlp.up_proj.weight", (f, d)),
                   (p + "mlp.down_proj.weight", (d, f)), (p + "input_layernorm.weight", (d,)),
                   (p + "post_attention_layernorm.weight", (d,))]
    shapes += [("model.norm.weight", (d,)), ("lm_head.weight", (v, d))]
    return shapes


GLM_GOLDEN = dict(padded_vocab_size=256, hidden_size=256, layernorm_epsilon=1e-5, multi_query_group_num=2,
                  num_attention_heads=4, ffn_hidden_size=352, num_layers=2, kv_channels=64)


def chatglm2_shapes(cfg):
    """Keys and shapes of a ChatGLM2 checkpoint as the reference holds it after the split of `query_key_value`
    into `query` / `key_value` and of `dense_h_to_4h` into `_1` (gate) / `_2` (up)
    (poptransformer/models/chatglm2/model.py:256-274)."""
    d, f, v = cfg["hidden_size"], cfg["ffn_hidden_size"], cfg["padded_vocab_size"]
    kv = 2 * cfg["multi_query_group_num"] * cfg["kv_channels"]
    shapes = [("transformer.embedding.word_embeddings.weight", (v, d))]
    for i in range(cfg["num_layers"]):
        p = f"transformer.encoder.layers.{i}."
        shapes += [(p + "input_layernorm.weight", (d,)), (p + "self_attention.query.weight", (d, d)),
                   (p + "self_attention.query.bias", (d,)), (p + "self_attention.key_value.weight", (kv, d)),
                   (p + "self_attention.key_value.bias", (kv,)), (p + "self_attention.dense.weight", (d, d)),
                   (p + "post_attention_layernorm.weight", (d,)), (p + "mlp.dense_h_to_4h_1.weight", (f, d)),
                   (p + "mlp.dense_h_to_4h_2.weight", (f, d)), (p + "mlp.dense_4h_to_h.weight", (d, f))]
    shapes += [("transformer.encoder.final_layernorm.weight", (d,)), ("transformer.output_layer.weight", (v, d))]
    return shapes


def glm_hf_state_dict(sd, cfg):
    """The ChatGLM2 checkpoint `sd` under the parameter names of Hugging Face's GlmForCausalLM, the same block
    (RMSNorm, q/k/v with bias over grouped KV heads, rotary embedding on interleaved pairs of the first half of
    each head, fused gate | up SwiGLU): `key_value` rows are k then v, `gate_up_proj` rows are gate then up."""
    half = cfg["multi_query_group_num"] * cfg["kv_channels"]
    out = {"model.embed_tokens.weight": sd["transformer.embedding.word_embeddings.weight"],
           "model.norm.weight": sd["transformer.encoder.final_layernorm.weight"],
           "lm_head.weight": sd["transformer.output_layer.weight"]}
    for i in range(cfg["num_layers"]):
        p, h = f"transformer.encoder.layers.{i}.", f"model.layers.{i}."
        out[h + "input_layernorm.weight"] = sd[p + "input_layernorm.weight"]
        out[h + "post_attention_layernorm.weight"] = sd[p + "post_attention_layernorm.weight"]
        out[h + "self_attn.q_proj.weight"] = sd[p + "self_attention.query.weight"]
        out[h + "self_attn.q_proj.bias"] = sd[p + "self_attention.query.bias"]
        out[h + "self_attn.k_proj.weight"] = sd[p + "self_attention.key_value.weight"][:half]
        out[h + "self_attn.k_proj.bias"] = sd[p + "self_attention.key_value.bias"][:half]
        out[h + "self_attn.v_proj.weight"] = sd[p + "self_attention.key_value.weight"][half:]
        out[h + "self_attn.v_proj.bias"] = sd[p + "self_attention.key_value.bias"][half:]
        out[h + "self_attn.o_proj.weight"] = sd[p + "self_attention.dense.weight"]
        out[h + "mlp.gate_up_proj.weight"] = np.concatenate([sd[p + "mlp.dense_h_to_4h_1.weight"],
                                                             sd[p + "mlp.dense_h_to_4h_2.weight"]], axis=0)
        out[h + "mlp.down_proj.weight"] = sd[p + "mlp.dense_4h_to_h.weight"]
    return out


def glm_logits():
    """ChatGLM2 block pinned end to end: Hugging Face GlmForCausalLM (built from a local config, nothing is
    downloaded) holding the seeded fp16 weights in fp32, logits of every position of two sequences."""
    from transformers import GlmConfig, GlmForCausalLM
    cfg = GLM_GOLDEN
    hf = GlmForCausalLM(GlmConfig(
        vocab_size=cfg["padded_vocab_size"], hidden_size=cfg["hidden_size"], intermediate_size=cfg["ffn_hidden_size"],
        num_hidden_layers=cfg["num_layers"], num_attention_heads=cfg["num_attention_heads"],
        num_key_value_heads=cfg["multi_query_group_num"], head_dim=cfg["kv_channels"], hidden_act="silu",
        rms_norm_eps=cfg["layernorm_epsilon"], max_position_embeddings=64, tie_word_embeddings=False,
        rope_parameters={"rope_type": "default", "rope_theta": 10000.0, "partial_rotary_factor": 0.5},
        attention_bias=True, pad_token_id=0)).eval()
    sd = seeded_state_dict(chatglm2_shapes(cfg), seed=2025)
    mapped = glm_hf_state_dict(sd, cfg)
    missing = hf.load_state_dict({k: torch.from_numpy(np.ascontiguousarray(v).astype(np.float32)) for k, v in mapped.items()},
                                 strict=False)
    assert not missing.unexpected_keys and all("rotary" in k for k in missing.missing_keys), missing
    toks = np.random.default_rng(6).integers(1, cfg["padded_vocab_size"], size=(2, 24)).astype(np.int32)
    with torch.no_grad():
        logits = hf(torch.from_numpy(toks.astype(np.int64))).logits.numpy()
    np.savez_compressed(os.path.join(HERE, "glm_hf.npz"), tokens=toks, logits=logits.astype(np.float32), seed=np.int64(2025))


def main():
    if len(sys.argv) > 1 and sys.argv[1] == "glm":      # only the fixture added last; the others stay byte-identical
        glm_logits()
        print("glm_hf.npz", os.path.getsize(os.path.join(HERE, "glm_hf.npz")))
        return
    # FP8: the fnuz formats of torch (e4m3fnuz = 1-4-3 bias 8, e5m2fnuz = 1-5-2 bias 16, NaN 0x80)
    codes = torch.arange(256, dtype=torch.uint8)
    rng = np.random.default_rng(12)
    # values inside each format's range only: beyond it torch's cast gives NaN where the Graphcore cast saturates
    x143 = np.concatenate([rng.standard_normal(3000) * 0.05, rng.uniform(-240, 240, 3000), [0.0, -0.0, 240.0, -240.0, 6e-8]]).astype(np.float16)
    x152 = np.concatenate([rng.standard_normal(3000) * 0.05, rng.uniform(-57344, 57344, 3000), [0.0, -0.0, 57344.0, -57344.0, 6e-8]]).astype(np.float16)
    np.savez_compressed(os.path.join(HERE, "fp8_fnuz.npz"),
                        table_F143=codes.view(torch.float8_e4m3fnuz).to(torch.float32).numpy(),
                        table_F152=codes.view(torch.float8_e5m2fnuz).to(torch.float32).numpy(),
                        x_F143=x143, x_F152=x152,
                        codes_F143=torch.from_numpy(x143.astype(np.float32)).to(torch.float8_e4m3fnuz).view(torch.uint8).numpy(),
                        codes_F152=torch.from_numpy(x152.astype(np.float32)).to(torch.float8_e5m2fnuz).view(torch.uint8).numpy())

    # INT4: two signed nibbles per byte, the high nibble first, by the definition of two's complement
    hi = np.array([(b >> 4) - 16 if (b >> 4) >= 8 else (b >> 4) for b in range(256)], np.int8)
    lo = np.array([(b & 15) - 16 if (b & 15) >= 8 else (b & 15) for b in range(256)], np.int8)
    np.savez_compressed(os.path.join(HERE, "int4_nibbles.npz"), byte=np.arange(256, dtype=np.uint8), high=hi, low=lo)

    # softmax (scipy), LayerNorm (torch), RMSNorm and rotary embedding (Hugging Face Llama)
    import scipy.special
    from transformers.models.llama.modeling_llama import LlamaRMSNorm, apply_rotary_pos_emb
    rng = np.random.default_rng(21)
    sx = (rng.standard_normal((6, 200)) * 3).astype(np.float16)
    lx = rng.standard_normal((3, 256)).astype(np.float16)
    lg, lb = rng.uniform(0.5, 1.5, 256).astype(np.float16), rng.standard_normal(256).astype(np.float16)
    ln = torch.nn.functional.layer_norm(torch.from_numpy(lx.astype(np.float32)), (256,), torch.from_numpy(lg.astype(np.float32)),
                                        torch.from_numpy(lb.astype(np.float32)), 1e-5).numpy()
    rx = rng.standard_normal((4, 128)).astype(np.float16)
    rw = rng.uniform(0.5, 1.5, 128).astype(np.float16)
    mod = LlamaRMSNorm(128, eps=1e-5)
    with torch.no_grad():
        mod.weight.copy_(torch.from_numpy(rw.astype(np.float32)))
        rms = mod(torch.from_numpy(rx.astype(np.float32))).numpy()
    D, steps = 128, np.array([0, 1, 37, 511], np.int32)
    q = rng.standard_normal((len(steps), 2, 3, 1, D)).astype(np.float16)
    rope = []
    for i, st in enumerate(steps):
        ang = st * (1.0 / (10000 ** (np.arange(0, D, 2) / D)))
        c = torch.from_numpy(np.concatenate([np.cos(ang), np.cos(ang)]).astype(np.float32)).reshape(1, 1, D)
        s = torch.from_numpy(np.concatenate([np.sin(ang), np.sin(ang)]).astype(np.float32)).reshape(1, 1, D)
        qt = torch.from_numpy(q[i].astype(np.float32))
        rope.append(apply_rotary_pos_emb(qt, qt, c, s)[0].numpy())
    np.savez_compressed(os.path.join(HERE, "operators.npz"), softmax_x=sx,
                        softmax_y=scipy.special.softmax(sx.astype(np.float64), axis=-1).astype(np.float32),
                        ln_x=lx, ln_gamma=lg, ln_beta=lb, ln_y=ln, rms_x=rx, rms_w=rw, rms_y=rms,
                        rope_steps=steps, rope_q=q, rope_y=np.stack(rope))

    # Llama: Hugging Face LlamaForCausalLM holding the seeded fp16 weights, logits of every position
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LLAMA_GOLDEN
    hf = LlamaForCausalLM(LlamaConfig(vocab_size=cfg["vocab_size"], hidden_size=cfg["hidden_size"],
                                      intermediate_size=cfg["intermediate_size"], num_hidden_layers=cfg["num_hidden_layers"],
                                      num_attention_heads=cfg["num_attention_heads"], num_key_value_heads=cfg["num_attention_heads"],
                                      rms_norm_eps=cfg["rms_norm_eps"], max_position_embeddings=64, rope_theta=10000.0,
                                      attention_bias=False, tie_word_embeddings=False)).eval()
    sd = seeded_state_dict(llama_shapes(cfg), seed=2024)
    missing = hf.load_state_dict({k: torch.from_numpy(v.astype(np.float32)) for k, v in sd.items()}, strict=False)
    assert not missing.unexpected_keys and all("rotary" in k for k in missing.missing_keys), missing
    toks = np.random.default_rng(5).integers(1, cfg["vocab_size"], size=(2, 24)).astype(np.int32)
    with torch.no_grad():
        logits = hf(torch.from_numpy(toks.astype(np.int64))).logits.numpy()
    np.savez_compressed(os.path.join(HERE, "llama_hf.npz"), tokens=toks, logits=logits.astype(np.float32), seed=np.int64(2024))
    glm_logits()
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
