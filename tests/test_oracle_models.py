"""Pins of the whole-model oracles against independent implementations of the same
architectures (Hugging Face transformers, random-init, CPU fp32): a wrong head split, a missing
query pre-scale, a transposed weight or a wrong rotary convention shows up as an O(1) error in
the logits, far above the fp16-vs-fp32 noise allowed here."""
import numpy as np
import pytest
import torch

from oracle import models as OM
from oracle import ops as O

f16, f32 = np.float16, np.float32


def _rel(a, b):
    return np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / np.abs(b).max()


def test_gpt2_oracle_against_hf():
    from transformers import GPT2Config, GPT2LMHeadModel
    torch.manual_seed(0)
    hf_cfg = GPT2Config(vocab_size=300, n_positions=32, n_embd=64, n_layer=2, n_head=2,
                        resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
    hf = GPT2LMHeadModel(hf_cfg).eval()
    with torch.no_grad():
        for p in hf.parameters():                      # make biases and LayerNorm affine non-trivial
            if p.dim() == 1:
                p.add_(torch.randn_like(p) * 0.05)
    cfg = dict(vocab_size=300, n_embd=64, layer_norm_epsilon=hf_cfg.layer_norm_epsilon, n_head=2, n_layer=2, n_positions=32)
    d, hd = 64, 32
    sd = {}
    for k, v in hf.state_dict().items():
        a = v.detach().numpy().astype(f32)
        if k.endswith(("attn.c_attn.weight", "attn.c_proj.weight", "mlp.c_fc.weight", "mlp.c_proj.weight")):
            a = a.T.copy()                             # HF Conv1D is [in, out]; the reference stores [out, in]
        if k.endswith("attn.c_attn.weight"):
            a[:d] *= 1 / hd ** 0.5                     # query pre-scale of gpt2/model.py:154-166
        if k.endswith("attn.c_attn.bias"):
            a = a.copy()
            a[:d] *= 1 / hd ** 0.5
        sd[k] = a.astype(f16)
    L, B = 16, 2
    model = OM.GPT2Oracle(sd, cfg, L, B)
    rng = np.random.default_rng(0)
    toks = rng.integers(0, 300, size=(B, L)).astype(np.int32)
    mask = np.full((B, L), -10000, f16)
    with torch.no_grad():
        ref_all = hf(torch.from_numpy(toks.astype(np.int64))).logits.numpy()
    for step in range(L):
        mask[:, step] = 0
        _, logits = model.step(toks[:, step].reshape(B, 1), step, mask)
        assert _rel(logits, ref_all[:, step]) < 2e-2, f"step {step}"


def test_llama2_oracle_against_hf():
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(1)
    hf_cfg = LlamaConfig(vocab_size=200, hidden_size=64, intermediate_size=176, num_hidden_layers=2,
                         num_attention_heads=2, num_key_value_heads=2, rms_norm_eps=1e-5, max_position_embeddings=64,
                         rope_theta=10000.0, attention_bias=False, tie_word_embeddings=False)
    hf = LlamaForCausalLM(hf_cfg).eval()
    with torch.no_grad():
        for n, p in hf.named_parameters():
            if "norm" in n:
                p.add_(torch.randn_like(p) * 0.1)
    cfg = dict(vocab_size=200, hidden_size=64, rms_norm_eps=1e-5, num_attention_heads=2, intermediate_size=176,
               num_hidden_layers=2)
    sd = {k: v.detach().numpy().astype(f16) for k, v in hf.state_dict().items()}
    L, B = 12, 2
    model = OM.Llama2Oracle(sd, cfg, L, B)
    rng = np.random.default_rng(1)
    toks = rng.integers(0, 200, size=(B, L)).astype(np.int32)
    mask = np.full((B, L), -10000, f16)
    with torch.no_grad():
        ref_all = hf(torch.from_numpy(toks.astype(np.int64))).logits.numpy()
    for step in range(L):
        mask[:, step] = 0
        _, logits = model.step(toks[:, step].reshape(B, 1), step, mask)
        assert _rel(logits, ref_all[:, step]) < 2e-2, f"step {step}"


def test_int4_model_equals_fp16_model_with_dequantised_weights():
    """The INT4 path must be exactly the fp16 path run on Int4ToHalf(weights)."""
    cfg = dict(vocab_size=64, hidden_size=32, rms_norm_eps=1e-5, num_attention_heads=2, intermediate_size=48,
               num_hidden_layers=1)
    sd = OM.make_llama2_state_dict(cfg, seed=5, int4=True)
    sd16 = dict(sd)
    for k in list(sd):
        if sd[k].dtype == np.int8:
            sd16[k] = np.ascontiguousarray(O.int4_to_half(sd[k], sd[k + "_scale"], 1).T)
    L, B = 8, 1
    ids = np.zeros((B, L), np.int32)
    ids[0, :3] = [5, 9, 11]
    ta, tb = [], []
    ca, _ = OM.run_decode_loop(OM.Llama2Oracle(sd, cfg, L, B), ids, L, L, 0, 2, trace=ta)
    cb, _ = OM.run_decode_loop(OM.Llama2Oracle(sd16, cfg, L, B), ids, L, L, 0, 2, trace=tb)
    assert np.array_equal(ca, cb)
    for (ia, la), (ib, lb) in zip(ta, tb):
        assert np.array_equal(la, lb)


def test_quantize_int4_roundtrip_error_bound():
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((8, 64)) * 0.02).astype(f16)
    p, s = OM.quantize_int4(w)
    assert p.dtype == np.int8 and p.shape == (8, 32) and s.dtype == f16
    wq = O.int4_to_half(p, s, 1).T.astype(f32)
    assert np.abs(wq - w.astype(f32)).max() <= 0.5 * s.astype(f32).max() * 1.01


def test_rwkv_oracle_against_hf():
    from transformers import RwkvConfig, RwkvForCausalLM
    torch.manual_seed(2)
    hf_cfg = RwkvConfig(vocab_size=150, context_length=32, hidden_size=64, num_hidden_layers=4, attention_hidden_size=64,
                        intermediate_size=128, layer_norm_epsilon=1e-5, rescale_every=2)
    hf = RwkvForCausalLM(hf_cfg).eval()
    with torch.no_grad():
        for n, p in hf.named_parameters():
            if "time_decay" in n:
                p.copy_(torch.empty_like(p).uniform_(-6, -1))
            elif "time_first" in n:
                p.copy_(torch.empty_like(p).uniform_(-1, 1))
            elif "time_mix" in n:
                p.copy_(torch.empty_like(p).uniform_(0.1, 0.9))
            elif "ln" in n:
                p.add_(torch.randn_like(p) * 0.05)
            else:
                p.mul_(3.0)                                     # make the projections matter
    cfg = dict(hidden_size=64, intermediate_size=128, attention_hidden_size=64, layer_norm_epsilon=1e-5, vocab_size=150,
               num_hidden_layers=4, rescale_every=2)
    # the reference's load-time processing (rwkv/model.py:150-155), applied to a copy
    sd = {}
    for k, v in hf.state_dict().items():
        a = v.detach().numpy().astype(f32).copy()
        if k.endswith("attention.output.weight") or k.endswith("feed_forward.value.weight"):
            a /= 2 ** (int(k.split(".")[2]) // 2)
        sd[k] = a.astype(f16)
    L, B = 10, 2
    model = OM.RWKVOracle(sd, cfg, L, B)
    rng = np.random.default_rng(3)
    toks = rng.integers(0, 150, size=(B, L)).astype(np.int32)
    with torch.no_grad():
        ref_all = hf(torch.from_numpy(toks.astype(np.int64))).logits.numpy()   # eval mode rescales the same way
    for step in range(L):
        _, logits = model.step(toks[:, step].reshape(B, 1), step)
        assert _rel(logits, ref_all[:, step]) < 3e-2, f"step {step}"
