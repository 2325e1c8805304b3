"""The fixtures of tests/golden/ (made by tests/golden/make_vectors.py from torch's fnuz casts, scipy,
torch.nn.functional and Hugging Face classes): the oracle against them on the CPU, and the kernels against
them directly - not through the oracle - on the GPU."""
import os

import numpy as np
import pytest

from oracle import models as OM
from oracle import ops as O
from tests.golden.make_vectors import GLM_GOLDEN, LLAMA_GOLDEN, chatglm2_shapes, llama_shapes, seeded_state_dict

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
f16, f32 = np.float16, np.float32


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def rel(got, ref):
    return np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() / np.abs(ref.astype(np.float64)).max()


# ------------------------------------------------------------------ oracle against the fixtures (CPU)
@pytest.mark.parametrize("fmt", ["F143", "F152"])
def test_oracle_fp8_codecs(fmt):
    g = load("fp8_fnuz.npz")
    tab = O.f8_table(fmt)
    ok = np.arange(256) != 0x80
    assert np.array_equal(tab[ok], g["table_" + fmt][ok]) and np.isnan(tab[0x80])
    assert np.array_equal(O.f8_encode(g["x_" + fmt], fmt, 0), g["codes_" + fmt])


def test_oracle_int4_nibbles():
    g = load("int4_nibbles.npz")
    packed = g["byte"].view(np.int8).reshape(256, 1)
    w = O.int4_to_half(packed, np.ones(256, f16), 1)            # [2, 256]: row 0 the high nibbles, row 1 the low ones
    assert np.array_equal(w[0], g["high"].astype(f16)) and np.array_equal(w[1], g["low"].astype(f16))


def test_oracle_operators():
    g = load("operators.npz")
    assert np.abs(O.softmax_ce(g["softmax_x"].astype(f32), -1, True) - g["softmax_y"]).max() < 1e-6
    assert np.abs(O.softmax_ce(g["softmax_x"], -1, True).astype(f32) - g["softmax_y"]).max() < 2e-3
    ln = O.layer_norm_ce(g["ln_x"], g["ln_gamma"], g["ln_beta"], 1e-5, 3, 1, 256)
    assert np.abs(ln.astype(f32).reshape(3, 256) - g["ln_y"]).max() <= 6e-3
    rms = O.rms_norm(g["rms_x"], g["rms_w"], 1e-5)
    assert np.abs(rms.astype(f32) - g["rms_y"]).max() <= 3 * 2.0 ** -10 * np.abs(g["rms_y"]).max()
    for i, st in enumerate(g["rope_steps"]):
        sin, cos = O.llama_sincos(int(st), 128)
        got = O.llama_rope(g["rope_q"][i], sin, cos).astype(f32)
        # the fp16 angle (step * inv_freq rounded to fp16) bounds the deviation from the fp32 rotation
        assert np.abs(got - g["rope_y"][i]).max() <= max(int(st), 1) * 2.0 ** -10 * 4 + 4e-3, f"step {st}"


def test_oracle_llama_logits():
    g = load("llama_hf.npz")
    sd = seeded_state_dict(llama_shapes(LLAMA_GOLDEN), int(g["seed"]))
    toks = g["tokens"]
    B, L = toks.shape
    model = OM.Llama2Oracle(sd, LLAMA_GOLDEN, L, B)
    mask = np.full((B, L), -10000, f16)
    for step in range(L):
        mask[:, step] = 0
        _, logits = model.step(toks[:, step].reshape(B, 1), step, mask)
        assert rel(logits, g["logits"][:, step]) < 2e-2, f"step {step}"


def test_oracle_chatglm2_logits():
    """ChatGLM2Oracle end to end (fp16) against Hugging Face's GlmForCausalLM - the same block: RMSNorm, q/k/v
    with bias over two KV heads, rotary embedding on interleaved pairs of the first half of each head, fused
    gate | up SwiGLU - holding the same seeded weights, position by position."""
    g = load("glm_hf.npz")
    sd = seeded_state_dict(chatglm2_shapes(GLM_GOLDEN), int(g["seed"]))
    toks = g["tokens"]
    B, L = toks.shape
    model = OM.ChatGLM2Oracle(sd, GLM_GOLDEN, L, B, "fp16")
    mask = np.full((B, L), -10000, f16)
    for step in range(L):
        mask[:, step] = 0
        _, logits = model.step(toks[:, step].reshape(B, 1), step, mask)
        assert rel(logits, g["logits"][:, step]) < 2e-2, f"step {step}"


# ------------------------------------------------------------------ kernels against the fixtures (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["F143", "F152"])
def test_kernel_fp8_codecs(fmt):
    import torch
    from poptransformer_amd import kernels as K
    g = load("fp8_fnuz.npz")
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    codes = torch.arange(256, dtype=torch.uint8, device="cuda")
    got = K.fp8_to_half(codes, zero, fmt).cpu().numpy().astype(f32)
    ok = np.arange(256) != 0x80
    assert np.array_equal(got[ok], g["table_" + fmt][ok]) and np.isnan(got[0x80])
    enc = K.half_to_fp8(torch.from_numpy(g["x_" + fmt]).cuda(), zero, fmt).cpu().numpy()
    assert np.array_equal(enc, g["codes_" + fmt])


@pytest.mark.gpu
def test_kernel_int4_nibbles():
    import torch
    from poptransformer_amd import kernels as K
    g = load("int4_nibbles.npz")
    packed = torch.from_numpy(g["byte"].view(np.int8).reshape(256, 1).copy()).cuda()
    w = K.int4_to_half(packed, torch.ones(256, dtype=torch.float16, device="cuda"), 1).cpu().numpy()
    assert np.array_equal(w[0], g["high"].astype(f16)) and np.array_equal(w[1], g["low"].astype(f16))


@pytest.mark.gpu
def test_kernel_operators():
    import torch
    from poptransformer_amd import kernels as K
    g = load("operators.npz")
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    assert np.abs(K.softmax_ce(d(g["softmax_x"]), True).cpu().numpy().astype(f32) - g["softmax_y"]).max() < 2e-3
    ln = K.layer_norm_ce(d(g["ln_x"]), d(g["ln_gamma"]), d(g["ln_beta"]), 1e-5).cpu().numpy().astype(f32)
    assert np.abs(ln - g["ln_y"]).max() <= 6e-3
    rms = K.rmsnorm(d(g["rms_x"]), d(g["rms_w"]), 1e-5).cpu().numpy().astype(f32)
    assert np.abs(rms - g["rms_y"]).max() <= 3 * 2.0 ** -10 * np.abs(g["rms_y"]).max()


@pytest.mark.gpu
def test_kernel_llama_logits_against_hugging_face():
    """The decoder on the GPU (fp16 weights, one launch per operator) against the logits Hugging Face's
    LlamaForCausalLM gives for the same weights and tokens, position by position."""
    import torch
    from poptransformer_amd.engine import fused, loader
    g = load("llama_hf.npz")
    sd = seeded_state_dict(llama_shapes(LLAMA_GOLDEN), int(g["seed"]))
    toks = g["tokens"]
    B, L = toks.shape
    dec = fused.FusedDecoder(loader.llama2_spec(LLAMA_GOLDEN, L + 1, B, pad_id=0, eos_id=-1), loader.llama2_weights(sd, LLAMA_GOLDEN))
    ids = np.zeros((B, L + 1), np.int32)
    ids[:, :L] = toks
    dec.reset(ids)
    for step in range(L):
        dec.step_fn()
        torch.cuda.synchronize()
        assert rel(dec.logits.cpu().numpy(), g["logits"][:, step]) < 2e-2, f"step {step}"


@pytest.mark.gpu
def test_kernel_chatglm2_logits_against_hugging_face():
    """The ChatGLM2 decoder on the GPU (fp16 weights, one launch per operator) against the logits of Hugging
    Face's GlmForCausalLM for the same weights and tokens, position by position."""
    import torch
    from poptransformer_amd.engine import fused, loader
    g = load("glm_hf.npz")
    sd = seeded_state_dict(chatglm2_shapes(GLM_GOLDEN), int(g["seed"]))
    toks = g["tokens"]
    B, L = toks.shape
    dec = fused.FusedDecoder(loader.chatglm2_spec(GLM_GOLDEN, L + 1, B, pad_id=0, eos_id=-1),
                             loader.chatglm2_weights(sd, GLM_GOLDEN, "fp16"))
    ids = np.zeros((B, L + 1), np.int32)
    ids[:, :L] = toks
    dec.reset(ids)
    for step in range(L):
        dec.step_fn()
        torch.cuda.synchronize()
        assert rel(dec.logits.cpu().numpy(), g["logits"][:, step]) < 2e-2, f"step {step}"
