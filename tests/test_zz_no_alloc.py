"""pta_llama_decode_step_static - the decode step whose workspace is an array built into the library, for callers
that cannot allocate - against pta_llama_decode_step with a workspace of its own: two generations in a row
through the same built-in array, the second of a smaller model at a smaller batch, bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import models as OM

pytestmark = pytest.mark.gpu

FIRST = dict(vocab_size=512, hidden_size=256, rms_norm_eps=1e-5, num_attention_heads=2, intermediate_size=688,
             num_hidden_layers=3)
SECOND = dict(vocab_size=384, hidden_size=128, rms_norm_eps=1e-5, num_attention_heads=1, intermediate_size=344,
              num_hidden_layers=2)


def _decoder(cfg, B, L, seed):
    from poptransformer_amd.engine import fused, loader
    sd = OM.make_llama2_state_dict(cfg, seed=seed, int4=True)
    dec = fused.FusedDecoder(loader.llama2_spec(cfg, L, B, 0, 2), loader.llama2_weights(sd, cfg))
    return dec.enable_persistent()


def _generate(dec, ids, steps, static):
    """`steps` loop iterations; returns the logits and ids of every iteration, the container and the KV rings."""
    dec.reset(ids)
    logits, picks = [], []
    for _ in range(steps):
        if static:
            dec.persistent.launch_static()
        else:
            dec.persistent.launch()
        torch.cuda.synchronize()
        logits.append(dec.logits.cpu().numpy().copy())
        picks.append(dec.next_ids.cpu().numpy().copy())
    return logits, picks, dec.container.cpu().numpy().copy(), [r.cpu().numpy().copy() for r in dec.rings], int(dec.step.item())


def _same(a, b):
    for x, y in zip(a[0], b[0]):
        assert np.array_equal(x.view(np.uint16), y.view(np.uint16)), "logits differ"
    for x, y in zip(a[1], b[1]):
        assert np.array_equal(x, y), "selected ids differ"
    assert np.array_equal(a[2], b[2]), "containers differ"
    for x, y in zip(a[3], b[3]):
        assert np.array_equal(x.view(np.uint16), y.view(np.uint16)), "KV rings differ"
    assert a[4] == b[4]


def test_decode_step_without_a_workspace_argument():
    rng = np.random.default_rng(3)
    cases = [(FIRST, 3, 48, 24, 5), (SECOND, 1, 32, 20, 6)]       # the second call is the smaller one
    for cfg, B, L, steps, seed in cases:
        print(f"case: static decode step, hidden {cfg['hidden_size']}, batch {B}", flush=True)
        ids = np.zeros((B, L), np.int32)
        ids[:, :6] = rng.integers(3, cfg["vocab_size"], size=(B, 6))
        own = _decoder(cfg, B, L, seed)
        ref = _generate(own, ids, steps, static=False)
        assert not own.persistent.failed() and ref[4] == steps
        builtin = _decoder(cfg, B, L, seed)
        got = _generate(builtin, ids, steps, static=True)
        _same(got, ref)
        # its own workspace was never used by the static launches
        assert int(builtin.persistent.workspace.view(torch.int32)[0].item()) == 0


def test_static_decode_step_of_many_sequences_after_a_larger_model():
    """Batch 8 and 16 (decode_step_wide_kernel: its arrival words and per-workgroup best logits sit behind the
    model-dependent slots of the shared array) after a launch of a different model with more layers through the same
    array, bit for bit against the entry point with a workspace of its own."""
    rng = np.random.default_rng(5)
    for cfg, B, L, steps, seed in [(FIRST, 3, 48, 8, 5), (SECOND, 16, 40, 24, 7), (FIRST, 8, 48, 24, 8)]:
        print(f"case: static decode step, hidden {cfg['hidden_size']}, batch {B}", flush=True)
        ids = np.zeros((B, L), np.int32)
        ids[:, :6] = rng.integers(3, cfg["vocab_size"], size=(B, 6))
        own = _decoder(cfg, B, L, seed)
        ref = _generate(own, ids, steps, static=False)
        assert not own.persistent.failed() and ref[4] == steps
        _same(_generate(_decoder(cfg, B, L, seed), ids, steps, static=True), ref)


def test_static_decode_step_refuses_what_the_built_in_array_cannot_hold():
    """A model whose workspace exceeds the 16 MiB array is refused before anything is launched (only sizes are
    read on the host: the pointers of this descriptor are never followed)."""
    from poptransformer_amd import _lib
    lib = _lib.load()
    keep = torch.zeros(64, dtype=torch.uint8, device="cuda")
    p = keep.data_ptr()
    model = _lib.DecodeModel(p, 4000, p, p, p, p, 4, 256, 2, 128, 688, 512, 64, 1e-5, 0, 2, 0)
    assert lib.pta_decode_step_workspace_bytes(ctypes.byref(model)) > (16 << 20)
    state = _lib.DecodeState(*([p] * 7))
    rc = lib.pta_llama_decode_step_static(ctypes.byref(model), ctypes.byref(state), 0, None)
    assert rc == _lib.PTA_EINVAL and b"built-in array" in lib.pta_last_error()
    torch.cuda.synchronize()
