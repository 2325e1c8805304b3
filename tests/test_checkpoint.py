"""Local checkpoint files <-> state dicts (poptransformer_amd/utils/checkpoint.py)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import models as OM
from oracle import ops as O
from poptransformer_amd.utils import checkpoint as C

CFG = dict(vocab_size=96, hidden_size=128, rms_norm_eps=1e-5, num_attention_heads=1, intermediate_size=256,
           num_hidden_layers=2)


def same(a, b):
    assert a.keys() == b.keys()
    for k in a:
        assert a[k].dtype == b[k].dtype and np.array_equal(a[k], b[k]), k


def test_safetensors_single_file_round_trip(tmp_path):
    sd = OM.make_llama2_state_dict(CFG, seed=3, int4=True)
    path = str(tmp_path / "model.safetensors")
    C.save_state_dict(sd, path)
    same(C.load_state_dict(path), sd)
    same(C.load_state_dict(str(tmp_path)), sd)          # the directory finds the file


def test_sharded_safetensors_with_index(tmp_path):
    sd = OM.make_llama2_state_dict(CFG, seed=4, int4=False)
    files = C.save_state_dict(sd, str(tmp_path), max_shard_bytes=64 * 1024)
    assert len(files) > 2
    index = json.load(open(tmp_path / "model.safetensors.index.json"))
    assert set(index["weight_map"]) == set(sd)
    same(C.load_state_dict(str(tmp_path)), sd)
    os.remove(files[1])
    with pytest.raises(Exception):
        C.load_state_dict(str(tmp_path))


def test_torch_state_dict_and_dtype_conversion(tmp_path):
    rng = np.random.default_rng(0)
    w32 = rng.standard_normal((8, 16)).astype(np.float32)
    tsd = {"a.weight": torch.from_numpy(w32), "b.weight": torch.from_numpy(w32).to(torch.bfloat16),
           "c.weight": torch.arange(-8, 8, dtype=torch.int8).reshape(2, 8)}
    path = str(tmp_path / "pytorch_model.bin")
    torch.save(tsd, path)
    sd = C.load_state_dict(path)
    assert sd["a.weight"].dtype == np.float16 and np.array_equal(sd["a.weight"], w32.astype(np.float16))
    assert sd["b.weight"].dtype == np.float16
    assert np.array_equal(sd["b.weight"], torch.from_numpy(w32).to(torch.bfloat16).to(torch.float16).numpy())
    assert sd["c.weight"].dtype == np.int8 and np.array_equal(sd["c.weight"], tsd["c.weight"].numpy())
    # bf16 in safetensors as well (numpy cannot hold it: read through torch)
    from safetensors.torch import save_file
    save_file({"b.weight": tsd["b.weight"]}, str(tmp_path / "m.safetensors"))
    assert np.array_equal(C.load_state_dict(str(tmp_path / "m.safetensors"))["b.weight"], sd["b.weight"])


def test_a_pickled_object_is_refused(tmp_path):
    import pickle

    class Boom:
        def __reduce__(self):
            return (os.system, ("true",))
    path = str(tmp_path / "evil.pt")
    with open(path, "wb") as f:
        pickle.dump({"x": Boom()}, f)
    with pytest.raises(Exception):
        C.load_state_dict(path)


def test_unknown_format_and_empty_directory(tmp_path):
    with pytest.raises(ValueError):
        C.load_state_dict(str(tmp_path / "weights.onnx"))
    with pytest.raises(FileNotFoundError):
        C.load_state_dict(str(tmp_path))


def test_pack_int4_matches_the_unpack_truth_table():
    rng = np.random.default_rng(1)
    q = rng.integers(-8, 8, size=(5, 12))
    packed = C.pack_int4(q)
    assert packed.dtype == np.int8 and packed.shape == (5, 6)
    assert np.array_equal(O.nibble_hi(packed), q[:, 0::2]) and np.array_equal(O.nibble_lo(packed), q[:, 1::2])
    assert np.array_equal(packed, O.pack_int4(q))
    with pytest.raises(ValueError):
        C.pack_int4(np.array([[8, 0]]))
    with pytest.raises(ValueError):
        C.pack_int4(np.zeros((2, 3), np.int64))


def test_quantize_int4_error_bound_and_layout():
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((16, 64)) * 0.02).astype(np.float16)
    packed, scale = C.quantize_int4(w)
    back = O.int4_to_half(packed, scale, 1).T.astype(np.float32)          # [out, in]
    assert np.all(np.abs(back - w.astype(np.float32)) <= 0.5 * scale.astype(np.float32)[:, None] * 1.001 + 1e-6)
    p2, s2 = OM.quantize_int4(w)
    assert np.array_equal(packed, p2) and np.array_equal(scale, s2)


def test_quantize_state_dict_selects_linear_weights_only():
    sd = OM.make_llama2_state_dict(CFG, seed=5, int4=False)
    q = C.quantize_state_dict_int4(sd)
    ref = OM.make_llama2_state_dict(CFG, seed=5, int4=True)
    same(q, ref)
