"""Checkpoints on the local disk <-> the state dicts the models take.

The reference obtains its weights with `AutoModel*.from_pretrained(<hub name>)`
(poptransformer/models/base_model.py:199-223, models/llama2/model.py:135-149), converts the
torch state dict to numpy and hands it to the layers, which look their tensors up by the
checkpoint's own key names (layers/linear.py:28-40).  There is no network here and nothing is
fetched: a checkpoint is a directory or a file on the local disk.

Formats read: `*.safetensors` (one file, or the shards listed in `*.safetensors.index.json`), and
torch `*.bin` / `*.pt` / `*.pth` state dicts, which are opened with `weights_only=True` (nothing in
the file is executed).  Floating-point tensors come back as fp16, which is what the reference's
graphs hold; integer tensors (packed INT4 weights, FP8 bytes) are left as they are.

INT4 checkpoints follow the layout of the reference's int4 path
(utils/param_handler/precision_strategy.py:24-42, examples/chatglm/conf/int4_sharding.yaml:20):
`<ctx>.weight` int8 [out, in/2] with two signed nibbles per byte (the high nibble is the even input
feature) and `<ctx>.weight_scale` fp16 [out].  The reference only loads such checkpoints;
`quantize_int4` / `quantize_state_dict_int4` produce them (symmetric per output channel,
scale = max|w| / 7).

`save_state_dict` writes safetensors: the counterpart of `saveInitializersExternally`
(utils/prepare.py:40-43), which moves the initializers out of the model proto into a file.
"""
import glob
import json
import os

import numpy as np

_TORCH_SUFFIXES = (".bin", ".pt", ".pth")


def _to_numpy(t):
    """torch tensor -> numpy; floating point becomes fp16."""
    import torch
    if t.is_floating_point():
        return t.to(torch.float16).contiguous().numpy()
    return t.contiguous().numpy()


def _read_safetensors(path):
    # through torch, so that bf16 tensors (which numpy cannot hold) are read too
    from safetensors import safe_open
    out = {}
    with safe_open(path, framework="pt", device="cpu") as f:
        for key in f.keys():
            out[key] = _to_numpy(f.get_tensor(key))
    return out


def _read_torch(path):
    import torch
    sd = torch.load(path, map_location="cpu", weights_only=True)
    if isinstance(sd, dict) and "state_dict" in sd and isinstance(sd["state_dict"], dict):
        sd = sd["state_dict"]
    if not isinstance(sd, dict):
        raise ValueError(f"{path} does not hold a state dict")
    return {k: _to_numpy(v) for k, v in sd.items() if hasattr(v, "is_floating_point")}


def load_state_dict(path):
    """path: a .safetensors / .bin / .pt / .pth file, a *.index.json shard index, or a directory
    holding any of these (Hugging Face layout).  Returns {key: numpy array}."""
    if os.path.isdir(path):
        for pattern in ("*.safetensors.index.json", "*.bin.index.json"):
            index = sorted(glob.glob(os.path.join(path, pattern)))
            if index:
                return load_state_dict(index[0])
        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            files = sorted(f for s in _TORCH_SUFFIXES for f in glob.glob(os.path.join(path, "*" + s)))
        if not files:
            raise FileNotFoundError(f"no checkpoint files (*.safetensors, *.bin, *.pt, *.pth) in {path}")
        out = {}
        for f in files:
            out.update(load_state_dict(f))
        return out
    if path.endswith(".index.json"):
        with open(path) as f:
            weight_map = json.load(f)["weight_map"]
        out = {}
        for shard in sorted(set(weight_map.values())):
            out.update(load_state_dict(os.path.join(os.path.dirname(path), shard)))
        missing = [k for k in weight_map if k not in out]
        if missing:
            raise KeyError(f"{path} lists tensors its shards do not hold: {missing[:3]} ...")
        return out
    if path.endswith(".safetensors"):
        return _read_safetensors(path)
    if path.endswith(_TORCH_SUFFIXES):
        return _read_torch(path)
    raise ValueError(f"unknown checkpoint format: {path}")


def save_state_dict(state_dict, path, max_shard_bytes=None):
    """Writes {key: numpy array} as safetensors.  With `max_shard_bytes`, `path` is a directory that
    receives model-XXXXX-of-YYYYY.safetensors shards and model.safetensors.index.json."""
    from safetensors.numpy import save_file
    arrays = {k: np.ascontiguousarray(v) for k, v in state_dict.items()}
    if max_shard_bytes is None:
        save_file(arrays, path)
        return [path]
    os.makedirs(path, exist_ok=True)
    shards, current, size = [], {}, 0
    for key, value in arrays.items():
        if current and size + value.nbytes > max_shard_bytes:
            shards.append(current)
            current, size = {}, 0
        current[key] = value
        size += value.nbytes
    if current:
        shards.append(current)
    weight_map, files = {}, []
    for i, shard in enumerate(shards):
        name = f"model-{i + 1:05d}-of-{len(shards):05d}.safetensors"
        save_file(shard, os.path.join(path, name))
        files.append(os.path.join(path, name))
        weight_map.update({k: name for k in shard})
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"total_size": int(sum(v.nbytes for v in arrays.values()))}, "weight_map": weight_map}, f)
    return files


def pack_int4(q):
    """q integer [out, in] in [-8, 7] -> int8 [out, in/2]: byte j of a row holds feature 2j in its
    high nibble and feature 2j+1 in its low nibble (custom_ops/int4_to_half_codelets.cpp:33-34)."""
    q = np.asarray(q)
    if q.ndim != 2 or q.shape[1] % 2:
        raise ValueError("pack_int4 needs a 2-D array with an even number of columns")
    if q.min() < -8 or q.max() > 7:
        raise ValueError("INT4 values must lie in [-8, 7]")
    u = (q.astype(np.int16) & 0xF).astype(np.uint8)
    return ((u[:, 0::2] << 4) | u[:, 1::2]).view(np.int8)


def quantize_int4(w):
    """w float [out, in] -> (packed int8 [out, in/2], scale fp16 [out]), symmetric per output channel."""
    w = np.asarray(w, np.float32)
    scale = (np.abs(w).max(axis=1) / 7.0).astype(np.float16)
    scale = np.maximum(scale, np.finfo(np.float16).tiny)
    q = np.clip(np.rint(w / scale.astype(np.float32)[:, None]), -8, 7).astype(np.int8)
    return pack_int4(q), scale


def quantize_state_dict_int4(state_dict, is_linear=None):
    """Returns a copy in which every Linear weight `<ctx>.weight` is packed INT4 with
    `<ctx>.weight_scale` beside it.  `is_linear(key, array)` selects them; by default every 2-D
    floating-point `*.weight` except embeddings, output heads and norm weights."""
    def default(key, value):
        if not key.endswith(".weight") or value.ndim != 2 or not np.issubdtype(value.dtype, np.floating):
            return False
        low = key.lower()
        if low.endswith("head.weight"):
            return False
        return not any(s in low for s in ("embed", "wte", "wpe", "output_layer", "norm", "ln_"))
    pick = is_linear or default
    out = {}
    for key, value in state_dict.items():
        if pick(key, value):
            out[key], out[key + "_scale"] = quantize_int4(value)
        else:
            out[key] = value
    return out
