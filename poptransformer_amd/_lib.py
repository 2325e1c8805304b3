"""ctypes binding of libpoptransformer_hip.so.

The reference loads its native ops with ``ctypes.cdll.LoadLibrary('../../custom_ops.so')`` at
import of ``poptransformer/ops/customized.py`` (lines 14-18); this module is the counterpart.
The library must have been built (``python -m poptransformer_amd.build`` or
``__graft_entry__.build()``): a missing library is an error, there is no fallback.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
# POPTRANSFORMER_HIP_LIB names another build of the library (e.g. one compiled with -DDS_TRACE)
LIB_PATH = os.environ.get("POPTRANSFORMER_HIP_LIB") or os.path.join(HERE, "libpoptransformer_hip.so")

PTA_OK, PTA_EINVAL, PTA_EUNSUPPORTED, PTA_EHIP = 0, -1, -2, -3
ACT_NONE, ACT_GELU_TANH, ACT_RELU_SQUARE, ACT_SIGMOID = 0, 1, 2, 3
F16, F32 = 0, 1
ROPE_NONE, ROPE_LLAMA, ROPE_GLM2 = 0, 1, 2
F143, F152 = 0, 1
FP8_FORMATS = {"F143": F143, "F152": F152}


NORM_NONE, NORM_RMS, NORM_LAYER = 0, 1, 2


class Weight(ctypes.Structure):
    _fields_ = [("kind", c_int), ("tiled", c_void_p), ("scale", c_void_p), ("N", c_int), ("K", c_int),
                ("x", c_void_p), ("act", c_int), ("mix", c_void_p)]


W_INT4, W_F16, W_F143, W_F152 = 0, 1, 2, 3


class DecodeLayer(ctypes.Structure):
    _fields_ = [(n, c_void_p) for n in ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "sq", "sk", "sv", "so", "sg", "su",
                                        "sd", "norm1", "norm2", "kv_ring")]


class DecodeModel(ctypes.Structure):
    _fields_ = [("layers", c_void_p), ("n_layer", c_int), ("embed", c_void_p), ("final_norm", c_void_p),
                ("head", c_void_p), ("inv_freq", c_void_p),
                ("batch", c_int), ("hidden", c_int), ("n_head", c_int), ("head_dim", c_int), ("ffn", c_int),
                ("vocab", c_int), ("max_len", c_int), ("eps", c_float),
                ("pad_id", c_int), ("eos_id", c_int), ("early_stop", c_int)]


class DecodeState(ctypes.Structure):
    _fields_ = [(n, c_void_p) for n in ("container", "mask", "stop_mask", "step", "keep_going", "next_ids", "logits")]


class Fusion(ctypes.Structure):
    _fields_ = [("bias", c_void_p), ("residual", c_void_p), ("act", c_int), ("mul", c_void_p), ("post_scale", c_float),
                ("norm", c_int),
                ("norm_weight", c_void_p), ("norm_bias", c_void_p), ("norm_eps", c_float),
                ("workspace", c_void_p), ("workspace_bytes", c_size_t),
                ("out_fp8_scale", c_void_p), ("out_fp8_format", c_int),
                ("mix_state", c_void_p), ("mix_step", c_void_p)]


# name -> (restype, argtypes); the order follows include/poptransformer_hip.h
SIGNATURES = {
    "pta_version": (c_int, []),
    "pta_last_error": (c_char_p, []),
    "pta_int4_to_half": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "pta_w4_tiled_bytes": (c_size_t, [c_int, c_int]),
    "pta_w4_tile": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "pta_w4a16_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, POINTER(Fusion), c_void_p]),
    "pta_w4a16_gemm_multi": (c_int, [c_void_p, c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                     POINTER(c_int), c_int, c_int, POINTER(Fusion), c_void_p]),
    "pta_w4a16_gemm_swiglu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                      POINTER(Fusion), c_void_p]),
    "pta_f16_tiled_bytes": (c_size_t, [c_int, c_int]),
    "pta_f16_tile": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "pta_f16_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, POINTER(Fusion), c_void_p]),
    "pta_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p]),
    "pta_layer_norm_ce": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p]),
    "pta_softmax_ce": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_kv_cache_update": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_kv_cache_append": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_kv_cache_read": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_kv_cache_pipeline_seq_last": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_qkv_rope_append": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_decode_attention_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "pta_decode_attention_qkv": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_decode_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                     c_int, c_int, c_void_p]),
    "pta_prompt_rope_append": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                       c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_prompt_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                     c_int, c_int, c_int, c_void_p]),
    "pta_prompt_rope_append_f8": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pta_prompt_attention_f8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                        c_int, c_int, c_int, c_int, c_void_p]),
    "pta_decode_attention_qkv_f8": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                            c_void_p]),
    "pta_decode_attention_qkv_grid": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                              c_int, c_void_p]),
    "pta_rmsnorm_fp8_grid": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "pta_linear_workspace_bytes": (c_size_t, [c_int, c_int]),
    "pta_argmax": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "pta_topk": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "pta_take_column": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "pta_beam_search_workspace_bytes": (c_size_t, [c_int, c_int]),
    "pta_beam_search_step": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                     c_int, c_int, c_void_p]),
    "pta_embedding": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "pta_half_to_fp8": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "pta_fp8_to_half": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "pta_fp8_tiled_bytes": (c_size_t, [c_int, c_int]),
    "pta_fp8_tile": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "pta_fp8_gemm_workspace_bytes": (c_size_t, [c_int, c_int]),
    "pta_fp8_gemm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                             c_void_p, POINTER(Fusion), c_void_p]),
    "pta_half_to_fp8_grid": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "pta_linear": (c_int, [c_void_p, c_void_p, c_int, POINTER(Weight), POINTER(c_void_p), POINTER(c_void_p), c_int, c_int,
                           POINTER(Fusion), c_void_p]),
    "pta_swiglu": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "pta_rwkv_mix": (c_int, [c_void_p] * 8 + [c_int, c_int, c_void_p]),
    "pta_layer_norm_ce_mix": (c_int, [c_void_p] * 11 + [c_int, c_int, c_float, c_void_p]),
    "pta_rwkv_wkv": (c_int, [c_void_p] * 9 + [c_int, c_int, c_void_p]),
    "pta_step_update": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                c_int, c_int, c_int, c_void_p]),
    "pta_decode_step_workspace_bytes": (c_size_t, [POINTER(DecodeModel)]),
    "pta_llama_decode_step": (c_int, [POINTER(DecodeModel), POINTER(DecodeState), c_void_p, c_void_p]),
    "pta_llama_decode_step_f8": (c_int, [POINTER(DecodeModel), POINTER(DecodeState), c_int, c_void_p, c_void_p]),
    "pta_decode_step_failed": (c_int, [c_void_p, POINTER(c_int), c_void_p]),
    "pta_llama_decode_step_static": (c_int, [POINTER(DecodeModel), POINTER(DecodeState), c_int, c_void_p]),
}

_lib = None


class PtaError(RuntimeError):
    pass


def load():
    """Load the shared library and declare every prototype. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise PtaError(
            f"{LIB_PATH} is missing: build it with `python -m poptransformer_amd.build` "
            "(there is no CPU fallback for the HIP kernels)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def check(rc, what=""):
    """Translate a status code into the exception the reference would have raised: invalid
    shapes/attributes are graph-build errors (ValueError), runtime failures RuntimeError."""
    if rc == PTA_OK:
        return
    msg = load().pta_last_error().decode()
    if rc == PTA_EINVAL:
        raise ValueError(msg or what)
    if rc == PTA_EUNSUPPORTED:
        raise NotImplementedError(msg or what)
    raise PtaError(msg or what)
