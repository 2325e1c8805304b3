"""Host-side (numpy) FP8 encoder used when Linear weights are bound under precision 'fp8' /
'fp8_weight'.  The reference calls poprt's `convert_float_to_uint8(w, 'F143', -1)` at the same point
(poptransformer/utils/param_handler/precision_strategy.py:44-51).  Same arithmetic as the device
encoder in csrc/fp8.hip: round to nearest even on the format grid, saturate, NaN -> 0x80."""
import numpy as np

_FORMATS = {"F143": (3, 8, 240.0), "F152": (2, 16, 57344.0)}


def f8_encode_host(x, fmt="F143", scale=0):
    if fmt not in _FORMATS:
        raise ValueError(f"Unsupport fp8 meata data {fmt}, it must be F143 or F152")
    mb, bias, vmax = _FORMATS[fmt]
    v = np.asarray(x, np.float64) * 2.0 ** (-int(scale))
    mag = np.abs(v)
    _, e = np.frexp(np.where(mag > 0, mag, 1.0))
    ef = np.maximum(e - 1 + bias, 1)
    q = np.rint(np.ldexp(mag, mb - (ef - bias)))
    carry = q >= (2 << mb)
    q = np.where(carry, q / 2, q)
    ef = np.where(carry, ef + 1, ef)
    sub = (ef == 1) & (q < (1 << mb))
    code = np.where(sub, q, ef * (1 << mb) + q - (1 << mb)).astype(np.int64)
    code = np.minimum(code, 0x7F)
    code = np.where(mag >= vmax, 0x7F, code)
    code = np.where(mag == 0, 0, code)
    code = np.where((v < 0) & (code != 0), code | 0x80, code)
    code = np.where(np.isnan(v), 0x80, code)
    return code.astype(np.uint8)
