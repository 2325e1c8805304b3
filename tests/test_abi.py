"""The C-ABI library loads on a machine without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "poptransformer_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pta_[a-z0-9_]+)\s*\(", text)))


def _library():
    from poptransformer_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from poptransformer_amd import build
        build.build(force=False)
    return _lib


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared()
    assert len(names) >= 20
    _lib = _library()
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes prototype in poptransformer_amd/_lib.py"
    for n in _lib.SIGNATURES:
        assert n in names, f"{n} is bound but not declared in the header"


def test_version_and_error_string_without_gpu():
    _lib = _library()
    lib = _lib.load()
    assert lib.pta_version() >= 100
    # argument validation happens on the host before any launch: no GPU is needed to see it
    rc = lib.pta_int4_to_half(None, None, None, 4, 4, 7, None)
    assert rc == _lib.PTA_EINVAL
    assert b"'axis' should be 0 or 1" in lib.pta_last_error()
    assert lib.pta_w4_tiled_bytes(11008, 4096) == 11008 * 4096 // 2
    assert lib.pta_w4_tiled_bytes(17, 130) == 2 * 2 * 1024
