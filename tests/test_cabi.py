"""The C-ABI library loads, exports every symbol include/ffk.h declares, and validates
arguments before touching the GPU (so these run without one)."""
import ctypes
import os
import re

import pytest

from fastfold_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    txt = open(os.path.join(ROOT, "include", "ffk.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(ffk_[a-z0-9_]+)\s*\(", txt)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert "ffk_softmax_fwd" in names and "ffk_layernorm_fwd" in names
    for n in names:
        assert hasattr(lib, n), "libffk.so does not export %s" % n
    assert lib.ffk_version() >= 100
    # every int-returning entry has a declared ctypes signature in the binding
    for n in names:
        if n not in ("ffk_version", "ffk_last_error_string"):
            assert n in _lib.SIGNATURES, "no ctypes signature for %s" % n


def test_argument_validation_without_gpu():
    lib = _lib.load()
    # null pointers
    rc = lib.ffk_softmax_fwd(None, None, None, None, 1, 1, 1, 4, 4, _lib.FFK_BF16, None)
    assert rc == 3 and b"null" in lib.ffk_last_error_string()
    rc = lib.ffk_layernorm_fwd(None, None, None, None, None, None, 4, 4, 1e-5, _lib.FFK_F32, None)
    assert rc == 3
    buf = ctypes.create_string_buffer(256)
    p = ctypes.cast(buf, ctypes.c_void_p)
    # bad shape / bad dtype are rejected before any launch
    assert lib.ffk_softmax_fwd(p, p, None, None, 1, 1, 1, 0, 4, _lib.FFK_BF16, None) == 2
    assert lib.ffk_softmax_fwd(p, p, None, None, 1, 1, 1, 2, 4, 77, None) == 1
    assert lib.ffk_layernorm_fwd(p, None, None, p, p, p, -1, 4, 1e-5, _lib.FFK_F32, None) == 2
    assert lib.ffk_layernorm_fwd(p, None, None, p, p, p, 1, 4, 1e-5, 9, None) == 1
    assert lib.ffk_bias_sigmoid_mul(p, p, None, p, 2, 4, _lib.FFK_F32, None) == 3
    with pytest.raises(RuntimeError):
        _lib.call("ffk_softmax_bwd", None, None, None, 1, 1, 0, None)


def test_library_exports_nothing_else():
    """The dynamic symbol table holds the declared entry points and no internal (C++-mangled) helpers."""
    import shutil
    import subprocess
    nm = shutil.which("nm")
    if nm is None:
        pytest.skip("binutils nm not available")
    out = subprocess.run([nm, "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    assert exported == _declared(), sorted(set(exported) ^ set(_declared()))
