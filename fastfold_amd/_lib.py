"""ctypes binding of libffk.so, the C-ABI kernel library (include/ffk.h).

The library is loaded from ``fastfold_amd/csrc/libffk.so`` (built in-tree by
``python -m fastfold_amd.csrc.build``).  There is no fallback: every op raises
``RuntimeError`` if the library is missing or a call returns a non-zero status.
Tensors cross the boundary as ``data_ptr()`` integers plus explicit shapes; the
launch stream is torch's current HIP stream.
"""
import ctypes
import os
from ctypes import c_int, c_int64, c_float, c_void_p, c_char_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libffk.so")

FFK_F32, FFK_BF16, FFK_F16 = 0, 1, 2
_DTYPE_TAG = {torch.float32: FFK_F32, torch.bfloat16: FFK_BF16, torch.float16: FFK_F16}

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float

# name -> argtypes; every entry of include/ffk.h that returns an int status
SIGNATURES = {
    "ffk_softmax_fwd": [_P, _P, _P, _P, _L, _L, _L, _L, _L, _I, _P],
    "ffk_softmax_bwd": [_P, _P, _P, _L, _L, _I, _P],
    "ffk_layernorm_fwd": [_P, _P, _P, _P, _P, _P, _L, _L, _F, _I, _P],
    "ffk_layernorm_bwd": [_P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _P],
    "ffk_bias_sigmoid_mul": [_P, _P, _P, _P, _L, _L, _I, _P],
    "ffk_bias_dropout_add": [_P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _L, _I, _P],
    "ffk_bias_ele_dropout_res": [_P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _L, _I, _P],
}

_lib = None


def load(path: str = None):
    """Loads libffk.so (once) and declares the prototypes."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise RuntimeError(
            "fastfold_amd: %s not found - build it with `python -m fastfold_amd.csrc.build` "
            "(there is no CPU or PyTorch fallback)" % p)
    lib = ctypes.CDLL(p)
    lib.ffk_version.restype = c_int
    lib.ffk_version.argtypes = []
    lib.ffk_last_error_string.restype = c_char_p
    lib.ffk_last_error_string.argtypes = []
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = argtypes
    _lib = lib
    return lib


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def dtype_tag(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_TAG[dtype]
    except KeyError:
        raise RuntimeError("fastfold_amd: unsupported dtype %s" % dtype)


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def ptr(t):
    """Device address of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


def check_device(*tensors):
    """The reference's CHECK_INPUT: every tensor on the GPU and contiguous
    (fastfold/model/fastnn/kernel/cuda_native/csrc/softmax_cuda_kernel.cu:12-16)."""
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("fastfold_amd: tensor must be a CUDA/HIP tensor (got %s)" % t.device)
        if not t.is_contiguous():
            raise RuntimeError("fastfold_amd: tensor must be contiguous")


def call(name: str, *args):
    """Calls an entry point; raises RuntimeError with the library's message on failure."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.ffk_last_error_string()
        raise RuntimeError("%s failed (status %d): %s" % (name, rc, msg.decode() if msg else "?"))
