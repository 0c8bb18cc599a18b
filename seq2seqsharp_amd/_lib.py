"""ctypes loader for libtship.so.  There is no fallback: if the library is missing or fails to load,
every entry point raises."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtship.so")
MAX_DIMS = 6


class TSHipError(RuntimeError):
    """Raised when a native call returns 0 (mirrors the InvalidOperationException of the managed side)."""


class TSHipTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("ndim", C.c_int32),
                ("sizes", C.c_int64 * MAX_DIMS), ("strides", C.c_int64 * MAX_DIMS)]


class TSHipGptConfig(C.Structure):
    _fields_ = [("n_layers", C.c_int32), ("hidden", C.c_int32), ("n_heads", C.c_int32), ("n_kv_heads", C.c_int32),
                ("ffn_dim", C.c_int32), ("vocab", C.c_int32), ("attn_type", C.c_int32), ("norm_type", C.c_int32),
                ("act", C.c_int32), ("n_experts", C.c_int32), ("experts_per_token", C.c_int32),
                ("norm_eps", C.c_float), ("rope_base", C.c_float), ("use_rope", C.c_int32), ("dtype", C.c_int32),
                ("max_batch", C.c_int32), ("max_seq_len", C.c_int32),
                ("max_segments", C.c_int32), ("sep_token_id", C.c_int32)]


_lib = None


def lib():
    """Load the native library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise TSHipError("libtship.so is not built: run `python -m seq2seqsharp_amd.build` "
                         "(needs hipcc; there is no CPU fallback)")
    L = C.CDLL(LIB_PATH)
    L.TSHip_GetLastError.restype = C.c_char_p
    _lib = L
    return L


def check(rc):
    if rc != 1:
        msg = lib().TSHip_GetLastError()
        raise TSHipError(msg.decode() if msg else "native call failed")
