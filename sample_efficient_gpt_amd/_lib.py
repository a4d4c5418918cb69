"""ctypes binding of libsegpt_attn.so (the C ABI declared in include/segpt_attn.h).

There is no CPU or eager fallback: if the shared library is missing, loading raises.
"""

from __future__ import annotations

import ctypes as C
import os
import threading

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libsegpt_attn.so")

SEGPT_ABI_VERSION = 2
SEGPT_DTYPE_BF16 = 0
SEGPT_DTYPE_FP32 = 1
SEGPT_FLAG_KV_PREPARED = 1
SEGPT_FLAG_RUNNING_MAX = 2
SEGPT_FLAG_DECODE = 4
SEGPT_FLAG_NO_NORM = 8
SEGPT_E_SCRATCH_LIMIT = -13
SEGPT_NOALLOC_SCRATCH_BYTES = 16 << 20
SEGPT_WS_KV = 0
SEGPT_WS_BWD = 1
FWD_STAGES = ("pre", "attn")  # SEGPT_FWD_STAGE_* = index
BWD_STAGES = ("pre", "dq", "dkdv", "reduce")  # SEGPT_BWD_STAGE_* = index

EXPORTED_SYMBOLS = (
    "segpt_abi_version",
    "segpt_strerror",
    "segpt_attn_workspace_bytes",
    "segpt_attn_fwd",
    "segpt_attn_bwd",
    "segpt_attn_bwd_stage",
    "segpt_attn_fwd_stage",
    "segpt_attn_fwd_noalloc",
)


class Tensor4(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_h", C.c_int64), ("stride_s", C.c_int64)]


class Tensor3(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_s", C.c_int64), ("stride_h", C.c_int64)]


class AttnParams(C.Structure):
    _fields_ = [
        ("struct_bytes", C.c_uint32),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("H", C.c_int32), ("Hkv", C.c_int32), ("Sq", C.c_int32), ("Sk", C.c_int32), ("D", C.c_int32),
        ("causal", C.c_int32),
        ("q_start", C.c_int32),
        ("gq_numel", C.c_int32),
        ("gk_numel", C.c_int32),
        ("eps", C.c_float), ("sm_scale", C.c_float), ("gate_scale", C.c_float),
        ("flags", C.c_int32),
        ("q", Tensor4), ("k", Tensor4), ("v", Tensor4), ("v_first", Tensor4),
        ("gate", Tensor3),
        ("o", Tensor4),
        ("lse", C.c_void_p),
        ("g_q", C.c_void_p), ("g_k", C.c_void_p), ("vr_coef", C.c_void_p),
        ("d_o", Tensor4), ("dq", Tensor4), ("dk", Tensor4), ("dv", Tensor4), ("dv_first", Tensor4),
        ("dgate", Tensor3),
        ("dg_q", C.c_void_p), ("dg_k", C.c_void_p), ("dvr_coef", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("kv_workspace", C.c_void_p),
        ("kv_workspace_bytes", C.c_size_t),
        ("rope_cos", C.c_void_p), ("rope_sin", C.c_void_p),
        ("rope_len", C.c_int32), ("rope_q_pos0", C.c_int32), ("rope_k_pos0", C.c_int32), ("reserved0", C.c_int32),
    ]


_lib = None
_lock = threading.Lock()


class SegptError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        super().__init__(f"{where} failed with code {code}: {strerror(code)}")


def load():
    """Load (once) and return the ctypes handle; raises if the library was not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} not found: build it with `python -m sample_efficient_gpt_amd.build` "
                "(hipcc, gfx950). There is no fallback path."
            )
        lib = C.CDLL(LIB_PATH)
        lib.segpt_abi_version.restype = C.c_int
        lib.segpt_abi_version.argtypes = []
        lib.segpt_strerror.restype = C.c_char_p
        lib.segpt_strerror.argtypes = [C.c_int]
        lib.segpt_attn_workspace_bytes.restype = C.c_size_t
        lib.segpt_attn_workspace_bytes.argtypes = [C.POINTER(AttnParams), C.c_int]
        lib.segpt_attn_fwd.restype = C.c_int
        lib.segpt_attn_fwd.argtypes = [C.POINTER(AttnParams), C.c_void_p]
        lib.segpt_attn_bwd.restype = C.c_int
        lib.segpt_attn_bwd.argtypes = [C.POINTER(AttnParams), C.c_void_p]
        lib.segpt_attn_bwd_stage.restype = C.c_int
        lib.segpt_attn_bwd_stage.argtypes = [C.POINTER(AttnParams), C.c_int, C.c_void_p]
        lib.segpt_attn_fwd_stage.restype = C.c_int
        lib.segpt_attn_fwd_stage.argtypes = [C.POINTER(AttnParams), C.c_int, C.c_void_p]
        lib.segpt_attn_fwd_noalloc.restype = C.c_int
        lib.segpt_attn_fwd_noalloc.argtypes = [C.POINTER(AttnParams), C.c_void_p]
        ver = lib.segpt_abi_version()
        if ver != SEGPT_ABI_VERSION:
            raise RuntimeError(f"libsegpt_attn.so ABI version {ver}, binding expects {SEGPT_ABI_VERSION}")
        _lib = lib
    return _lib


def strerror(code: int) -> str:
    return load().segpt_strerror(int(code)).decode()


def new_params() -> AttnParams:
    p = AttnParams()
    p.struct_bytes = C.sizeof(AttnParams)
    return p


def t4(t) -> Tensor4:
    """View of a [B, heads, S, D] torch tensor (any strides with a contiguous last dim)."""
    if t is None:
        return Tensor4(None, 0, 0, 0)
    assert t.dim() == 4 and t.stride(3) == 1, "expected a 4-D tensor with a contiguous last dimension"
    return Tensor4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def t3(t) -> Tensor3:
    """View of a [B, S, H] torch tensor."""
    if t is None:
        return Tensor3(None, 0, 0, 0)
    assert t.dim() == 3
    return Tensor3(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def ptr(t):
    return None if t is None else t.data_ptr()


def alloc_workspace(lib, p, which: int, device):
    """Allocate (torch, uint8) the scratch buffer of kind `which` for filled params; returns the tensor."""
    import torch

    nbytes = max(int(lib.segpt_attn_workspace_bytes(p, which)), 256)
    return torch.empty(nbytes, dtype=torch.uint8, device=device)
