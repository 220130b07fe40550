"""ctypes binding of libfluxhip.so (the C ABI declared in include/flux_hip.h).

PyTorch supplies device memory and the current HIP stream; every computation on the hot path is a
hand-written gfx950 kernel behind this binding. There is no fallback: if the library is missing,
or a tensor is not on a GPU, the call raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int32, c_int64, c_void_p

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libfluxhip.so")
_lib = None

FLUX_BF16, FLUX_F32 = 0, 1
ACT_NONE, ACT_GELU_TANH, ACT_SILU = 0, 1, 2
LINEAR_SHARED_GPU = 1
E_NULL, E_SHAPE, E_DTYPE, E_ALIGN, E_TOO_WIDE, E_UNSUPPORTED = -1, -2, -3, -4, -5, -6
MAX_ROW = 65536

_DTYPE_CODE = {torch.bfloat16: FLUX_BF16, torch.float32: FLUX_F32}


class Src4(Structure):
    _fields_ = [("ptr", c_void_p), ("sb", c_int64), ("sh", c_int64), ("sl", c_int64)]


class QkvPrepArgs(Structure):
    _fields_ = [
        ("q_txt", Src4), ("k_txt", Src4), ("v_txt", Src4),
        ("q_img", Src4), ("k_img", Src4), ("v_img", Src4),
        ("q_out", c_void_p), ("k_out", c_void_p), ("v_out", c_void_p),
        ("q_scale_txt", c_void_p), ("k_scale_txt", c_void_p),
        ("q_scale_img", c_void_p), ("k_scale_img", c_void_p),
        ("pe", c_void_p), ("pe_batch_stride", c_int64),
        ("B", c_int64), ("H", c_int64), ("Lt", c_int64), ("Li", c_int64),
        ("D", c_int32), ("dtype", c_int32), ("scale_dtype", c_int32), ("eps", c_float),
    ]


class LinearQKFusion(Structure):
    _fields_ = [
        ("q_out", c_void_p), ("k_out", c_void_p),
        ("q_scale", c_void_p), ("k_scale", c_void_p),
        ("pe", c_void_p), ("pe_batch_stride", c_int64),
        ("heads", c_int64), ("seq_len", c_int64), ("out_len", c_int64), ("pos0", c_int64),
        ("eps", c_float),
    ]


class LinearArgs(Structure):
    _fields_ = [
        ("A", c_void_p), ("W", c_void_p), ("bias", c_void_p),
        ("Y", c_void_p), ("Y2", c_void_p),
        ("resid", c_void_p), ("gate", c_void_p),
        ("M", c_int64), ("N", c_int64), ("K", c_int64),
        ("lda", c_int64), ("ldw", c_int64), ("ldy", c_int64), ("ldy2", c_int64),
        ("split_n", c_int64), ("y2_col0", c_int64),
        ("ldresid", c_int64), ("gate_batch_stride", c_int64), ("rows_per_batch", c_int64),
        ("act", c_int32), ("in_act", c_int32), ("act_begin", c_int64),
        ("qk", POINTER(LinearQKFusion)),
        ("flags", c_int64),
    ]


class AttnArgs(Structure):
    _fields_ = [
        ("q", Src4), ("k", Src4), ("v", Src4),
        ("o", c_void_p), ("o_sb", c_int64), ("o_sh", c_int64), ("o_sl", c_int64),
        ("lse", c_void_p),
        ("B", c_int64), ("H", c_int64), ("L", c_int64),
        ("D", c_int32), ("sm_scale", c_float),
    ]


# name -> (restype, argtypes); also the list the symbol-export test walks.
SIGNATURES = {
    "flux_abi_version": (c_int32, []),
    "flux_last_error": (c_char_p, []),
    "flux_rms_norm": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int32,
                                c_int64, c_int64, c_int64, c_int32, c_int32, c_float, c_void_p]),
    "flux_rms_norm_bwd": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32,
                                    c_int32, c_int32, c_void_p]),
    "flux_layer_norm_modulation": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32,
                                             c_int64, c_int32, c_float, c_void_p]),
    "flux_qkv_prep": (c_int32, [POINTER(QkvPrepArgs), c_void_p]),
    "flux_linear_bf16": (c_int32, [POINTER(LinearArgs), c_void_p]),
    "flux_attention_fwd_bf16": (c_int32, [POINTER(AttnArgs), c_void_p]),
    "flux_silu": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    "flux_gelu_tanh": (c_int32, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int32, c_void_p]),
    "flux_modulation_scale_shift": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                              c_int32, c_int32, c_void_p]),
    "flux_gate_residual": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                     c_int32, c_int32, c_void_p]),
}


def lib_path() -> str:
    return _LIB_PATH


def lib():
    """Load libfluxhip.so once. torch is imported first on purpose: both link libamdhip64.so.7 and
    the process must end up with a single HIP runtime (the one torch already mapped)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: the HIP kernels are not built. Run "
                "`python -c 'import __graft_entry__ as g; g.build()'` at the repository root "
                "(or `make -C triton-kernels_amd/csrc`). There is no fallback path."
            )
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.flux_abi_version() != 4:
            raise RuntimeError("libfluxhip.so: ABI version mismatch")
        _lib = handle
    return _lib


def last_error() -> str:
    msg = lib().flux_last_error()
    return msg.decode() if msg else ""


def check(rc: int, what: str) -> None:
    if rc == 0:
        return
    msg = last_error() or what
    if rc == E_TOO_WIDE:
        raise RuntimeError(msg)
    if rc == E_DTYPE:
        raise TypeError(msg)
    if rc in (E_SHAPE, E_NULL, E_ALIGN):
        raise ValueError(msg)
    if rc == E_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(f"{msg} (hipError {rc})")


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}: the HIP kernels take bfloat16 or float32") from None


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("triton_kernels (HIP build): tensors must live on a GPU; there is no CPU path")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


class on_device:
    """Make `dev` current for the duration of a launch (no-op when it already is)."""

    __slots__ = ("dev", "prev")

    def __init__(self, dev: torch.device):
        self.dev = dev
        self.prev = None

    def __enter__(self):
        idx = self.dev.index if self.dev.index is not None else torch.cuda.current_device()
        cur = torch.cuda.current_device()
        if idx != cur:
            self.prev = cur
            torch.cuda.set_device(idx)
        return self

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def src4(t: torch.Tensor | None) -> Src4:
    """[B,H,L,D] view -> pointer + (sb, sh, sl). The caller guarantees stride(-1) == 1."""
    if t is None:
        return Src4(None, 0, 0, 0)
    return Src4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


__all__ = [
    "lib", "lib_path", "check", "last_error", "dtype_code", "require_gpu", "stream_ptr", "on_device", "ptr", "src4",
    "Src4", "QkvPrepArgs", "LinearArgs", "AttnArgs", "SIGNATURES", "byref",
    "FLUX_BF16", "FLUX_F32", "ACT_NONE", "ACT_GELU_TANH", "ACT_SILU", "LINEAR_SHARED_GPU", "MAX_ROW",
]
