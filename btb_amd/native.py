"""ctypes bindings of libbtb_hip.so: the counterpart of the reference's `Native` / `_Cuda` pair
(btb/engine/native.py:559-608, 1243-1493) for the decode weight-matvec path on one MI355X.

`Native.card_kernels()` binds the library once per process and returns a `HipCard`, whose methods take torch
tensors on the GPU, check dtype / shape / contiguity before anything is launched (a refusal raises ValueError and
launches nothing, as the reference's convenience wrappers do) and queue the kernels on torch's current stream, so
they record into a graph capture like any other node. A missing library or GPU is an error, never a fallback:
there is no CPU or torch path behind these calls.
"""

from __future__ import annotations

import ctypes
import os
from collections.abc import Sequence
from typing import Any

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbtb_hip.so")

OK, ERR_NULL, ERR_OVERFLOW, ERR_DOMAIN, ERR_PANIC = 0, -1, -5, -6, -7
_CODES = {ERR_NULL: "ERR_NULL", ERR_OVERFLOW: "ERR_OVERFLOW", ERR_DOMAIN: "ERR_DOMAIN", ERR_PANIC: "ERR_PANIC"}

_vp, _sz, _i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32

# every exported symbol: name -> (restype, argtypes); the header include/btb_hip.h declares the same list
SIGNATURES: dict[str, tuple[Any, list[Any]]] = {
    "btb_hip_init": (_i32, [_i32]),
    "btb_hip_arch": (ctypes.c_char_p, []),
    "btb_hip_sms": (_i32, []),
    "btb_hip_last_error": (ctypes.c_char_p, []),
    "btb_hip_set_tuning": (_i32, [ctypes.c_char_p, _i32]),
    "btb_hip_gemv_bf16": (_i32, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_gemv_silu_bf16": (_i32, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
}


class HipError(RuntimeError):
    """a call the library refused or the HIP runtime failed: `[hip] <what> failed: <code> <message>`"""


def load_library(path: str | os.PathLike[str] = LIB_PATH) -> ctypes.CDLL:
    """the shared library with every symbol's signature set; RuntimeError where it has not been built"""
    if not os.path.exists(path):
        raise RuntimeError(f"[hip] the kernels are missing: {path} (run `python -m btb_amd.build`)")
    lib = ctypes.CDLL(os.fspath(path))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class HipCard:
    """The card's operators over torch tensors. `GEMV_ROWS` are the pass widths the reference's card graphs are
    captured at (btb/engine/native.py:1918); any M up to 1024 is taken here."""

    GEMV_ROWS = (1, 2, 4, 8, 16, 32)

    def __init__(self, path: str | os.PathLike[str] = LIB_PATH) -> None:
        if not torch.cuda.is_available():
            raise RuntimeError("[hip] no GPU is visible to torch: the HIP kernels cannot run")
        self.lib = load_library(path)
        torch.cuda.init()
        torch.empty(1, device="cuda")
        self.device = torch.cuda.current_device()
        self._call("btb_hip_init", self.device)
        self.sms = int(self.lib.btb_hip_sms())
        self.arch = self.lib.btb_hip_arch().decode()

    # -- plumbing ---------------------------------------------------------------------------------------------

    def _call(self, name: str, *args: Any) -> None:
        rc = getattr(self.lib, name)(*args)
        if rc != OK:
            msg = self.lib.btb_hip_last_error().decode(errors="replace")
            raise HipError(f"[hip] {name} failed: {rc} {_CODES.get(rc, '?')} {msg}")

    @staticmethod
    def ptr(t: torch.Tensor) -> ctypes.c_void_p:
        return ctypes.c_void_p(t.data_ptr())

    def set_tuning(self, key: str, value: int) -> None:
        self._call("btb_hip_set_tuning", key.encode(), int(value))

    @staticmethod
    def _need(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
        if not isinstance(t, torch.Tensor) or t.dtype != dtype or not t.is_cuda or not t.is_contiguous():
            raise ValueError(f"[hip] {what} must be a contiguous {dtype} tensor on the GPU, got "
                             f"{getattr(t, 'dtype', type(t))} {getattr(t, 'device', '')}")

    # -- bf16 matvec ------------------------------------------------------------------------------------------

    def gemv(self, w: torch.Tensor, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """y [M, R] = x [M, C] @ w [R, C]^T, bf16 in and out, f32 accumulate (`btb_gemv_bf16_m{M}`)"""
        self._need(w, torch.bfloat16, "w")
        self._need(x, torch.bfloat16, "x")
        R, C = (int(s) for s in w.shape)
        x2 = x.reshape(-1, C)
        M = int(x2.shape[0])
        if y is None:
            y = torch.empty(M, R, dtype=torch.bfloat16, device=w.device)
        else:
            self._need(y, torch.bfloat16, "y")
            if y.numel() != M * R:
                raise ValueError(f"[hip] gemv: y holds {y.numel()} elements, the product has {M * R}")
        self._call("btb_hip_gemv_bf16", self.ptr(w), self.ptr(x2), self.ptr(y), R, C, M, _stream())
        return y

    def gemv_silu(self, w: torch.Tensor, gu: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """the down projection over gu [M, 2C] (gate then up) with bf16(bf16(silu(g)) * u) folded into the x load"""
        self._need(w, torch.bfloat16, "w")
        self._need(gu, torch.bfloat16, "gu")
        R, C = (int(s) for s in w.shape)
        g2 = gu.reshape(-1, 2 * C)
        M = int(g2.shape[0])
        if y is None:
            y = torch.empty(M, R, dtype=torch.bfloat16, device=w.device)
        else:
            self._need(y, torch.bfloat16, "y")
            if y.numel() != M * R:
                raise ValueError(f"[hip] gemv_silu: y holds {y.numel()} elements, the product has {M * R}")
        self._call("btb_hip_gemv_silu_bf16", self.ptr(w), self.ptr(g2), self.ptr(y), R, C, M, _stream())
        return y


class Native:
    """Lazy binding, once per process (the reference's `Native.card_kernels`, btb/engine/native.py:1209-1226):
    `card_kernels()` returns the bound `HipCard` or raises with the reason; it never falls back."""

    _card: HipCard | None = None
    reason: str | None = None

    @classmethod
    def card_kernels(cls) -> HipCard:
        if cls._card is None:
            try:
                cls._card = HipCard()
                cls.reason = None
            except Exception as e:  # the reason is kept for whoever asks again
                cls.reason = str(e)
                raise
        return cls._card
