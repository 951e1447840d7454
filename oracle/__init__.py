"""TEST INFRASTRUCTURE - the CPU oracle of the decode weight-matvec path.

Only `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import this package; nothing
under `btb_amd/` does. It restates the reference's CPU arithmetic (the Rust crate under native/src, which cannot be
built in this image: no rustc / cargo) in C (`btb_oracle.c`, loaded here through ctypes) and numpy (`codecs.py`,
`moe.py`), each function citing the reference lines it follows.

`lib()` loads `oracle/libbtb_oracle.so`, building it with `make -C oracle` when it is missing.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbtb_oracle.so")

OK, ERR_NULL, ERR_OVERFLOW, ERR_DOMAIN, ERR_PANIC = 0, -1, -5, -6, -7
TIER_SCALAR, TIER_AVX2, TIER_AVX512 = 0, 1, 2

_lib: ctypes.CDLL | None = None

_sz, _i32, _vp = ctypes.c_size_t, ctypes.c_int32, ctypes.c_void_p

_SIGS = {
    "btb_isa": (ctypes.c_char_p, []),
    "btb_oracle_set_tier": (ctypes.c_int, [ctypes.c_int]),
    "btb_gemv_bf16_rows": (_i32, [_vp, _sz, _sz, _vp, _sz, _vp, _sz]),
    "btb_gemv_bf16_group": (_i32, [_sz, _vp, _vp, _vp, _vp, _vp, _vp, _sz]),
    "btb_gemv_p12_rows": (_i32, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _sz, _vp, _sz]),
    "btb_gemv_mxfp4_rows": (_i32, [_vp, _vp, _sz, _sz, _vp, _sz, _vp, _sz]),
    "btb_gemv_mxfp4_ggml_rows": (_i32, [_vp, _sz, _sz, _vp, _sz, _vp, _sz]),
    "btb_gemv_mxfp4_group": (_i32, [_sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz]),
    "btb_gemv_fp8_rows": (_i32, [_vp, _vp, _sz, _sz, _sz, _sz, _vp, _sz, _vp, _sz]),
    "btb_gemv_fp8_group": (_i32, [_sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz]),
    "btb_oracle_unpack_p12": (_i32, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _vp]),
    "btb_oracle_widen_mxfp4": (_i32, [_vp, _vp, _sz, _vp]),
    "btb_oracle_widen_fp8": (_i32, [_vp, _vp, _sz, _sz, _sz, _sz, _vp]),
    "btb_oracle_round_bf16": (ctypes.c_float, [ctypes.c_float]),
    "btb_oracle_f8_value": (ctypes.c_float, [ctypes.c_uint8]),
    "btb_oracle_fp4_value": (ctypes.c_float, [ctypes.c_uint8]),
    "btb_oracle_mx_scale": (ctypes.c_float, [ctypes.c_uint8]),
    "btb_oracle_fold16": (ctypes.c_float, [_vp]),
}


def build() -> str:
    r = subprocess.run(["make", "-C", HERE, "-B", "libbtb_oracle.so"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"oracle build failed:\n{r.stdout}\n{r.stderr}")
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _p(a: np.ndarray | None) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if a is None else a.ctypes.data)


def isa() -> str:
    return lib().btb_isa().decode()


def set_tier(t: int) -> int:
    """force the kernel tier (0 scalar, 1 AVX2, 2 AVX-512; -1 the machine's best); returns the tier in force"""
    return int(lib().btb_oracle_set_tier(int(t)))


def _c(a: np.ndarray, dtype) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def gemv_bf16(w: np.ndarray, x: np.ndarray, threads: int = 1) -> np.ndarray:
    """y [b, rows] f32 = x [b, cols] f32 times w [rows, cols] bf16 bit patterns (uint16), the host's order"""
    w = _c(w, np.uint16)
    x = _c(np.atleast_2d(x), np.float32)
    rows, cols = w.shape
    y = np.empty((x.shape[0], rows), dtype=np.float32)
    rc = lib().btb_gemv_bf16_rows(_p(w), rows, cols, _p(x), x.shape[0], _p(y), threads)
    if rc != OK:
        raise ValueError(f"btb_gemv_bf16_rows: {rc}")
    return y


def gemv_p12(lo, hi4, table, esc_idx, esc_val, rows: int, cols: int, x: np.ndarray, threads: int = 1) -> np.ndarray:
    lo, hi4, table = _c(lo, np.uint8), _c(hi4, np.uint8), _c(table, np.uint8)
    esc_idx = _c(esc_idx, np.int32)
    esc_val = _c(esc_val, np.uint8)
    x = _c(np.atleast_2d(x), np.float32)
    y = np.empty((x.shape[0], rows), dtype=np.float32)
    rc = lib().btb_gemv_p12_rows(_p(lo), _p(hi4), _p(table), _p(esc_idx) if esc_idx.size else None,
                                 _p(esc_val) if esc_val.size else None, esc_idx.size, rows, cols, _p(x), x.shape[0],
                                 _p(y), threads)
    if rc != OK:
        raise ValueError(f"btb_gemv_p12_rows: {rc}")
    return y


def gemv_mxfp4_ggml(raw: np.ndarray, rows: int, cols: int, x: np.ndarray, threads: int = 1):
    """the MXFP4 matvec over ggml's layout: 17-byte blocks, scale first (btb_gemv_mxfp4_ggml_rows, lib.rs:162-183)"""
    raw = _c(raw, np.uint8)
    x = _c(np.atleast_2d(x), np.float32)
    y = np.empty((x.shape[0], rows), dtype=np.float32)
    rc = lib().btb_gemv_mxfp4_ggml_rows(_p(raw), rows, cols, _p(x), x.shape[0], _p(y), threads)
    if rc != OK:
        raise ValueError(f"btb_gemv_mxfp4_ggml_rows: {rc}")
    return y


def gemv_mxfp4(blocks: np.ndarray, scales: np.ndarray, rows: int, cols: int, x: np.ndarray, threads: int = 1):
    blocks, scales = _c(blocks, np.uint8), _c(scales, np.uint8)
    x = _c(np.atleast_2d(x), np.float32)
    y = np.empty((x.shape[0], rows), dtype=np.float32)
    rc = lib().btb_gemv_mxfp4_rows(_p(blocks), _p(scales), rows, cols, _p(x), x.shape[0], _p(y), threads)
    if rc != OK:
        raise ValueError(f"btb_gemv_mxfp4_rows: {rc}")
    return y


def gemv_fp8(w: np.ndarray, scales: np.ndarray, x: np.ndarray, threads: int = 1) -> np.ndarray:
    w = _c(w, np.uint8)
    scales = _c(scales, np.float32)
    rows, cols = w.shape
    sr, sc = scales.shape
    x = _c(np.atleast_2d(x), np.float32)
    y = np.empty((x.shape[0], rows), dtype=np.float32)
    rc = lib().btb_gemv_fp8_rows(_p(w), _p(scales), rows, cols, sr, sc, _p(x), x.shape[0], _p(y), threads)
    if rc != OK:
        raise ValueError(f"btb_gemv_fp8_rows: {rc}")
    return y


def unpack_p12(lo, hi4, table, esc_idx, esc_val, n: int) -> np.ndarray:
    """the bf16 bit patterns (uint16 [n]) of a packed tensor"""
    lo, hi4, table = _c(lo, np.uint8), _c(hi4, np.uint8), _c(table, np.uint8)
    esc_idx, esc_val = _c(esc_idx, np.int32), _c(esc_val, np.uint8)
    out = np.empty(n, dtype=np.uint16)
    rc = lib().btb_oracle_unpack_p12(_p(lo), _p(hi4), _p(table), _p(esc_idx) if esc_idx.size else None,
                                     _p(esc_val) if esc_val.size else None, esc_idx.size, n, _p(out))
    if rc != OK:
        raise ValueError(f"btb_oracle_unpack_p12: {rc}")
    return out


def widen_mxfp4(blocks: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """f32 [nblocks * 32]: fp4 * 2^(scale - 127), the CPU matvec's weight"""
    blocks, scales = _c(blocks, np.uint8), _c(scales, np.uint8)
    n = scales.size
    out = np.empty(n * 32, dtype=np.float32)
    rc = lib().btb_oracle_widen_mxfp4(_p(blocks), _p(scales), n, _p(out))
    if rc != OK:
        raise ValueError(f"btb_oracle_widen_mxfp4: {rc}")
    return out


def widen_fp8(w: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """f32 [rows, cols] holding bf16(e4m3 * scale), the weight every tier multiplies"""
    w, scales = _c(w, np.uint8), _c(scales, np.float32)
    rows, cols = w.shape
    out = np.empty((rows, cols), dtype=np.float32)
    rc = lib().btb_oracle_widen_fp8(_p(w), _p(scales), rows, cols, scales.shape[0], scales.shape[1], _p(out))
    if rc != OK:
        raise ValueError(f"btb_oracle_widen_fp8: {rc}")
    return out
