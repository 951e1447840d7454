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
from typing import Any, Sequence

import torch

from .card_launch import CardLaunch

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
    "btb_hip_stream_probe": (_i32, [_vp, _sz, _vp, _vp]),
    "btb_hip_gemv_bf16": (_i32, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_gemv_silu_bf16": (_i32, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_gemv_glu_silu_bf16": (_i32, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_gemv_bf16_norm": (_i32, [_vp, _vp, _vp, _vp, ctypes.c_float, _i32, _vp, _vp, _sz, _sz, _sz, _i32, _vp]),
    "btb_hip_gemv_bf16_embed_norm": (_i32, [_vp, _vp, _vp, _sz, _vp, ctypes.c_float, _i32, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_gemv_p12_embed_norm": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _vp, ctypes.c_float,
                                           _i32, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_gemv_p12_norm": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, ctypes.c_float, _i32, _vp,
                                     _vp, _sz, _sz, _sz, _i32, _vp]),
    "btb_hip_gemv_p12": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_p12_pairs": (_i32, [_vp, _vp, _vp]),
    "btb_hip_p12_row_esc": (_i32, [_vp, _vp, _vp, _sz, _vp, _sz, _sz, _vp, _vp]),
    "btb_hip_p12_row_ptr": (_i32, [_vp, _sz, _sz, _sz, _vp, _vp]),
    "btb_hip_p12_check": (_i32, [_vp, _sz, _sz, _vp, _vp]),
    "btb_hip_p12_widen": (_i32, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _vp, _vp]),
    "btb_hip_gemv_fp8": (_i32, [_vp, _vp, _sz, _sz, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_fp8_widen": (_i32, [_vp, _vp, _sz, _sz, _sz, _sz, _vp, _i32, _vp]),
    "btb_hip_round_bf16": (_i32, [_vp, _vp, _sz, _vp]),
    "btb_hip_gemv_mxfp4": (_i32, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_mx4_widen": (_i32, [_vp, _vp, _vp, _sz, ctypes.c_int64, _vp, _i32, _vp]),
    "btb_hip_gemv_bf16_rows": (_i32, [_vp, _sz, _sz, _vp, _sz, _vp, _vp]),
    "btb_hip_gemv_bf16_group": (_i32, [_sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_gemv_p12_rows": (_i32, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _sz, _vp, _vp]),
    "btb_hip_gemv_mxfp4_rows": (_i32, [_vp, _vp, _sz, _sz, _vp, _sz, _vp, _vp]),
    "btb_hip_gemv_mxfp4_ggml_rows": (_i32, [_vp, _sz, _sz, _vp, _sz, _vp, _vp]),
    "btb_hip_gemv_mxfp4_group": (_i32, [_sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_gemv_fp8_rows": (_i32, [_vp, _vp, _sz, _sz, _sz, _sz, _vp, _sz, _vp, _vp]),
    "btb_hip_gemv_fp8_group": (_i32, [_sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_moe_route": (_i32, [_vp, _i32, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _vp]),
    "btb_hip_moe_group_picks": (_i32, [_vp, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_moe_router_bf16": (_i32, [_vp, _vp, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_moe_experts_bf16": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _vp]),
    "btb_hip_moe_experts_mxfp4": (_i32, [_vp] * 11 + [_sz] * 5 + [_i32, ctypes.c_float, ctypes.c_float, _vp]),
    "btb_hip_embed": (_i32, [_vp, _vp, _vp, _sz, _sz, _sz, _vp]),
    "btb_hip_add_rmsnorm": (_i32, [_vp, _vp, _vp, ctypes.c_float, _vp, _sz, _sz, _i32, _vp]),
    "btb_hip_norm_rope_kv": (_i32, [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz,
                                    _sz, ctypes.c_int64, ctypes.c_int64, _i32, _vp]),
    "btb_hip_norm_rope_kv_seqs": (_i32, [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz,
                                         ctypes.c_int64, ctypes.c_int64, _i32, _vp]),
    "btb_hip_norm_rope_kv_tbl": (_i32, [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz,
                                        _sz, ctypes.c_int64, ctypes.c_int64, _i32, _vp, _vp]),
    "btb_hip_attn_decode_win": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, ctypes.c_int64, ctypes.c_int64,
                                       ctypes.c_float, _sz, _sz, ctypes.c_int64, _vp, _vp, _vp]),
    "btb_hip_publish_only": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_attn_scratch_floats": (_sz, [_sz, _sz, _sz, _sz, _sz]),
    "btb_hip_attn_decode": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, ctypes.c_int64, ctypes.c_int64,
                                   ctypes.c_float, _sz, _sz, _vp, _vp]),
    "btb_hip_attn_decode_parts": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, ctypes.c_int64, ctypes.c_int64,
                                         ctypes.c_float, _sz, _sz, ctypes.c_int64, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_attn_decode_seqs": (_i32, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, ctypes.c_int64, ctypes.c_int64,
                                        ctypes.c_float, _sz, _sz, ctypes.c_int64, _vp, _vp, _vp, _vp]),
    "btb_hip_attn_decode_noalloc": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, ctypes.c_int64,
                                           ctypes.c_int64, ctypes.c_float, _sz, _sz, _vp]),
    "btb_hip_attn_decode_qkv": (_i32, [_vp, _vp, _vp, ctypes.c_float, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz,
                                       ctypes.c_int64, ctypes.c_int64, ctypes.c_float, _sz, _sz, _vp, _vp]),
    "btb_hip_attn_rows_fused": (_i32, [_sz, _sz, _sz, _sz, _sz, _sz]),
    "btb_hip_attn_decode_qkv_rows": (_i32, [_vp, _vp, _vp, ctypes.c_float, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                            _sz, _sz, _sz, _sz, ctypes.c_int64, ctypes.c_int64, ctypes.c_float, _sz,
                                            _sz, _vp, _vp]),
    "btb_hip_silu_mul": (_i32, [_vp, _vp, _sz, _sz, _vp]),
    "btb_hip_argmax": (_i32, [_vp, _vp, _sz, _sz, _vp]),
    "btb_hip_publish": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "btb_hip_argmax_publish": (_i32, [_vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
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


def _p(t: torch.Tensor) -> ctypes.c_void_p:
    """a tensor's device address as a pointer argument of the C ABI"""
    return ctypes.c_void_p(t.data_ptr())



def _launch_table() -> dict[str, tuple[int, Any]]:
    """reference kernel name -> (its parameter count, parameters -> (entry point, its arguments less the stream))"""
    t: dict[str, tuple[int, Any]] = {}
    for M in (1, 2, 4, 8, 16, 32):
        t[f"btb_gemv_bf16_m{M}"] = (5, lambda v, g, card, M=M: ("btb_hip_gemv_bf16", (v[0], v[1], v[2], v[3], v[4], M)))
        t[f"btb_gemv_silu_bf16_m{M}"] = (5, lambda v, g, card, M=M: ("btb_hip_gemv_silu_bf16", (v[0], v[1], v[2], v[3], v[4], M)))
        t[f"btb_gemv_lane16_f32_m{M}"] = (5, lambda v, g, card, M=M: ("btb_hip_gemv_bf16_rows", (v[0], v[3], v[4], v[1], M, v[2])))
        t[f"btb_gemv_lane16_mx4_f32_m{M}"] = (
            6, lambda v, g, card, M=M: ("btb_hip_gemv_mxfp4_rows", (v[0], v[1], v[4], v[5], v[2], M, v[3])))
    for n in ("btb_gemv_mma_bf16", "btb_gemv_mma8_bf16"):
        t[n] = (6, lambda v, g, card: ("btb_hip_gemv_bf16", (v[0], v[1], v[2], v[3], v[4], v[5])))
    t["btb_gemv_mma_glu_silu"] = (6, lambda v, g, card: ("btb_hip_gemv_glu_silu_bf16", (v[0], v[1], v[2], v[3], v[4], v[5])))
    t["btb_silu_mul"] = (4, lambda v, g, card: ("btb_hip_silu_mul", (v[0], v[1], v[2], v[3])))
    # btb_add_rmsnorm(h, y, w, eps, x, H, centered), a block a row
    t["btb_add_rmsnorm"] = (7, lambda v, g, card: ("btb_hip_add_rmsnorm", (v[0], v[1], v[2], v[3], v[4], g[0], v[5], v[6])))
    for D in (64, 128, 256):
        # (qkv, wq, wk, eps, cos, sin, n0, depth, K, V, q, T, Hq, Hk, hs, rs, centered)
        t[f"btb_norm_rope_kv_d{D}"] = (17, lambda v, g, card, D=D: ("btb_hip_norm_rope_kv", (
            v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9], v[10], v[11], v[12], v[13], D, v[14], v[15], v[16])))
    # btb_moe_route(logits bf16, ls, E, k, idx, w, hidx, hw, cnt, seq, hseq), a block a row; the host copies are the
    # reference's way of fetching experts from the host tier and are not made here
    t["btb_moe_route"] = (11, lambda v, g, card: ("btb_hip_moe_route", (v[0], 0, v[1], v[2], v[3], g[0], v[4], v[5], None)))
    for D in (64, 128, 256):  # the same with the cache's row map as the last parameter
        t[f"btb_norm_rope_kv_tbl_d{D}"] = (18, lambda v, g, card, D=D: ("btb_hip_norm_rope_kv_tbl", (
            v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9], v[10], v[11], v[12], v[13], D, v[14], v[15], v[16],
            v[17])))
    # btb_attn_flash_d128(q, K, V, out, n0p, par, T, Hq, Hk, hs, rs, scale, part_m, part_l, part_acc, cnt, win, tbl) on
    # a grid (row tiles, key groups, kv heads): grid[1] key groups of 512 keys each reach the cache's capacity. The
    # groups' states go into the caller's own part_m / part_l / part_acc (S T Hq and S T Hq D floats, the sizes the
    # reference's card graph gives them), so the launch allocates nothing and a captured graph keeps its arrays; the
    # arrival counter is left alone (the groups are folded by a second launch, not by the last arriver)
    t["btb_attn_flash_d128"] = (18, lambda v, g, card: ("btb_hip_attn_decode_parts", (
        v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], 128, v[9], v[10], v[11], 512, max(int(g[1]), 1), v[16],
        v[17], v[12], v[13], v[14])))
    # the same pair for a pass whose rows are sequences of their own (`rw`, the rows layout):
    # btb_norm_rope_kv_rows_d{D}(qkv, wq, wk, eps, cos, sin, rw, K, V, q, T, Hq, Hk, hs, rs, centered) and
    # btb_attn_flash_rows_d128(q, K, V, out, rw, T, Hq, Hk, hs, rs, scale, part_m, part_l, part_acc, cnt, win)
    for D in (64, 128, 256):
        t[f"btb_norm_rope_kv_rows_d{D}"] = (16, lambda v, g, card, D=D: ("btb_hip_norm_rope_kv_seqs", (
            v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9], v[10], v[11], v[12], D, v[13], v[14], v[15])))
    t["btb_attn_flash_rows_d128"] = (16, lambda v, g, card: ("btb_hip_attn_decode_seqs", (
        v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], 128, v[8], v[9], v[10], 512, max(int(g[1]), 1), v[15], v[11],
        v[12], v[13])))
    # btb_publish(n0, ids, out_tok, out_n0, out_ts)
    t["btb_publish"] = (5, lambda v, g, card: ("btb_hip_publish_only", (v[0], v[1], v[2], v[3], v[4])))
    # btb_mx4_widen(blocks, scales, seats, groups, out), grid.y seats
    t["btb_mx4_widen"] = (5, lambda v, g, card: ("btb_hip_mx4_widen", (v[0], v[1], v[2], g[1], v[3], v[4], 0)))
    return t


_LAUNCH = _launch_table()

class HipCard(CardLaunch):
    """The card's operators over torch tensors: the reference's `_Cuda` (`CardLaunch` + `launch`,
    btb/engine/native.py:1243) over this library. `launch` takes the reference's kernel names; `CardLaunch` adds the
    typed launchers (`k.btb_add_rmsnorm(grid, block, ...)`, `k.btb_gemv_bf16(M, grid, block, ...)`) and
    `ptr(role, tensor)`, which is all the reference's `_card_body` asks of its `k`. `GEMV_ROWS` are the pass widths the
    reference's card graphs are captured at (btb/engine/native.py:1918); any M up to 1024 is taken here."""

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

    def stream_probe(self, a: torch.Tensor) -> None:
        """the streaming matvec's loads over a bf16 [R, 2560] matrix, without the matvec (a measurement aid)"""
        self._need(a, torch.bfloat16, "a")
        if a.dim() != 2 or a.shape[1] != 2560 or a.shape[0] % 2:
            raise ValueError("[hip] stream_probe reads a bf16 [R, 2560] matrix, R even")
        self._call("btb_hip_stream_probe", _p(a), int(a.shape[0]), None, _stream())

    def set_tuning(self, key: str, value: int) -> None:
        self._call("btb_hip_set_tuning", key.encode(), int(value))

    @staticmethod
    def _need(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
        if not isinstance(t, torch.Tensor) or t.dtype != dtype or not t.is_cuda or not t.is_contiguous():
            raise ValueError(f"[hip] {what} must be a contiguous {dtype} tensor on the GPU, got "
                             f"{getattr(t, 'dtype', type(t))} {getattr(t, 'device', '')}")

    # -- the reference's launcher surface: kernels by name -------------------------------------------------------

    def launch(self, name: str, grid: tuple[int, int, int], block: tuple[int, int, int], args: Sequence[Any],
               stream: torch.cuda.Stream | None = None, shared: int = 0) -> None:
        """The reference's `Launcher.launch` (btb/engine/card_launch.py:428-440) for the kernels of this path: `name`
        is the reference kernel's name, `args` its parameters in its own order (native/cuda/btb_kernels.cu,
        btb_gemv_mma.cuh), one ctypes value (or int / float) each. `block` and `shared` are the CUDA kernel's and
        mean nothing here - the library picks its own wave64 geometry - and of `grid` only what carries a size is
        read (rows in grid[0] for btb_add_rmsnorm and btb_moe_route, seats in grid[1] for btb_mx4_widen). The
        parameter count is checked before anything is launched; an unknown name is a KeyError naming it."""
        entry = _LAUNCH.get(name)
        if entry is None:
            raise KeyError(f"[hip] {name} is not a kernel of this path ({len(_LAUNCH)} are: see HipCard.fn)")
        count, call = entry
        if len(args) != count:
            raise ValueError(f"[hip] {name} takes {count} parameters, got {len(args)}")
        vals = [a.value if isinstance(a, ctypes._SimpleCData) else a for a in args]
        st = ctypes.c_void_p((stream or torch.cuda.current_stream()).cuda_stream)
        sym, cargs = call(vals, tuple(int(g) for g in grid), self)
        self._call(sym, *cargs, st)

    @property
    def fn(self) -> dict[str, str]:
        """kernel name -> the library entry point that serves it (the reference keeps its loaded kernels here)"""
        return {n: call([0] * count, (1, 1, 1), None)[0] for n, (count, call) in _LAUNCH.items()}

    def close(self) -> None:
        """the reference's `_Cuda.close` unloads its module (btb/engine/native.py:1484-1492); the card here owns no
        device memory and the library stays loaded for the process, so there is nothing to drop. Idempotent."""

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
        self._call("btb_hip_gemv_bf16", _p(w), _p(x2), _p(y), R, C, M, _stream())
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
        self._call("btb_hip_gemv_silu_bf16", _p(w), _p(g2), _p(y), R, C, M, _stream())
        return y


    def gemv_glu_silu(self, w: torch.Tensor, x: torch.Tensor, m: torch.Tensor | None = None) -> torch.Tensor:
        """m [M, I] = bf16(bf16(silu(g)) * u) with [g, u] = x @ w^T, w [2I, C]: gate, up and the activation in one
        kernel (`btb_gemv_mma_glu_silu`)"""
        self._need(w, torch.bfloat16, "w")
        self._need(x, torch.bfloat16, "x")
        R, C = (int(s) for s in w.shape)
        x2 = x.reshape(-1, C)
        M = int(x2.shape[0])
        m = self._out(m, M, R // 2, x.device, "gemv_glu_silu")
        self._call("btb_hip_gemv_glu_silu_bf16", _p(w), _p(x2), _p(m), R // 2, C, M, _stream())
        return m

    def gemv_norm(self, w: Any, h_in: torch.Tensor, y: torch.Tensor | None, norm_w: torch.Tensor, eps: float,
                  h_out: torch.Tensor | None, out: torch.Tensor, glu: bool = False, centered: bool = False) -> torch.Tensor:
        """out = W . rmsnorm(h_in + y) with the add and the norm folded into the matvec's x load; the new residual
        goes to `h_out` (a different tensor than `h_in`). `w` is a bf16 matrix or a `P12Weight`; `glu` folds the
        SwiGLU activation into the epilogue (out is then [M, R / 2])."""
        for t, what in ((h_in, "h_in"), (norm_w, "norm_w"), (out, "out")):
            self._need(t, torch.bfloat16, what)
        for t, what in ((y, "y"), (h_out, "h_out")):
            if t is not None:
                self._need(t, torch.bfloat16, what)
        R, C = (int(s) for s in w.shape)
        M = int(h_in.numel()) // C
        if h_in.numel() != M * C or norm_w.numel() != C or out.numel() != M * (R // 2 if glu else R) \
                or (y is not None and y.numel() != M * C) or (h_out is not None and h_out.numel() != M * C):
            raise ValueError("[hip] gemv_norm: the rows, the norm weight and the output do not fit the matrix")
        if h_out is not None and h_out.data_ptr() == h_in.data_ptr():
            raise ValueError("[hip] gemv_norm: the new residual cannot be written over the one being read")
        p = lambda t: None if t is None else _p(t)
        if isinstance(w, torch.Tensor):
            self._need(w, torch.bfloat16, "w")
            self._call("btb_hip_gemv_bf16_norm", _p(w), _p(h_in), p(y), _p(norm_w), float(eps),
                       int(centered), p(h_out), _p(out), R, C, M, int(glu), _stream())
        else:
            ne = int(w.esc_idx.numel())
            self._call("btb_hip_gemv_p12_norm", _p(w.lo), _p(w.hi4), _p(w.table), self._pairs(w),
                       _p(w.esc_idx) if ne else None, _p(w.esc_val) if ne else None, ne, _p(w.row_ptr),
                       self._row_esc(w), _p(h_in), p(y), _p(norm_w), float(eps), int(centered), p(h_out), _p(out), R, C,
                       M, int(glu), _stream())
        return out

    def gemv_embed_norm(self, w: Any, table: torch.Tensor, ids: torch.Tensor, norm_w: torch.Tensor, eps: float,
                        h_out: torch.Tensor | None, out: torch.Tensor, centered: bool = False) -> torch.Tensor:
        """`embed` + `gemv_norm` in one launch: the residual rows are table[ids], written to `h_out`; out = W . rmsnorm"""
        for t, what in ((table, "table"), (norm_w, "norm_w"), (out, "out")):
            self._need(t, torch.bfloat16, what)
        self._need(ids, torch.int32, "ids")
        if h_out is not None:
            self._need(h_out, torch.bfloat16, "h_out")
        R, C = (int(s) for s in w.shape)
        M, vocab = int(ids.numel()), int(table.shape[0])
        if table.dim() != 2 or table.shape[1] != C or norm_w.numel() != C or out.numel() != M * R \
                or (h_out is not None and h_out.numel() != M * C):
            raise ValueError("[hip] gemv_embed_norm: the table, the norm weight and the outputs do not fit the matrix")
        p = lambda t: None if t is None else _p(t)
        if isinstance(w, torch.Tensor):
            self._need(w, torch.bfloat16, "w")
            self._call("btb_hip_gemv_bf16_embed_norm", _p(w), _p(table), _p(ids), vocab,
                       _p(norm_w), float(eps), int(centered), p(h_out), _p(out), R, C, M, _stream())
        else:
            ne = int(w.esc_idx.numel())
            self._call("btb_hip_gemv_p12_embed_norm", _p(w.lo), _p(w.hi4), _p(w.table), self._pairs(w),
                       _p(w.esc_idx) if ne else None, _p(w.esc_val) if ne else None, ne, _p(w.row_ptr),
                       self._row_esc(w), _p(table), _p(ids), vocab, _p(norm_w), float(eps), int(centered), p(h_out),
                       _p(out), R, C, M, _stream())
        return out

    # -- the stored forms ---------------------------------------------------------------------------------------

    def _out(self, y: torch.Tensor | None, M: int, R: int, dev: torch.device, what: str) -> torch.Tensor:
        if y is None:
            return torch.empty(M, R, dtype=torch.bfloat16, device=dev)
        self._need(y, torch.bfloat16, "y")
        if y.numel() != M * R:
            raise ValueError(f"[hip] {what}: y holds {y.numel()} elements, the product has {M * R}")
        return y

    def p12_check(self, esc_idx: torch.Tensor, n: int) -> None:
        """ValueError unless the escape list is strictly ascending inside [0, n): checked on the GPU, once, at upload"""
        self._need(esc_idx, torch.int32, "esc_idx")
        if esc_idx.numel() == 0:
            return
        flag = torch.zeros(1, dtype=torch.int32, device=esc_idx.device)
        rc = self.lib.btb_hip_p12_check(_p(esc_idx), esc_idx.numel(), int(n), _p(flag), _stream())
        if rc == ERR_DOMAIN:
            raise ValueError(f"[hip] pack12: {self.lib.btb_hip_last_error().decode(errors='replace')}")
        if rc != OK:
            raise HipError(f"[hip] btb_hip_p12_check failed: {rc} {_CODES.get(rc, '?')}")

    @staticmethod
    def _pairs(w: Any) -> ctypes.c_void_p | None:
        t = getattr(w, "pairs", None)
        return None if t is None else _p(t)

    @staticmethod
    def _row_esc(w: Any) -> ctypes.c_void_p | None:
        t = getattr(w, "row_esc", None)
        return None if t is None else _p(t)

    def p12_row_esc(self, lo: torch.Tensor, esc_idx: torch.Tensor, esc_val: torch.Tensor, row_ptr: torch.Tensor,
                    rows: int, cols: int) -> torch.Tensor | None:
        """int32 [rows, S] (read as u32; S = 8 up to 4096 columns, else 16): every row's first S escapes, a word each
        (low byte, true high byte, column; bit 31: the row has more), which the matvecs ask for ahead of the row's
        weights (built once at upload). None for rows wider than 32767, whose columns a word cannot hold: the matvecs
        then walk the list."""
        if cols > 0x7FFF:
            return None
        self._need(lo, torch.uint8, "lo")
        self._need(esc_idx, torch.int32, "esc_idx")
        self._need(esc_val, torch.uint8, "esc_val")
        self._need(row_ptr, torch.int32, "row_ptr")
        if row_ptr.numel() != rows + 1 or lo.numel() != rows * cols or esc_val.numel() != esc_idx.numel():
            raise ValueError("[hip] p12_row_esc: lo holds rows * cols bytes, row_ptr rows + 1 entries, the list's two "
                             "arrays one entry an escape")
        out = torch.empty(rows, 8 if cols <= 4096 else 16, dtype=torch.int32, device=lo.device)
        ne = int(esc_idx.numel())
        self._call("btb_hip_p12_row_esc", _p(lo), _p(esc_idx) if ne else None, _p(esc_val) if ne else None, ne,
                   _p(row_ptr), rows, cols, _p(out), _stream())
        return out

    def p12_pairs(self, table: torch.Tensor) -> torch.Tensor:
        """int16 [256] (read as u16): the high bytes of the two weights each byte of codes stands for, the escape code
        as 0 (built once at upload; the matvecs keep a copy in LDS)"""
        self._need(table, torch.uint8, "table")
        if table.numel() != 16:
            raise ValueError("[hip] p12_pairs: the table holds 16 bytes")
        out = torch.empty(256, dtype=torch.int16, device=table.device)
        self._call("btb_hip_p12_pairs", _p(table), _p(out), _stream())
        return out

    def p12_row_ptr(self, esc_idx: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
        """int32 [rows + 1]: the first escape at or past each row's first weight (built once at upload)"""
        self._need(esc_idx, torch.int32, "esc_idx")
        out = torch.empty(rows + 1, dtype=torch.int32, device=esc_idx.device)
        self._call("btb_hip_p12_row_ptr", _p(esc_idx) if esc_idx.numel() else None, esc_idx.numel(), rows, cols,
                   _p(out), _stream())
        return out

    def gemv_p12(self, w: Any, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """y [M, R] = x [M, C] over a `P12Weight`, the 12-bit form widened in registers"""
        R, C = w.shape
        self._need(x, torch.bfloat16, "x")
        x2 = x.reshape(-1, C)
        M = int(x2.shape[0])
        y = self._out(y, M, R, x.device, "gemv_p12")
        ne = int(w.esc_idx.numel())
        self._call("btb_hip_gemv_p12", _p(w.lo), _p(w.hi4), _p(w.table), self._pairs(w),
                   _p(w.esc_idx) if ne else None, _p(w.esc_val) if ne else None, ne, _p(w.row_ptr),
                   self._row_esc(w), _p(x2), _p(y), R, C, M, _stream())
        return y

    def p12_widen(self, lo, hi4, table, esc_idx, esc_val, n: int, shape: Sequence[int],
                  out: torch.Tensor | None = None) -> torch.Tensor:
        """a packed tensor back to bf16 on the GPU (`unpack_bf16`), through the matvec's own in-register widen"""
        for t, what in ((lo, "lo"), (hi4, "hi4"), (table, "table")):
            self._need(t, torch.uint8, what)
        if out is None:
            out = torch.empty(tuple(shape), dtype=torch.bfloat16, device=lo.device)
        else:
            self._need(out, torch.bfloat16, "out")
            if out.numel() != int(n):
                raise ValueError(f"[hip] p12_widen: out holds {out.numel()} values, the tensor has {int(n)}")
        ne = 0 if esc_idx is None else int(esc_idx.numel())
        if ne:
            self._need(esc_idx, torch.int32, "esc_idx")
            self._need(esc_val, torch.uint8, "esc_val")
        self._call("btb_hip_p12_widen", _p(lo), _p(hi4), _p(table), _p(esc_idx) if ne else None,
                   _p(esc_val) if ne else None, ne, n, _p(out), _stream())
        return out

    def gemv_fp8(self, w: Any, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """y [M, R] = x [M, C] over an `F8Weight`: each weight bf16(e4m3 * scale), made in registers"""
        R, C = w.shape
        sr, sc = w.grid
        self._need(w.w, torch.uint8, "w")
        self._need(w.scales, torch.float32, "scales")
        self._need(x, torch.bfloat16, "x")
        x2 = x.reshape(-1, C)
        M = int(x2.shape[0])
        y = self._out(y, M, R, x.device, "gemv_fp8")
        self._call("btb_hip_gemv_fp8", _p(w.w), _p(w.scales), sr, sc, _p(x2), _p(y), R, C, M,
                   _stream())
        return y

    def round_bf16(self, x: torch.Tensor) -> torch.Tensor:
        """float32 values as stored bf16, by the rounding every bf16 output of the library goes through (nearest even,
        a NaN the quiet NaN of its sign and upper payload: the crate's `round_bf16` with torch's NaN rule)"""
        self._need(x, torch.float32, "x")
        out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
        self._call("btb_hip_round_bf16", _p(x), _p(out), int(x.numel()), _stream())
        return out

    def fp8_widen(self, w: Any, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        """an `F8Weight` as the held matrix (`fp8.held`), bf16 or the same values as f32"""
        R, C = w.shape
        sr, sc = w.grid
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("[hip] fp8_widen writes bf16 or float32")
        out = torch.empty(R, C, dtype=dtype, device=w.w.device)
        self._call("btb_hip_fp8_widen", _p(w.w), _p(w.scales), R, C, sr, sc, _p(out),
                   int(dtype == torch.float32), _stream())
        return out

    def gemv_mx4(self, w: Any, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """y [M, R] = x [M, C] over an `MxWeight` (checkpoint layout), fp4 * 2^(scale - 127) made in registers"""
        R, C = w.shape
        self._need(w.blocks, torch.uint8, "blocks")
        self._need(w.scales, torch.uint8, "scales")
        self._need(x, torch.bfloat16, "x")
        x2 = x.reshape(-1, C)
        M = int(x2.shape[0])
        y = self._out(y, M, R, x.device, "gemv_mx4")
        self._call("btb_hip_gemv_mxfp4", _p(w.blocks), _p(w.scales), _p(x2), _p(y), R, C, M,
                   _stream())
        return y

    def mx4_widen(self, blocks: torch.Tensor, scales: torch.Tensor, seats: torch.Tensor | None = None,
                  out: torch.Tensor | None = None, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        """MXFP4 experts at `seats` of the stacks `blocks` [S, .., 16] and `scales` [S, ..] widened to
        [len(seats), groups * 32] in one pass (the reference's `_Cuda.mx4_widen`, btb/engine/native.py:1494-1530);
        `dtype` float32 keeps the unrounded f32 product the CPU matvec multiplies"""
        groups = int(scales[0].numel())
        if (blocks.dtype != torch.uint8 or scales.dtype != torch.uint8
                or not (blocks.is_contiguous() and scales.is_contiguous())
                or int(blocks[0].numel()) != 16 * groups or blocks.device != scales.device or not blocks.is_cuda):
            raise ValueError(f"[hip] mx4_widen: blocks {tuple(blocks.shape)} {blocks.dtype} and scales "
                             f"{tuple(scales.shape)} {scales.dtype} are not a contiguous uint8 stack of 16-byte "
                             f"blocks and their scales on the GPU")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("[hip] mx4_widen writes bf16 or float32")
        if seats is not None:
            seats = seats.to(blocks.device, torch.int32).contiguous()
            n = int(seats.numel())
        else:
            n = int(scales.shape[0])
        if out is None:
            out = torch.empty(n, groups * 32, dtype=dtype, device=blocks.device)
        elif out.dtype != dtype or not out.is_contiguous() or out.numel() != n * groups * 32:
            raise ValueError(f"[hip] mx4_widen: out must be {n * groups * 32} contiguous {dtype}")
        if n:
            self._call("btb_hip_mx4_widen", _p(blocks), _p(scales), None if seats is None else _p(seats),
                       n, groups, _p(out), int(dtype == torch.float32), _stream())
        return out


    # -- the host's bits on the card: f32 rows in, f32 rows out ------------------------------------------------------

    def _rows_io(self, x: torch.Tensor, y: torch.Tensor | None, R: int, C: int, what: str):
        self._need(x, torch.float32, "x")
        x2 = x.reshape(-1, C)
        b = int(x2.shape[0])
        if y is None:
            y = torch.empty(b, R, dtype=torch.float32, device=x.device)
        else:
            self._need(y, torch.float32, "y")
            if y.numel() != b * R:
                raise ValueError(f"[hip] {what}: y holds {y.numel()} elements, the product has {b * R}")
        return x2, b, y

    def gemv_lane16(self, w: torch.Tensor, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """the host's bf16 x f32 matvec to the bit (the reference's `_Cuda.gemv_lane16`, btb/engine/native.py:2342-2365):
        w bf16 [R, C], x f32 [n, C] -> f32 [n, R]"""
        self._need(w, torch.bfloat16, "w")
        R, C = (int(s) for s in w.shape)
        x2, b, y = self._rows_io(x, y, R, C, "gemv_lane16")
        self._call("btb_hip_gemv_bf16_rows", _p(w), R, C, _p(x2), b, _p(y), _stream())
        return y

    def gemv_lane16_p12(self, w: Any, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        R, C = w.shape
        x2, b, y = self._rows_io(x, y, R, C, "gemv_lane16_p12")
        ne = int(w.esc_idx.numel())
        self._call("btb_hip_gemv_p12_rows", _p(w.lo), _p(w.hi4), _p(w.table),
                   _p(w.esc_idx) if ne else None, _p(w.esc_val) if ne else None, ne, R, C, _p(x2), b,
                   _p(y), _stream())
        return y

    def gemv_lane16_mx4(self, w: Any, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """the host's MXFP4 matvec to the bit (`_Cuda.gemv_lane16_mx4`, btb/engine/native.py:2367-2390)"""
        R, C = w.shape
        x2, b, y = self._rows_io(x, y, R, C, "gemv_lane16_mx4")
        self._call("btb_hip_gemv_mxfp4_rows", _p(w.blocks), _p(w.scales), R, C, _p(x2), b, _p(y),
                   _stream())
        return y

    def gemv_lane16_mx4_ggml(self, raw: torch.Tensor, rows: int, cols: int, x: torch.Tensor,
                             y: torch.Tensor | None = None) -> torch.Tensor:
        """the same over ggml's layout: raw u8 [rows * cols / 32 * 17], 17-byte blocks with the scale first
        (`btb_gemv_mxfp4_ggml_rows`, native/src/lib.rs:162-183); the bits of `gemv_lane16_mx4` for the same weights"""
        self._need(raw, torch.uint8, "raw")
        if raw.numel() != rows * cols // 32 * 17:
            raise ValueError(f"[hip] gemv_lane16_mx4_ggml: {raw.numel()} bytes are not {rows} x {cols} weights in 17-byte blocks")
        x2, b, y = self._rows_io(x, y, rows, cols, "gemv_lane16_mx4_ggml")
        self._call("btb_hip_gemv_mxfp4_ggml_rows", _p(raw), rows, cols, _p(x2), b, _p(y), _stream())
        return y

    def gemv_lane16_fp8(self, w: Any, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        R, C = w.shape
        sr, sc = w.grid
        x2, b, y = self._rows_io(x, y, R, C, "gemv_lane16_fp8")
        self._call("btb_hip_gemv_fp8_rows", _p(w.w), _p(w.scales), R, C, sr, sc, _p(x2), b, _p(y),
                   _stream())
        return y

    # -- routed experts -----------------------------------------------------------------------------------------

    def moe_route(self, logits: torch.Tensor, k: int, E: int | None = None):
        """(idx int32 [T, k], weights bf16 [T, k], weights f32 [T, k]) of logits [T, ls] (bf16 or f32): softmax over
        the first E, top k by (p descending, index ascending), renormalised (`btb_moe_route`)"""
        if logits.dtype not in (torch.bfloat16, torch.float32) or not logits.is_cuda or logits.dim() != 2 \
                or logits.stride(1) != 1:
            raise ValueError("[hip] moe_route: logits must be a [T, ls] bf16 or f32 tensor on the GPU, rows contiguous")
        T, ls = int(logits.shape[0]), int(logits.stride(0))
        E = int(logits.shape[1]) if E is None else int(E)
        idx = torch.empty(T, k, dtype=torch.int32, device=logits.device)
        w = torch.empty(T, k, dtype=torch.bfloat16, device=logits.device)
        w32 = torch.empty(T, k, dtype=torch.float32, device=logits.device)
        self._call("btb_hip_moe_route", _p(logits), int(logits.dtype == torch.float32), ls, E, k, T, _p(idx),
                   _p(w), _p(w32), _stream())
        return idx, w, w32

    def moe_group_picks(self, idx: torch.Tensor, num_experts: int):
        """(pick position i32 [T k], row i32 [T k], offsets i32 [E], counts i32 [E]) of the picks idx i32 [T, k] sorted
        by expert, stable over idx.T.reshape(-1) (`group_picks`, btb/engine/host.py:283-296), all on the device"""
        self._need(idx, torch.int32, "idx")
        if idx.dim() != 2 or not idx.is_contiguous():
            raise ValueError("[hip] moe_group_picks: idx must be a contiguous [T, k] int32 tensor on the GPU")
        T, k = (int(s) for s in idx.shape)
        dev = idx.device
        slot = torch.empty(T * k, dtype=torch.int32, device=dev)
        token = torch.empty(T * k, dtype=torch.int32, device=dev)
        offs = torch.empty(int(num_experts), dtype=torch.int32, device=dev)
        counts = torch.empty(int(num_experts), dtype=torch.int32, device=dev)
        self._call("btb_hip_moe_group_picks", _p(idx), T, k, int(num_experts), _p(slot), _p(token),
                   _p(offs), _p(counts), _stream())
        return slot, token, offs, counts

    def moe_router(self, router: torch.Tensor, x: torch.Tensor, k: int):
        """(logits f32 [T, E], logits bf16 [T, E], idx int32 [T, k], weights bf16 [T, k], weights f32 [T, k]) of bf16
        rows x [T, H] against the bf16 router matrix [E, H]: the host-order logits and their routing, two launches"""
        self._need(router, torch.bfloat16, "router")
        self._need(x, torch.bfloat16, "x")
        E, H = (int(s) for s in router.shape)
        if x.dim() != 2 or int(x.shape[1]) != H:
            raise ValueError(f"[hip] moe_router: x {tuple(x.shape)} is not [T, {H}]")
        T = int(x.shape[0])
        dev = x.device
        logits = torch.empty(T, E, dtype=torch.float32, device=dev)
        logits16 = torch.empty(T, E, dtype=torch.bfloat16, device=dev)
        idx = torch.empty(T, k, dtype=torch.int32, device=dev)
        w = torch.empty(T, k, dtype=torch.bfloat16, device=dev)
        w32 = torch.empty(T, k, dtype=torch.float32, device=dev)
        self._call("btb_hip_moe_router_bf16", _p(router), _p(x), T, E, H, k, _p(logits),
                   _p(logits16), _p(idx), _p(w), _p(w32), _stream())
        return logits, logits16, idx, w, w32

    def moe_experts(self, gate_up: torch.Tensor, down: torch.Tensor, x: torch.Tensor, idx: torch.Tensor,
                    w: torch.Tensor, y: torch.Tensor | None = None, gu: torch.Tensor | None = None) -> torch.Tensor:
        """y [T, H]: the routed experts of x [T, H] over the stacks gate_up [E, 2I, H] and down [E, H, I] (bf16),
        picks idx int32 [T, k] and weights w bf16 [T, k], summed in ascending expert order"""
        for t, what in ((gate_up, "gate_up"), (down, "down"), (x, "x"), (w, "w")):
            self._need(t, torch.bfloat16, what)
        self._need(idx, torch.int32, "idx")
        E, I2, H = (int(s) for s in gate_up.shape)
        if tuple(down.shape) != (E, H, I2 // 2) or x.shape[-1] != H or idx.shape != w.shape:
            raise ValueError(f"[hip] moe_experts: gate_up {tuple(gate_up.shape)}, down {tuple(down.shape)}, x "
                             f"{tuple(x.shape)}, idx {tuple(idx.shape)}, w {tuple(w.shape)} do not fit together")
        T, k = (int(s) for s in idx.shape)
        if gu is None:
            gu = torch.empty(T, k, I2, dtype=torch.bfloat16, device=x.device)
        if y is None:
            y = torch.empty(T, H, dtype=torch.bfloat16, device=x.device)
        self._call("btb_hip_moe_experts_bf16", _p(gate_up), _p(down), _p(x), _p(idx), _p(w),
                   _p(gu), _p(y), T, k, E, H, I2 // 2, _stream())
        return y

    def moe_experts_mx4(self, ex: Any, x: torch.Tensor, idx: torch.Tensor, w: torch.Tensor,
                        y: torch.Tensor | None = None, h: torch.Tensor | None = None, oss: bool = True,
                        alpha: float = 1.702, limit: float = 7.0) -> torch.Tensor:
        """y [T, H]: the routed experts of x [T, H] over a layer's MXFP4 stacks as stored (`MxExperts`: gate_up blocks
        [E, 2I, H / 32, 16] + scales, down blocks [E, H, I / 32, 16] + scales, optional bf16 biases), picks idx int32
        [T, k], weights w bf16 [T, k], summed in ascending expert order. `oss`: gpt-oss's experts (interleaved gate /
        up rows, biases, the clamped gate with `alpha` and `limit`); else concatenated halves and SiLU."""
        for t, what in ((ex.gate_up_blocks, "gate_up_blocks"), (ex.gate_up_scales, "gate_up_scales"),
                        (ex.down_blocks, "down_blocks"), (ex.down_scales, "down_scales")):
            self._need(t, torch.uint8, what)
        for t, what in ((x, "x"), (w, "w")):
            self._need(t, torch.bfloat16, what)
        self._need(idx, torch.int32, "idx")
        E, H, I = int(ex.experts), int(ex.hidden), int(ex.intermediate)
        gb, db = getattr(ex, "gate_up_bias", None), getattr(ex, "down_bias", None)
        for t, what, n in ((gb, "gate_up_bias", E * 2 * I), (db, "down_bias", E * H)):
            if t is not None:
                self._need(t, torch.bfloat16, what)
                if t.numel() != n or not oss:
                    raise ValueError(f"[hip] moe_experts_mx4: {what} holds {t.numel()} values; the gpt-oss form takes {n}")
        if x.shape[-1] != H or idx.shape != w.shape or idx.dim() != 2:
            raise ValueError(f"[hip] moe_experts_mx4: x {tuple(x.shape)}, idx {tuple(idx.shape)}, w {tuple(w.shape)} do "
                             f"not fit a layer of hidden {H}")
        T, k = (int(s) for s in idx.shape)
        if h is None:
            h = torch.empty(T, k, I, dtype=torch.bfloat16, device=x.device)
        elif h.dtype != torch.bfloat16 or h.numel() < T * k * I or not h.is_contiguous():
            raise ValueError(f"[hip] moe_experts_mx4: h is contiguous bf16 scratch of at least {T * k * I} values")
        y = self._out(y, T, H, x.device, "moe_experts_mx4")
        p = lambda t: None if t is None else _p(t)
        self._call("btb_hip_moe_experts_mxfp4", _p(ex.gate_up_blocks), _p(ex.gate_up_scales), _p(ex.down_blocks),
                   _p(ex.down_scales), p(gb), p(db), _p(x), _p(idx), _p(w), _p(h), _p(y), T, k, E, H, I, int(bool(oss)),
                   float(alpha), float(limit), _stream())
        return y


    # -- the decode step's kernels between the matvecs ------------------------------------------------------------

    def embed(self, table: torch.Tensor, ids: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
        self._need(table, torch.bfloat16, "table")
        self._need(ids, torch.int32, "ids")
        self._need(h, torch.bfloat16, "h")
        V, H = (int(s) for s in table.shape)
        self._call("btb_hip_embed", _p(table), _p(ids), _p(h), int(ids.numel()), H, V, _stream())
        return h

    def add_rmsnorm(self, h: torch.Tensor, y: torch.Tensor | None, w: torch.Tensor, eps: float, x: torch.Tensor,
                    centered: bool = False) -> torch.Tensor:
        """h += y in place (bf16 add), x = rmsnorm(h) * w (`btb_add_rmsnorm`)"""
        for t, what in ((h, "h"), (w, "w"), (x, "x")):
            self._need(t, torch.bfloat16, what)
        if y is not None:
            self._need(y, torch.bfloat16, "y")
        H = int(w.numel())
        T = int(h.numel()) // H
        if h.numel() != T * H or x.numel() != T * H or (y is not None and y.numel() != T * H):
            raise ValueError("[hip] add_rmsnorm: h, y and x are [T, H] with H the weight's length")
        self._call("btb_hip_add_rmsnorm", _p(h), None if y is None else _p(y), _p(w), float(eps),
                   _p(x), T, H, int(bool(centered)), _stream())
        return x

    def norm_rope_kv(self, qkv: torch.Tensor, wq: torch.Tensor | None, wk: torch.Tensor | None, eps: float,
                     cos: torch.Tensor, sin: torch.Tensor, n0: torch.Tensor, K: torch.Tensor, V: torch.Tensor,
                     q: torch.Tensor, Hq: int, Hk: int, D: int, depth: torch.Tensor | None = None,
                     centered: bool = False, tbl: torch.Tensor | None = None) -> None:
        """q/k norm, rope and the cache write for the pass's rows (`btb_norm_rope_kv_d{D}`); K, V are one layer's
        [Hk, cap, D] views (any strides with D contiguous). `tbl` (int32, one entry a logical slot): the cache's row
        map - row t lands in cache row tbl[n0 + t] (`btb_norm_rope_kv_tbl_d{D}`)"""
        for t, what in ((qkv, "qkv"), (cos, "cos"), (sin, "sin"), (q, "q")):
            self._need(t, torch.bfloat16, what)
        self._need(n0, torch.int32, "n0")
        if K.dtype != torch.bfloat16 or V.dtype != torch.bfloat16 or K.stride(2) != 1 or K.stride() != V.stride():
            raise ValueError("[hip] norm_rope_kv: K and V are bf16 [Hk, cap, D] views with the same strides")
        T = int(qkv.numel()) // ((Hq + 2 * Hk) * D)
        args = (_p(qkv), None if wq is None else _p(wq), None if wk is None else _p(wk), float(eps),
                _p(cos), _p(sin), _p(n0), None if depth is None else _p(depth), _p(K),
                _p(V), _p(q), T, Hq, Hk, D, int(K.stride(0)), int(K.stride(1)), int(bool(centered)))
        if tbl is None:
            self._call("btb_hip_norm_rope_kv", *args, _stream())
        else:
            self._need(tbl, torch.int32, "tbl")
            self._call("btb_hip_norm_rope_kv_tbl", *args, _p(tbl), _stream())

    @staticmethod
    def rows_layout(base: int, steps: int, W: int, rows: Sequence[tuple[int, int, int]], pad_to: int = 0,
                    device: Any = "cuda") -> torch.Tensor:
        """The layout of a pass whose rows are sequences of their own (the reference fills the same array before a
        rows step, btb/engine/cuda.py:3457-3464): int32 [base, steps, W, then (col, off, len) a row] - row t's prefix is
        `len` cache slots from `off`, its own step i lies at slot base + i * W + col. Rows past `rows` up to `pad_to`
        are padding (len -1), which the kernels skip."""
        lay = [int(base), int(steps), int(W)]
        for col, off, n in rows:
            lay += [int(col), int(off), int(n)]
        lay += [0, 0, -1] * max(0, int(pad_to) - len(rows))
        return torch.tensor(lay, dtype=torch.int32, device=device)

    def norm_rope_kv_seqs(self, qkv: torch.Tensor, wq: torch.Tensor | None, wk: torch.Tensor | None, eps: float,
                          cos: torch.Tensor, sin: torch.Tensor, rw: torch.Tensor, K: torch.Tensor, V: torch.Tensor,
                          q: torch.Tensor, Hq: int, Hk: int, D: int, centered: bool = False) -> None:
        """`norm_rope_kv` for a pass whose rows are sequences of their own, laid out by `rw` (`rows_layout`): row t is
        roped at its own position len + steps and written to its step's slot (`btb_norm_rope_kv_rows_d{D}`)"""
        for t, what in ((qkv, "qkv"), (cos, "cos"), (sin, "sin"), (q, "q")):
            self._need(t, torch.bfloat16, what)
        self._need(rw, torch.int32, "rw")
        if K.dtype != torch.bfloat16 or V.dtype != torch.bfloat16 or K.stride(2) != 1 or K.stride() != V.stride():
            raise ValueError("[hip] norm_rope_kv_seqs: K and V are bf16 [Hk, cap, D] views with the same strides")
        T = int(qkv.numel()) // ((Hq + 2 * Hk) * D)
        if rw.numel() < 3 + 3 * T:
            raise ValueError(f"[hip] norm_rope_kv_seqs: the layout holds {rw.numel()} words, {T} rows take {3 + 3 * T}")
        self._call("btb_hip_norm_rope_kv_seqs", _p(qkv), None if wq is None else _p(wq), None if wk is None else _p(wk),
                   float(eps), _p(cos), _p(sin), _p(rw), _p(K), _p(V), _p(q), T, Hq, Hk, D, int(K.stride(0)),
                   int(K.stride(1)), int(bool(centered)), _stream())

    def attn_decode_seqs(self, q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, att: torch.Tensor, rw: torch.Tensor,
                         Hq: int, Hk: int, D: int, scale: float, span: int, S: int, part_m: torch.Tensor,
                         part_l: torch.Tensor, part_acc: torch.Tensor, win: int = 0) -> None:
        """decode attention for a pass whose rows are sequences of their own (`rw`): row t over its own prefix and
        steps, in S spans of `span` keys; the spans' states go into the caller's three arrays
        (`btb_attn_flash_rows_d128`)"""
        for t, what in ((q, "q"), (att, "att")):
            self._need(t, torch.bfloat16, what)
        self._need(rw, torch.int32, "rw")
        for t, what in ((part_m, "part_m"), (part_l, "part_l"), (part_acc, "part_acc")):
            self._need(t, torch.float32, what)
        if K.dtype != torch.bfloat16 or V.dtype != torch.bfloat16 or K.stride(2) != 1 or K.stride() != V.stride():
            raise ValueError("[hip] attn_decode_seqs: K and V are bf16 [Hk, cap, D] views with the same strides")
        T = int(q.numel()) // (Hq * D)
        if q.numel() != T * Hq * D or att.numel() != T * Hq * D or rw.numel() < 3 + 3 * T:
            raise ValueError("[hip] attn_decode_seqs: q and att are [T, Hq D], the layout holds 3 + 3 T words")
        if part_m.numel() < T * Hq * S or part_l.numel() < T * Hq * S or part_acc.numel() < T * Hq * S * D:
            raise ValueError(f"[hip] attn_decode_seqs: part_m / part_l hold T Hq S = {T * Hq * S} floats, part_acc D times that")
        self._call("btb_hip_attn_decode_seqs", _p(q), _p(K), _p(V), _p(att), _p(rw), T, Hq, Hk, D, int(K.stride(0)),
                   int(K.stride(1)), float(scale), int(span), int(S), int(win), _p(part_m), _p(part_l), _p(part_acc),
                   _stream())

    def attn_scratch(self, T: int, Hq: int, Hk: int, D: int, S: int, device: Any = "cuda") -> torch.Tensor:
        """the f32 scratch `attn_decode` leaves its spans' states in, at these sizes"""
        n = int(self.lib.btb_hip_attn_scratch_floats(T, Hq, Hk, D, S))
        return torch.empty(n, dtype=torch.float32, device=device)

    def attn_decode(self, q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, att: torch.Tensor, n0: torch.Tensor,
                    Hq: int, Hk: int, D: int, scale: float, S: int, scratch: torch.Tensor,
                    par: torch.Tensor | None = None, win: int = 0, tbl: torch.Tensor | None = None) -> None:
        """att [T, Hq * D] = the rows' attention over the cache: row t sees keys 0 .. n0 + t, or with `par` (int32 [T],
        a verify pass's tree: the row's parent among the pass's rows, -1 at a root) the cache's n0 keys and, of the
        pass's rows, its ancestors and itself. `win` > 0: only the last `win` positions up to the row's own; `tbl`
        (int32, one entry a logical slot): the cache's row map"""
        self._need(q, torch.bfloat16, "q")
        self._need(att, torch.bfloat16, "att")
        self._need(n0, torch.int32, "n0")
        self._need(scratch, torch.float32, "scratch")
        if K.dtype != torch.bfloat16 or V.dtype != torch.bfloat16 or K.stride(2) != 1 or K.stride() != V.stride():
            raise ValueError("[hip] attn_decode: K and V are bf16 [Hk, cap, D] views with the same strides")
        T = int(q.numel()) // (Hq * D)
        need = int(self.lib.btb_hip_attn_scratch_floats(T, Hq, Hk, D, S))
        if scratch.numel() < need:
            raise ValueError(f"[hip] attn_decode: scratch holds {scratch.numel()} floats, {need} are needed")
        if par is not None:
            self._need(par, torch.int32, "par")
            if par.numel() != T:
                raise ValueError(f"[hip] attn_decode: par names {par.numel()} rows, the pass has {T}")
        if win or tbl is not None:
            if tbl is not None:
                self._need(tbl, torch.int32, "tbl")
                if tbl.numel() < int(K.shape[1]):
                    raise ValueError(f"[hip] attn_decode: tbl maps {tbl.numel()} slots, the cache has {int(K.shape[1])}")
            self._call("btb_hip_attn_decode_win", _p(q), _p(K), _p(V), _p(att), _p(n0),
                       None if par is None else _p(par), T, Hq, Hk, D, int(K.stride(0)), int(K.stride(1)),
                       float(scale), int(K.shape[1]), S, int(win), None if tbl is None else _p(tbl),
                       _p(scratch), _stream())
            return
        self._call("btb_hip_attn_decode", _p(q), _p(K), _p(V), _p(att), _p(n0),
                   None if par is None else _p(par), T, Hq, Hk, D, int(K.stride(0)), int(K.stride(1)),
                   float(scale), int(K.shape[1]), S, _p(scratch), _stream())

    def attn_decode_noalloc(self, q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, att: torch.Tensor,
                            n0: torch.Tensor, Hq: int, Hk: int, D: int, scale: float, S: int,
                            par: torch.Tensor | None = None) -> None:
        """`attn_decode` without a workspace: the spans' states go into the array the library holds on the GPU (4 MiB;
        larger passes are refused). For callers that may not allocate; calls that overlap on one GPU race on it."""
        self._need(q, torch.bfloat16, "q")
        self._need(att, torch.bfloat16, "att")
        self._need(n0, torch.int32, "n0")
        if K.dtype != torch.bfloat16 or V.dtype != torch.bfloat16 or K.stride(2) != 1 or K.stride() != V.stride():
            raise ValueError("[hip] attn_decode_noalloc: K and V are bf16 [Hk, cap, D] views with the same strides")
        T = int(q.numel()) // (Hq * D)
        if att.numel() != T * Hq * D:
            raise ValueError(f"[hip] attn_decode_noalloc: att holds {att.numel()} values, the pass makes {T * Hq * D}")
        if par is not None:
            self._need(par, torch.int32, "par")
            if par.numel() != T:
                raise ValueError(f"[hip] attn_decode_noalloc: par names {par.numel()} rows, the pass has {T}")
        self._call("btb_hip_attn_decode_noalloc", _p(q), _p(K), _p(V), _p(att), _p(n0),
                   None if par is None else _p(par), T, Hq, Hk, D, int(K.stride(0)), int(K.stride(1)),
                   float(scale), int(K.shape[1]), S, _stream())

    def attn_decode_qkv(self, qkv: torch.Tensor, wq: torch.Tensor | None, wk: torch.Tensor | None, eps: float,
                        cos_t: torch.Tensor, sin_t: torch.Tensor, n0: torch.Tensor, K: torch.Tensor, V: torch.Tensor,
                        att: torch.Tensor, Hq: int, Hk: int, D: int, scale: float, S: int, scratch: torch.Tensor,
                        centered: bool = False) -> None:
        """the step's own attention straight from the fused qkv row: `norm_rope_kv` + `attn_decode` at one row, one
        launch less (q stays on the chip; the new K / V row is written by the workgroup whose span holds slot n0)"""
        for t, what in ((qkv, "qkv"), (att, "att"), (cos_t, "cos"), (sin_t, "sin")):
            self._need(t, torch.bfloat16, what)
        for t, what in ((wq, "wq"), (wk, "wk")):
            if t is not None:
                self._need(t, torch.bfloat16, what)
                if t.numel() != D:
                    raise ValueError(f"[hip] attn_decode_qkv: {what} holds {t.numel()} values, head_dim is {D}")
        self._need(n0, torch.int32, "n0")
        self._need(scratch, torch.float32, "scratch")
        if K.dtype != torch.bfloat16 or V.dtype != torch.bfloat16 or K.stride(2) != 1 or K.stride() != V.stride():
            raise ValueError("[hip] attn_decode_qkv: K and V are bf16 [Hk, cap, D] views with the same strides")
        if qkv.numel() != (Hq + 2 * Hk) * D or att.numel() != Hq * D:
            raise ValueError("[hip] attn_decode_qkv: one row of qkv [(Hq + 2 Hk) D] and of att [Hq D]")
        if cos_t.shape[-1] != D or cos_t.shape != sin_t.shape or cos_t.shape[0] < K.shape[1]:
            raise ValueError("[hip] attn_decode_qkv: rope tables are [positions >= cap, D]")
        need = int(self.lib.btb_hip_attn_scratch_floats(1, Hq, Hk, D, S))
        if scratch.numel() < need:
            raise ValueError(f"[hip] attn_decode_qkv: scratch holds {scratch.numel()} floats, {need} are needed")
        p = lambda t: None if t is None else _p(t)
        self._call("btb_hip_attn_decode_qkv", _p(qkv), p(wq), p(wk), float(eps), 1 if centered else 0,
                   _p(cos_t), _p(sin_t), _p(n0), _p(K), _p(V), _p(att), Hq, Hk, D,
                   int(K.stride(0)), int(K.stride(1)), float(scale), int(K.shape[1]), S, _p(scratch), _stream())

    def attn_rows_fused(self, T: int, Hq: int, Hk: int, D: int, cap: int, S: int) -> bool:
        """whether `attn_decode_qkv_rows` takes a pass of this shape"""
        return bool(self.lib.btb_hip_attn_rows_fused(T, Hq, Hk, D, cap, S))

    def attn_decode_qkv_rows(self, qkv: torch.Tensor, wq: torch.Tensor | None, wk: torch.Tensor | None, eps: float,
                             cos_t: torch.Tensor, sin_t: torch.Tensor, n0: torch.Tensor, K: torch.Tensor,
                             V: torch.Tensor, att: torch.Tensor, Hq: int, Hk: int, D: int, scale: float, S: int,
                             scratch: torch.Tensor, depth: torch.Tensor | None = None,
                             par: torch.Tensor | None = None, centered: bool = False) -> None:
        """a pass's attention straight from its fused qkv rows [T, (Hq + 2 Hk) D]: `norm_rope_kv` + `attn_decode`, one
        launch less (q stays on the chip; the new K / V rows are written by the workgroups whose spans hold them)"""
        for t, what in ((qkv, "qkv"), (att, "att"), (cos_t, "cos"), (sin_t, "sin")):
            self._need(t, torch.bfloat16, what)
        for t, what in ((wq, "wq"), (wk, "wk")):
            if t is not None:
                self._need(t, torch.bfloat16, what)
                if t.numel() != D:
                    raise ValueError(f"[hip] attn_decode_qkv_rows: {what} holds {t.numel()} values, head_dim is {D}")
        self._need(n0, torch.int32, "n0")
        self._need(scratch, torch.float32, "scratch")
        if K.dtype != torch.bfloat16 or V.dtype != torch.bfloat16 or K.stride(2) != 1 or K.stride() != V.stride():
            raise ValueError("[hip] attn_decode_qkv_rows: K and V are bf16 [Hk, cap, D] views with the same strides")
        width = (Hq + 2 * Hk) * D
        T = qkv.numel() // width
        if T < 1 or qkv.numel() != T * width or att.numel() != T * Hq * D:
            raise ValueError("[hip] attn_decode_qkv_rows: qkv is [T, (Hq + 2 Hk) D], att [T, Hq D]")
        if cos_t.shape[-1] != D or cos_t.shape != sin_t.shape or cos_t.shape[0] < K.shape[1]:
            raise ValueError("[hip] attn_decode_qkv_rows: rope tables are [positions >= cap, D]")
        for t, what in ((depth, "depth"), (par, "par")):
            if t is not None:
                self._need(t, torch.int32, what)
                if t.numel() != T:
                    raise ValueError(f"[hip] attn_decode_qkv_rows: {what} names {t.numel()} rows, the pass has {T}")
        need = int(self.lib.btb_hip_attn_scratch_floats(T, Hq, Hk, D, S))
        if scratch.numel() < need:
            raise ValueError(f"[hip] attn_decode_qkv_rows: scratch holds {scratch.numel()} floats, {need} are needed")
        p = lambda t: None if t is None else _p(t)
        self._call("btb_hip_attn_decode_qkv_rows", _p(qkv), p(wq), p(wk), float(eps), 1 if centered else 0,
                   _p(cos_t), _p(sin_t), _p(n0), p(depth), p(par), _p(K), _p(V),
                   _p(att), T, Hq, Hk, D, int(K.stride(0)), int(K.stride(1)), float(scale), int(K.shape[1]), S,
                   _p(scratch), _stream())

    def silu_mul(self, gu: torch.Tensor, m: torch.Tensor) -> torch.Tensor:
        self._need(gu, torch.bfloat16, "gu")
        self._need(m, torch.bfloat16, "m")
        I = int(gu.shape[-1]) // 2
        self._call("btb_hip_silu_mul", _p(gu), _p(m), int(gu.numel()) // (2 * I), I, _stream())
        return m

    def argmax(self, logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        self._need(logits, torch.bfloat16, "logits")
        self._need(out, torch.int32, "out")
        V = int(logits.shape[-1])
        self._call("btb_hip_argmax", _p(logits), _p(out), int(logits.numel()) // V, V, _stream())
        return out

    def publish(self, n0: torch.Tensor, picked: torch.Tensor, next_ids: torch.Tensor | None = None,
                out_tok: torch.Tensor | None = None, out_n0: torch.Tensor | None = None,
                out_ts: torch.Tensor | None = None) -> None:
        """the step's end: next_ids = picked, n0 += 1, and the token / clock / length into pinned host tensors"""
        p = lambda t: None if t is None else _p(t)
        self._call("btb_hip_publish", _p(n0), _p(picked), p(next_ids), p(out_tok), p(out_n0), p(out_ts),
                   _stream())

    def publish_only(self, n0: torch.Tensor, ids: torch.Tensor, out_tok: torch.Tensor, out_n0: torch.Tensor | None = None,
                     out_ts: torch.Tensor | None = None) -> None:
        """the reference's `btb_publish`: token, clock and length into pinned host tensors, nothing else"""
        p = lambda t: None if t is None else _p(t)
        self._call("btb_hip_publish_only", _p(n0), _p(ids), _p(out_tok), p(out_n0), p(out_ts), _stream())

    def argmax_publish(self, logits: torch.Tensor, picked: torch.Tensor, n0: torch.Tensor,
                       next_ids: torch.Tensor | None = None, out_tok: torch.Tensor | None = None,
                       out_n0: torch.Tensor | None = None, out_ts: torch.Tensor | None = None) -> None:
        """`argmax` over one row and `publish` in one launch"""
        self._need(logits, torch.bfloat16, "logits")
        self._need(picked, torch.int32, "picked")
        self._need(n0, torch.int32, "n0")
        V = int(logits.shape[-1])
        if logits.numel() != V:
            raise ValueError("[hip] argmax_publish: one row of logits")
        p = lambda t: None if t is None else _p(t)
        self._call("btb_hip_argmax_publish", _p(logits), V, _p(picked), _p(n0), p(next_ids),
                   p(out_tok), p(out_n0), p(out_ts), _stream())


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
