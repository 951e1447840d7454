"""The C ABI as a maintainer binds it: the shared library loads where no GPU is, exports every function the header
declares, and the Python binder's signature table names exactly that list (no compute call is made here)."""

from __future__ import annotations

import ctypes
import os
import re

from btb_amd import native

from .helpers import ROOT

HEADER = os.path.join(ROOT, "include", "btb_hip.h")


def declared() -> list[str]:
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(btb_hip_\w+)\s*\(", text)))


def test_header_declares_functions():
    names = declared()
    assert "btb_hip_gemv_bf16" in names and len(names) >= 7


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(native.LIB_PATH)
    for name in declared():
        assert hasattr(lib, name), f"{name} is declared in include/btb_hip.h but not exported"


def test_binder_covers_the_header():
    assert sorted(native.SIGNATURES) == declared()
    native.load_library()


def test_process_entry_points_without_a_gpu():
    lib = native.load_library()
    assert lib.btb_hip_arch() == b"gfx950"
    assert lib.btb_hip_set_tuning(b"no_such_knob", 1) == native.ERR_DOMAIN
    assert lib.btb_hip_set_tuning(None, 1) == native.ERR_NULL
    assert lib.btb_hip_set_tuning(b"gemv_wgs_per_cu", -1) == native.OK
    assert b"unknown" in lib.btb_hip_last_error()


class _Recorder:
    """a launcher that keeps what it is handed"""

    def __init__(self):
        self.calls = []

    def launch(self, name, grid, block, args, stream=None, shared=0):
        self.calls.append((name, grid, block, list(args), stream, shared))


def test_typed_launchers_name_the_kernels_the_card_serves():
    """the typed launchers (btb/engine/card_launch.py's surface for this path) and the card's launch table agree:
    every kernel name a launcher can produce is served, with the parameter count the launcher packs; `ptr(role, t)`
    is the reference's (`role(t.data_ptr())`, None the null address)"""
    from btb_amd import card_launch as cl

    assert set(native._LAUNCH) == set(cl.KERNELS)
    for fam, (variant, params) in cl.SPEC.items():
        n = len(params.split())
        for name in cl.kernel_names(fam):
            if name in native._LAUNCH:
                assert native._LAUNCH[name][0] == n, name
    assert issubclass(native.HipCard, cl.CardLaunch)

    class T:  # anything with data_ptr()
        def data_ptr(self):
            return 0x1000

    assert cl.ptr(cl.Weight, T()) == 0x1000 and cl.ptr(cl.RowMap, None) == 0
    assert native.HipCard.ptr(cl.Query, T()) == 0x1000
    rec = _Recorder()
    cl.btb_gemv_bf16(rec, 4, (3, 1, 1), (128, 1, 1), 0x1000, 0x2000, 0x3000, 12, 64, shared=16)
    name, grid, block, args, stream, shared = rec.calls[0]
    assert (name, grid, block, stream, shared) == ("btb_gemv_bf16_m4", (3, 1, 1), (128, 1, 1), None, 16)
    assert [type(a) for a in args] == [ctypes.c_void_p] * 3 + [ctypes.c_int] * 2
    assert [a.value for a in args] == [0x1000, 0x2000, 0x3000, 12, 64]
    cl.btb_attn_flash(rec, 128, (1, 2, 8), (256, 1, 1), 1, 2, 3, 4, 5, 0, 1, 32, 8, 128, 1024, 0.125, 6, 7, 8, 9, 0, 0)
    name, _, _, args, _, _ = rec.calls[1]
    assert name == "btb_attn_flash_d128" and len(args) == 18 and args[5].value is None and args[17].value is None
    assert isinstance(args[11], ctypes.c_float) and isinstance(args[16], ctypes.c_int)
    cl.btb_mx4_widen(rec, (1, 3, 1), (256, 1, 1), 1, 2, 3, groups=1 << 33, out=4)
    assert isinstance(rec.calls[2][3][3], ctypes.c_longlong) and rec.calls[2][3][3].value == 1 << 33
