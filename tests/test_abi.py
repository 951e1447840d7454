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
