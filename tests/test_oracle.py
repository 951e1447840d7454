"""Pins the CPU oracle (oracle/btb_oracle.c) before anything is checked against it: the reference's own hand cases
and constants, the f64 bound its tests hold, a brute force in exact rational arithmetic of the 16-lane order, the
invariance laws (threads, batch width, ISA tier move no bit) and the error codes of the C ABI."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from oracle import codecs

from .helpers import bits16, conditioned_err, f32_bits, lane16_row, weights_bf16


def bf(v) -> np.ndarray:
    """exact small values as bf16 bit patterns"""
    return bits16(torch.tensor(v, dtype=torch.float32).to(torch.bfloat16))


# -- the reference's hand cases (native/src/gemv.rs:5023-5032; native/tests/gemv.rs:355-368) ---------------------


def test_hand_cases():
    y = oracle.gemv_bf16(bf([[1, 2, -3], [0.5, -1, 4]]), np.array([[2, 3, 1]], dtype=np.float32))
    assert y.tolist() == [[5.0, 2.0]]
    assert oracle.gemv_bf16(bf([[1.5, 2.5]]), np.array([[2, 4]], np.float32)).tolist() == [[13.0]]
    assert oracle.gemv_bf16(bf([[1.5], [2.5]]), np.array([[3]], np.float32)).tolist() == [[4.5, 7.5]]


def test_bf16_widen_is_a_shift():
    for bits in (0x3F80, 0xBF80, 0x0001, 0x7F7F, 0x3EAB):  # (-0 + 0 is +0, so 0x8000 is not in the list)
        y = oracle.gemv_bf16(np.array([[bits]], np.uint16), np.array([[1.0]], np.float32))
        assert f32_bits(y)[0, 0] == bits << 16


# -- the summation order, by brute force in exact arithmetic --------------------------------------------------------


@pytest.mark.parametrize("rows,cols", [(3, 70), (5, 16), (2, 33), (1, 1), (4, 529)])
def test_lane_order_brute_force(rows, cols):
    """a dropped term, a wrong lane or a different fold order changes low bits on these ill-conditioned rows"""
    rng = np.random.default_rng(rows * 1000 + cols)
    # wide dynamic range, so the order of the additions shows in the result
    w = codecs.f32_to_bf16_bits((rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-6, 6, (rows, cols))))
                                .astype(np.float32))
    x = (rng.standard_normal((1, cols)) * np.exp2(rng.integers(-6, 6, (1, cols)))).astype(np.float32)
    y = oracle.gemv_bf16(w, x)
    wf = codecs.bf16_bits_to_f32(w)
    for r in range(rows):
        want = lane16_row(wf[r], x[0])
        assert f32_bits(y[0, r]) == f32_bits(want), (r, y[0, r], want)


def test_fold16_order():
    a = (np.arange(16, dtype=np.float32) + 1) * np.float32(1e-3) + np.float32(1e4) * (np.arange(16) % 3 == 0)
    got = oracle.lib().btb_oracle_fold16(a.ctypes.data)
    t = [np.float32(a[2 * j] + a[2 * j + 1]) for j in range(8)]
    u = [np.float32(t[2 * j] + t[2 * j + 1]) for j in range(4)]
    want = np.float32(np.float32(u[0] + u[1]) + np.float32(u[2] + u[3]))
    assert np.float32(got) == want


# -- f64 bound (native/src/gemv.rs:5034-5073: conditioned error < 1e-6) ------------------------------------------------


@pytest.mark.parametrize("rows,cols,b", [(48, 512, 1), (37, 1031, 3), (8, 5120, 2), (129, 17, 9)])
def test_against_f64(rows, cols, b):
    w = weights_bf16(rows, cols, 1, std=1.0)
    x = torch.randn(b, cols, generator=torch.Generator().manual_seed(2)).numpy()
    y = oracle.gemv_bf16(bits16(w), x, threads=3)
    assert conditioned_err(y, w.double().numpy(), x.astype(np.float64)) < 1e-6


# -- the laws: threads, batch width and tier move no bit (native/src/gemv.rs:5112-5145) --------------------------------


def test_threads_batch_and_tier_move_no_bit():
    rows, cols = 67, 1100
    w = bits16(weights_bf16(rows, cols, 3))
    x = torch.randn(17, cols, generator=torch.Generator().manual_seed(4)).numpy()
    oracle.set_tier(oracle.TIER_SCALAR)
    base = oracle.gemv_bf16(w, x, threads=1)
    try:
        for tier in (oracle.TIER_SCALAR, oracle.TIER_AVX2, oracle.TIER_AVX512):
            oracle.set_tier(tier)
            for threads in (1, 2, 7, 0):
                y = oracle.gemv_bf16(w, x, threads=threads)
                assert np.array_equal(f32_bits(y), f32_bits(base)), (tier, threads)
            for i in (0, 5, 16):  # a row of a batch is its own one-row call
                solo = oracle.gemv_bf16(w, x[i : i + 1], threads=2)
                assert np.array_equal(f32_bits(solo[0]), f32_bits(base[i]))
    finally:
        oracle.set_tier(-1)


def test_group_equals_single_calls():
    L = oracle.lib()
    shapes = [(12, 64), (5, 48), (33, 512)]
    ws = [bits16(weights_bf16(r, c, 10 + i)) for i, (r, c) in enumerate(shapes)]
    xs = [np.random.default_rng(i).standard_normal((2, c)).astype(np.float32) for i, (_, c) in enumerate(shapes)]
    ys = [np.zeros((2, r), np.float32) for r, _ in shapes]
    n = len(shapes)
    P = ctypes.c_void_p * n
    S = ctypes.c_size_t * n
    rc = L.btb_gemv_bf16_group(n, P(*[w.ctypes.data for w in ws]), S(*[r for r, _ in shapes]),
                               S(*[c for _, c in shapes]), P(*[x.ctypes.data for x in xs]), S(*[2] * n),
                               P(*[y.ctypes.data for y in ys]), 3)
    assert rc == 0
    for w, x, y in zip(ws, xs, ys):
        assert np.array_equal(f32_bits(y), f32_bits(oracle.gemv_bf16(w, x)))


# -- pack12: the packed matvec is the bf16 matvec, bit for bit (native/tests/gemv.rs:297-299) ------------------------


@pytest.mark.parametrize("rows,cols", [(16, 512), (7, 33), (9, 1030), (1, 1)])
def test_p12_equals_bf16_bits(rows, cols):
    w = weights_bf16(rows, cols, 20)
    wb = bits16(w).copy()
    # force escapes: a few high bytes far from the palette
    flat = wb.reshape(-1)
    at = np.arange(0, flat.size, max(1, flat.size // 37))
    flat[at] = (flat[at] & 0x00FF) | ((0x10 + np.arange(at.size) % 24).astype(np.uint16) << 8)
    packed = codecs.pack12_pack(wb)
    assert packed[3].size > 0 or flat.size < 16
    x = np.random.default_rng(1).standard_normal((3, cols)).astype(np.float32)
    want = oracle.gemv_bf16(wb.reshape(rows, cols), x)
    for tier in (oracle.TIER_SCALAR, oracle.TIER_AVX2):
        oracle.set_tier(tier)
        got = oracle.gemv_p12(*packed, rows, cols, x, threads=2)
        assert np.array_equal(f32_bits(got), f32_bits(want))
    oracle.set_tier(-1)
    assert np.array_equal(oracle.unpack_p12(*packed, rows * cols), flat)


# -- MXFP4 constants (native/src/gemv.rs:5260-5274) and the closed form ldexp(fp4, s - 127) -----------------------------


def test_mxfp4_table_and_scale_constants():
    L = oracle.lib()
    want = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    got = [L.btb_oracle_fp4_value(c) for c in range(16)]
    assert got == want and np.signbit(np.float32(got[8]))
    assert L.btb_oracle_mx_scale(127) == 1.0 and L.btb_oracle_mx_scale(128) == 2.0
    assert L.btb_oracle_mx_scale(126) == 0.5
    assert L.btb_oracle_mx_scale(1) == 2.0**-126 and L.btb_oracle_mx_scale(0) == 2.0**-127


def test_mxfp4_widen_every_byte_every_scale():
    """all 256 bytes x all 256 scales against numpy's ldexp (one rounding), and against the numpy codec"""
    blocks = np.tile(np.arange(256, dtype=np.uint8).reshape(16, 16), (256, 1))  # [4096, 16]
    scales = np.repeat(np.arange(256, dtype=np.uint8), 16)                      # [4096]
    got = oracle.widen_mxfp4(blocks, scales).reshape(4096, 32)
    lut = codecs.FP4_VALUES
    vals = np.empty((4096, 32), np.float32)
    vals[:, 0::2] = lut[blocks & 15]
    vals[:, 1::2] = lut[blocks >> 4]
    with np.errstate(over="ignore", invalid="ignore"):
        want = np.ldexp(vals.astype(np.float64), scales.astype(np.int64)[:, None] - 127).astype(np.float32)
    finite = scales != 255
    assert np.array_equal(f32_bits(got[finite]), f32_bits(want[finite]))
    # scale 255 is +inf: 0 * inf is NaN, anything else +-inf
    assert np.all(np.isnan(got[~finite]) | np.isinf(got[~finite]))
    assert np.array_equal(f32_bits(got[finite]),
                          f32_bits(codecs.mxfp4_dequantize(blocks.reshape(4096, 1, 16), scales.reshape(4096, 1))[finite]))


def test_mxfp4_gemv_against_f64():
    rng = np.random.default_rng(5)
    rows, cols = 24, 256
    blocks = rng.integers(0, 256, (rows, cols // 32, 16), dtype=np.uint8)
    scales = rng.integers(118, 132, (rows, cols // 32), dtype=np.uint8)
    x = rng.standard_normal((2, cols)).astype(np.float32)
    y = oracle.gemv_mxfp4(blocks, scales, rows, cols, x, threads=2)
    w = codecs.mxfp4_dequantize(blocks, scales).astype(np.float64)
    assert conditioned_err(y, w, x.astype(np.float64)) < 1e-6


@pytest.mark.parametrize("rows,cols", [(1, 32), (5, 96), (17, 1024), (33, 2880)])
def test_mxfp4_ggml_layout_gives_the_checkpoint_layouts_bits(rows, cols):
    """native/src/gemv.rs:5215-5250: the same weights in ggml's 17-byte blocks give the same bits, any b, any threads"""
    from .helpers import mx4_ggml

    rng = np.random.default_rng(rows)
    blocks = rng.integers(0, 256, (rows, cols // 32, 16), dtype=np.uint8)
    scales = rng.integers(0, 255, (rows, cols // 32), dtype=np.uint8)
    raw = mx4_ggml(blocks, scales)
    for b in (1, 3, 16):
        x = rng.uniform(-1, 1, (b, cols)).astype(np.float32)
        want = oracle.gemv_mxfp4(blocks, scales, rows, cols, x, threads=2)
        got = oracle.gemv_mxfp4_ggml(raw, rows, cols, x, threads=3)
        assert np.all((f32_bits(got) == f32_bits(want)) | (np.isnan(got) & np.isnan(want)))
    # a hand case: scale 127 (2^0), weight 0 = code 2 (1.0) in the low nibble of byte 1, weight 16 = code 4 (2.0) in its high
    one = np.zeros(17, np.uint8)
    one[0], one[1] = 127, 0x42
    xx = np.zeros((1, 32), np.float32)
    xx[0, 0], xx[0, 16] = 3.0, 5.0
    assert oracle.gemv_mxfp4_ggml(one, 1, 32, xx)[0, 0] == 1.0 * 3.0 + 2.0 * 5.0
    L = oracle.lib()
    y = np.zeros((1, 1), np.float32)
    assert L.btb_gemv_mxfp4_ggml_rows(None, 1, 32, xx.ctypes.data, 1, y.ctypes.data, 1) == oracle.ERR_NULL
    assert L.btb_gemv_mxfp4_ggml_rows(one.ctypes.data, 1, 24, xx.ctypes.data, 1, y.ctypes.data, 1) == oracle.ERR_DOMAIN


# -- FP8 (native/src/gemv.rs:5383-5430) --------------------------------------------------------------------------


def test_f8_value_all_bytes_against_torch():
    L = oracle.lib()
    b = torch.arange(256, dtype=torch.uint8)
    want = b.view(torch.float8_e4m3fn).float().numpy()
    got = np.array([L.btb_oracle_f8_value(i) for i in range(256)], np.float32)
    nan = np.isnan(want)
    assert set(np.nonzero(nan)[0]) == {0x7F, 0xFF} and np.all(np.isnan(got[nan]))
    assert np.array_equal(f32_bits(got[~nan]), f32_bits(want[~nan]))
    assert got[0x7E] == 448.0 and got[0x01] == 1 / 512
    assert np.array_equal(f32_bits(codecs.e4m3_decode(b.numpy())[~nan]), f32_bits(want[~nan]))


def test_round_bf16_against_torch_and_ties():
    L = oracle.lib()
    assert L.btb_oracle_round_bf16(1 + 2.0**-8) == 1.0              # tie to even: down
    assert L.btb_oracle_round_bf16(1 + 3 * 2.0**-8) == 1 + 2.0**-6  # tie to even: up
    v = torch.randn(100_000, generator=torch.Generator().manual_seed(7)) * 37.0
    want = v.to(torch.bfloat16).float().numpy()
    got = codecs.round_bf16(v.numpy())
    assert np.array_equal(f32_bits(got), f32_bits(want))
    some = v.numpy()[:2000]
    assert all(L.btb_oracle_round_bf16(float(s)) == w for s, w in zip(some, want[:2000]))


@pytest.mark.parametrize("rows,cols,grid", [(32, 64, (2, 2)), (48, 111 * 3, (3, 3)), (16, 256, (1, 1)), (8, 37, (8, 37))])
def test_fp8_widen_and_gemv(rows, cols, grid):
    rng = np.random.default_rng(rows + cols)
    q = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0x3C  # no NaN bytes
    scales = (rng.random(grid, dtype=np.float32) * 0.01 + 1e-4).astype(np.float32)
    held = oracle.widen_fp8(q, scales)
    want = torch.from_numpy(q).view(torch.float8_e4m3fn).float().reshape(grid[0], rows // grid[0], grid[1],
                                                                          cols // grid[1])
    want = (want * torch.from_numpy(scales).reshape(grid[0], 1, grid[1], 1)).to(torch.bfloat16).float()
    assert np.array_equal(f32_bits(held), f32_bits(want.reshape(rows, cols).numpy()))
    assert np.array_equal(f32_bits(held), f32_bits(codecs.fp8_held(q, scales)))
    x = rng.standard_normal((3, cols)).astype(np.float32)
    y = oracle.gemv_fp8(q, scales, x, threads=2)
    assert conditioned_err(y, held.astype(np.float64), x.astype(np.float64)) < 1e-6
    # the FP8 matvec is the bf16 matvec over the held matrix, bit for bit
    hb = (f32_bits(held) >> 16).astype(np.uint16)
    assert np.array_equal(f32_bits(y), f32_bits(oracle.gemv_bf16(hb, x)))


# -- error codes (native/src/gemv.rs:5075-5110; native/tests/gemv.rs:413-580) ---------------------------------------------


def test_error_codes():
    L = oracle.lib()
    w = np.zeros((4, 8), np.uint16)
    x = np.zeros((1, 8), np.float32)
    y = np.full((1, 4), 7.0, np.float32)
    P = lambda a: ctypes.c_void_p(a.ctypes.data)
    assert L.btb_gemv_bf16_rows(None, 4, 8, P(x), 1, P(y), 1) == oracle.ERR_NULL
    assert L.btb_gemv_bf16_rows(P(w), 0, 8, P(x), 1, P(y), 1) == oracle.ERR_DOMAIN
    assert L.btb_gemv_bf16_rows(P(w), 4, 8, P(x), 1, P(y), 1025) == oracle.ERR_DOMAIN
    assert L.btb_gemv_bf16_rows(P(w), 1 << 62, 8, P(x), 1, P(y), 1) == oracle.ERR_DOMAIN
    assert L.btb_gemv_bf16_rows(P(w), 4, 8, ctypes.c_void_p(x.ctypes.data + 2), 1, P(y), 1) == oracle.ERR_DOMAIN
    assert L.btb_gemv_bf16_rows(None, 0, 8, P(x), 1, P(y), 1) == oracle.ERR_NULL  # null before domain
    assert np.all(y == 7.0)  # a refused call writes nothing
    lo, hi4, tab = np.zeros(32, np.uint8), np.zeros(16, np.uint8), np.zeros(16, np.uint8)
    ev = np.zeros(2, np.uint8)
    for bad in ([5, 5], [9, 3], [0, 32], [-1, 4]):
        ei = np.array(bad, np.int32)
        assert L.btb_gemv_p12_rows(P(lo), P(hi4), P(tab), P(ei), P(ev), 2, 4, 8, P(x), 1, P(y), 1) == oracle.ERR_DOMAIN
    assert L.btb_gemv_p12_rows(P(lo), P(hi4), P(tab), None, None, 2, 4, 8, P(x), 1, P(y), 1) == oracle.ERR_NULL
    assert L.btb_gemv_mxfp4_rows(P(lo), P(tab), 4, 24, P(x), 1, P(y), 1) == oracle.ERR_DOMAIN  # cols % 32
    sc = np.ones((3, 1), np.float32)
    assert L.btb_gemv_fp8_rows(P(lo), P(sc), 4, 8, 3, 1, P(x), 1, P(y), 1) == oracle.ERR_DOMAIN  # 3 does not divide 4
    assert np.all(y == 7.0)
