"""The device twins of the crate's CPU entry points (f32 x and y, the host's order) against the CPU oracle: BIT-EXACT,
for every stored form, batch width and ragged shape - the reference's own law for its lane16 card kernels
(tests/kernels/test_mx4_lane16.py:29-60: "card == host bits")."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from btb_amd import fp8, mxfp4
from btb_amd.pack12 import P12Weight
from oracle import codecs

from .helpers import bits16, f32_bits, weights_bf16

pytestmark = pytest.mark.gpu


def xs(b: int, cols: int, seed: int) -> torch.Tensor:
    return torch.randn(b, cols, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("rows,cols", [(128, 2048), (67, 1100), (16, 16), (5, 33), (1, 1), (1536, 2048)])
@pytest.mark.parametrize("b", [1, 2, 3, 5, 8, 9])
def test_bf16_rows_bits(card, rows, cols, b):
    w = weights_bf16(rows, cols, seed=400, std=1.0)
    x = xs(b, cols, 401)
    got = card.gemv_lane16(w.cuda(), x.cuda()).cpu().numpy()
    want = oracle.gemv_bf16(bits16(w), x.numpy(), threads=0)
    assert np.array_equal(f32_bits(got), f32_bits(want))


@pytest.mark.parametrize("rows,cols", [(64, 512), (9, 1040), (3, 16)])
def test_p12_rows_bits(card, rows, cols):
    w = weights_bf16(rows, cols, seed=410)
    wb = bits16(w).copy().reshape(-1)
    at = np.arange(0, wb.size, max(1, wb.size // 101))
    wb[at] = (wb[at] & 0x00FF) | ((0x30 + np.arange(at.size) % 24).astype(np.uint16) << 8)
    w = torch.from_numpy(wb.view(np.int16).reshape(rows, cols)).view(torch.bfloat16)
    pw = P12Weight.pack(w.cuda(), card)
    assert pw.esc_idx.numel() > 0
    x = xs(3, cols, 411)
    got = card.gemv_lane16_p12(pw, x.cuda()).cpu().numpy()
    want = oracle.gemv_p12(*codecs.pack12_pack(wb), rows, cols, x.numpy(), threads=0)
    assert np.array_equal(f32_bits(got), f32_bits(want))
    # ... which is the bf16 matvec's bits (native/tests/gemv.rs:297-299)
    assert np.array_equal(f32_bits(got), f32_bits(card.gemv_lane16(w.cuda(), x.cuda()).cpu().numpy()))


@pytest.mark.parametrize("rows,cols", [(2880, 2880 // 32 * 32), (64, 256), (5, 32)])
@pytest.mark.parametrize("b", [1, 4])
def test_mxfp4_rows_bits(card, rows, cols, b):
    rng = np.random.default_rng(rows)
    blocks = rng.integers(0, 256, (rows, cols // 32, 16), dtype=np.uint8)
    scales = rng.integers(0, 255, (rows, cols // 32), dtype=np.uint8)  # subnormal scales included
    scales[:, ::3] = rng.integers(118, 132, scales[:, ::3].shape, dtype=np.uint8)
    x = xs(b, cols, 421)
    w = mxfp4.MxWeight(torch.from_numpy(blocks).reshape(-1).cuda(), torch.from_numpy(scales).reshape(-1).cuda(), rows, cols)
    got = card.gemv_lane16_mx4(w, x.cuda()).cpu().numpy()
    want = oracle.gemv_mxfp4(blocks, scales, rows, cols, x.numpy(), threads=0)
    same = f32_bits(got) == f32_bits(want)
    assert np.all(same | (np.isnan(got) & np.isnan(want)))


@pytest.mark.parametrize("rows,cols", [(1, 32), (17, 1024), (33, 2880)])
@pytest.mark.parametrize("b", [1, 3, 16])
def test_mxfp4_ggml_rows_bits(card, rows, cols, b):
    """`btb_gemv_mxfp4_ggml_rows` on the device: the oracle's bits, which are the checkpoint layout's for the same
    weights (native/src/gemv.rs:5215-5250)"""
    from .helpers import mx4_ggml

    rng = np.random.default_rng(rows + b)
    blocks = rng.integers(0, 256, (rows, cols // 32, 16), dtype=np.uint8)
    scales = rng.integers(0, 255, (rows, cols // 32), dtype=np.uint8)
    raw = mx4_ggml(blocks, scales)
    x = xs(b, cols, 423)
    got = card.gemv_lane16_mx4_ggml(torch.from_numpy(raw).cuda(), rows, cols, x.cuda()).cpu().numpy()
    want = oracle.gemv_mxfp4_ggml(raw, rows, cols, x.numpy(), threads=0)
    assert np.all((f32_bits(got) == f32_bits(want)) | (np.isnan(got) & np.isnan(want)))
    w = mxfp4.MxWeight(torch.from_numpy(blocks).reshape(-1).cuda(), torch.from_numpy(scales).reshape(-1).cuda(), rows, cols)
    other = card.gemv_lane16_mx4(w, x.cuda()).cpu().numpy()
    assert np.all((f32_bits(got) == f32_bits(other)) | (np.isnan(got) & np.isnan(other)))


@pytest.mark.parametrize("rows,cols,block", [(256, 512, (128, 128)), (48, 111, (16, 37)), (8, 64, (8, 64))])
def test_fp8_rows_bits(card, rows, cols, block):
    src = weights_bf16(rows, cols, seed=430).float()
    q, s = fp8.quantize(src, block)
    x = xs(3, cols, 431)
    w = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), rows, cols)
    got = card.gemv_lane16_fp8(w, x.cuda()).cpu().numpy()
    want = oracle.gemv_fp8(q.view(torch.uint8).numpy(), s.numpy(), x.numpy(), threads=0)
    assert np.array_equal(f32_bits(got), f32_bits(want))


def test_group_equals_single_calls_and_refusals(card):
    L = card.lib
    shapes = [(12, 64), (5, 48), (33, 512)]
    ws = [weights_bf16(r, c, 440 + i).cuda() for i, (r, c) in enumerate(shapes)]
    x = [xs(2, c, 450 + i).cuda() for i, (_, c) in enumerate(shapes)]
    y = [torch.zeros(2, r, device="cuda") for r, _ in shapes]
    n = len(shapes)
    P, S = ctypes.c_void_p * n, ctypes.c_size_t * n
    rows, cols, bs = S(*[r for r, _ in shapes]), S(*[c for _, c in shapes]), S(*[2] * n)
    assert L.btb_hip_gemv_bf16_group(n, P(*[t.data_ptr() for t in ws]), rows, cols, P(*[t.data_ptr() for t in x]), bs,
                                     P(*[t.data_ptr() for t in y]), None) == 0
    for w, xi, yi in zip(ws, x, y):
        assert torch.equal(yi.view(torch.int32), card.gemv_lane16(w, xi).view(torch.int32))
    # a bad task anywhere refuses the whole call before anything is launched
    before = [t.clone() for t in y]
    bad = S(12, 0, 33)
    assert L.btb_hip_gemv_bf16_group(n, P(*[t.data_ptr() for t in ws]), bad, cols, P(*[t.data_ptr() for t in x]), bs,
                                     P(*[t.data_ptr() for t in y]), None) == -6
    assert L.btb_hip_gemv_bf16_group(0, None, None, None, None, None, None, None) == -1
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(before, y))
    w0, x0, y0 = ws[0], x[0], y[0]
    assert L.btb_hip_gemv_bf16_rows(card.ptr(ctypes.c_void_p, w0), 12, 64, ctypes.c_void_p(x0.data_ptr() + 2), 2, card.ptr(ctypes.c_void_p, y0), None) == -6
    assert L.btb_hip_gemv_bf16_rows(None, 0, 64, card.ptr(ctypes.c_void_p, x0), 2, card.ptr(ctypes.c_void_p, y0), None) == -1


@pytest.mark.parametrize("rows,cols", [(128, 2048), (67, 1100)])
@pytest.mark.parametrize("b", [1, 8, 17])
def test_bf16_rows_at_an_odd_address_and_width(card, rows, cols, b):
    """the reference's sweep moves every pointer by one element and takes 17 vectors (native/tests/gemv.rs:20-45,
    262-329): the bits do not move - here the matrix one element off a 16-byte boundary leaves the wide-load kernel
    for the element-load one, which must give the very same bits"""
    w = weights_bf16(rows, cols, seed=440, std=1.0)
    x = xs(b, cols, 441)
    want = oracle.gemv_bf16(bits16(w), x.numpy(), threads=0)
    wbuf = torch.zeros(rows * cols + 1, dtype=torch.bfloat16, device="cuda")
    wbuf[1:] = w.reshape(-1).cuda()
    xbuf = torch.zeros(b * cols + 1, dtype=torch.float32, device="cuda")
    xbuf[1:] = x.reshape(-1).cuda()
    ybuf = torch.zeros(b * rows + 1, dtype=torch.float32, device="cuda")
    rc = card.lib.btb_hip_gemv_bf16_rows(ctypes.c_void_p(wbuf.data_ptr() + 2), rows, cols,
                                         ctypes.c_void_p(xbuf.data_ptr() + 4), b, ctypes.c_void_p(ybuf.data_ptr() + 4),
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    got = ybuf[1:].reshape(b, rows).cpu().numpy()
    assert np.array_equal(f32_bits(got), f32_bits(want))
    assert np.array_equal(f32_bits(card.gemv_lane16(w.cuda(), x.cuda()).cpu().numpy()), f32_bits(want))
