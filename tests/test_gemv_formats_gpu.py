"""The fused widen + matvec of the three stored forms on the GPU against the CPU oracle's matvec over the same bytes.

Bar: max |y_gpu - y_ref| / max |y_ref| <= 1e-2 on bf16 outputs (both sides accumulate in f32; the widened weights are
bit-identical - tests/test_widen_gpu.py - so only the order of the f32 additions and the final bf16 rounding differ),
and the reference card's own bar of one bf16 ulp of the largest output.
"""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from btb_amd import fp8, mxfp4, pack12
from btb_amd.pack12 import P12Weight
from oracle import codecs

from .helpers import acts_bf16, bits16, weights_bf16

pytestmark = pytest.mark.gpu


def check(y: torch.Tensor, ref_f32: np.ndarray) -> None:
    ref = codecs.round_bf16(ref_f32)
    got = y.float().cpu().numpy()
    peak = np.abs(ref).max()
    err = np.abs(got - ref).max()
    assert err <= 1e-2 * peak and err <= peak * 2.0**-7, (err, peak)


@pytest.mark.parametrize("R,C", [(9728, 2560), (2560, 9728), (2560, 4096), (2048, 768), (100, 272), (5, 16)])
@pytest.mark.parametrize("M", [1, 3])
def test_gemv_p12(card, R, C, M):
    w = weights_bf16(R, C, seed=300)
    wb = bits16(w).copy().reshape(-1)
    at = np.arange(0, wb.size, max(1, wb.size // 2003))  # forced escapes on top of the natural ones
    wb[at] = (wb[at] & 0x00FF) | ((0x30 + np.arange(at.size) % 24).astype(np.uint16) << 8)
    w = torch.from_numpy(wb.view(np.int16).reshape(R, C)).view(torch.bfloat16)
    x = acts_bf16(M, C, seed=301)
    pw = P12Weight.pack(w.cuda(), card)
    assert pw.esc_idx.numel() > 0
    y = card.gemv_p12(pw, x.cuda())
    packed = codecs.pack12_pack(wb)
    ref = oracle.gemv_p12(*packed, R, C, x.float().numpy(), threads=0)
    check(y, ref)
    # the packed matvec and the bf16 matvec over the unpacked matrix agree to the same bar (the CPU pair is bit-equal)
    check(card.gemv(w.cuda(), x.cuda()), ref)


def test_gemv_p12_no_escapes(card):
    R, C = 64, 512
    w = (weights_bf16(R, C, seed=302).float().clamp(0.011, 0.03)).to(torch.bfloat16)  # few high bytes: no escapes
    pw = P12Weight.pack(w.cuda(), card)
    assert pw.esc_idx.numel() == 0
    x = acts_bf16(8, C, seed=303)
    ref = oracle.gemv_bf16(bits16(w), x.float().numpy())
    check(card.gemv_p12(pw, x[:2].contiguous().cuda()), ref[:2])
    check(card.gemv_p12(pw, x.cuda()), ref)  # eight rows: the matrix-core kernel, whose escape lists are null here


@pytest.mark.parametrize("R,C,block", [(2048, 7168, (128, 128)), (512, 1024, (128, 128)), (64, 256, (16, 16)),
                                       (48, 96, (48, 96))])
@pytest.mark.parametrize("M", [1, 4])
def test_gemv_fp8(card, R, C, block, M):
    src = weights_bf16(R, C, seed=310).float()
    q, s = fp8.quantize(src, block)
    x = acts_bf16(M, C, seed=311)
    w = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), R, C)
    y = card.gemv_fp8(w, x.cuda())
    ref = oracle.gemv_fp8(q.view(torch.uint8).numpy(), s.numpy(), x.float().numpy(), threads=0)
    check(y, ref)


@pytest.mark.parametrize("R,C", [(2048, 7168), (1536, 2048), (2048, 768), (24, 64), (3, 32)])
@pytest.mark.parametrize("M", [1, 4])
def test_gemv_mxfp4(card, R, C, M):
    src = weights_bf16(R, C, seed=320).float()
    blocks, scales = mxfp4.quantize(src)
    x = acts_bf16(M, C, seed=321)
    w = mxfp4.MxWeight(blocks.reshape(-1).cuda(), scales.reshape(-1).cuda(), R, C)
    y = card.gemv_mx4(w, x.cuda())
    ref = oracle.gemv_mxfp4(blocks.numpy(), scales.numpy(), R, C, x.float().numpy(), threads=0)
    check(y, ref)


@pytest.mark.parametrize("form,R,C", [("bf16", 2560, 4096), ("bf16", 2560, 9728), ("p12", 2560, 4096), ("p12", 2560, 9728),
                                      ("mxfp4", 9216, 2048), ("bf16", 2304, 1024)])
def test_the_grid_changes_no_bit(card, form, R, C):
    """how a launch is cut over the CUs - workgroups of five waves where four leave the CUs uneven, a tile more a wave
    where that fills the turns evenly - is the launch's own business: with either choice switched off (knobs
    gemv_five_waves, gemv_even_grid) the one-row matvec gives the same bits"""
    x = acts_bf16(1, C, seed=402).cuda()
    if form == "bf16":
        w = weights_bf16(R, C, seed=401).cuda()
        run = lambda: card.gemv(w, x)
    elif form == "p12":
        pw = P12Weight.pack(weights_bf16(R, C, seed=401).cuda(), card)
        run = lambda: card.gemv_p12(pw, x)
    else:
        blocks, scales = mxfp4.quantize(weights_bf16(R, C, seed=401).float())
        mw = mxfp4.MxWeight(blocks.reshape(-1).cuda(), scales.reshape(-1).cuda(), R, C)
        run = lambda: card.gemv_mx4(mw, x)
    want = run()
    try:
        for knob in ("gemv_five_waves", "gemv_even_grid"):
            card.set_tuning(knob, 0)
            got = run()
            card.set_tuning(knob, -1)
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), knob
    finally:
        card.set_tuning("gemv_five_waves", -1)
        card.set_tuning("gemv_even_grid", -1)


def test_format_refusals(card):
    L = card.lib
    z = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    x = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    s = torch.ones(16, dtype=torch.float32, device="cuda")
    p = lambda t: card.ptr(ctypes.c_void_p, t)
    assert L.btb_hip_gemv_mxfp4(p(z), p(z), p(x), p(y), 4, 48, 1, None) == -6          # C % 32
    assert L.btb_hip_gemv_mxfp4(None, p(z), p(x), p(y), 4, 64, 1, None) == -1
    assert L.btb_hip_gemv_fp8(p(z), p(s), 3, 1, p(x), p(y), 4, 64, 1, None) == -6       # 3 does not divide 4
    assert L.btb_hip_gemv_fp8(p(z), p(s), 1, 8, p(x), p(y), 4, 64, 1, None) == -6       # 8-column blocks: not 16
    assert L.btb_hip_gemv_p12(p(z), p(z), p(z), None, None, None, 2, p(s), None, p(x), p(y), 4, 64, 1, None) == -1
    assert L.btb_hip_gemv_p12(p(z), p(z), p(z), None, None, None, 0, p(s), None, p(x), p(y), 4, 60, 1, None) == -6  # C % 16


# ---- the verify widths (M >= 8): FP8 and MXFP4 widened into bf16 fragments for the matrix cores -------------------

def _width_law(card, op, w, x, ref):
    """the bar against the oracle at the full width; rows of an 8-row pass are the rows of the wide pass bit for bit
    (native/cuda/btb_kernels.cu:84-88 for the family of tensor-core passes); the vector-ALU passes of the same rows
    stay within the same bar of the matrix-core pass"""
    y = op(w, x)
    check(y, ref)
    y8 = op(w, x[:8].contiguous())
    assert torch.equal(y8.view(torch.int16), y[:8].view(torch.int16))
    y5 = op(w, x[:5].contiguous())  # the narrowest pass the matrix cores take
    assert torch.equal(y5.view(torch.int16), y[:5].view(torch.int16))
    card.set_tuning("gemv_no_mfma", 1)
    try:
        v = op(w, x)
    finally:
        card.set_tuning("gemv_no_mfma", -1)
    check(v, ref)
    peak = float(y.float().abs().max())
    assert float((v.float() - y.float()).abs().max()) <= peak * 2.0**-7
    # two to four rows: large block-scaled matrices go to the matrix cores from two or three rows on, the others stay
    # on the vector kernels; whichever family takes the pass, its rows are that family's rows, bit for bit
    for m in (2, 3, 4):
        ym = op(w, x[:m].contiguous())
        check(ym, ref[:m])
        matrix = torch.equal(ym.view(torch.int16), y[:m].view(torch.int16))
        vector = torch.equal(ym.view(torch.int16), v[:m].view(torch.int16))
        assert matrix or vector, m
    card.set_tuning("gemv_mfma_from", 5)  # every form's threshold back at five rows: the vector family to four
    try:
        y4 = op(w, x[:4].contiguous())
    finally:
        card.set_tuning("gemv_mfma_from", -1)
    assert torch.equal(y4.view(torch.int16), v[:4].view(torch.int16))


@pytest.mark.parametrize("R,C,block", [(18432, 7168, (128, 128)), (2048, 7168, (128, 128)), (512, 1024, (128, 128)),
                                       (1024, 2560, (128, 128)), (64, 256, (16, 16)), (50, 96, (50, 96)),
                                       (256, 9728, (128, 128))])
@pytest.mark.parametrize("M", [8, 16, 12])
def test_gemv_fp8_verify_widths(card, R, C, block, M):
    """config C5a at its full shape and at shapes that take each of the matrix-core kernel's forms (rows of 2, 4, 8
    waves; the wide form; rows past 7168 columns, whose x fragments are streamed) and its fall-backs (rows not a
    multiple of 16)"""
    src = weights_bf16(R, C, seed=330).float()
    q, s = fp8.quantize(src, block)
    x = acts_bf16(M, C, seed=331)
    w = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), R, C)
    ref = oracle.gemv_fp8(q.view(torch.uint8).numpy(), s.numpy(), x.float().numpy(), threads=0)
    _width_law(card, card.gemv_fp8, w, x.cuda(), ref)


@pytest.mark.parametrize("R,C", [(18432, 7168), (2048, 7168), (1536, 2048), (2048, 768), (1024, 2560), (24, 64), (48, 32),
                                 (256, 9728)])
@pytest.mark.parametrize("M", [8, 16, 12])
def test_gemv_mxfp4_verify_widths(card, R, C, M):
    """config C5b at its full shape, the MoE expert shapes, and small shapes"""
    src = weights_bf16(R, C, seed=340).float()
    blocks, scales = mxfp4.quantize(src)
    x = acts_bf16(M, C, seed=341)
    w = mxfp4.MxWeight(blocks.reshape(-1).cuda(), scales.reshape(-1).cuda(), R, C)
    ref = oracle.gemv_mxfp4(blocks.numpy(), scales.numpy(), R, C, x.float().numpy(), threads=0)
    _width_law(card, card.gemv_mx4, w, x.cuda(), ref)


@pytest.mark.parametrize("form,block", [("fp8", (128, 128)), ("fp8", (64, 256)), ("fp8", (16, 32)), ("mxfp4", None)])
@pytest.mark.parametrize("M", [5, 16, 24, 33])
def test_long_rows_straight_into_lds(card, form, block, M):
    """Rows of 7168 columns at the verify widths take the kernel whose weights go from memory straight into LDS
    (sixteen rows of x a pass, so 24 and 33 are two and three passes, the last of 8 and of 1): against the oracle,
    against the staged kernel it replaces (knob mfma_direct = 0; the two differ in f32 summation order only), and a
    row's bits do not depend on which pass or which other rows it came with."""
    R, C = 9728, 7168  # 608 tiles: three turns of a grid of 203 workgroups, the last of which has two
    src = weights_bf16(R, C, seed=350).float()
    x = acts_bf16(M, C, seed=351)
    if form == "fp8":
        q, s = fp8.quantize(src, block)
        w = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), R, C)
        ref = oracle.gemv_fp8(q.view(torch.uint8).numpy(), s.numpy(), x.float().numpy(), threads=0)
        op = card.gemv_fp8
    else:
        blocks, scales = mxfp4.quantize(src)
        w = mxfp4.MxWeight(blocks.reshape(-1).cuda(), scales.reshape(-1).cuda(), R, C)
        ref = oracle.gemv_mxfp4(blocks.numpy(), scales.numpy(), R, C, x.float().numpy(), threads=0)
        op = card.gemv_mx4
    xg = x.cuda()
    y = op(w, xg)
    check(y, ref)
    card.set_tuning("mfma_direct", 0)
    try:
        staged = op(w, xg)
    finally:
        card.set_tuning("mfma_direct", -1)
    check(staged, ref)
    peak = float(y.float().abs().max())
    assert float((staged.float() - y.float()).abs().max()) <= peak * 2.0**-7
    last = op(w, xg[M - 5:].contiguous())  # the last five rows in a pass of their own (the narrowest wide pass)
    assert torch.equal(last.view(torch.int16), y[M - 5:].view(torch.int16))
    assert torch.equal(op(w, xg).view(torch.int16), y.view(torch.int16))  # and the same bits every time


@pytest.mark.parametrize("R,C", [(9728, 2560), (320, 4096), (208, 9728), (256, 3200), (144, 9216), (96, 10752)])
@pytest.mark.parametrize("M,crowd", [(5, False), (16, False), (21, True)])
def test_packed_rows_straight_into_lds(card, R, C, M, crowd):
    """12-bit rows of the lengths the direct-to-LDS kernel has shapes for - 2560 (ten waves), 3073..4096 (eight) and
    9217..10752 columns (seven, sub-blocks of 256 columns); 3200, 9216 and 9728 leave some waves without a last
    sub-block - at the verify widths: against the oracle, against the staged kernel it replaces (knob mfma_direct = 0;
    the two differ in f32 summation order only), a row's bits whatever pass it came with, the same bits every time.
    `crowd`: high bytes spread over far more than fifteen values, so that a tile's escapes are many times the
    thirty-two its escape wave takes at once; otherwise the natural handful, with tiles that have none."""
    g = torch.Generator().manual_seed(390 + M)
    if crowd:
        w = (torch.randn(R, C, generator=g) * torch.exp2(torch.randint(-12, 4, (R, C), generator=g).float())).to(torch.bfloat16)
    else:
        w = weights_bf16(R, C, seed=391)
    pw = P12Weight.pack(w.cuda(), card)
    assert (pw.esc_idx.numel() > R * C // 10) if crowd else (0 < pw.esc_idx.numel() < R * C // 100)
    x = acts_bf16(M, C, seed=392)
    ref = oracle.gemv_bf16(bits16(w), x.float().numpy())  # the packed matrix is the bf16 matrix, bit for bit
    xg = x.cuda()
    y = card.gemv_p12(pw, xg)
    check(y, ref)
    card.set_tuning("mfma_direct", 0)
    try:
        staged = card.gemv_p12(pw, xg)
    finally:
        card.set_tuning("mfma_direct", -1)
    check(staged, ref)
    peak = float(y.float().abs().max())
    assert float((staged.float() - y.float()).abs().max()) <= peak * 2.0**-7
    last = card.gemv_p12(pw, xg[M - 5:].contiguous())
    assert torch.equal(last.view(torch.int16), y[M - 5:].view(torch.int16))
    assert torch.equal(card.gemv_p12(pw, xg).view(torch.int16), y.view(torch.int16))


@pytest.mark.parametrize("form", ["fp8", "mxfp4"])
@pytest.mark.parametrize("R,C", [(4864, 2560), (320, 4096), (208, 9728), (256, 3584), (96, 10752), (144, 9216)])
@pytest.mark.parametrize("M", [7, 19])
def test_block_scaled_rows_of_the_models_lengths_straight_into_lds(card, form, R, C, M):
    """the direct-to-LDS kernel's other row lengths for the block-scaled forms - 2560, up to 4096, around 9728 columns;
    3584 and 9216 / 9728 leave some waves without a last sub-block: against the oracle, the staged kernel, and a
    row's bits whatever pass it came with (19 rows: a pass of 16 and one of 3)"""
    src = weights_bf16(R, C, seed=370).float()
    x = acts_bf16(M, C, seed=371)
    if form == "fp8":
        q, s = fp8.quantize(src, (16, 128) if R % 128 else (128, 128))
        w = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), R, C)
        ref = oracle.gemv_fp8(q.view(torch.uint8).numpy(), s.numpy(), x.float().numpy(), threads=0)
        op = card.gemv_fp8
    else:
        blocks, scales = mxfp4.quantize(src)
        w = mxfp4.MxWeight(blocks.reshape(-1).cuda(), scales.reshape(-1).cuda(), R, C)
        ref = oracle.gemv_mxfp4(blocks.numpy(), scales.numpy(), R, C, x.float().numpy(), threads=0)
        op = card.gemv_mx4
    xg = x.cuda()
    y = op(w, xg)
    check(y, ref)
    card.set_tuning("mfma_direct", 0)
    try:
        staged = op(w, xg)
    finally:
        card.set_tuning("mfma_direct", -1)
    check(staged, ref)
    peak = float(y.float().abs().max())
    assert float((staged.float() - y.float()).abs().max()) <= peak * 2.0**-7
    last = op(w, xg[M - 5:].contiguous())
    assert torch.equal(last.view(torch.int16), y[M - 5:].view(torch.int16))
    assert torch.equal(op(w, xg).view(torch.int16), y.view(torch.int16))


@pytest.mark.parametrize("form", ["fp8", "mxfp4"])
def test_long_rows_with_scales_of_every_size(card, form):
    """the direct-to-LDS kernel's scales travel through LDS by loads of their own: random bytes under scales that differ
    from block to block by factors up to 2^40 (MXFP4: e8m0 bytes 107..147; FP8: f32 scales 2^-20..2^20, a zero scale
    and a negative one among them) against the oracle over the same bytes, at 16 rows and at 7 (one pass each)"""
    R, C = 1024, 7168
    rng = np.random.default_rng(380)
    x = acts_bf16(16, C, seed=381)
    if form == "fp8":
        q = rng.integers(0, 256, (R, C), dtype=np.uint8)
        q[(q & 0x7F) == 0x7F] = 0x3C  # no NaN bytes: e4m3fn has no infinities, 0x7F / 0xFF are its NaNs
        sc = np.exp2(rng.integers(-20, 21, (R // 128, C // 128))).astype(np.float32) * rng.uniform(1.0, 2.0, (R // 128, C // 128)).astype(np.float32)
        sc[1, 3] = 0.0
        sc[2, 5] = -sc[2, 5]
        w = fp8.F8Weight(torch.from_numpy(q).cuda(), torch.from_numpy(sc).cuda(), R, C)
        ref = oracle.gemv_fp8(q, sc, x.float().numpy(), threads=0)
        op = card.gemv_fp8
    else:
        blocks = rng.integers(0, 256, (R, C // 32, 16), dtype=np.uint8)
        scales = rng.integers(107, 148, (R, C // 32), dtype=np.uint8)
        w = mxfp4.MxWeight(torch.from_numpy(blocks).reshape(-1).cuda(), torch.from_numpy(scales).reshape(-1).cuda(), R, C)
        ref = oracle.gemv_mxfp4(blocks, scales, R, C, x.float().numpy(), threads=0)
        op = card.gemv_mx4
    xg = x.cuda()
    y = op(w, xg)
    # weight rows of very different size: each weight row's sixteen outputs are held to 2^-6 of the largest of them
    # (two bf16 ulps: the f32 sums run in another order than the oracle's, and blocks 2^40 apart cancel little)
    got = y.float().cpu().numpy()
    want = codecs.round_bf16(ref)
    assert np.all(np.isfinite(want)) and np.all(np.isfinite(got))
    peak = np.abs(want).max(axis=0, keepdims=True)  # per weight row, over the x rows
    assert np.all(np.abs(got - want) <= 2.0**-6 * np.maximum(peak, 1e-30)), float((np.abs(got - want) / np.maximum(peak, 1e-30)).max())
    y7 = op(w, xg[:7].contiguous())
    assert torch.equal(y7.view(torch.int16), y[:7].view(torch.int16))


@pytest.mark.parametrize("form", ["fp8", "mxfp4"])
def test_full_shape_one_row_and_linearity(card, form):
    """C5 at M = 1 on the full [18432, 7168] matrix against the oracle, and a size-independent property on top: the
    matvec is linear in x up to the output's rounding - y(x1) + y(x2) against y over the f32 sum, each within the bar"""
    R, C = 18432, 7168
    src = weights_bf16(R, C, seed=350).float()
    x = acts_bf16(2, C, seed=351)
    if form == "fp8":
        q, s = fp8.quantize(src, (128, 128))
        w = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), R, C)
        op = card.gemv_fp8
        ref = oracle.gemv_fp8(q.view(torch.uint8).numpy(), s.numpy(), x.float().numpy(), threads=0)
    else:
        blocks, scales = mxfp4.quantize(src)
        w = mxfp4.MxWeight(blocks.reshape(-1).cuda(), scales.reshape(-1).cuda(), R, C)
        op = card.gemv_mx4
        ref = oracle.gemv_mxfp4(blocks.numpy(), scales.numpy(), R, C, x.float().numpy(), threads=0)
    y1 = op(w, x[:1].contiguous().cuda())
    check(y1, ref[:1])
    both = op(w, x.cuda())
    check(both, ref)
    if form == "fp8":  # two rows of FP8 stay on the vector kernel: row 0 of the 2-row pass has the one-row pass's bits
        assert torch.equal(both[:1].view(torch.int16), y1.view(torch.int16))
    else:  # two rows of MXFP4 on a matrix this large go to the matrix cores: the rows of an 8-row pass, bit for bit
        y8 = op(w, torch.cat([x, acts_bf16(6, C, seed=352)]).cuda())
        assert torch.equal(both.view(torch.int16), y8[:2].view(torch.int16))
        assert not torch.equal(both[:1].view(torch.int16), y1.view(torch.int16))  # (and so not the vector kernel's)
    total = both.float().sum(dim=0).cpu().numpy()
    want = ref.sum(axis=0)
    assert np.abs(total - want).max() <= 1e-2 * np.abs(want).max()


@pytest.mark.parametrize("R,C", [(9728, 2560), (2560, 4096), (1024, 7168), (2048, 768), (64, 256), (50, 96),
                                 (2560, 9728)])
@pytest.mark.parametrize("M", [8, 16, 12, 24])
def test_gemv_p12_verify_widths(card, R, C, M):
    """12-bit matrices at the verify widths: the matrix-core kernel's forms (rows of 2, 4, 8 waves; the wide form; two
    tiles of x rows at M = 24) and its fall-back (rows not a multiple of 16), with escapes forced on top of the natural
    ones so that every 16-row tile holds some"""
    w = weights_bf16(R, C, seed=360)
    wb = bits16(w).copy().reshape(-1)
    at = np.arange(0, wb.size, max(1, wb.size // 4001))
    wb[at] = (wb[at] & 0x00FF) | ((0x30 + np.arange(at.size) % 24).astype(np.uint16) << 8)
    w = torch.from_numpy(wb.view(np.int16).reshape(R, C)).view(torch.bfloat16)
    pw = P12Weight.pack(w.cuda(), card)
    assert pw.esc_idx.numel() > 0
    x = acts_bf16(M, C, seed=361)
    ref = oracle.gemv_p12(*codecs.pack12_pack(wb), R, C, x.float().numpy(), threads=0)
    _width_law(card, card.gemv_p12, pw, x.cuda(), ref)


def test_gemv_p12_verify_width_many_escapes(card):
    """a matrix whose high bytes are spread over far more than fifteen values: a sixth of the weights are escapes, and
    the matrix-core pass still meets the bar against the matvec over the unpacked matrix"""
    R, C, M = 256, 1024, 8
    g = torch.Generator().manual_seed(362)
    w = (torch.randn(R, C, generator=g) * torch.exp2(torch.randint(-12, 4, (R, C), generator=g).float())).to(torch.bfloat16)
    pw = P12Weight.pack(w.cuda(), card)
    assert pw.esc_idx.numel() > R * C // 10
    x = acts_bf16(M, C, seed=363)
    y = card.gemv_p12(pw, x.cuda())
    check(y, oracle.gemv_bf16(bits16(w), x.float().numpy()))


@pytest.mark.parametrize("R,C", [(6144, 2560), (2560, 9728), (512, 4096), (96, 272), (64, 1024)])
@pytest.mark.parametrize("M,glu,wild", [(1, False, False), (1, True, False), (3, False, True), (2, True, True)])
def test_packed_norm_forms_with_the_pair_table_change_no_bit(card, R, C, M, glu, wild):
    """The add + norm matvecs over a pack12 matrix look the high bytes up in a 256-entry pair table in LDS; the plain
    packed matvec does the lookup in registers. The widened weights are the same bf16 values and the sums run in the
    same lane order, so: folded form == add_rmsnorm, then the plain packed matvec (then silu_mul), bit for bit; the
    same with the table switched off (knob p12_pair_table = 0); and within the bar of the oracle's matvec over the
    unpacked matrix. `wild`: high bytes spread over far more than fifteen values, a sixth of the weights escapes."""
    g = torch.Generator().manual_seed(370 + R + M)
    if wild:
        w = (torch.randn(R, C, generator=g) * torch.exp2(torch.randint(-12, 4, (R, C), generator=g).float())).to(torch.bfloat16)
    else:
        w = weights_bf16(R, C, seed=371 + R)
    pw = P12Weight.pack(w.cuda(), card)
    if wild:
        assert pw.esc_idx.numel() > R * C // 10
    h = acts_bf16(M, C, seed=372).cuda()
    y = acts_bf16(M, C, seed=373).cuda()
    nw = (1.0 + 0.1 * torch.randn(C, generator=g)).to(torch.bfloat16).cuda()
    h1, x1 = h.clone(), torch.empty_like(h)
    card.add_rmsnorm(h1, y, nw, 1e-6, x1)
    want = card.gemv_p12(pw, x1)
    if glu:
        half = torch.empty(M, R // 2, dtype=torch.bfloat16, device="cuda")
        card.silu_mul(want, half)
        want = half
    outs = []
    try:
        for knob in (-1, 0):
            card.set_tuning("p12_pair_table", knob)
            h2 = torch.empty_like(h)
            out = torch.empty(M, R // 2 if glu else R, dtype=torch.bfloat16, device="cuda")
            card.gemv_norm(pw, h, y, nw, 1e-6, h2, out, glu=glu)
            assert torch.equal(h2.view(torch.int16), h1.view(torch.int16))
            outs.append(out)
    finally:
        card.set_tuning("p12_pair_table", -1)
    assert torch.equal(outs[0].view(torch.int16), want.view(torch.int16))
    assert torch.equal(outs[1].view(torch.int16), want.view(torch.int16))
    if not glu:
        check(outs[0], oracle.gemv_bf16(bits16(w), x1.float().cpu().numpy()))


@pytest.mark.parametrize("packed", [False, True])
def test_the_head_shape(card, packed):
    """the largest matrix of the step, the [151936, 2560] head (778 MB of bf16), stored as bf16 and as 12 bits a weight:
    every logit against the oracle"""
    R, C = 151936, 2560
    w = weights_bf16(R, C, seed=370)
    x = acts_bf16(1, C, seed=371)
    ref = oracle.gemv_bf16(bits16(w), x.float().numpy())
    if packed:
        y = card.gemv_p12(P12Weight.pack(w.cuda(), card), x.cuda())
    else:
        y = card.gemv(w.cuda(), x.cuda())
    check(y, ref)


def test_pair_table_made_at_upload(card):
    """pairs[b] = table[b & 15] | table[b >> 4] << 8 with the escape code's slot taken as 0, whatever byte the store
    left in table[15]; the matrix's own table carries 0 there too"""
    table = torch.arange(16, dtype=torch.uint8) * 7 + 33
    table[15] = 0xFF
    got = card.p12_pairs(table.cuda()).cpu().numpy().view(np.uint16)
    t = table.numpy().astype(np.uint16).copy()
    t[15] = 0
    b = np.arange(256)
    assert np.array_equal(got, t[b & 15] | (t[b >> 4] << 8))
    w = weights_bf16(32, 64, seed=380)
    lo, hi4, tb, ei, ev = (t_.cuda() for t_ in pack12.pack_bf16(w))
    tb[15] = 0x7F
    pw = P12Weight(lo, hi4, tb, ei, ev, 32, 64, card)
    assert int(pw.table[15]) == 0 and int(tb[15]) == 0x7F and pw.pairs.numel() == 256   # its own copy, the caller's left


def escapes_in_rows(R, C, counts, seed):
    """a bf16 matrix whose row r holds counts[r % len(counts)] forced escapes (rare high bytes, low bytes of both
    halves) at scattered columns"""
    w = weights_bf16(R, C, seed=seed)
    wb = bits16(w).copy()
    rng = np.random.default_rng(seed)
    for r in range(R):
        k = counts[r % len(counts)]
        if k:
            cols = np.sort(rng.choice(C, size=k, replace=False))
            wb[r, cols] = (wb[r, cols] & 0x00FF) | ((0x20 + (np.arange(k) + r) % 40).astype(np.uint16) << 8)
    return torch.from_numpy(wb.view(np.int16)).view(torch.bfloat16)


@pytest.mark.parametrize("R,C,S", [(48, 272, 8), (40, 4096, 8), (24, 4112, 16)])
def test_rows_words_made_at_upload(card, R, C, S):
    """row_esc[r, k] = row r's escape k as (low byte, true high byte << 8, column << 16), 0x7FFF for the column where
    the row has no such escape, bit 31 of all the row's words where it has more than words (8 a row up to 4096
    columns, 16 beyond); rows too wide for a word's column field get none"""
    w = escapes_in_rows(R, C, [0, 1, 2, 8, 9, 17, 0, 3, 16, 20], seed=390)
    lo, hi4, tb, ei, ev = (t_.cuda() for t_ in pack12.pack_bf16(w))
    pw = P12Weight(lo, hi4, tb, ei, ev, R, C, card)
    got = pw.row_esc.cpu().numpy().view(np.uint32)
    idx, val, lob = ei.cpu().numpy().astype(np.int64), ev.cpu().numpy(), lo.cpu().numpy().reshape(-1)
    assert got.shape == (R, S)
    want = np.zeros((R, S), dtype=np.uint32)
    for r in range(R):
        mine = np.flatnonzero((idx >= r * C) & (idx < (r + 1) * C))
        for k in range(S):
            if k < mine.size:
                e = mine[k]
                want[r, k] = int(lob[idx[e]]) | (int(val[e]) << 8) | (int(idx[e] - r * C) << 16)
            else:
                want[r, k] = 0x7FFF << 16
        if mine.size > S:
            want[r] |= 0x80000000
    assert np.array_equal(got, want)
    assert (got[:, 0] >> 31).sum() > 0 and ((got[:, 0] >> 16) & 0x7FFF == 0x7FFF).sum() > 0   # both kinds of row met
    assert card.p12_row_esc(lo, ei, ev, pw.row_ptr, R, 40000) is None          # a column a word cannot hold
    L, p_ = card.lib, (lambda t: t.data_ptr())
    out = torch.empty(16 * R, dtype=torch.int32, device="cuda")
    assert L.btb_hip_p12_row_esc(p_(lo), p_(ei), p_(ev), ei.numel(), p_(pw.row_ptr), 1, 0x8000, p_(out), None) == -6
    assert L.btb_hip_p12_row_esc(None, p_(ei), p_(ev), ei.numel(), p_(pw.row_ptr), R, C, p_(out), None) == -1


@pytest.mark.parametrize("R,C", [(2560, 4096), (6144, 2560), (96, 272), (2560, 9728), (64, 1024)])
@pytest.mark.parametrize("M", [1, 2, 4])
def test_packed_matvec_with_the_rows_words_and_through_the_list(card, R, C, M):
    """a row's first four escapes come out of the row's own words, asked for ahead of its weights; a caller without
    them (row_esc NULL) walks the list: the same bits - with rows of none, one, eight, nine, sixteen and forty escapes, the plain
    matvec, the one with the residual add + norm folded in and its gate / up form - and the oracle's values"""
    w = escapes_in_rows(R, C, [0, 1, 0, 8, 9, 2, 40, 0, 1, 3, 16, 17], seed=391 + M)
    x = acts_bf16(M, C, seed=392).cuda()
    lo, hi4, tb, ei, ev = (t_.cuda() for t_ in pack12.pack_bf16(w))
    pw = P12Weight(lo, hi4, tb, ei, ev, R, C, card)
    assert pw.row_esc is not None and pw.esc_idx.numel() > R
    h = acts_bf16(M, C, seed=393).cuda()
    nw = (1.0 + 0.1 * torch.randn(C, generator=torch.Generator().manual_seed(394))).to(torch.bfloat16).cuda()
    def run():
        y = card.gemv_p12(pw, x)
        h2 = torch.empty_like(h)
        yn = card.gemv_norm(pw, h, x, nw, 1e-6, h2, torch.empty(M, R, dtype=torch.bfloat16, device="cuda"))
        yg = card.gemv_norm(pw, h, x, nw, 1e-6, torch.empty_like(h),
                            torch.empty(M, R // 2, dtype=torch.bfloat16, device="cuda"), glu=True)
        return y, yn, h2, yg
    with_words = run()
    words, pw.row_esc = pw.row_esc, None
    try:
        through_list = run()
    finally:
        pw.row_esc = words
    for a, b in zip(with_words, through_list):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    check(with_words[0], oracle.gemv_bf16(bits16(w), x.float().cpu().numpy(), threads=0))


@pytest.mark.parametrize("R,C", [(9728, 2560), (2560, 4096), (2560, 9728), (96, 272)])
@pytest.mark.parametrize("M", [1, 4, 8, 16])
def test_plain_packed_matvec_with_and_without_the_pair_table(card, R, C, M):
    """the plain packed matvec looks its high bytes up in the pair table too (brought into LDS from the copy made at
    upload); the in-register lookup (knob p12_pair_table = 0, or a caller without the table) gives the same bits. And a
    store whose unused table slot 15 holds 0xFF - where the streamed stand-in of an escaped weight would be NaN - gives
    the bits of the store that holds 0 there, at one row and at the matrix-core widths."""
    w = weights_bf16(R, C, seed=381)
    wb = bits16(w).copy().reshape(-1)
    at = np.arange(0, wb.size, max(1, wb.size // 1009))          # forced escapes, low bytes >= 0x80 among them
    wb[at] = (wb[at] & 0x00FF) | ((0x20 + np.arange(at.size) % 40).astype(np.uint16) << 8)
    w = torch.from_numpy(wb.view(np.int16).reshape(R, C)).view(torch.bfloat16)
    x = acts_bf16(M, C, seed=382).cuda()
    lo, hi4, tb, ei, ev = (t_.cuda() for t_ in pack12.pack_bf16(w))
    pw = P12Weight(lo, hi4, tb, ei, ev, R, C, card)
    assert pw.esc_idx.numel() >= 500
    y = card.gemv_p12(pw, x)
    try:
        card.set_tuning("p12_pair_table", 0)
        y0 = card.gemv_p12(pw, x)
        card.set_tuning("p12_pair_table", 1)
        y1 = card.gemv_p12(pw, x)
    finally:
        card.set_tuning("p12_pair_table", -1)
    assert torch.equal(y.view(torch.int16), y0.view(torch.int16)) and torch.equal(y.view(torch.int16), y1.view(torch.int16))
    check(y, oracle.gemv_bf16(bits16(w), x.float().cpu().numpy(), threads=0))
    foreign = tb.clone()
    foreign[15] = 0xFF
    yf = card.gemv_p12(P12Weight(lo, hi4, foreign, ei, ev, R, C, card), x)
    assert torch.equal(yf.view(torch.int16), y.view(torch.int16)) and bool(torch.isfinite(yf.float()).all())
    if M >= 8 and C in (2560, 4096):
        # a caller of the C ABI that hands over the table as stored (0xFF in slot 15) beside the pair table made from
        # it: on the matrix-core kernel that takes the pair table an escaped weight streams as slot 15 = 0 all the same
        pw.table[15] = 0xFF
        yr = card.gemv_p12(pw, x)
        assert torch.equal(yr.view(torch.int16), y.view(torch.int16))
