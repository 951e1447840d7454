"""The bf16 decode matvec on the GPU (through the C ABI) against the CPU oracle on the same seeded inputs.

Bar: max |y_gpu - y_ref| / max |y_ref| <= 1e-2 on the bf16 outputs, y_ref the oracle's f32
result rounded to bf16. Both sides accumulate in f32 with one fused multiply-add per weight; they differ only in the
order of the additions (<= ~sqrt(C) * 2^-24 relative to sum |w x|, far below a bf16 ulp), so what is seen is at most a
bf16 rounding flip: 2^-8 relative to the output. The reference's own card bar, one bf16 ulp of the largest output
(tests/kernels/test_card_kernels.py:135-148), is asserted too.
"""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from oracle import codecs

from .helpers import acts_bf16, bits16, weights_bf16

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def oracle_bf16_out(w: torch.Tensor, x: torch.Tensor) -> np.ndarray:
    """the CPU path's answer as the card stores it: f32 lane sums, rounded to bf16 (kept as f32)"""
    y = oracle.gemv_bf16(bits16(w), x.float().numpy(), threads=0)
    return codecs.round_bf16(y)


def check(y: torch.Tensor, ref: np.ndarray) -> None:
    got = y.float().cpu().numpy()
    peak = np.abs(ref).max()
    err = np.abs(got - ref).max()
    assert err <= REL_TOL * peak, (err, peak)
    assert err <= peak * 2.0**-7, (err, peak)


@pytest.mark.parametrize("R,C", [(9728, 2560), (2560, 9728), (6144, 2560), (2560, 4096), (2048, 768), (1536, 2048),
                                 (128, 2048), (1000, 264), (7, 8), (3, 1032)])
@pytest.mark.parametrize("M", [1, 4])
def test_gemv_bf16_matches_oracle(card, R, C, M):
    w = weights_bf16(R, C, seed=100)
    x = acts_bf16(M, C, seed=101)
    y = card.gemv(w.cuda(), x.cuda())
    check(y, oracle_bf16_out(w, x))


@pytest.mark.parametrize("M", [2, 3, 4, 5, 7])
def test_row_of_a_wide_pass_is_its_one_row_pass(card, M):
    """native/cuda/btb_kernels.cu:84-88 and tests/kernels/test_card_kernels.py:145-148: row m does not depend on M"""
    R, C = 2560, 4096
    w = weights_bf16(R, C, seed=110).cuda()
    x = acts_bf16(M, C, seed=111).cuda()
    y = card.gemv(w, x)
    check(y, oracle_bf16_out(w.cpu(), x.cpu()))
    for m in (0, M - 1):
        solo = card.gemv(w, x[m : m + 1].contiguous())
        assert torch.equal(solo[0].view(torch.int16), y[m].view(torch.int16))


@pytest.mark.parametrize("R,C", [(2560, 9728), (2561, 5128), (7, 10240), (1, 6152), (5000, 8192), (3000, 9736)])
def test_long_rows_by_two_waves(card, R, C):
    """rows of 5121 .. 10240 values are summed by two waves, a half each (`gemv_halves`): against the oracle at one to
    four rows of x; row m of a pass is its one-row pass bit for bit; the add + norm in the x load gives the bits of
    add_rmsnorm followed by the plain matvec, the gate / up fold those of the plain matvec followed by silu_mul; with
    the split switched off (knob gemv_halves = 0: the whole-row kernel,
    another order of summation) the outputs stay within one bf16 ulp of the largest. Shapes: the down projection, odd
    row counts, the shortest and the longest row the split takes, rows of an odd number of units, and a matrix tall
    enough that workgroups take several turns."""
    w = weights_bf16(R, C, seed=120)
    x = acts_bf16(4, C, seed=121)
    ref = oracle_bf16_out(w, x)
    wd, xd = w.cuda(), x.cuda()
    y4 = card.gemv(wd, xd)
    check(y4, ref)
    for M in (1, 2, 3):
        ym = card.gemv(wd, xd[:M].contiguous())
        assert torch.equal(ym.view(torch.int16), y4[:M].view(torch.int16)), M
    solo = card.gemv(wd, xd[3:4].contiguous())
    assert torch.equal(solo[0].view(torch.int16), y4[3].view(torch.int16))
    # the add + norm form (workgroups of four waves) against the two launches (ten waves): the same bits
    for M in (1, 3):
        h = acts_bf16(M, C, seed=122).cuda()
        d = acts_bf16(M, C, seed=123).cuda()
        nw = (1.0 + 0.1 * torch.randn(C, generator=torch.Generator().manual_seed(124))).to(torch.bfloat16).cuda()
        h1, x1 = h.clone(), torch.empty_like(h)
        card.add_rmsnorm(h1, d, nw, 1e-6, x1)
        want = card.gemv(wd, x1)
        h2 = torch.empty_like(h)
        out = torch.empty(M, R, dtype=torch.bfloat16, device="cuda")
        card.gemv_norm(wd, h, d, nw, 1e-6, h2, out, glu=False)
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))
        assert torch.equal(h2.view(torch.int16), h1.view(torch.int16))
    # the gate / up fold over such rows (four waves an output): the plain matvec, then silu_mul, bit for bit
    if R % 2 == 0:
        for M in (1, 3):
            xm = xd[:M].contiguous()
            want = torch.empty(M, R // 2, dtype=torch.bfloat16, device="cuda")
            card.silu_mul(card.gemv(wd, xm), want)
            got = card.gemv_glu_silu(wd, xm)
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), M
    card.set_tuning("gemv_halves", 0)
    try:
        whole = card.gemv(wd, xd)
    finally:
        card.set_tuning("gemv_halves", -1)
    check(whole, ref)
    peak = float(np.abs(ref).max())
    assert float((whole.float() - y4.float()).abs().max()) <= peak * 2.0**-7


def test_long_rows_by_two_waves_over_drawn_shapes(card):
    """twenty drawn shapes in and around the split's range of row lengths (any multiple of 8 from 5000 to 10400 values,
    1 .. 3000 rows, 1 .. 4 rows of x): the oracle's bar, and every row of the pass the bits of its one-row pass"""
    rng = np.random.default_rng(20261)
    for i in range(20):
        R = int(rng.integers(1, 3001))
        C = 8 * int(rng.integers(625, 1301))
        M = int(rng.integers(1, 5))
        w = weights_bf16(R, C, seed=2000 + i)
        x = acts_bf16(M, C, seed=3000 + i)
        wd, xd = w.cuda(), x.cuda()
        y = card.gemv(wd, xd)
        check(y, oracle_bf16_out(w, x))
        for m in range(M):
            solo = card.gemv(wd, xd[m : m + 1].contiguous())
            assert torch.equal(solo[0].view(torch.int16), y[m].view(torch.int16)), (R, C, M, m)


@pytest.mark.parametrize("R,C", [(9728, 2560), (2560, 9728), (2560, 4096), (1000, 96), (18, 32)])
@pytest.mark.parametrize("M", [8, 16, 32, 12, 40])
def test_verify_widths_on_the_matrix_cores(card, R, C, M):
    """M >= 8 runs on MFMA: within the oracle's bar, and a row's bits are the same at every verify width (the
    reference's tensor-core matvec keeps that law within its family: tests/kernels/test_card_kernels.py:513-524)"""
    w = weights_bf16(R, C, seed=112).cuda()
    x = acts_bf16(M, C, seed=113).cuda()
    y = card.gemv(w, x)
    check(y, oracle_bf16_out(w.cpu(), x.cpu()))
    y8 = card.gemv(w, x[:8].contiguous())
    assert torch.equal(y8.view(torch.int16), y[:8].view(torch.int16))
    # the vector-ALU form of the same pass agrees to the same bar and equals the one-row pass bit for bit
    card.set_tuning("gemv_no_mfma", 1)
    try:
        v = card.gemv(w, x)
        solo = card.gemv(w, x[M - 1 :].contiguous())
    finally:
        card.set_tuning("gemv_no_mfma", -1)
    check(v, oracle_bf16_out(w.cpu(), x.cpu()))
    assert torch.equal(solo[0].view(torch.int16), v[M - 1].view(torch.int16))


def test_repeat_runs_are_bit_stable(card):
    w = weights_bf16(9728, 2560, seed=120).cuda()
    x = acts_bf16(1, 2560, seed=121).cuda()
    a = card.gemv(w, x).clone()
    for _ in range(5):
        assert torch.equal(card.gemv(w, x).view(torch.int16), a.view(torch.int16))


@pytest.mark.parametrize("M", [1, 4])
def test_silu_fold_equals_two_steps(card, M):
    """tests/kernels/test_card_kernels.py:376-391: the folded down projection equals act-mul then the plain matvec"""
    R, C = 2560, 9728
    w = weights_bf16(R, C, seed=130).cuda()
    gu = acts_bf16(M, 2 * C, seed=131).cuda()
    g, u = gu[:, :C].float(), gu[:, C:].float()
    s = (g / (1 + torch.exp(-g))).to(torch.bfloat16).float()
    x = (s * u).to(torch.bfloat16)
    folded = card.gemv_silu(w, gu)
    plain = card.gemv(w, x.contiguous())
    # the activation's exp may differ from torch's in the last bit, which can flip a bf16 rounding of x here and there
    ref = oracle_bf16_out(w.cpu(), x.cpu())
    check(folded, ref)
    frac = (folded != plain).float().mean().item()
    assert frac < 0.02, frac


@pytest.mark.parametrize("I,C", [(9728, 2560), (768, 2048), (96, 4096), (64, 9728), (40, 64)])
@pytest.mark.parametrize("M", [8, 16, 24])
def test_glu_kernel_at_the_verify_widths(card, I, C, M):
    """gate, up and the activation in the matrix-core kernel: the bits of its matvec followed by silu_mul, for each of
    the kernel's forms (and the vector passes where I is no multiple of 16)"""
    w = weights_bf16(2 * I, C, seed=152).cuda()
    x = acts_bf16(M, C, seed=153).cuda()
    gu = card.gemv(w, x)
    want = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
    card.silu_mul(gu, want)
    got = card.gemv_glu_silu(w, x)
    if I % 16 == 0:
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    else:  # vector passes against a matrix-core matvec: the bar, not the bits
        assert float((got.float() - want.float()).abs().max()) <= 2.0**-7 * float(want.float().abs().max())


@pytest.mark.parametrize("M", [1, 3])
def test_glu_kernel_equals_matvec_then_silu_mul(card, M):
    I, C = 9728, 2560
    w = weights_bf16(2 * I, C, seed=150).cuda()
    x = acts_bf16(M, C, seed=151).cuda()
    gu = card.gemv(w, x)
    want = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
    card.silu_mul(gu, want)
    got = card.gemv_glu_silu(w, x)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("M,with_y,glu,C", [(1, True, False, 2560), (1, False, False, 2560), (2, True, True, 2560),
                                              (1, True, True, 2560), (5, True, False, 2560), (8, True, True, 2560),
                                              (8, False, False, 2560), (16, True, True, 2560), (13, True, False, 2560),
                                              (7, True, True, 2048), (16, True, False, 1536), (4, True, False, 1280),
                                              (17, True, False, 2560), (35, True, True, 2560)])
def test_norm_folded_into_the_x_load_changes_no_bit(card, M, with_y, glu, C):
    """the residual add + norm made by the matvec itself (the vector kernels up to four rows a pass; from five rows
    the matrix cores, where the kernel makes the rows for rows of 1312 .. 2560 values, 16 rows a launch) against
    add_rmsnorm followed by the matvec: the same output and the same new residual, bit for bit"""
    R = 6144
    w = weights_bf16(R, C, seed=160).cuda()
    h = acts_bf16(M, C, seed=161).cuda()
    y = acts_bf16(M, C, seed=162).cuda() if with_y else None
    nw = (1.0 + 0.1 * torch.randn(C, generator=torch.Generator().manual_seed(163))).to(torch.bfloat16).cuda()
    h1, x1 = h.clone(), torch.empty_like(h)
    card.add_rmsnorm(h1, y, nw, 1e-6, x1)
    want = card.gemv_glu_silu(w, x1) if glu else card.gemv(w, x1)
    h2 = torch.empty_like(h)
    out = torch.empty(M, R // 2 if glu else R, dtype=torch.bfloat16, device="cuda")
    card.gemv_norm(w, h, y, nw, 1e-6, h2, out, glu=glu)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    assert torch.equal(h2.view(torch.int16), h1.view(torch.int16))
    with pytest.raises(ValueError):
        card.gemv_norm(w, h, y, nw, 1e-6, h, out, glu=glu)


@pytest.mark.parametrize("M", [1, 3, 8, 16])
def test_embedding_rows_gathered_by_the_first_matvec(card, M):
    """`gemv_embed_norm` against embed + add_rmsnorm + gemv: the same output and residual rows, ids outside the table
    clamped into it - on the vector kernels and, from five rows, on the matrix cores"""
    R, C, vocab = 4096, 2560, 300
    w = weights_bf16(R, C, seed=170).cuda()
    table = acts_bf16(vocab, C, seed=171).cuda()
    nw = (1.0 + 0.1 * torch.randn(C, generator=torch.Generator().manual_seed(172))).to(torch.bfloat16).cuda()
    ids = torch.randint(0, vocab, (M,), generator=torch.Generator().manual_seed(173), dtype=torch.int32)
    ids[0] = vocab + 5
    ids = ids.cuda()
    h1 = torch.empty(M, C, dtype=torch.bfloat16, device="cuda")
    card.embed(table, ids, h1)
    x1 = torch.empty_like(h1)
    card.add_rmsnorm(h1, None, nw, 1e-6, x1)
    want = card.gemv(w, x1)
    h2 = torch.empty_like(h1)
    out = torch.empty(M, R, dtype=torch.bfloat16, device="cuda")
    card.gemv_embed_norm(w, table, ids, nw, 1e-6, h2, out)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    assert torch.equal(h2.view(torch.int16), h1.view(torch.int16))


def test_rows_a_tile_change_no_bit_over_drawn_shapes(card):
    """the matrix-core matvec takes tiles of twelve or ten rows where sixteen would leave CUs idle (knob mfma_tile_rows
    = 0: always sixteen): over thirty drawn shapes - any multiple of 16 rows, the row lengths of the kernel's classes,
    5 .. 32 rows of x - the same bits either way, within the bar of an f32 product"""
    rng = np.random.default_rng(20252)
    lower = 0
    for _ in range(30):
        R = 16 * int(rng.integers(1, 700))
        C = int(rng.choice([2560, 4096, 1536, 5120, 9728, 7168]))
        M = int(rng.integers(5, 33))
        w = weights_bf16(R, C, seed=int(rng.integers(1 << 30))).cuda()
        x = acts_bf16(M, C, seed=int(rng.integers(1 << 30))).cuda()
        y = card.gemv(w, x)
        card.set_tuning("mfma_tile_rows", 0)
        try:
            y16 = card.gemv(w, x)
        finally:
            card.set_tuning("mfma_tile_rows", -1)
        assert torch.equal(y.view(torch.int16), y16.view(torch.int16)), (R, C, M)
        ref = x.float() @ w.float().t()
        assert float((y.float() - ref).abs().max()) <= 2.0**-7 * float(ref.abs().max()), (R, C, M)
        lower += int(R % 12 == 0 or R % 10 == 0)
    assert lower >= 5  # the draw holds row counts the lower tiles apply to


def test_refusals_launch_nothing(card):
    w = weights_bf16(16, 64, seed=140).cuda()
    x = acts_bf16(1, 64, seed=141).cuda()
    with pytest.raises(ValueError):
        card.gemv(w.float(), x)
    with pytest.raises(ValueError):
        card.gemv(w, x.cpu())
    with pytest.raises(ValueError):
        card.gemv(w, x, torch.empty(3, dtype=torch.bfloat16, device="cuda"))
    L = card.lib
    y = torch.full((1, 16), 7.0, dtype=torch.bfloat16, device="cuda")
    assert L.btb_hip_gemv_bf16(None, card.ptr(ctypes.c_void_p, x), card.ptr(ctypes.c_void_p, y), 16, 64, 1, None) == -1
    assert L.btb_hip_gemv_bf16(card.ptr(ctypes.c_void_p, w), card.ptr(ctypes.c_void_p, x), card.ptr(ctypes.c_void_p, y), 0, 64, 1, None) == -6
    assert L.btb_hip_gemv_bf16(card.ptr(ctypes.c_void_p, w), card.ptr(ctypes.c_void_p, x), card.ptr(ctypes.c_void_p, y), 16, 60, 1, None) == -6  # C % 8
    assert L.btb_hip_gemv_bf16(None, card.ptr(ctypes.c_void_p, x), card.ptr(ctypes.c_void_p, y), 0, 64, 1, None) == -1  # null before domain
    torch.cuda.synchronize()
    assert torch.all(y == 7.0)
