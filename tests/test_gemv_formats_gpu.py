"""The fused widen + matvec of the three stored forms on the GPU against the CPU oracle's matvec over the same bytes.

Bar: max |y_gpu - y_ref| / max |y_ref| <= 1e-2 on bf16 outputs (both sides accumulate in f32; the widened weights are
bit-identical - tests/test_widen_gpu.py - so only the order of the f32 additions and the final bf16 rounding differ),
and the reference card's own bar of one bf16 ulp of the largest output.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

import oracle
from btb_amd import fp8, mxfp4
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
    x = acts_bf16(2, C, seed=303)
    ref = oracle.gemv_bf16(bits16(w), x.float().numpy())
    check(card.gemv_p12(pw, x.cuda()), ref)


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


def test_format_refusals(card):
    L = card.lib
    z = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    x = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    s = torch.ones(16, dtype=torch.float32, device="cuda")
    p = card.ptr
    assert L.btb_hip_gemv_mxfp4(p(z), p(z), p(x), p(y), 4, 48, 1, None) == -6          # C % 32
    assert L.btb_hip_gemv_mxfp4(None, p(z), p(x), p(y), 4, 64, 1, None) == -1
    assert L.btb_hip_gemv_fp8(p(z), p(s), 3, 1, p(x), p(y), 4, 64, 1, None) == -6       # 3 does not divide 4
    assert L.btb_hip_gemv_fp8(p(z), p(s), 1, 8, p(x), p(y), 4, 64, 1, None) == -6       # 8-column blocks: not 16
    assert L.btb_hip_gemv_p12(p(z), p(z), p(z), None, None, 2, p(s), p(x), p(y), 4, 64, 1, None) == -1
    assert L.btb_hip_gemv_p12(p(z), p(z), p(z), None, None, 0, p(s), p(x), p(y), 4, 60, 1, None) == -6  # C % 16
