"""The in-register widen of every stored form, on the GPU through the C ABI, against the CPU oracle: BIT-EXACT.

The widen kernels run the same policy code the matvec instantiates (btb_formats.hpp), so what is pinned here is the
value every weight takes inside the fused matvec. Covered exhaustively where the domain is small: every e4m3 byte under
a sweep of scales, every fp4 byte under every e8m0 scale (the reference's tests/kernels/test_mx4_widen.py:34-42),
and pack12 over the reference's committed fixture plus seeded matrices with forced escapes, odd tails and empty
escape lists.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

import oracle
from btb_amd import fp8, mxfp4, pack12
from oracle import codecs

from .helpers import bits16, f32_bits, weights_bf16
from .test_codecs import load_dir

pytestmark = pytest.mark.gpu


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return (t if dtype is None else t.view(dtype)).cuda()


# -- pack12 ------------------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("rows,cols", [(9728, 2560), (64, 96), (7, 33), (1, 1), (3, 16), (128, 40)])
@pytest.mark.parametrize("escapes", [True, False])
def test_p12_widen_bit_exact(card, rows, cols, escapes):
    w = weights_bf16(rows, cols, seed=200)
    wb = bits16(w).copy().reshape(-1)
    if escapes:
        at = np.arange(0, wb.size, max(1, wb.size // 997))
        wb[at] = (wb[at] & 0x00FF) | ((0x10 + np.arange(at.size) % 40).astype(np.uint16) << 8)
    lo, hi4, table, esc_idx, esc_val = codecs.pack12_pack(wb)
    want = oracle.unpack_p12(lo, hi4, table, esc_idx, esc_val, wb.size)
    assert np.array_equal(want, wb)
    got = card.p12_widen(dev(lo), dev(hi4), dev(table), dev(esc_idx), dev(esc_val), wb.size, (rows, cols))
    assert np.array_equal(bits16(got).reshape(-1), want)


def test_p12_widen_reference_fixture(card):
    """every packed tensor of the reference's tiny_qwen3-pack12 store widens to its parent's bytes on the GPU"""
    store, parent = load_dir("tiny_qwen3-pack12"), load_dir("tiny_qwen3")
    for name in [k[: -len(".pack12")] for k in store if k.endswith(".pack12")]:
        lo, hi4, table, esc_idx, esc_val, shape = pack12.split(store[name + ".pack12"], store[name + ".pack12.meta"])
        n = parent[name].numel()
        got = card.p12_widen(lo.contiguous().cuda(), hi4.contiguous().cuda(), table.cuda(), esc_idx.cuda(),
                             esc_val.contiguous().cuda(), n, shape)
        assert torch.equal(got.cpu().view(torch.int16), parent[name].view(torch.int16)), name


def test_p12_row_ptr(card):
    rows, cols = 37, 48
    esc = np.sort(np.random.default_rng(3).choice(rows * cols, 200, replace=False)).astype(np.int32)
    got = card.p12_row_ptr(dev(esc), rows, cols).cpu().numpy()
    want = np.searchsorted(esc, np.arange(rows + 1) * cols, side="left")
    assert np.array_equal(got, want)
    empty = card.p12_row_ptr(torch.empty(0, dtype=torch.int32, device="cuda"), rows, cols)
    assert torch.all(empty == 0)


@pytest.mark.parametrize("bad", [[5, 5], [9, 3], [0, 32], [-1, 4]])   # the lists native/src/gemv.rs:4171-4189 refuses
def test_p12_bad_escape_lists_are_refused_at_upload(card, bad):
    """btb_hip_p12_check returns ERR_DOMAIN for them, raw through the C ABI, and `P12Weight` refuses to come into
    being - so no matvec or widen kernel is ever handed such a list"""
    import ctypes

    from btb_amd import native
    from btb_amd.pack12 import P12Weight

    ei = torch.tensor(bad, dtype=torch.int32, device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert card.lib.btb_hip_p12_check(P(ei), 2, 32, P(flag), st) == native.ERR_DOMAIN
    assert card.lib.btb_hip_p12_check(None, 2, 32, P(flag), st) == native.ERR_NULL
    assert card.lib.btb_hip_p12_check(P(ei), 33, 32, P(flag), st) == native.ERR_DOMAIN   # more escapes than weights
    good = torch.tensor([3, 9], dtype=torch.int32, device="cuda")
    assert card.lib.btb_hip_p12_check(P(good), 2, 32, P(flag), st) == native.OK
    assert card.lib.btb_hip_p12_check(None, 0, 32, None, st) == native.OK                # no list: nothing to check
    z = lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError):
        P12Weight(z(32), z(16), z(16), ei, z(2), 4, 8, card)
    with pytest.raises(ValueError):
        card.p12_check(ei, 32)
    P12Weight(z(32), z(16), z(16), good, z(2), 4, 8, card)


def test_p12_widen_skips_escape_indices_outside_the_tensor(card):
    """the patch kernel itself never writes outside `out`, whatever the list holds (the fences stay as they were)"""
    n = 64
    lo = torch.arange(n, dtype=torch.uint8, device="cuda")
    hi4 = torch.zeros(n // 2, dtype=torch.uint8, device="cuda")
    table = torch.zeros(16, dtype=torch.uint8, device="cuda")
    ei = torch.tensor([-7, 5, n, 2**30], dtype=torch.int32, device="cuda")
    ev = torch.tensor([1, 2, 3, 4], dtype=torch.uint8, device="cuda")
    buf = torch.full((n + 64,), 0x7777, dtype=torch.int16, device="cuda")
    out = buf[32 : 32 + n].view(torch.bfloat16)
    card.p12_widen(lo, hi4, table, ei, ev, n, (n,), out=out)
    torch.cuda.synchronize()
    assert bool((buf[:32] == 0x7777).all()) and bool((buf[32 + n :] == 0x7777).all())
    got = out.view(torch.int16).cpu().numpy().astype(np.uint16)
    want = np.arange(n, dtype=np.uint16)
    want[5] |= 2 << 8
    assert np.array_equal(got, want)


# -- fp8 ---------------------------------------------------------------------------------------------------------------


def test_fp8_widen_every_byte_under_many_scales(card):
    """256 bytes x 512 scales (powers of two across the f32 range, tiny, huge and seeded ordinary ones), 16-column
    blocks: the held weight bf16(e4m3 * scale) bit for bit, NaN bytes and subnormal products included"""
    rng = np.random.default_rng(11)
    scales = np.concatenate([np.exp2(np.arange(-140, 116, dtype=np.float64)).astype(np.float32),
                             (rng.random(256) * 1e-3 + 1e-6).astype(np.float32)])
    sr = scales.size
    q = np.tile(np.arange(256, dtype=np.uint8), (sr, 1))          # [sr, 256]: every byte in every row
    grid = np.repeat(scales[:, None], 16, axis=1)                  # [sr, 16] blocks of 16 columns
    want = oracle.widen_fp8(q, grid)
    w = fp8.F8Weight(dev(q), dev(grid), sr, 256)
    got32 = card.fp8_widen(w, torch.float32).cpu().numpy()
    got16 = card.fp8_widen(w, torch.bfloat16)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got32), nan)
    assert np.array_equal(f32_bits(got32)[~nan], f32_bits(want)[~nan])
    assert np.array_equal(bits16(got16)[~nan], (f32_bits(want)[~nan] >> 16).astype(np.uint16))


@pytest.mark.parametrize("rows,cols,block", [(256, 7168, (128, 128)), (64, 256, (16, 16)), (48, 96, (48, 96))])
def test_fp8_widen_quantized_matrix(card, rows, cols, block):
    src = weights_bf16(rows, cols, seed=210).float()
    q, s = fp8.quantize(src, block)
    w = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), rows, cols)
    got = card.fp8_widen(w, torch.bfloat16)
    want = oracle.widen_fp8(q.view(torch.uint8).numpy(), s.numpy())
    assert np.array_equal(bits16(got), (f32_bits(want) >> 16).astype(np.uint16))
    assert torch.equal(got.cpu().view(torch.int16), fp8.held(q, s).view(torch.int16))


# -- mxfp4 -------------------------------------------------------------------------------------------------------------


def test_mx4_widen_every_byte_every_scale(card):
    blocks = np.tile(np.arange(256, dtype=np.uint8).reshape(16, 16), (256, 1)).reshape(256, 16, 16)
    scales = np.repeat(np.arange(256, dtype=np.uint8), 16).reshape(256, 16)
    want = oracle.widen_mxfp4(blocks, scales).reshape(256, 16 * 32)
    got32 = card.mx4_widen(dev(blocks), dev(scales), dtype=torch.float32).cpu().numpy()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got32), nan)
    assert np.array_equal(f32_bits(got32)[~nan], f32_bits(want)[~nan])
    # the bf16 form equals torch's ldexp widening (btb/mxfp4_torch.py:71-80) wherever it is finite
    got16 = card.mx4_widen(dev(blocks), dev(scales))
    ref16 = mxfp4.dequant_blocks(torch.from_numpy(blocks), torch.from_numpy(scales))
    ok = torch.isfinite(ref16.float())
    assert torch.equal(got16.cpu().view(torch.int16)[ok], ref16.view(torch.int16).reshape(256, -1)[ok])


def test_mx4_widen_seats(card):
    rng = np.random.default_rng(5)
    S, groups = 6, 40
    blocks = rng.integers(0, 256, (S, groups, 16), dtype=np.uint8)
    scales = rng.integers(100, 140, (S, groups), dtype=np.uint8)
    seats = torch.tensor([4, 0, 5], dtype=torch.int32)
    got = card.mx4_widen(dev(blocks), dev(scales), seats.cuda())
    want = mxfp4.dequant_blocks(torch.from_numpy(blocks[[4, 0, 5]]), torch.from_numpy(scales[[4, 0, 5]]))
    assert torch.equal(got.cpu().view(torch.int16), want.reshape(3, -1).view(torch.int16))
    with pytest.raises(ValueError):
        card.mx4_widen(dev(blocks).float(), dev(scales))


def test_round_bf16_is_the_integer_rule(card):
    """the device's f32 -> bf16 rounding (one conversion instruction) against the integer rule the reference and the
    oracle state (native/src/gemv.rs:3003-3007; a NaN: the quiet NaN a torch cast writes) on bit patterns of every
    kind: anything, NaNs of every payload and both signs, denormals, exact ties, the values round the largest finite"""
    rng = np.random.default_rng(960)
    bits = np.concatenate([
        rng.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32),
        (0x7F800000 | rng.integers(1, 2**23, 300_000, dtype=np.uint64)).astype(np.uint32),
        (0xFF800000 | rng.integers(1, 2**23, 300_000, dtype=np.uint64)).astype(np.uint32),
        rng.integers(0, 2**23, 300_000, dtype=np.uint64).astype(np.uint32),
        ((rng.integers(0, 2**16, 300_000, dtype=np.uint64).astype(np.uint32) << 16) | 0x8000).astype(np.uint32),
        np.array([0x7F800000, 0xFF800000, 0x7F7FFFFF, 0x7F7F8000, 0x7F7F7FFF, 0, 0x80000000, 0x7F800001, 0x7FC00000,
                  0x7FFFFFFF, 0xFFFFFFFF, 0x00000001, 0x00008000, 0x00018000], dtype=np.uint32),
    ])
    x = torch.from_numpy(bits.view(np.float32).copy()).cuda()
    got = card.round_bf16(x).view(torch.int16).cpu().numpy().view(np.uint16)
    want = codecs.f32_to_bf16_bits(bits.view(np.float32))
    assert np.array_equal(got, want)

