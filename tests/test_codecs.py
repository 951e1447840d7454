"""The storage codecs against the golden pairs the reference's own tests hold (copied as data under tests/golden):

  tiny_qwen3-pack12/pack12-00000.safetensors  is `btb pack` of tiny_qwen3 (every `layers.` bf16 tensor)
  tiny_qwen3-f8_e4m3/                         is fp8.quantize(parent, (16, 16)) of tiny_qwen3's linears

and the product codecs (btb_amd.pack12 / fp8 / mxfp4, torch) against the oracle's (oracle/codecs.py, numpy)."""

from __future__ import annotations

import glob
import os

import numpy as np
import pytest
import torch
from safetensors import safe_open

import oracle
from btb_amd import fp8, mxfp4, pack12
from oracle import codecs

from .helpers import GOLDEN, bits16, f32_bits, weights_bf16


def load_dir(name: str) -> dict[str, torch.Tensor]:
    out = {}
    for path in sorted(glob.glob(os.path.join(GOLDEN, name, "*.safetensors"))):
        with safe_open(path, framework="pt") as f:
            for k in f.keys():
                out[k] = f.get_tensor(k)
    return out


@pytest.fixture(scope="module")
def parent():
    return load_dir("tiny_qwen3")


# -- pack12 ------------------------------------------------------------------------------------------------------------


def test_pack12_fixture_unpacks_to_parent(parent):
    """the reference's law: a packed store widens to its parent's bytes (tests/integration/test_engine_units.py:555-568)"""
    store = load_dir("tiny_qwen3-pack12")
    names = [k[: -len(".pack12")] for k in store if k.endswith(".pack12")]
    assert len(names) > 20
    escapes = 0
    for name in names:
        body, meta = store[name + ".pack12"], store[name + ".pack12.meta"]
        want = bits16(parent[name]).reshape(-1)
        # oracle: numpy split + the C unpack
        lo, hi4, table, esc_idx, esc_val, shape = codecs.pack12_split(body.numpy().tobytes(), meta.numpy().tobytes())
        assert list(parent[name].shape) == shape
        assert np.array_equal(oracle.unpack_p12(lo, hi4, table, esc_idx, esc_val, want.size), want), name
        assert np.array_equal(codecs.pack12_unpack(lo, hi4, table, want.size, esc_idx, esc_val), want), name
        escapes += esc_idx.size
        # product: torch split + unpack
        tlo, thi4, ttab, tei, tev, tshape = pack12.split(body, meta)
        got = pack12.unpack_bf16(tlo, thi4, ttab, want.size, tshape, tei, tev)
        assert np.array_equal(bits16(got).reshape(-1), want), name
    assert escapes > 0  # the fixture exercises the escape list


def test_pack12_packers_write_the_fixture_bytes(parent):
    """packing the parent reproduces the stored bytes: table order (frequency, ties by byte value), nibble order,
    padding and the meta record"""
    store = load_dir("tiny_qwen3-pack12")
    for name in [k[: -len(".pack12")] for k in store if k.endswith(".pack12")]:
        body, meta = store[name + ".pack12"], store[name + ".pack12.meta"]
        obody, ometa = codecs.pack12_blob(bits16(parent[name]), parent[name].shape)
        assert obody == body.numpy().tobytes() and ometa == meta.numpy().tobytes(), name
        pbody, pmeta = pack12.blob(parent[name])
        assert torch.equal(pbody, body) and torch.equal(pmeta, meta), name


@pytest.mark.parametrize("shape,scale", [((64, 96), 0.02), ((7, 33), 1.0), ((1, 1), 0.5), ((128, 40), 30.0)])
def test_pack12_round_trip(shape, scale):
    """tests/unit/test_unit.py:52-69: bit-exact at several shapes and scales; ~0.75 of the bf16 bytes"""
    w = weights_bf16(*shape, seed=31, std=scale)
    lo, hi4, table, esc_idx, esc_val = pack12.pack_bf16(w)
    back = pack12.unpack_bf16(lo, hi4, table, w.numel(), w.shape, esc_idx, esc_val)
    assert torch.equal(back.view(torch.int16), w.view(torch.int16))
    olo, ohi4, otab, oei, oev = codecs.pack12_pack(bits16(w))
    assert np.array_equal(lo.numpy(), olo) and np.array_equal(hi4.numpy(), ohi4) and np.array_equal(table.numpy(), otab)
    assert np.array_equal(esc_idx.numpy(), oei) and np.array_equal(esc_val.numpy(), oev)


def test_pack12_escape_kat():
    """tests/unit/test_unit.py:72-86: 17 powers of four, four of each -> 17 distinct high bytes, 15 in the table,
    the 2 x 4 = 8 elements of the two largest byte values (ties go to the smaller byte) escape"""
    vals = torch.tensor([4.0**k for k in range(-8, 9)], dtype=torch.float32).repeat_interleave(4).to(torch.bfloat16)
    lo, hi4, table, esc_idx, esc_val = pack12.pack_bf16(vals.reshape(17, 4))
    assert esc_idx.numel() == 8
    hi = (bits16(vals) >> 8).astype(np.uint8)
    assert sorted(set(esc_val.tolist())) == sorted(set(hi.tolist()))[-2:]
    assert table[:15].tolist() == sorted(set(hi.tolist()))[:15] and int(table[15]) == 0


# -- fp8 ---------------------------------------------------------------------------------------------------------------


def test_fp8_fixture_is_quantize_of_parent(parent):
    """tests/make_fixtures.py:1134-1169 wrote the store as fp8.quantize(parent, (16, 16)); both codecs reproduce its
    bytes and scales, and the held matrix is bf16(e4m3 * scale)"""
    store = load_dir("tiny_qwen3-f8_e4m3")
    names = [k for k, t in store.items() if t.dtype == torch.float8_e4m3fn]
    assert len(names) >= 20
    for name in names:
        q = store[name].view(torch.uint8)
        s = store[name[: -len(".weight")] + ".weight_scale_inv"]
        src = parent[name]
        pq, ps = fp8.quantize(src, (16, 16))
        assert torch.equal(pq.view(torch.uint8), q) and torch.equal(ps, s), name
        oq, os_ = codecs.fp8_quantize(src.float().numpy(), (16, 16))
        assert np.array_equal(oq, q.numpy()) and np.array_equal(f32_bits(os_), f32_bits(s.numpy())), name
        held = fp8.held(q, s)
        assert np.array_equal(f32_bits(oracle.widen_fp8(q.numpy(), s.numpy())), f32_bits(held.float().numpy())), name


def test_e4m3_encode_matches_torch_cast():
    v = torch.cat([torch.randn(50_000, generator=torch.Generator().manual_seed(3)) * 100.0,
                   torch.linspace(-448, 448, 20_001), torch.tensor([0.0, -0.0, 2.0**-10, 2.0**-9, 1.5 * 2.0**-9, 3e-4])])
    v = v.clamp(-448, 448)
    want = v.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(codecs.e4m3_encode(v.numpy()), want)


# -- mxfp4 -------------------------------------------------------------------------------------------------------------


def test_mxfp4_table_is_transformers():
    """tests/kernels/test_mxfp4.py:17-20"""
    tm = pytest.importorskip("transformers.integrations.mxfp4")
    assert tuple(tm.FP4_VALUES) == mxfp4.FP4_VALUES == tuple(float(v) for v in codecs.FP4_VALUES)


def test_mxfp4_dequantize_matches_transformers():
    """tests/kernels/test_mxfp4.py:23-34: bits over the whole e8m0 range (a scale of 255 aside)"""
    tm = pytest.importorskip("transformers.integrations.mxfp4")
    g = torch.Generator().manual_seed(5)
    E, rows, G = 2, 8, 4
    blocks = torch.randint(0, 256, (E, rows, G, 16), generator=g, dtype=torch.uint8)
    scales = torch.randint(0, 255, (E, rows, G), generator=g, dtype=torch.uint8)
    want = tm.convert_moe_packed_tensors(blocks, scales, dtype=torch.float32).transpose(1, 2)  # [E, rows, K]
    got = mxfp4.dequantize(blocks, scales)
    ok = torch.isfinite(want)
    assert torch.equal(got[ok].view(torch.int32), want[ok].view(torch.int32))
    assert np.array_equal(f32_bits(codecs.mxfp4_dequantize(blocks.numpy(), scales.numpy())), f32_bits(got.numpy()))
    assert torch.equal(mxfp4.dequant_blocks(blocks, scales, torch.float32)[ok].view(torch.int32),
                       want[ok].view(torch.int32))


def test_mxfp4_encoder_round_trip_and_agreement():
    """the encoder has no counterpart in the reference; beside the brute-force test below: the two restatements
    agree on N(0, 0.02) weights, every representable matrix survives encode -> decode, and the error stays within the
    rule's bound: half the widest grid gap, or the saturation of a block's peak (below 8 units) at 6"""
    w = weights_bf16(16, 256, 41).float()
    pb, ps = mxfp4.quantize(w)
    ob, os_ = codecs.mxfp4_encode(w.numpy())
    assert np.array_equal(pb.numpy(), ob) and np.array_equal(ps.numpy(), os_)
    deq = mxfp4.dequantize(pb, ps)
    pb2, ps2 = mxfp4.quantize(deq)
    assert torch.equal(mxfp4.dequantize(pb2, ps2), deq)
    unit = mxfp4.scale_factors(ps)[..., None]
    assert torch.all((deq - w).abs().reshape(16, 8, 32) <= 2.0 * unit)


def _nearest_e2m1(v: float, scale_byte: int) -> int:
    """the code of the e2m1 value nearest to v / 2^(scale - 127), by exhaustive search in exact arithmetic: ties go to
    the code with an even mantissa bit (0, 1, 2, 4: codes 0, 2, 4, 6), magnitudes past 6 saturate at 6; the sign bit is
    v's (a negative zero keeps it)"""
    import math
    from fractions import Fraction

    a = abs(Fraction(float(v))) / Fraction(2) ** (scale_byte - 127)
    mags = [Fraction(x) for x in (0, 0.5, 1, 1.5, 2, 3, 4, 6)]
    best = min(range(8), key=lambda c: (abs(mags[c] - a), c & 1))   # nearest, then the even code
    return best | (8 if math.copysign(1.0, float(v)) < 0 else 0)


def test_mxfp4_encoder_is_the_ocp_rule_by_brute_force():
    """The reference has no MXFP4 encoder (it reads checkpoints; its tests draw random bytes), so there is nothing to
    be in parity with; what fixes an encoder is the OCP MX rule itself: shared exponent floor(log2(amax)) - 2, elements
    to the NEAREST e2m1 value, ties to even, saturation at 6. Every element of blocks built around the grid's exact
    midpoints, their neighbours one f32 step either side, the saturation edge, zeros and negative zeros is held to an
    exhaustive nearest-value search in exact rationals; the scale byte is held to the exponent rule on powers of two
    and just below them. An encoder that rounds toward zero (or ties away from even) fails on the midpoints."""
    rng = np.random.default_rng(7)
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], np.float32)
    rows = []
    want_scale = []
    for k in (-20, -9, -3, 0, 5):                        # the block's unit 2^k: its peak fixes the shared exponent
        unit = np.float32(2.0) ** np.float32(k)
        for peak in (4.0, 5.9, 6.0, 7.999):             # floor(log2(peak * unit)) - 2 == k for each of these
            v = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(9)),
                                [0.0, -0.0, 0.1, 6.0, 6.5, 7.5]]).astype(np.float32)
            v = np.concatenate([v, -v[:4]])[:31]
            v = np.concatenate([v, np.zeros(31 - v.size, np.float32), [np.float32(peak)]]).astype(np.float32)
            sign = np.where(rng.random(32) < 0.5, np.float32(-1), np.float32(1))
            sign[-1] = 1
            rows.append((v * sign * unit).astype(np.float32))
            want_scale.append(127 + k)
    rows.append(np.zeros(32, np.float32))                # an all-zero block: scale byte 127, every code a zero
    want_scale.append(127)
    t = np.stack(rows)
    ob, os_ = codecs.mxfp4_encode(t)
    pb, ps = mxfp4.quantize(torch.from_numpy(t))
    assert np.array_equal(ob, pb.numpy()) and np.array_equal(os_, ps.numpy())
    assert os_.reshape(-1).tolist() == want_scale
    codes = np.stack([ob & 0x0F, ob >> 4], axis=-1).reshape(len(rows), 32)
    want = np.array([[_nearest_e2m1(x, sb) for x in row] for row, sb in zip(t, want_scale)], np.uint8)
    assert np.array_equal(codes, want)
    # the test's own teeth: an encoder that truncates toward zero differs from the search on these very inputs
    mags = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6], np.float64)
    scaled = np.abs(t.astype(np.float64)) / np.exp2(np.array(want_scale, np.float64) - 127)[:, None]
    trunc = (np.searchsorted(mags, np.minimum(scaled, 6.0), side="right") - 1).astype(np.uint8)
    assert np.count_nonzero(trunc != (want & 7)) > 50


# -- a damaged 12-bit store is refused before it reaches a kernel -----------------------------------------------------


@pytest.mark.parametrize("bad", [[5, 5], [9, 3], [0, 32], [-1, 4]])   # the lists native/src/gemv.rs:4171-4189 refuses
def test_pack12_bad_escape_lists_are_refused(bad):
    with pytest.raises(ValueError):
        pack12.check_escapes(torch.tensor(bad, dtype=torch.int32), torch.zeros(2, dtype=torch.uint8), 32)


def test_pack12_escape_list_checks():
    pack12.check_escapes(torch.tensor([0, 7, 31], dtype=torch.int32), torch.zeros(3, dtype=torch.uint8), 32)
    pack12.check_escapes(torch.empty(0, dtype=torch.int32), torch.empty(0, dtype=torch.uint8), 32)
    with pytest.raises(ValueError):   # as many values as indices
        pack12.check_escapes(torch.tensor([1, 2], dtype=torch.int32), torch.zeros(3, dtype=torch.uint8), 32)


def test_pack12_split_refuses_a_body_of_the_wrong_length(parent):
    w = parent["model.layers.0.mlp.down_proj.weight"]
    body, meta = pack12.blob(w)
    lo, hi4, table, ei, ev, shape = pack12.split(body, meta)
    assert shape == list(w.shape) and ei.numel() == ev.numel()
    assert torch.equal(pack12.unpack_bf16(lo, hi4, table, w.numel(), shape, ei, ev).view(torch.int16), w.view(torch.int16))
    with pytest.raises(ValueError):
        pack12.split(body[:-4], meta)
    with pytest.raises(ValueError):
        pack12.split(torch.cat([body, body.new_zeros(4)]), meta)
    more = meta.clone()
    more[16] += 1                      # one more escape than the body holds
    with pytest.raises(ValueError):
        pack12.split(body, more)
    with pytest.raises(ValueError):
        pack12.entry(bytes(meta[:20].numpy().tobytes()))
