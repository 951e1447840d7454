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
    """the encoder has no counterpart in the reference (parity unpinned); what is checked: the two restatements
    agree, every representable matrix survives encode -> decode, and the error stays within the rule's bound: half
    the widest grid gap, or the saturation of a block's peak (below 8 units) at 6"""
    w = weights_bf16(16, 256, 41).float()
    pb, ps = mxfp4.quantize(w)
    ob, os_ = codecs.mxfp4_encode(w.numpy())
    assert np.array_equal(pb.numpy(), ob) and np.array_equal(ps.numpy(), os_)
    deq = mxfp4.dequantize(pb, ps)
    pb2, ps2 = mxfp4.quantize(deq)
    assert torch.equal(mxfp4.dequantize(pb2, ps2), deq)
    unit = mxfp4.scale_factors(ps)[..., None]
    assert torch.all((deq - w).abs().reshape(16, 8, 32) <= 2.0 * unit)


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
