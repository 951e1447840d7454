"""TEST INFRASTRUCTURE - numpy restatements of the reference's storage codecs, used only as checkers.

  pack12   btb/pack12.py:48-67 (pack), :70-97 (unpack), :100-133 (blob / entry layout)
  fp8      btb/fp8.py:29-62, 97-100 (scale grid, widen, quantize, held)
  mxfp4    btb/mxfp4.py:41, 102-124 (table, dequantize, scale factors)

The MXFP4 *encoder* has no counterpart in the reference (it only ever decodes checkpoints or draws random bytes:
tests/helpers.py:305-316), so no reference result exists for it to match; `mxfp4_encode` follows the OCP MX rule and
is held to that rule by an exhaustive nearest-value search in exact arithmetic (tests/test_codecs.py).
"""

from __future__ import annotations

import struct

import numpy as np

# ------------------------------------------------------------------------------------------------------------
# bf16
# ------------------------------------------------------------------------------------------------------------


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """nearest bf16, ties to even, as uint16 bit patterns (a NaN becomes a quiet NaN)"""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    r = ((b + np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
    nan = (b & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    return np.where(nan, ((b >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16), r)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_bf16(a: np.ndarray) -> np.ndarray:
    return bf16_bits_to_f32(f32_to_bf16_bits(a))


# ------------------------------------------------------------------------------------------------------------
# pack12
# ------------------------------------------------------------------------------------------------------------

ESC = 15


def pack12_pack(bits: np.ndarray):
    """bf16 bit patterns (uint16, any shape) to (lo, hi4, table, esc_idx, esc_val): the table lists the 15 most
    frequent high bytes, frequency descending, ties by byte value ascending"""
    v = np.ascontiguousarray(bits, dtype=np.uint16).reshape(-1)
    lo = (v & 0xFF).astype(np.uint8)
    hi = (v >> 8).astype(np.uint8)
    counts = np.bincount(hi, minlength=256)
    order = sorted(range(256), key=lambda b: (-int(counts[b]), b))[:ESC]
    order = [b for b in order if counts[b] > 0]
    lut = np.full(256, ESC, dtype=np.uint8)
    for code, b in enumerate(order):
        lut[b] = code
    code = lut[hi]
    esc = np.nonzero(code == ESC)[0]
    esc_idx = esc.astype(np.int32)
    esc_val = hi[esc]
    if code.size % 2:
        code = np.concatenate([code, np.zeros(1, dtype=np.uint8)])
    hi4 = (code[0::2] | (code[1::2] << 4)).astype(np.uint8)
    table = np.zeros(16, dtype=np.uint8)
    table[: len(order)] = order
    return lo, hi4, table, esc_idx, esc_val


def pack12_unpack(lo, hi4, table, n: int, esc_idx=None, esc_val=None) -> np.ndarray:
    """the bf16 bit patterns back (uint16 [n])"""
    lo = np.asarray(lo, dtype=np.uint8)[:n]
    hi4 = np.asarray(hi4, dtype=np.uint8)
    codes = np.empty(hi4.size * 2, dtype=np.uint8)
    codes[0::2] = hi4 & 0x0F
    codes[1::2] = hi4 >> 4
    out = (np.asarray(table, dtype=np.uint8)[codes[:n]].astype(np.uint16) << 8) | lo
    if esc_idx is not None and len(esc_idx):
        idx = np.asarray(esc_idx, dtype=np.int64)
        out[idx] = (np.asarray(esc_val, dtype=np.uint8).astype(np.uint16) << 8) | lo[idx]
    return out


def pack12_blob(bits: np.ndarray, shape) -> tuple[bytes, bytes]:
    """the two on-disk entries of one tensor: body (`<name>.pack12`) and meta (`<name>.pack12.meta`)"""
    lo, hi4, table, esc_idx, esc_val = pack12_pack(bits)
    pad = (-(lo.nbytes + hi4.nbytes)) % 4
    body = lo.tobytes() + hi4.tobytes() + b"\0" * pad + esc_idx.astype("<i4").tobytes() + esc_val.tobytes()
    body += b"\0" * ((-len(body)) % 4)
    shape = [int(d) for d in shape]
    meta = table.tobytes() + struct.pack(f"<II{len(shape)}q", int(esc_idx.size), len(shape), *shape)
    return body, meta


def pack12_split(body: bytes, meta: bytes):
    """(lo, hi4, table, esc_idx, esc_val, shape) out of a tensor's two on-disk entries"""
    table = np.frombuffer(meta[:16], dtype=np.uint8)
    n_esc, rank = struct.unpack("<II", meta[16:24])
    shape = [int(d) for d in struct.unpack(f"<{rank}q", meta[24 : 24 + 8 * rank])]
    n = int(np.prod(shape)) if shape else 1
    a1 = n
    a2 = a1 + (n + 1) // 2
    a2p = a2 + ((-a2) % 4)
    a3 = a2p + 4 * n_esc
    buf = np.frombuffer(body, dtype=np.uint8)
    lo, hi4 = buf[:a1], buf[a1:a2]
    esc_idx = np.frombuffer(bytes(buf[a2p:a3]), dtype="<i4").astype(np.int32)
    esc_val = buf[a3 : a3 + n_esc]
    return lo, hi4, table, esc_idx, esc_val, shape


# ------------------------------------------------------------------------------------------------------------
# fp8 e4m3fn with block scales
# ------------------------------------------------------------------------------------------------------------

FP8_MAX = 448.0


def e4m3_decode(b: np.ndarray) -> np.ndarray:
    """e4m3fn bytes to f32: exponent 0 is m * 2^-9, 0x7F / 0xFF NaN, no infinity (native/src/gemv.rs:3009-3020)"""
    b = np.asarray(b, dtype=np.uint8)
    a = (b & 0x7F).astype(np.uint32)
    sub = (a.astype(np.float32) * np.float32(1.0 / 512.0)).view(np.uint32)
    nrm = (a << np.uint32(20)) + np.uint32(120 << 23)
    mag = np.where(a == 0x7F, np.uint32(0x7FC00000), np.where(a < 8, sub, nrm)).astype(np.uint32)
    return (mag | ((b & 0x80).astype(np.uint32) << np.uint32(24))).view(np.float32)


def e4m3_encode(v: np.ndarray) -> np.ndarray:
    """f32 to the nearest e4m3fn byte, ties to even; |v| is expected within 448 (a larger one or a NaN is NaN)"""
    v = np.asarray(v, dtype=np.float32)
    sign = (v.view(np.uint32) >> np.uint32(24)).astype(np.uint8) & np.uint8(0x80)
    a = np.abs(v).astype(np.float64)
    out = np.zeros(v.shape, dtype=np.uint8)
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0))).astype(np.int64)
    e = np.maximum(e, -6)  # below the smallest normal the spacing stays 2^-9
    q = np.rint(a / np.exp2(e - 3.0))  # in units of the binade's spacing: 8..16 for a normal
    up = q >= 16
    e = np.where(up, e + 1, e)
    q = np.where(up, 8, q)
    normal = q >= 8
    code = np.where(normal, ((e + 7) << 3) | (q.astype(np.int64) - 8), q.astype(np.int64))
    bad = ~np.isfinite(v) | (code > 0x7E)
    out = np.where(bad, 0x7F, code).astype(np.uint8)
    return out | sign


def fp8_quantize(t: np.ndarray, block: tuple[int, int] | None):
    """btb/fp8.py:49-62: each block scaled so its largest magnitude is 448; returns (bytes uint8, scale_inv f32)"""
    t = np.asarray(t, dtype=np.float32)
    rows, cols = t.shape
    bm, bn = block if block is not None else (rows, cols)
    if rows % bm or cols % bn:
        raise ValueError(f"[fp8] a {rows}x{cols} matrix does not split into {bm}x{bn} blocks")
    tiles = t.reshape(rows // bm, bm, cols // bn, bn)
    peak = np.abs(tiles).max(axis=(1, 3))
    # torch evaluates `448 / peak` (a Python scalar over a tensor) as reciprocal(peak) * 448: two f32 roundings,
    # which is what the reference's stored scales hold
    recip = (np.float32(1.0) / np.where(peak > 0, peak, np.float32(1.0))).astype(np.float32)
    scale = np.where(peak > 0, recip * np.float32(FP8_MAX), np.float32(1.0)).astype(np.float32)
    scaled = np.clip((tiles * scale[:, None, :, None]).astype(np.float32), -FP8_MAX, FP8_MAX)
    q = e4m3_encode(scaled).reshape(rows, cols)
    return q, (np.float32(1.0) / scale).astype(np.float32)


def fp8_held(q: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """bf16(e4m3 * scale) as f32 [rows, cols] (btb/fp8.py:36-46, 97-100)"""
    q = np.asarray(q, dtype=np.uint8)
    g = np.asarray(scales, dtype=np.float32)
    rows, cols = q.shape
    sr, sc = g.shape
    f = e4m3_decode(q).reshape(sr, rows // sr, sc, cols // sc) * g.reshape(sr, 1, sc, 1)
    return round_bf16(f.astype(np.float32)).reshape(rows, cols)


# ------------------------------------------------------------------------------------------------------------
# MXFP4
# ------------------------------------------------------------------------------------------------------------

FP4_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
                      dtype=np.float32)


def e8m0_scale(s: np.ndarray) -> np.ndarray:
    """2^(s - 127) as f32 for every byte: s == 0 is 2^-127 (btb/mxfp4.py:120-124)"""
    s = np.asarray(s, dtype=np.uint8).astype(np.uint32)
    f = (np.maximum(s, 1) << np.uint32(23)).view(np.float32)
    return np.where(s == 0, f * np.float32(0.5), f).astype(np.float32)


def mxfp4_dequantize(blocks: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """blocks [..., K/32, 16] and scales [..., K/32] to f32 [..., K]: low nibble first (btb/mxfp4.py:102-117)"""
    blocks = np.asarray(blocks, dtype=np.uint8)
    scales = np.asarray(scales, dtype=np.uint8)
    out = np.empty((*blocks.shape[:-1], 32), dtype=np.float32)
    out[..., 0::2] = FP4_VALUES[blocks & 0x0F]
    out[..., 1::2] = FP4_VALUES[blocks >> 4]
    out *= e8m0_scale(scales)[..., None]
    return out.reshape(*blocks.shape[:-2], blocks.shape[-2] * 32)


def mxfp4_encode(t: np.ndarray):
    """f32 [rows, K] to (blocks [rows, K/32, 16], scales [rows, K/32]) by the OCP MX rule: the block's shared
    exponent is floor(log2(amax)) - 2, elements round to the nearest e2m1 value (ties to the even code) and
    saturate at 6. No counterpart in the reference (it reads MXFP4 checkpoints and never writes one), so there is
    no reference result to be in parity with; the rule itself is pinned by tests/test_codecs.py: every element against
    an exhaustive nearest-value search in exact rationals over the grid's midpoints, their neighbours and the
    saturation edge, the scale byte against the exponent rule."""
    t = np.asarray(t, dtype=np.float32)
    rows, K = t.shape
    if K % 32:
        raise ValueError(f"[mxfp4] K = {K} is not a multiple of 32")
    g = t.reshape(rows, K // 32, 32).astype(np.float64)
    amax = np.abs(g).max(axis=-1)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(amax > 0, amax, 1.0))).astype(np.int64) - 2
    s = np.clip(e + 127, 0, 254)
    s = np.where(amax > 0, s, 127).astype(np.uint8)
    a = np.abs(g) / np.exp2(s.astype(np.float64) - 127.0)[..., None]
    mids = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    code = np.zeros(a.shape, dtype=np.uint8)
    for i, m in enumerate(mids):
        code += (a >= m) if i % 2 else (a > m)
    code |= (np.signbit(g).astype(np.uint8) << 3)
    blocks = (code[..., 0::2] | (code[..., 1::2] << 4)).astype(np.uint8)
    return blocks, s
