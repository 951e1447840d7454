"""The 12-bit lossless weight format (pack12, version 1): codec and the on-device container.

Same interface and byte layout as the reference's `btb/pack12.py` (:48-67 `pack_bf16`, :70-97 `unpack_bf16`,
:100-110 `blob`, :113-133 `entry`): a bf16 tensor is a low byte per element (`lo`), a 4-bit code per element into a
15-entry table of high bytes (`hi4`, the earlier element in the low nibble) and an escape list (ascending int32
indices and their high bytes) for the elements whose high byte is not in the table. The table lists high bytes by
frequency, ties by byte value, so a tensor packs to the same bytes every time. Everything here runs in torch on
whatever device the tensor is on, so a whole model packs on the GPU in seconds.

`P12Weight` is a packed matrix as the kernels read it: the five arrays on the GPU plus the per-row escape offsets
(`row_ptr`, built once at upload by `btb_hip_p12_row_ptr`) that let a wave find its row's escapes without a search.
"""

from __future__ import annotations

import struct
from collections.abc import Sequence
from typing import Any

import torch

VERSION = 1
ESC = 15
MAX_ELEMENTS = 2**31 - 1  # the escape indices are int32
META = 24  # table (16), escape count (u32), rank (u32); the shape (int64 x rank) follows


def check_size(n: int) -> None:
    if int(n) > MAX_ELEMENTS:
        raise ValueError(
            f"{int(n)} elements: the format's escape indices are int32, so a tensor packs up to {MAX_ELEMENTS}"
        )


def pack_bf16(t: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(lo u8[n], hi4 u8[ceil(n/2)], table u8[16], esc_idx i32[e], esc_val u8[e]) of a bf16 tensor, on its device"""
    if t.dtype != torch.bfloat16:
        raise ValueError(f"[pack12] a bf16 tensor packs, got {t.dtype}")
    check_size(t.numel())
    v = t.detach().contiguous().view(torch.int16).reshape(-1).to(torch.int32) & 0xFFFF
    lo = (v & 0xFF).to(torch.uint8)
    hi = (v >> 8).to(torch.int64)
    counts = torch.bincount(hi, minlength=256)
    # frequency descending; a stable sort leaves equal counts in ascending byte order
    top = torch.argsort(-counts, stable=True)[:ESC]
    top = top[counts[top] > 0]
    lut = torch.full((256,), ESC, dtype=torch.uint8, device=t.device)
    lut[top] = torch.arange(top.numel(), dtype=torch.uint8, device=t.device)
    code = lut[hi]
    esc = torch.nonzero(code == ESC).reshape(-1)
    esc_idx = esc.to(torch.int32)
    esc_val = hi[esc].to(torch.uint8)
    if code.numel() % 2:
        code = torch.cat([code, code.new_zeros(1)])
    hi4 = code[0::2] | (code[1::2] << 4)
    table = torch.zeros(16, dtype=torch.uint8, device=t.device)
    table[: top.numel()] = top.to(torch.uint8)
    return lo, hi4, table, esc_idx, esc_val


def unpack_bf16(
    lo: torch.Tensor,
    hi4: torch.Tensor,
    table: torch.Tensor,
    n: int,
    shape: Sequence[int],
    esc_idx: Any = None,
    esc_val: Any = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """the bf16 tensor back, bit for bit (torch ops; the GPU's fused path is `HipCard.p12_widen`)"""
    if out is None:
        out = torch.empty(tuple(shape), dtype=torch.bfloat16, device=lo.device)
    o16 = out.view(torch.int16).view(-1)
    codes = torch.stack([hi4 & 15, hi4 >> 4], dim=-1).reshape(-1)[:n].to(torch.int64)
    hi = table.to(torch.int16)[codes] << 8
    o16[:n] = hi | lo[:n].to(torch.int16)
    if esc_idx is not None and esc_idx.numel():
        at = esc_idx.to(torch.int64)
        o16[at] = (esc_val.to(torch.int16) << 8) | lo[at].to(torch.int16)
    return out


def blob(t: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """the two on-disk entries of a tensor, uint8: `<name>.pack12` = lo | hi4 | pad to 4 | esc_idx (int32 LE) | esc_val
    | pad to 4, and `<name>.pack12.meta` = table[16] | n_esc u32 | rank u32 | shape int64 x rank"""
    lo, hi4, table, esc_idx, esc_val = (a.cpu() for a in pack_bf16(t))
    pad = (-(lo.numel() + hi4.numel())) % 4
    body = lo.numpy().tobytes() + hi4.numpy().tobytes() + b"\0" * pad
    body += esc_idx.numpy().astype("<i4").tobytes() + esc_val.numpy().tobytes()
    body += b"\0" * ((-len(body)) % 4)
    shape = [int(d) for d in t.shape]
    meta = table.numpy().tobytes() + struct.pack(f"<II{len(shape)}q", int(esc_idx.numel()), len(shape), *shape)
    return (torch.frombuffer(bytearray(body), dtype=torch.uint8), torch.frombuffer(bytearray(meta), dtype=torch.uint8))


def entry(meta: bytes) -> dict[str, Any]:
    """a packed tensor's layout from its meta: shape, element count, the byte lengths of lo / hi4 / pad, the escape
    count and the table"""
    n_esc, rank = struct.unpack("<II", meta[16:24])
    shape = [int(d) for d in struct.unpack(f"<{rank}q", meta[24 : 24 + 8 * rank])]
    n = 1
    for d in shape:
        n *= d
    lo, hi4 = n, (n + 1) // 2
    return {"shape": shape, "n": n, "lo": lo, "hi4": hi4, "pad": (-(lo + hi4)) % 4, "esc": int(n_esc),
            "table": list(meta[:16])}


def split(body: torch.Tensor, meta: torch.Tensor):
    """(lo, hi4, table, esc_idx, esc_val, shape): views into a tensor's on-disk entries (uint8 tensors)"""
    e = entry(bytes(meta.cpu().numpy().tobytes()))
    a1 = e["lo"]
    a2 = a1 + e["hi4"] + e["pad"]
    a3 = a2 + 4 * e["esc"]
    table = torch.tensor(e["table"], dtype=torch.uint8, device=body.device)
    esc_idx = body[a2:a3].clone().view(torch.int32) if e["esc"] else torch.empty(0, dtype=torch.int32, device=body.device)
    esc_val = body[a3 : a3 + e["esc"]]
    return body[:a1], body[a1 : a1 + e["hi4"]], table, esc_idx, esc_val, e["shape"]


class P12Weight:
    """One packed matrix on the GPU as the kernels read it; `shape` = (rows, cols). `row_ptr[r]` is the index of the
    first escape at or past row r's first weight (int32 [rows + 1]), filled by the card at construction."""

    __slots__ = ("esc_idx", "esc_val", "hi4", "lo", "row_ptr", "shape", "table")

    def __init__(self, lo, hi4, table, esc_idx, esc_val, rows: int, cols: int, card: Any) -> None:
        dev = lo.device
        if dev.type != "cuda":
            raise ValueError("[pack12] a P12Weight lives on the GPU")
        n = rows * cols
        if lo.numel() != n or hi4.numel() != (n + 1) // 2 or table.numel() != 16:
            raise ValueError(f"[pack12] [{rows}, {cols}] needs {n} low bytes, {(n + 1) // 2} code bytes and a "
                             f"16-byte table")
        self.lo, self.hi4, self.table = lo.contiguous(), hi4.contiguous(), table.contiguous()
        self.esc_idx = esc_idx.to(torch.int32).contiguous()
        self.esc_val = esc_val.to(torch.uint8).contiguous()
        self.shape = (int(rows), int(cols))
        self.row_ptr = card.p12_row_ptr(self.esc_idx, rows, cols)

    @classmethod
    def pack(cls, w: torch.Tensor, card: Any) -> "P12Weight":
        rows, cols = (int(s) for s in w.shape)
        return cls(*pack_bf16(w), rows, cols, card)

    @property
    def nbytes(self) -> int:
        return (self.lo.numel() + self.hi4.numel() + 16 + 5 * self.esc_idx.numel() + 4 * self.row_ptr.numel())

    def __repr__(self) -> str:
        return f"P12Weight[{self.shape[0]}, {self.shape[1]}, {self.esc_idx.numel()} escapes]"
