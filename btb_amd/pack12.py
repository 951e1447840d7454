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

from collections.abc import Sequence
from typing import Any

import numpy as np
import torch

VERSION = 1
ESC = 15                  # the code that means "look in the escape list"
MAX_ELEMENTS = 2**31 - 1  # escape indices are int32
META = 24                 # bytes of a meta entry before the shape: table (16), escape count (u32), rank (u32)


def check_size(n: int) -> None:
    """refuses a tensor the int32 escape indices cannot address"""
    n = int(n)
    if n > MAX_ELEMENTS:
        raise ValueError(f"[pack12] {n} elements do not pack: an escape index is an int32, the limit is {MAX_ELEMENTS}")


def _table_of(hi: torch.Tensor) -> torch.Tensor:
    """the (at most 15) high bytes that get a code, most frequent first, equal counts by ascending byte value: the top
    15 of the keys count * 256 + (255 - byte), which are all distinct, so the order does not depend on the sort"""
    counts = torch.bincount(hi, minlength=256)
    byte = torch.arange(256, device=hi.device)
    key = counts * 256 + (255 - byte)
    best = torch.topk(key, ESC, sorted=True).indices
    return best[counts[best] > 0]


def pack_bf16(t: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """A bf16 tensor's five arrays, on its device: lo u8[n], hi4 u8[ceil(n / 2)] (element 2k in byte k's low nibble, an
    odd tail padded with code 0), table u8[16] (slot 15 and unused slots 0), esc_idx i32[e] ascending, esc_val u8[e]."""
    if t.dtype != torch.bfloat16:
        raise ValueError(f"[pack12] only bf16 tensors pack, this one is {t.dtype}")
    check_size(t.numel())
    dev = t.device
    bits = t.detach().contiguous().view(torch.uint8).reshape(-1, 2)   # little-endian: [:, 0] low byte, [:, 1] high byte
    lo = bits[:, 0].contiguous()
    hi = bits[:, 1].to(torch.int64)
    chosen = _table_of(hi)
    table = torch.zeros(16, dtype=torch.uint8, device=dev)
    table[: chosen.numel()] = chosen.to(torch.uint8)
    code_of = torch.full((256,), ESC, dtype=torch.uint8, device=dev)
    code_of.scatter_(0, chosen, torch.arange(chosen.numel(), dtype=torch.uint8, device=dev))
    code = code_of[hi]
    escaped = (code == ESC).nonzero(as_tuple=True)[0]
    pairs = torch.nn.functional.pad(code, (0, code.numel() & 1)).view(-1, 2)
    hi4 = pairs[:, 0] | (pairs[:, 1] << 4)
    return lo, hi4, table, escaped.to(torch.int32), hi[escaped].to(torch.uint8)


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
    """the bf16 tensor back, bit for bit, in torch ops on the arrays' device (`HipCard.p12_widen` is the GPU kernel)"""
    n = int(n)
    if out is None:
        out = torch.empty(tuple(shape), dtype=torch.bfloat16, device=lo.device)
    dst = out.view(torch.uint8).view(-1, 2)                            # the same two bytes an element as pack_bf16 reads
    nib = torch.stack((hi4 & 0x0F, hi4 >> 4), dim=1).view(-1)[:n]
    dst[:n, 0] = lo[:n]
    dst[:n, 1] = table[nib.to(torch.int64)]
    if esc_idx is not None and esc_idx.numel() > 0:
        dst[esc_idx.to(torch.int64), 1] = esc_val.to(torch.uint8)
    return out


def _pad4(n: int) -> int:
    return -n % 4


def blob(t: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """A tensor's two store entries (uint8 tensors). `<name>.pack12`: lo, hi4, zeros up to a multiple of 4, esc_idx as
    little-endian int32, esc_val, zeros up to a multiple of 4. `<name>.pack12.meta`: the 16 table bytes, the escape
    count and the rank as u32, the shape as int64."""
    lo, hi4, table, esc_idx, esc_val = (a.cpu().numpy() for a in pack_bf16(t))
    head = lo.size + hi4.size
    at_idx = head + _pad4(head)
    at_val = at_idx + 4 * esc_idx.size
    body = np.zeros(at_val + esc_val.size + _pad4(at_val + esc_val.size), dtype=np.uint8)
    body[: lo.size] = lo
    body[lo.size : head] = hi4
    body[at_idx:at_val] = esc_idx.astype("<i4").view(np.uint8)
    body[at_val : at_val + esc_val.size] = esc_val
    dims = np.asarray(t.shape, dtype="<i8")
    meta = np.concatenate([table, np.asarray([esc_idx.size, dims.size], dtype="<u4").view(np.uint8), dims.view(np.uint8)])
    return torch.from_numpy(body), torch.from_numpy(meta.astype(np.uint8))


def entry(meta: bytes) -> dict[str, Any]:
    """What a meta entry says about its tensor: `shape`, `n` elements, the byte lengths `lo` and `hi4`, the `pad` after
    them, `esc` escapes and the 16 `table` bytes."""
    raw = np.frombuffer(bytes(meta), dtype=np.uint8)
    if raw.size < META:
        raise ValueError(f"[pack12] a meta entry has at least {META} bytes, this one {raw.size}")
    n_esc, rank = (int(v) for v in raw[16:META].view("<u4"))
    if raw.size < META + 8 * rank:
        raise ValueError(f"[pack12] a meta entry of rank {rank} has {META + 8 * rank} bytes, this one {raw.size}")
    shape = [int(d) for d in raw[META : META + 8 * rank].view("<i8")]
    if any(d < 0 for d in shape):
        raise ValueError(f"[pack12] a meta entry with a negative dimension: {shape}")
    n = int(np.prod(shape, dtype=np.int64)) if shape else 1
    check_size(n)
    codes = (n + 1) // 2
    return {"shape": shape, "n": n, "lo": n, "hi4": codes, "pad": _pad4(n + codes), "esc": n_esc,
            "table": raw[:16].tolist()}


def split(body: torch.Tensor, meta: torch.Tensor):
    """(lo, hi4, table, esc_idx, esc_val, shape) of a stored tensor: views into its `.pack12` bytes (esc_idx a copy,
    for its alignment), on the bytes' device. A body whose length is not what the meta entry implies is refused."""
    e = entry(meta.cpu().numpy().tobytes())
    at_hi4 = e["lo"]
    at_idx = at_hi4 + e["hi4"] + e["pad"]
    at_val = at_idx + 4 * e["esc"]
    end = at_val + e["esc"]
    if e["esc"] > e["n"] or body.dtype != torch.uint8 or body.numel() != end + _pad4(end):
        raise ValueError(f"[pack12] a store entry of {body.numel()} bytes does not hold {e['n']} weights with {e['esc']} "
                         f"escapes ({end + _pad4(end)} bytes)")
    esc_idx = body[at_idx:at_val].clone().view(torch.int32)
    table = torch.tensor(e["table"], dtype=torch.uint8, device=body.device)
    return body[:at_hi4], body[at_hi4 : at_hi4 + e["hi4"]], table, esc_idx, body[at_val:end], e["shape"]


def check_escapes(esc_idx: torch.Tensor, esc_val: torch.Tensor, n: int) -> None:
    """ValueError unless the list is what the kernels index with: as many values as indices, every index in [0, n),
    strictly ascending (the reference refuses the same lists with ERR_DOMAIN: native/src/gemv.rs:4171-4189). Runs where
    the list lies (a few torch reductions; on the GPU for an uploaded matrix), once, at upload."""
    if esc_idx.numel() != esc_val.numel():
        raise ValueError(f"[pack12] {esc_idx.numel()} escape indices but {esc_val.numel()} escape values")
    if esc_idx.numel() == 0:
        return
    if esc_idx.numel() > int(n):
        raise ValueError(f"[pack12] {esc_idx.numel()} escapes for {int(n)} weights")
    idx = esc_idx.to(torch.int64)
    ok = bool(idx[0] >= 0) and bool(idx[-1] < int(n)) and bool((idx[1:] > idx[:-1]).all())
    if not ok:
        raise ValueError(f"[pack12] the escape list is not strictly ascending inside [0, {int(n)})")


class P12Weight:
    """One packed matrix on the GPU as the kernels read it; `shape` = (rows, cols). Three arrays are made here, once, by
    the card: `row_ptr[r]`, the index of the first escape at or past row r's first weight (int32 [rows + 1]), `pairs`,
    the 256 two-byte entries the matvecs look a byte of codes up in, and `row_esc`, every row's first 8 (16 beyond 4096
    columns) escapes as words of the row's own (None for rows wider than 32767). The table is the matrix's own copy with
    slot 15 - the escape code, which names no table entry - set to 0: a store that left another byte there (0x7F or
    0xFF would make the streamed stand-in of an escaped weight inf or NaN, and its correction NaN) is as good as one
    that wrote the 0 the packer writes."""

    __slots__ = ("esc_idx", "esc_val", "hi4", "lo", "pairs", "row_esc", "row_ptr", "shape", "table")

    def __init__(self, lo, hi4, table, esc_idx, esc_val, rows: int, cols: int, card: Any) -> None:
        dev = lo.device
        if dev.type != "cuda":
            raise ValueError("[pack12] a P12Weight lives on the GPU")
        n = rows * cols
        if lo.numel() != n or hi4.numel() != (n + 1) // 2 or table.numel() != 16:
            raise ValueError(f"[pack12] [{rows}, {cols}] needs {n} low bytes, {(n + 1) // 2} code bytes and a "
                             f"16-byte table")
        check_size(n)
        self.lo, self.hi4 = lo.contiguous(), hi4.contiguous()
        self.table = table.to(torch.uint8).clone().contiguous()
        self.table[15] = 0
        self.esc_idx = esc_idx.to(torch.int32).contiguous()
        self.esc_val = esc_val.to(torch.uint8).contiguous()
        self.shape = (int(rows), int(cols))
        # the kernels index the low bytes and x with these: a list from a damaged store must never reach them
        check_escapes(self.esc_idx, self.esc_val, n)
        card.p12_check(self.esc_idx, n)
        self.row_ptr = card.p12_row_ptr(self.esc_idx, rows, cols)
        self.pairs = card.p12_pairs(self.table)
        self.row_esc = card.p12_row_esc(self.lo, self.esc_idx, self.esc_val, self.row_ptr, rows, cols)

    @classmethod
    def pack(cls, w: torch.Tensor, card: Any) -> "P12Weight":
        rows, cols = (int(s) for s in w.shape)
        return cls(*pack_bf16(w), rows, cols, card)

    @property
    def nbytes(self) -> int:
        return (self.lo.numel() + self.hi4.numel() + 16 + 512 + 5 * self.esc_idx.numel() + 4 * self.row_ptr.numel()
                + (0 if self.row_esc is None else 4 * self.row_esc.numel()))

    def __repr__(self) -> str:
        return f"P12Weight[{self.shape[0]}, {self.shape[1]}, {self.esc_idx.numel()} escapes]"
