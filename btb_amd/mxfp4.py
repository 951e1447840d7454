"""MXFP4 as gpt-oss stores it: 32 weights along K share 16 bytes of packed fp4 (e2m1, the earlier weight of a pair in
the LOW nibble) and one uint8 e8m0 exponent; weight = fp4 * 2^(scale - 127).

Same interface as the reference's `btb/mxfp4.py` (:41 `FP4_VALUES`, :102-117 `dequantize`, :120-124
`scale_factors`, :127-168 `MxWeight`) and `btb/mxfp4_torch.py:71-80` (`dequant_blocks`). The reference has no
encoder (it reads checkpoints); `quantize` here follows the OCP MX rule and exists so a benchmark can make MXFP4
matrices from seeded bf16 ones.
"""

from __future__ import annotations

import torch

FP4_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)
BLOCK = 32
BLOCK_BYTES = 16
BIAS = 127


def blocks_per_row(k: int) -> int:
    """how many 32-weight blocks a row of k weights is cut into"""
    n, rest = divmod(int(k), BLOCK)
    if rest or n < 0:
        raise ValueError(f"[mxfp4] a row of {k} weights is not a whole number of {BLOCK}-weight blocks")
    return n


def matrix_bytes(rows: int, k: int) -> tuple[int, int]:
    """(bytes of packed codes, bytes of scales) a [rows, k] matrix takes"""
    blocks = int(rows) * blocks_per_row(k)
    return blocks * BLOCK_BYTES, blocks


def scale_factors(scales: torch.Tensor) -> torch.Tensor:
    """Every e8m0 byte s as the f32 2^(s - 127), built from its bits so that nothing rounds: s >= 1 is a normal number
    with exponent field s, s = 0 is the subnormal 2^-127 (mantissa 0x400000), s = 255 comes out as +inf."""
    field = scales.to(torch.int32)
    bits = torch.where(field > 0, field * (1 << 23), torch.full_like(field, 0x0040_0000))
    return bits.view(torch.float32)


def _codes_to_values(blocks: torch.Tensor) -> torch.Tensor:
    """[..., 16] packed bytes -> [..., 32] fp4 values as f32, the low nibble first"""
    lut = torch.tensor(FP4_VALUES, dtype=torch.float32, device=blocks.device)
    idx = torch.stack((blocks & 0x0F, blocks >> 4), dim=-1).to(torch.int64)
    return lut[idx].flatten(-2)


def _check_pair(blocks: torch.Tensor, scales: torch.Tensor) -> None:
    if blocks.shape[-1] != BLOCK_BYTES:
        raise ValueError(f"[mxfp4] the last dim of blocks is the {BLOCK_BYTES} bytes of one block, not {blocks.shape[-1]}")
    if tuple(blocks.shape[:-1]) != tuple(scales.shape):
        raise ValueError(f"[mxfp4] one scale a block: blocks {tuple(blocks.shape)} need scales {tuple(blocks.shape[:-1])}, "
                         f"got {tuple(scales.shape)}")


def dequantize(blocks: torch.Tensor, scales: torch.Tensor, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """blocks [..., rows, K/32, 16] and scales [..., rows, K/32] (uint8) -> [..., rows, K]: the f32 product
    fp4 * 2^(scale - 127) - exact but for the subnormal results - cast to `dtype`"""
    _check_pair(blocks, scales)
    wide = _codes_to_values(blocks) * scale_factors(scales).unsqueeze(-1)
    return wide.flatten(-2).to(dtype)


def dequant_blocks(blocks: torch.Tensor, scales: torch.Tensor, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """the widening the card's `mx4_widen` matches bit for bit: ldexp(fp4, scale - 127) rounded to `dtype`"""
    _check_pair(blocks, scales)
    wide = torch.ldexp(_codes_to_values(blocks), (scales.to(torch.int32) - BIAS).unsqueeze(-1))
    return wide.flatten(-2).to(dtype)


def quantize(t: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """[rows, K] floats to (blocks [rows, K/32, 16], scales [rows, K/32]) by the OCP MX rule: the shared exponent is
    floor(log2(amax)) - 2, elements round to the nearest e2m1 value (ties to the even code) and saturate at 6"""
    rows, k = (int(s) for s in t.shape)
    g = blocks_per_row(k)
    v = t.float().reshape(rows, g, BLOCK)
    amax = v.abs().amax(dim=-1)
    # floor(log2(amax)) from the f32 exponent field (a subnormal amax clamps to the smallest scale below)
    e = ((amax.view(torch.int32) >> 23) & 0xFF) - 127 - 2
    s = torch.where(amax > 0, torch.clamp(e + BIAS, 0, 254), torch.full_like(e, BIAS)).to(torch.uint8)
    a = (v / scale_factors(s)[..., None]).abs()
    code = torch.zeros_like(a, dtype=torch.uint8)
    for i, m in enumerate((0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0)):
        code += ((a >= m) if i % 2 else (a > m)).to(torch.uint8)
    code |= (torch.signbit(v).to(torch.uint8) << 3)
    blocks = code[..., 0::2] | (code[..., 1::2] << 4)
    return blocks.contiguous(), s.contiguous()


class MxWeight:
    """One MXFP4 matrix as stored (the checkpoint's layout): `blocks` rows * K/32 * 16 bytes, `scales` rows * K/32
    bytes, `shape` = (rows, K)."""

    __slots__ = ("blocks", "scales", "shape")

    def __init__(self, blocks: torch.Tensor, scales: torch.Tensor, rows: int, k: int) -> None:
        nb, ns = matrix_bytes(rows, k)
        if blocks.numel() != nb or scales.numel() != ns:
            raise ValueError(f"[mxfp4] [{rows}, {k}] needs {nb} block bytes and {ns} scales, got {blocks.numel()} "
                             f"and {scales.numel()}")
        if blocks.dtype != torch.uint8 or scales.dtype != torch.uint8:
            raise ValueError("[mxfp4] blocks and scales are uint8")
        self.blocks = blocks.contiguous()
        self.scales = scales.contiguous()
        self.shape = (int(rows), int(k))

    @property
    def nbytes(self) -> int:
        return self.blocks.numel() + self.scales.numel()

    def __repr__(self) -> str:
        return f"MxWeight[{self.shape[0]}, {self.shape[1]}]"

    def dequantize(self, dtype: torch.dtype = torch.float32) -> torch.Tensor:
        rows, k = self.shape
        return dequantize(self.blocks.reshape(rows, k // BLOCK, BLOCK_BYTES), self.scales.reshape(rows, k // BLOCK),
                          dtype)
