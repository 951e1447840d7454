"""Shared test helpers: seeded inputs in the benchmark configurations' shapes, an exact model of the f32 fused multiply-add for
brute-force checks, the f64 reference and the error measures the reference's own tests use."""

from __future__ import annotations

import os
from fractions import Fraction

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
SEED0 = 0x0B7B0000


def gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(SEED0 + seed)


def weights_bf16(rows: int, cols: int, seed: int, std: float = 0.02) -> torch.Tensor:
    """bf16 [rows, cols] ~ N(0, std), rounded to nearest even: the seeded weights of every config"""
    return (torch.randn(rows, cols, generator=gen(seed)) * std).to(torch.bfloat16)


def acts_bf16(m: int, cols: int, seed: int) -> torch.Tensor:
    return torch.randn(m, cols, generator=gen(seed)).to(torch.bfloat16)


def bits16(t: torch.Tensor) -> np.ndarray:
    """a bf16 tensor's bit patterns as uint16"""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits16(b: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(b, dtype=np.uint16).view(np.int16).copy()).view(torch.bfloat16)


def f32_bits(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# -- exact f32 arithmetic in rationals --------------------------------------------------------------------


def _frac(x: float) -> Fraction:
    return Fraction(float(np.float32(x)))


def _round_f32(q: Fraction) -> np.float32:
    """the f32 nearest to the rational q, ties to even, subnormals included (no overflow in these tests)"""
    if q == 0:
        return np.float32(0.0)
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)
    m = round(a / Fraction(2) ** (e - 23))  # Fraction.__round__ rounds half to even
    return np.float32(sign * float(Fraction(m) * Fraction(2) ** (e - 23)))


def fma_exact(a: float, b: float, c: float) -> np.float32:
    return _round_f32(_frac(a) * _frac(b) + _frac(c))


def add_exact(a: float, b: float) -> np.float32:
    return _round_f32(_frac(a) + _frac(b))


def lane16_row(w: np.ndarray, x: np.ndarray) -> np.float32:
    """one output of the host matvec in exact arithmetic: 16 lane sums, lane j <- columns = j mod 16 in ascending
    order with one fused multiply-add each, then the pairwise fold (native/src/gemv.rs:45-58, 84-123)"""
    acc = [np.float32(0.0)] * 16
    for c in range(len(w)):
        acc[c % 16] = fma_exact(float(w[c]), float(x[c]), float(acc[c % 16]))
    t = [add_exact(acc[2 * j], acc[2 * j + 1]) for j in range(8)]
    u = [add_exact(t[2 * j], t[2 * j + 1]) for j in range(4)]
    return add_exact(add_exact(u[0], u[1]), add_exact(u[2], u[3]))


def conditioned_err(y: np.ndarray, w64: np.ndarray, x64: np.ndarray) -> float:
    """max |y - W x| / sum |w x| per output: the reference's conditioned error (native/tests/gemv.rs:113-130)"""
    ref = x64 @ w64.T
    scale = np.abs(x64) @ np.abs(w64).T
    return float(np.max(np.abs(y.astype(np.float64) - ref) / np.maximum(scale, 1e-300)))


def reference_logits(cfg, get, prompt):
    """the last position's logits of a Qwen3-style dense stack in f32 torch: the textbook forward pass"""
    H, D, Hq, Hk = cfg.hidden, cfg.head_dim, cfg.q_heads, cfg.kv_heads
    x = get("model.embed_tokens.weight")[torch.tensor(prompt)]
    T = x.shape[0]
    pos = torch.arange(T, dtype=torch.float32)
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, D // 2, dtype=torch.float32) * 2.0 / D))
    ang = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=-1)
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]

    def norm(v, wname):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + cfg.eps) * get(wname)

    def rope(v):
        rot = torch.cat([-v[..., D // 2 :], v[..., : D // 2]], dim=-1)
        return v * cos + rot * sin

    for i in range(cfg.layers):
        L = f"model.layers.{i}."
        h = norm(x, L + "input_layernorm.weight")
        q = (h @ get(L + "self_attn.q_proj.weight").T).reshape(T, Hq, D)
        k = (h @ get(L + "self_attn.k_proj.weight").T).reshape(T, Hk, D)
        v = (h @ get(L + "self_attn.v_proj.weight").T).reshape(T, Hk, D)
        q, k = rope(norm(q, L + "self_attn.q_norm.weight")), rope(norm(k, L + "self_attn.k_norm.weight"))
        k, v = k.repeat_interleave(Hq // Hk, dim=1), v.repeat_interleave(Hq // Hk, dim=1)
        s = torch.einsum("thd,shd->hts", q, k) / D**0.5
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
        a = torch.einsum("hts,shd->thd", s.softmax(-1), v).reshape(T, Hq * D)
        x = x + a @ get(L + "self_attn.o_proj.weight").T
        h = norm(x, L + "post_attention_layernorm.weight")
        g, u = h @ get(L + "mlp.gate_proj.weight").T, h @ get(L + "mlp.up_proj.weight").T
        x = x + (torch.nn.functional.silu(g) * u) @ get(L + "mlp.down_proj.weight").T
    x = norm(x, "model.norm.weight")
    return (x[-1] @ get("model.embed_tokens.weight").T).numpy()


def mx4_ggml(blocks, scales):
    """a checkpoint-layout MXFP4 matrix (blocks u8 [..., 16], scales u8 [...]) in ggml's layout: 17-byte blocks, the
    scale first, weights 0..15 in the low nibbles and 16..31 in the high (the reference's own test helper does the
    same repacking, native/src/gemv.rs:5192-5213)"""
    import numpy as np

    b = np.asarray(blocks, np.uint8).reshape(-1, 16)
    codes = np.stack([b & 0x0F, b >> 4], axis=-1).reshape(-1, 32)  # weight order
    raw = np.empty((b.shape[0], 17), np.uint8)
    raw[:, 0] = np.asarray(scales, np.uint8).reshape(-1)
    raw[:, 1:] = codes[:, :16] | (codes[:, 16:] << 4)
    return raw.reshape(-1)
