"""TEST INFRASTRUCTURE - one dense decode step as the reference computes it with bf16 rows, in numpy over the oracle's
C matvec. The op sequence and every bf16 rounding point follow the reference's card graph and fused modules:

  residual + RMSNorm      native/cuda/btb_kernels.cu:360-393; btb/engine/fused.py:14-30 (f32 throughout, one rounding)
  q/k norm, rope          native/cuda/btb_kernels.cu:295-326; btb/engine/fused.py:45-58 (q*cos rounded, then addcmul)
  matvecs                 native/src/gemv.rs (the host's 16-lane order, f32), output rounded to bf16
  attention               native/src/attn.rs via native/src/lib.rs:554-598: f32 scores, softmax, p . V (here in f64,
                          the reference's own yardstick: native/tests/common/refs.rs:202-211), output rounded to bf16
  SwiGLU                  native/cuda/btb_kernels.cu:157-166, 470-479: bf16(bf16(silu(g)) * u)
  greedy pick             native/src/sample.rs:53-67: the largest logit, the lowest index on ties

Weights are bf16 bit patterns (uint16 arrays); activations are f32 arrays holding bf16 values.

Every function takes `dt`: "bf16" (the card's rounding points, what the GPU path computes) or "f32" (no rounding of
activations anywhere: the reference's default host path, btb/engine/fused.py:14-67 with f32 rows), the form the
reference's banked receipts were written with (tests/make_fixtures.py:1230-1264).

Pinned on the CPU by tests/test_oracle_decode.py: `step` in f32 against the reference's receipts_qwen3.pt (logits to
1e-4, the cached K / V rows, the greedy tokens) and in bf16 at the card's bar; `attention` against a brute-force
f64 softmax written out key by key; `norm_rope` against the textbook rotate-half on hand cases; `add_rmsnorm` and
`silu_mul` against closed forms.
"""

from __future__ import annotations

import numpy as np

import oracle
from oracle import codecs

R = codecs.round_bf16


def _r(dt: str):
    """the rounding applied at a rounding point: bf16 RNE for bf16 rows, nothing for f32 rows"""
    if dt == "bf16":
        return R
    if dt == "f32":
        return lambda a: np.asarray(a, np.float32)
    raise ValueError(f"dt is 'bf16' or 'f32', got {dt!r}")


def f32(bits: np.ndarray) -> np.ndarray:
    return codecs.bf16_bits_to_f32(bits)


def add_rmsnorm(h: np.ndarray, y, w_bits: np.ndarray, eps: float, dt: str = "bf16"):
    """(h', x): h' = bf16(h + y), x = bf16(h' * rsqrt(mean(h'^2) + eps) * w)"""
    R = _r(dt)
    if y is not None:
        h = R((h + y).astype(np.float32))
    ss = np.sum(h.astype(np.float64) ** 2, axis=-1, keepdims=True)
    rstd = (1.0 / np.sqrt(ss / h.shape[-1] + eps)).astype(np.float32)
    return h, R((h * rstd * f32(w_bits)).astype(np.float32))


def matvec(w_bits: np.ndarray, x: np.ndarray, dt: str = "bf16") -> np.ndarray:
    return _r(dt)(oracle.gemv_bf16(w_bits, x.astype(np.float32), threads=0))


def rope_tables(head_dim: int, theta: float, positions: int, dt: str = "bf16"):
    half = head_dim // 2
    inv = (1.0 / (np.float32(theta) ** (np.arange(0, half, dtype=np.float32) * np.float32(2.0) / np.float32(head_dim))))
    ang = np.arange(positions, dtype=np.float32)[:, None] * inv.astype(np.float32)[None, :]
    emb = np.concatenate([ang, ang], axis=-1).astype(np.float32)
    return _r(dt)(np.cos(emb).astype(np.float32)), _r(dt)(np.sin(emb).astype(np.float32))


def norm_rope(v: np.ndarray, wn_bits, eps: float, cos: np.ndarray, sin: np.ndarray, dt: str = "bf16") -> np.ndarray:
    """v [heads, D] bf16 values -> normed and rotated, bf16 values"""
    R = _r(dt)
    D = v.shape[-1]
    if wn_bits is not None:
        ss = np.sum(v.astype(np.float64) ** 2, axis=-1, keepdims=True)
        rstd = (1.0 / np.sqrt(ss / D + eps)).astype(np.float32)
        v = R((v * rstd * f32(wn_bits)).astype(np.float32))
    rot = np.concatenate([-v[:, D // 2 :], v[:, : D // 2]], axis=-1)
    qc = R((v * cos).astype(np.float32))
    return R((rot.astype(np.float64) * sin.astype(np.float64) + qc.astype(np.float64)).astype(np.float32))


def attention(q: np.ndarray, K: np.ndarray, V: np.ndarray, scale: float, dt: str = "bf16") -> np.ndarray:
    """q [Hq, D], K / V [Hk, n, D] (bf16 values) -> [Hq, D] bf16 values; query head j reads kv head j // (Hq / Hk)"""
    Hq, D = q.shape
    Hk = K.shape[0]
    G = Hq // Hk
    out = np.empty((Hq, D), np.float32)
    for j in range(Hq):
        g = j // G
        s = (K[g].astype(np.float64) @ q[j].astype(np.float64)) * scale
        p = np.exp(s - s.max())
        out[j] = (p @ V[g].astype(np.float64) / p.sum()).astype(np.float32)
    return _r(dt)(out)


def silu_mul(gu: np.ndarray, dt: str = "bf16") -> np.ndarray:
    R = _r(dt)
    I = gu.shape[-1] // 2
    g, u = gu[..., :I], gu[..., I:]
    s = R((g / (np.float32(1.0) + np.exp(-g).astype(np.float32))).astype(np.float32))
    return R((s * u).astype(np.float32))


def step(cfg, W: dict, token: int, kv: np.ndarray, n0: int, dt: str = "bf16", trace: list | None = None):
    """One row's step. cfg has layers, hidden, q_heads, kv_heads, head_dim, intermediate, vocab, eps, rope_theta; W
    maps names to bf16 bit patterns; kv [layers, 2, Hk, cap, D] f32 holding values of dt, updated in place at slot n0.
    Returns (logits as values of dt [vocab], picked token). `trace`, when a list, receives what stands between the
    layers: entry i is (h, y) as layer i finds them - the residual and the block output not yet added to it (None
    before layer 0) - and entry `layers` what the last layer leaves."""
    Hq, Hk, D = cfg.q_heads, cfg.kv_heads, cfg.head_dim
    cos, sin = rope_tables(D, cfg.rope_theta, n0 + 1, dt)
    cos, sin = cos[n0], sin[n0]
    h = f32(W["embed"][token])[None, :]
    y = None
    for i in range(cfg.layers):
        L = f"layers.{i}."
        if trace is not None:
            trace.append((h.copy(), None if y is None else y.copy()))
        h, x = add_rmsnorm(h, y, W[L + "ln1"], cfg.eps, dt)
        qkv = matvec(W[L + "qkv"], x, dt)[0]
        q = norm_rope(qkv[: Hq * D].reshape(Hq, D), W.get(L + "wq"), cfg.eps, cos, sin, dt)
        k = norm_rope(qkv[Hq * D : (Hq + Hk) * D].reshape(Hk, D), W.get(L + "wk"), cfg.eps, cos, sin, dt)
        v = qkv[(Hq + Hk) * D :].reshape(Hk, D)
        kv[i, 0, :, n0] = k
        kv[i, 1, :, n0] = v
        att = attention(q, kv[i, 0, :, : n0 + 1], kv[i, 1, :, : n0 + 1], 1.0 / np.sqrt(D), dt)
        y = matvec(W[L + "o"], att.reshape(1, -1), dt)
        h, x = add_rmsnorm(h, y, W[L + "ln2"], cfg.eps, dt)
        gu = matvec(W[L + "gu"], x, dt)
        y = matvec(W[L + "down"], silu_mul(gu, dt), dt)
    if trace is not None:
        trace.append((h.copy(), None if y is None else y.copy()))
    h, x = add_rmsnorm(h, y, W["norm"], cfg.eps, dt)
    logits = matvec(W["head"], x, dt)[0]
    return logits, int(np.argmax(logits))
