"""TEST INFRASTRUCTURE - the routed MoE layer as the reference's CPU path computes it, in numpy over the oracle's C
matvec. Follows:

  router     btb/engine/families/qwen4/router.py:43-51: logits = W_r x (f32, the host matvec), f32 softmax over all
             experts, top k (torch.topk: value descending; on equal values the lower index, the rule the card's
             kernel states at native/cuda/btb_kernels.cu:848-851), weights / their sum, cast to the rows' dtype
  experts    btb/engine/host.py:508-569 (one row) and :906-967 (several): per selected expert gu = W_gu x (f32) ->
             rows' dtype -> silu(gate) * up on the two halves (host.py:439-441) -> f32 -> W_dn h (f32) -> rows' dtype
             -> times the pick's weight -> summed into the row in ASCENDING expert order, every step in the rows'
             dtype

  grouping   btb/engine/host.py:283-296 (`group_picks`): the call's (pick, row) pairs in one stable sort by expert, an
             expert's pairs pick-major then row, with each expert's offset and count

  MXFP4 experts  the same experts over `btb_gemv_mxfp4_rows` on the stacks as stored (host.py:459-461 picks
             `Native.gemv_mx4_group` for them); gpt-oss's form of the middle (host.py:414-451): the expert's bias added
             to the rounded gate_up product, the halves INTERLEAVED (gate the even rows), gate clamped to <= limit, up
             to +-limit, (up + 1) * (gate * sigmoid(alpha * gate)), every torch operation a rounding in the rows'
             dtype; the down bias added after the down product's rounding and before the pick's weight (:427-432)

`dt` is the rows' dtype: "bf16" (the engine running bf16 rows, what the GPU path computes) or "f32".

Pinned on the CPU by tests/test_oracle_moe.py: the f32 layer against an independent plain-torch layer (softmax,
torch.topk, renormalisation, dense per-token expert sums) to 1e-5; hand cases that a swapped gate / up half, a dropped
renormalisation, a descending expert sum (bf16, where the order shows) or the wrong tie rule fail; `group_picks`
against the one-hot / torch.where listing the reference's docstring names; the gpt-oss experts (f32) against
transformers' `GptOssExperts` over the dequantised stacks, its rounding points (bf16) against the same expression
evaluated by torch on bf16 tensors, and planted mistakes (concatenated halves, no clamp, `up` without its + 1, the bias
after the gate) that each move the result past the bar.
"""

from __future__ import annotations

import numpy as np

import oracle
from oracle import codecs


def _as(dt: str, a: np.ndarray) -> np.ndarray:
    a = np.asarray(a, dtype=np.float32)
    return codecs.round_bf16(a) if dt == "bf16" else a


def router(w_router_bits: np.ndarray, x: np.ndarray, k: int, dt: str = "bf16", norm_topk: bool = True):
    """x [T, H] (values of the rows' dtype, as f32) -> (logits f32 [T, E], weights [T, k] in dt, experts int64 [T, k])"""
    logits = oracle.gemv_bf16(w_router_bits, np.asarray(x, np.float32), threads=0)
    m = logits.max(axis=-1, keepdims=True)
    e = np.exp((logits - m).astype(np.float32)).astype(np.float32)
    probs = (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)
    # value descending, index ascending on ties: a stable sort of the negated values
    order = np.argsort(-probs, axis=-1, kind="stable")[:, :k]
    top = np.take_along_axis(probs, order, axis=-1)
    if norm_topk:
        s = np.zeros(top.shape[0], np.float32)
        for j in range(k):
            s = (s + top[:, j]).astype(np.float32)
        top = (top / s[:, None]).astype(np.float32)
    return logits, _as(dt, top), order.astype(np.int64)


def group_picks(picks: np.ndarray, num_experts: int):
    """picks [T, k] -> (pick position, row) of every pair sorted by expert (stable, so pick-major then row within an
    expert), and each expert's offset and count into them (btb/engine/host.py:283-296)"""
    picks = np.asarray(picks)
    T = picks.shape[0]
    flat = picks.T.reshape(-1)
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=int(num_experts)).astype(np.int64)
    offs = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int64)
    return order // T, order % T, offs, counts


def silu(g: np.ndarray) -> np.ndarray:
    g = np.asarray(g, np.float32)
    return (g / (np.float32(1.0) + np.exp(-g).astype(np.float32))).astype(np.float32)


def experts(gate_up_bits: np.ndarray, down_bits: np.ndarray, x: np.ndarray, picks: np.ndarray, weights: np.ndarray,
            dt: str = "bf16") -> np.ndarray:
    """gate_up [E, 2I, H] and down [E, H, I] as bf16 bit patterns, x [T, H], picks [T, k], weights [T, k] (values of
    dt) -> [T, H] in dt"""
    x = np.asarray(x, np.float32)
    T, H = x.shape
    I = down_bits.shape[2]
    final = np.zeros((T, H), np.float32)
    for e in sorted(set(int(v) for v in picks.reshape(-1))):
        tok, pos = np.nonzero(picks == e)
        cur = x[tok]
        gu = _as(dt, oracle.gemv_bf16(gate_up_bits[e], cur, threads=0))
        act = _as(dt, silu(gu[:, :I]))            # the activation is one op in the rows' dtype ...
        h = _as(dt, act * gu[:, I:])               # ... and the product another
        d = _as(dt, oracle.gemv_bf16(down_bits[e], h, threads=0))
        contrib = _as(dt, d * np.asarray(weights, np.float32)[tok, pos, None])
        for i, t in enumerate(tok):                # index_add_ in ascending expert order, each add in dt
            final[t] = _as(dt, final[t] + contrib[i])
    return final


def sigmoid(v: np.ndarray) -> np.ndarray:
    v = np.asarray(v, np.float32)
    return (np.float32(1.0) / (np.float32(1.0) + np.exp(-v).astype(np.float32))).astype(np.float32)


def gpt_oss_gate(gate_up: np.ndarray, alpha: float, limit: float, dt: str = "bf16") -> np.ndarray:
    """[n, 2I] (values of dt) -> [n, I]: `gpt_oss_gate` (btb/engine/host.py:443-451), one rounding an operation"""
    gate, up = gate_up[..., 0::2], gate_up[..., 1::2]
    gate = np.minimum(gate, np.float32(limit))
    up = np.clip(up, np.float32(-limit), np.float32(limit))
    t = _as(dt, gate * np.float32(alpha))
    glu = _as(dt, gate * _as(dt, sigmoid(t)))
    return _as(dt, _as(dt, up + np.float32(1.0)) * glu)


def experts_mx4(gu_blocks, gu_scales, dn_blocks, dn_scales, x, picks, weights, dt: str = "bf16", oss: bool = True,
                gu_bias=None, dn_bias=None, alpha: float = 1.702, limit: float = 7.0) -> np.ndarray:
    """MXFP4 stacks as stored - gu_blocks u8 [E, 2I, H/32, 16], gu_scales u8 [E, 2I, H/32], dn_blocks u8
    [E, H, I/32, 16], dn_scales u8 [E, H, I/32] - x [T, H], picks and weights [T, k], the biases (values of dt, [E, 2I]
    and [E, H]) or None -> [T, H] in dt. `oss`: gpt-oss's middle; else silu(gate) * up on concatenated halves."""
    x = np.asarray(x, np.float32)
    T, H = x.shape
    I = dn_scales.shape[2] * 32
    final = np.zeros((T, H), np.float32)
    for e in sorted(set(int(v) for v in picks.reshape(-1))):
        tok, pos = np.nonzero(picks == e)
        gu = _as(dt, oracle.gemv_mxfp4(gu_blocks[e], gu_scales[e], 2 * I, H, x[tok], threads=0))
        if oss:
            if gu_bias is not None:
                gu = _as(dt, gu + np.asarray(gu_bias, np.float32)[e][None, :])
            h = gpt_oss_gate(gu, alpha, limit, dt)
        else:
            h = _as(dt, _as(dt, silu(gu[:, :I])) * gu[:, I:])
        d = _as(dt, oracle.gemv_mxfp4(dn_blocks[e], dn_scales[e], H, I, h, threads=0))
        if dn_bias is not None:
            d = _as(dt, d + np.asarray(dn_bias, np.float32)[e][None, :])
        contrib = _as(dt, d * np.asarray(weights, np.float32)[tok, pos, None])
        for i, t in enumerate(tok):
            final[t] = _as(dt, final[t] + contrib[i])
    return final


def layer(w_router_bits, gate_up_bits, down_bits, x, k: int, dt: str = "bf16"):
    logits, w, picks = router(w_router_bits, x, k, dt)
    return experts(gate_up_bits, down_bits, x, picks, w, dt), logits, w, picks
