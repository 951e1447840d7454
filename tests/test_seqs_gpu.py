"""A pass whose rows are sequences of their own, a token each (the reference's rows layout,
native/cuda/btb_kernels.cu:232-249: a fork's rows share one prefix, a batch's prefixes lie end to end, every row's step
i in one stretch of W cache slots): `btb_hip_norm_rope_kv_seqs` + `btb_hip_attn_decode_seqs`, and the same two by the
reference's kernel names.

The law the reference states for the layout - "a row's bits are its own decode's whatever rows step beside it" - is
the test: each row's sequence is gathered into a cache of its own, stepped alone through `btb_hip_norm_rope_kv` and
`btb_hip_attn_decode_parts` at one row with the same spans, and the pass must leave those bits (q, the K / V row
written, the attention output). The values themselves are held to the CPU restatement (oracle/decode.py) over the
gathered keys, at the attention's yardstick (worst error against f64 over the largest value, 2^-7)."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from btb_amd import card_launch as cl
from btb_amd.decode import StackConfig, rope_tables
from oracle import decode as od

from .helpers import gen

pytestmark = pytest.mark.gpu

D = 128


def _slots(base, steps, W, row):
    """cache slots of a row's keys in logical order: its prefix, its earlier steps, and this pass's step"""
    col, off, n = row
    return [off + j for j in range(n)] + [base + i * W + col for i in range(steps + 1)]


def _case(kind: str, seed: int):
    g = gen(seed)
    if kind == "fork":      # four rows over one prefix of 700 keys, three steps taken so far
        rows = [(c, 16, 700) for c in (0, 1, 2, 3)]
        base, steps, W = 1024, 3, 4
    elif kind == "batch":   # five rows, prefixes of their own end to end, the pass's columns out of order
        lens = [0, 1, 127, 300, 513]
        offs = np.concatenate([[0], np.cumsum(lens)[:-1]]).tolist()
        rows = [(c, o, n) for c, o, n in zip((4, 2, 0, 1, 3), offs, lens)]
        base, steps, W = 960, 0, 6
    else:                   # one row, deep into its own steps
        rows = [(0, 5, 40)]
        base, steps, W = 64, 200, 1
    cap = base + (steps + 1) * W + 8
    return g, rows, base, steps, W, cap


@pytest.mark.parametrize("kind,Hq,Hk,span,S,win,pad", [("fork", 32, 8, 128, 6, 0, 0), ("batch", 16, 4, 256, 3, 0, 3),
                                                       ("batch", 8, 8, 512, 2, 100, 0), ("alone", 8, 2, 128, 2, 0, 1),
                                                       ("fork", 16, 2, 512, 2, 64, 2)])
def test_a_pass_of_sequences_is_each_sequences_own_step(card, kind, Hq, Hk, span, S, win, pad):
    g, rows, base, steps, W, cap = _case(kind, 4100 + Hq + S)
    B, T = len(rows), len(rows) + pad
    cfg = StackConfig(layers=1, hidden=64, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=64, vocab=8)
    cos, sin = rope_tables(cfg, 2048, "cuda")
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
    wq = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    wk = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    scale = 1.0 / np.sqrt(D)
    K0, V0 = K.clone(), V.clone()

    # each sequence alone: its keys gathered into a cache of its own, one row stepped through the two kernels
    alone = []
    for t, row in enumerate(rows):
        sl = torch.tensor(_slots(base, steps, W, row), device="cuda")
        pos = len(sl) - 1
        K1 = torch.zeros(Hk, pos + 4, D, dtype=torch.bfloat16, device="cuda")
        V1 = torch.zeros_like(K1)
        K1[:, :pos], V1[:, :pos] = K0[:, sl[:-1]], V0[:, sl[:-1]]
        q1 = torch.zeros(1, Hq * D, dtype=torch.bfloat16, device="cuda")
        n0t = torch.tensor([pos], dtype=torch.int32, device="cuda")
        card.norm_rope_kv(qkv[t : t + 1].contiguous(), wq, wk, 1e-6, cos, sin, n0t, K1, V1, q1, Hq, Hk, D)
        att1 = torch.zeros(1, Hq * D, dtype=torch.bfloat16, device="cuda")
        pm, pl = (torch.zeros(Hq * S, dtype=torch.float32, device="cuda") for _ in range(2))
        pa = torch.zeros(Hq * S * D, dtype=torch.float32, device="cuda")
        p = lambda x: ctypes.c_void_p(x.data_ptr())
        rc = card.lib.btb_hip_attn_decode_parts(p(q1), p(K1), p(V1), p(att1), p(n0t), None, 1, Hq, Hk, D, K1.stride(0),
                                                K1.stride(1), scale, span, S, win, None, p(pm), p(pl), p(pa), None)
        assert rc == 0, card.lib.btb_hip_last_error()
        alone.append((q1, K1[:, pos].clone(), V1[:, pos].clone(), att1, K1, V1, pos))
    torch.cuda.synchronize()

    # the pass: all the rows at once over the shared cache, padding rows behind them
    rw = card.rows_layout(base, steps, W, rows, pad_to=T)
    q = torch.full((T, Hq * D), 7.0, dtype=torch.bfloat16, device="cuda")
    att = torch.full((T, Hq * D), 9.0, dtype=torch.bfloat16, device="cuda")
    card.norm_rope_kv_seqs(qkv, wq, wk, 1e-6, cos, sin, rw, K, V, q, Hq, Hk, D)
    pm, pl = (torch.zeros(T * Hq * S, dtype=torch.float32, device="cuda") for _ in range(2))
    pa = torch.zeros(T * Hq * S * D, dtype=torch.float32, device="cuda")
    card.attn_decode_seqs(q, K, V, att, rw, Hq, Hk, D, scale, span, S, pm, pl, pa, win=win)
    torch.cuda.synchronize()
    written = set()
    for t, row in enumerate(rows):
        q1, k1, v1, att1, K1, V1, pos = alone[t]
        slot = _slots(base, steps, W, row)[-1]
        written.add(slot)
        assert torch.equal(q[t], q1[0]), t
        assert torch.equal(K[:, slot], k1) and torch.equal(V[:, slot], v1), t
        assert torch.equal(att[t], att1[0]), t
        first = max(pos + 1 - win, 0) if win else 0
        want = od.attention(q1[0].float().cpu().numpy().reshape(Hq, D), K1[:, first : pos + 1].float().cpu().numpy(),
                            V1[:, first : pos + 1].float().cpu().numpy(), scale)
        got = att[t].float().cpu().numpy().reshape(Hq, D)
        assert np.abs(got - want).max() / np.abs(want).max() <= 2.0**-7, t
    # padding rows: nothing computed; the cache: the rows' own step slots and nothing else
    assert torch.all(q[B:] == 7.0) and torch.all(att[B:] == 9.0)
    keep = torch.ones(cap, dtype=torch.bool, device="cuda")
    keep[torch.tensor(sorted(written), device="cuda")] = False
    assert torch.equal(K[:, keep], K0[:, keep]) and torch.equal(V[:, keep], V0[:, keep])
    assert len(written) == B


def test_the_rows_kernels_by_the_references_names(card):
    """`k.btb_norm_rope_kv_rows(D, ...)` and `k.btb_attn_flash_rows(D, ...)` as the reference's step calls them
    (btb/engine/cuda.py:1737-1756; parameters in the kernels' own order, grid[1] key groups of 512 keys) leave the bits
    of the library's own two calls"""
    Hq, Hk, S = 16, 4, 2
    g, rows, base, steps, W, cap = _case("batch", 4200)
    T = len(rows) + 1
    cfg = StackConfig(layers=1, hidden=64, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=64, vocab=8)
    cos, sin = rope_tables(cfg, 2048, "cuda")
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
    wq = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    scale = 1.0 / np.sqrt(D)
    rw = card.rows_layout(base, steps, W, rows, pad_to=T)
    outs = []
    for by_name in (False, True):
        Kc, Vc = K.clone(), V.clone()
        q = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        pm, pl = (torch.zeros(T * Hq * S, dtype=torch.float32, device="cuda") for _ in range(2))
        pa = torch.zeros(T * Hq * S * D, dtype=torch.float32, device="cuda")
        if by_name:
            k = card
            hs, rs = cl.CacheHeadStride(Kc.stride(0)), cl.CacheRowStride(Kc.stride(1))
            k.btb_norm_rope_kv_rows(D, (Hq + 2 * Hk, T, 1), (32, 1, 1), k.ptr(cl.Qkv, qkv), k.ptr(cl.QNorm, wq),
                                    k.ptr(cl.KNorm, None), cl.NormEps(1e-6), k.ptr(cl.RopeCos, cos), k.ptr(cl.RopeSin, sin),
                                    k.ptr(cl.RowsLayout, rw), k.ptr(cl.KCache, Kc), k.ptr(cl.VCache, Vc), k.ptr(cl.Query, q),
                                    cl.Rows(T), cl.QHeads(Hq), cl.KvHeads(Hk), hs, rs, cl.NormCentered(0))
            k.btb_attn_flash_rows(D, (T, S, Hk), (128, 1, 1), k.ptr(cl.Query, q), k.ptr(cl.KCache, Kc), k.ptr(cl.VCache, Vc),
                                  k.ptr(cl.AttnOut, att), k.ptr(cl.RowsLayout, rw), cl.Rows(T), cl.QHeads(Hq),
                                  cl.KvHeads(Hk), hs, rs, cl.AttnScale(scale), k.ptr(cl.PartMax, pm), k.ptr(cl.PartSum, pl),
                                  k.ptr(cl.PartAcc, pa), k.ptr(cl.Arrivals, None), cl.Window(0))
        else:
            card.norm_rope_kv_seqs(qkv, wq, None, 1e-6, cos, sin, rw, Kc, Vc, q, Hq, Hk, D)
            card.attn_decode_seqs(q, Kc, Vc, att, rw, Hq, Hk, D, scale, 512, S, pm, pl, pa)
        torch.cuda.synchronize()
        outs.append((q, att, Kc, Vc))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert bool(outs[0][1].float().abs().sum() > 0)
    assert card.fn["btb_attn_flash_rows_d128"] == "btb_hip_attn_decode_seqs"
    assert card.fn["btb_norm_rope_kv_rows_d128"] == "btb_hip_norm_rope_kv_seqs"


def test_refusals(card):
    Hq, Hk, S, T = 8, 2, 2, 2
    z = lambda *s, dt=torch.bfloat16: torch.zeros(*s, dtype=dt, device="cuda")
    K, V, q, att = z(Hk, 256, D), z(Hk, 256, D), z(T, Hq * D), z(T, Hq * D)
    rw = card.rows_layout(128, 0, 2, [(0, 0, 10), (1, 10, 20)])
    pm, pl, pa = z(T * Hq * S, dt=torch.float32), z(T * Hq * S, dt=torch.float32), z(T * Hq * S * D, dt=torch.float32)
    p = lambda x: None if x is None else ctypes.c_void_p(x.data_ptr())
    call = lambda rwp, span: card.lib.btb_hip_attn_decode_seqs(p(q), p(K), p(V), p(att), rwp, T, Hq, Hk, D, K.stride(0),
                                                               K.stride(1), 0.1, span, S, 0, p(pm), p(pl), p(pa), None)
    assert call(None, 128) == -1                       # no layout
    assert call(p(rw), 100) == -6                      # a span that is not whole batches of 128 keys
    assert call(p(rw), 128) == 0
    with pytest.raises(ValueError):                    # a layout too short for the pass's rows
        card.attn_decode_seqs(q, K, V, att, rw[:6].contiguous(), Hq, Hk, D, 0.1, 128, S, pm, pl, pa)
    with pytest.raises(ValueError):
        card.attn_decode_seqs(q, K, V, att, rw, Hq, Hk, D, 0.1, 128, S, pm[:3], pl, pa)
    torch.cuda.synchronize()
