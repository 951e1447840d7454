"""Writes stay inside their buffers: every output of every operator sits between two poisoned fences, and the fences
must come back untouched - at the benchmark's real shapes and at odd ones (the reference fences its CPU kernels'
buffers with guard pages and poison the same way: native/tests/common/mod.rs:1-120, refs.rs:14-27, 116-142; there
is no sanitizer for the card in its CI either). Inputs are fenced with NaN so that a read past an input's end shows
up in the result wherever it is compared with an unfenced run."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from btb_amd import fp8, mxfp4
from btb_amd.decode import StackConfig, rope_tables
from btb_amd.moe import Experts, Router
from btb_amd.pack12 import P12Weight

from .helpers import acts_bf16, gen, weights_bf16

pytestmark = pytest.mark.gpu

FENCE = 512  # elements either side
POISON = {torch.bfloat16: 0x7FC1, torch.float32: 0x7FC0BAD0, torch.int32: 0x5A5A5A5A}
BITS = {torch.bfloat16: torch.int16, torch.float32: torch.int32, torch.int32: torch.int32}


class Fenced:
    """a contiguous tensor of `shape` inside a poisoned allocation"""

    def __init__(self, shape, dtype, fill=None):
        n = int(np.prod(shape))
        self.raw = torch.empty(n + 2 * FENCE, dtype=dtype, device="cuda")
        self.raw.view(BITS[dtype]).fill_(POISON[dtype])
        self.t = self.raw[FENCE : FENCE + n].view(*shape)
        if fill is not None:
            self.t.copy_(fill)
        self.before = self.raw[:FENCE].clone()
        self.after = self.raw[FENCE + n :].clone()
        self.n = n

    def check(self, what: str) -> None:
        torch.cuda.synchronize()
        b = BITS[self.raw.dtype]
        assert torch.equal(self.raw[:FENCE].view(b), self.before.view(b)), f"{what}: wrote before its output"
        assert torch.equal(self.raw[FENCE + self.n :].view(b), self.after.view(b)), f"{what}: wrote past its output"


def fin(t: torch.Tensor) -> torch.Tensor:
    """an input inside NaN fences"""
    return Fenced(tuple(t.shape), t.dtype, t.cuda()).t


@pytest.mark.parametrize("R,C", [(9728, 2560), (2560, 9728), (1000, 264), (7, 8), (3, 1032), (50, 96)])
@pytest.mark.parametrize("M", [1, 3, 4, 8, 17])
def test_matvec_outputs_stay_inside(card, R, C, M):
    w = fin(weights_bf16(R, C, seed=900))
    x = fin(acts_bf16(M, C, seed=901))
    y = Fenced((M, R), torch.bfloat16)
    card.gemv(w, x, y.t)
    y.check("gemv")
    assert torch.equal(y.t, card.gemv(w.clone(), x.clone()))            # and nothing of the fences was read
    f = Fenced((M, R), torch.float32)
    card.gemv_lane16(w, fin(x.float()), f.t)
    f.check("gemv_lane16")
    if R % 2 == 0:
        g = Fenced((M, R // 2), torch.bfloat16)
        card.gemv_glu_silu(w, x, g.t)
        g.check("gemv_glu_silu")
        assert torch.equal(g.t, card.gemv_glu_silu(w.clone(), x.clone()))
    if C % 16 == 0:
        pw = P12Weight.pack(w.clone(), card)
        y = Fenced((M, R), torch.bfloat16)
        card.gemv_p12(pw, x, y.t)
        y.check("gemv_p12")
    if C % 32 == 0:
        blocks, scales = mxfp4.quantize(w.float().cpu())
        mw = mxfp4.MxWeight(blocks.reshape(-1).cuda(), scales.reshape(-1).cuda(), R, C)
        y = Fenced((M, R), torch.bfloat16)
        card.gemv_mx4(mw, x, y.t)
        y.check("gemv_mx4")
    if R % 2 == 0 and C % 16 == 0:
        q, s = fp8.quantize(w.float().cpu(), (R // 2, 16))
        fw = fp8.F8Weight(q.view(torch.uint8).cuda(), s.cuda(), R, C)
        y = Fenced((M, R), torch.bfloat16)
        card.gemv_fp8(fw, x, y.t)
        y.check("gemv_fp8")


@pytest.mark.parametrize("M", [1, 2, 4])
def test_fused_matvec_outputs_stay_inside(card, M):
    H, I = 2560, 1216
    wgu = fin(weights_bf16(2 * I, H, seed=910))
    wd = fin(weights_bf16(H, I, seed=911))
    h = fin(acts_bf16(M, H, seed=912))
    yb = fin(acts_bf16(M, H, seed=913))
    ln = fin((1.0 + 0.1 * torch.randn(H, generator=gen(914))).to(torch.bfloat16))
    m = Fenced((M, I), torch.bfloat16)
    card.gemv_glu_silu(wgu, h, m.t)
    m.check("gemv_glu_silu")
    h2 = Fenced((M, H), torch.bfloat16)
    m2 = Fenced((M, I), torch.bfloat16)
    card.gemv_norm(wgu, h, yb, ln, 1e-6, h2.t, m2.t, glu=True)
    h2.check("gemv_norm: h_out")
    m2.check("gemv_norm: out")
    gu = Fenced((M, 2 * I), torch.bfloat16)
    card.gemv(wgu, h, gu.t)
    y = Fenced((M, H), torch.bfloat16)
    card.gemv_silu(wd, gu.t, y.t)
    y.check("gemv_silu")
    mm = Fenced((M, I), torch.bfloat16)
    card.silu_mul(gu.t, mm.t)
    mm.check("silu_mul")
    hh = Fenced((M, H), torch.bfloat16, h)
    x = Fenced((M, H), torch.bfloat16)
    card.add_rmsnorm(hh.t, yb, ln, 1e-6, x.t)
    hh.check("add_rmsnorm: h")
    x.check("add_rmsnorm: x")


@pytest.mark.parametrize("n0,T,S", [(4095, 1, 32), (100, 1, 5), (63, 3, 7), (0, 1, 1), (125, 8, 2), (250, 3, 2)])
def test_attention_outputs_stay_inside(card, n0, T, S):
    Hq, Hk, D = 32, 8, 128
    cap = n0 + T + 2
    g = gen(920 + n0)
    K = Fenced((Hk, cap, D), torch.bfloat16, torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda())
    V = Fenced((Hk, cap, D), torch.bfloat16, torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda())
    qkv = fin(torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16))
    wq = fin(torch.ones(D, dtype=torch.bfloat16))
    cfg = StackConfig(layers=1, hidden=256, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=256, vocab=256)
    cos, sin = rope_tables(cfg, cap, "cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scratch = Fenced((int(card.lib.btb_hip_attn_scratch_floats(T, Hq, Hk, D, S)),), torch.float32)
    q = Fenced((T, Hq * D), torch.bfloat16)
    att = Fenced((T, Hq * D), torch.bfloat16)
    card.norm_rope_kv(qkv, wq, wq, 1e-6, cos, sin, n0t, K.t, V.t, q.t, Hq, Hk, D)
    card.attn_decode(q.t, K.t, V.t, att.t, n0t, Hq, Hk, D, D**-0.5, S, scratch.t)
    for f, what in ((K, "K"), (V, "V"), (q, "q"), (att, "att"), (scratch, "scratch")):
        f.check(f"norm_rope_kv + attn_decode: {what}")
    if T == 1:
        att2 = Fenced((1, Hq * D), torch.bfloat16)
        card.attn_decode_qkv(qkv, wq, wq, 1e-6, cos, sin, n0t, K.t, V.t, att2.t, Hq, Hk, D, D**-0.5, S, scratch.t)
        for f, what in ((K, "K"), (V, "V"), (att2, "att"), (scratch, "scratch")):
            f.check(f"attn_decode_qkv: {what}")
        assert torch.equal(att2.t, att.t)
    if card.attn_rows_fused(T, Hq, Hk, D, cap, S):
        att3 = Fenced((T, Hq * D), torch.bfloat16)
        card.attn_decode_qkv_rows(qkv, wq, wq, 1e-6, cos, sin, n0t, K.t, V.t, att3.t, Hq, Hk, D, D**-0.5, S, scratch.t)
        for f, what in ((K, "K"), (V, "V"), (att3, "att"), (scratch, "scratch")):
            f.check(f"attn_decode_qkv_rows: {what}")
        assert torch.equal(att3.t, att.t)


@pytest.mark.parametrize("n0", [100, 117, 127])
def test_step_attention_writes_no_row_past_the_caches_end(card, n0):
    """spans are whole 128-key batches, so a span can reach past the cache's last slot: a cache length at or past the
    capacity (a caller that did not count its rows) must leave K and V - fenced - untouched"""
    Hq, Hk, D, cap, S = 32, 8, 128, 100, 1
    g = gen(925)
    K = Fenced((Hk, cap, D), torch.bfloat16, torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda())
    V = Fenced((Hk, cap, D), torch.bfloat16, torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda())
    K0, V0 = K.t.clone(), V.t.clone()
    qkv = fin(torch.randn(1, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16))
    wq = fin(torch.ones(D, dtype=torch.bfloat16))
    cfg = StackConfig(layers=1, hidden=256, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=256, vocab=256)
    cos, sin = rope_tables(cfg, 128, "cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scratch = Fenced((int(card.lib.btb_hip_attn_scratch_floats(1, Hq, Hk, D, S)),), torch.float32)
    att = Fenced((1, Hq * D), torch.bfloat16)
    card.attn_decode_qkv(qkv, wq, wq, 1e-6, cos, sin, n0t, K.t, V.t, att.t, Hq, Hk, D, D**-0.5, S, scratch.t)
    for f, what in ((K, "K"), (V, "V"), (att, "att"), (scratch, "scratch")):
        f.check(f"attn_decode_qkv past the end: {what}")
    assert torch.equal(K.t, K0) and torch.equal(V.t, V0)


@pytest.mark.parametrize("T", [1, 5])
def test_moe_outputs_stay_inside(card, T):
    E, k, H, I = 16, 4, 2048, 768
    g = gen(930)
    wr = fin((torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16))
    gu = fin((torch.randn(E, 2 * I, H, generator=g) * 0.02).to(torch.bfloat16))
    dn = fin((torch.randn(E, H, I, generator=g) * 0.02).to(torch.bfloat16))
    x = fin(acts_bf16(T, H, seed=931))
    _, weights, picks = Router(card, wr, k)(x)
    y = Fenced((T, H), torch.bfloat16)
    scratch = Fenced((T, k, 2 * I), torch.bfloat16)
    card.moe_experts(gu, dn, x, picks, weights, y.t, scratch.t)
    y.check("moe_experts: y")
    scratch.check("moe_experts: scratch")
    want = Experts(card, gu.clone(), dn.clone())(x.clone(), picks, weights)
    assert torch.equal(y.t, want)
