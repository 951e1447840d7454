"""The decode step's kernels between the matvecs, each against its numpy restatement in oracle/decode.py.

Elementwise kernels round to bf16 where the reference's card kernels do; their f32 intermediates (rsqrt, exp) may
differ from numpy's in the last bit, which can flip a bf16 rounding: outputs are held to one bf16 ulp (2^-7 relative,
elementwise, plus an absolute floor of one ulp of the row's largest value). Attention is held to the reference's own
yardstick, the worst relative error against f64 (native/tests/common/refs.rs:202-211), at the full 4096-key context."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from btb_amd.decode import StackConfig, rope_tables
from oracle import codecs
from oracle import decode as od

from .helpers import acts_bf16, bits16, gen, weights_bf16

pytestmark = pytest.mark.gpu


def ulp_close(got: torch.Tensor, want: np.ndarray, ulps: float = 1.0) -> None:
    g = got.float().cpu().numpy().reshape(want.shape)
    tol = ulps * 2.0**-7 * (np.abs(want) + np.abs(want).max() * 2.0**-7)
    bad = np.abs(g - want) > tol
    assert not bad.any(), (int(bad.sum()), float(np.abs(g - want).max()))


@pytest.mark.parametrize("T,H", [(1, 2560), (3, 2048), (2, 100)])
@pytest.mark.parametrize("with_y", [True, False])
def test_add_rmsnorm(card, T, H, with_y):
    h = acts_bf16(T, H, seed=600)
    y = acts_bf16(T, H, seed=601) if with_y else None
    w = (1.0 + 0.1 * torch.randn(H, generator=gen(602))).to(torch.bfloat16)
    hg, x = h.clone().cuda(), torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
    card.add_rmsnorm(hg, None if y is None else y.cuda(), w.cuda(), 1e-6, x)
    h2, want = od.add_rmsnorm(h.float().numpy(), None if y is None else y.float().numpy(), bits16(w), 1e-6)
    assert np.array_equal(hg.float().cpu().numpy(), h2)          # the residual add is exact bf16 arithmetic
    ulp_close(x, want)


@pytest.mark.parametrize("T", [1, 3])
def test_norm_rope_kv(card, T):
    Hq, Hk, D, cap, n0 = 8, 2, 128, 64, 37
    qkv = acts_bf16(T, (Hq + 2 * Hk) * D, seed=610)
    wq = (1.0 + 0.1 * torch.randn(D, generator=gen(611))).to(torch.bfloat16)
    wk = (1.0 + 0.1 * torch.randn(D, generator=gen(612))).to(torch.bfloat16)
    from btb_amd.decode import StackConfig, rope_tables

    cfg = StackConfig(layers=1, hidden=256, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=256, vocab=256)
    cos, sin = rope_tables(cfg, cap, "cuda")
    ocos, osin = od.rope_tables(D, cfg.rope_theta, cap)
    ulp_close(cos, ocos)   # the two tables agree to a rounding of cos / sin
    K = torch.zeros(Hk, cap, D, dtype=torch.bfloat16, device="cuda")
    V = torch.zeros_like(K)
    q = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    card.norm_rope_kv(qkv.cuda(), wq.cuda(), wk.cuda(), 1e-6, cos, sin, n0t, K, V, q, Hq, Hk, D)
    cosn, sinn = cos.float().cpu().numpy(), sin.float().cpu().numpy()
    for t in range(T):
        row = qkv[t].float().numpy()
        wantq = od.norm_rope(row[: Hq * D].reshape(Hq, D), bits16(wq), 1e-6, cosn[n0 + t], sinn[n0 + t])
        wantk = od.norm_rope(row[Hq * D : (Hq + Hk) * D].reshape(Hk, D), bits16(wk), 1e-6, cosn[n0 + t], sinn[n0 + t])
        ulp_close(q[t], wantq, 2.0)
        ulp_close(K[:, n0 + t], wantk, 2.0)
        assert np.array_equal(V[:, n0 + t].float().cpu().numpy().reshape(-1), row[(Hq + Hk) * D :])  # v rows copied
    assert torch.all(K[:, :n0] == 0) and torch.all(K[:, n0 + T :] == 0)                              # nothing else written


@pytest.mark.parametrize("n0,T,Hq,Hk,S", [(4096, 1, 32, 8, 64), (100, 1, 32, 8, 4), (0, 1, 8, 8, 1), (63, 3, 16, 2, 7),
                                           (500, 1, 8, 1, 16)])
def test_attn_decode_against_f64(card, n0, T, Hq, Hk, S):
    D = 128
    cap = n0 + T + 5
    g = gen(620 + n0)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    q = torch.randn(T, Hq * D, generator=g).to(torch.bfloat16)
    att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    for rep in range(2):  # a second launch over the same scratch gives the same bits
        card.attn_decode(q.cuda(), K.cuda(), V.cuda(), att, n0t, Hq, Hk, D, scale, S, scratch)
        got = att.clone()
        if rep:
            assert torch.equal(got, first)
        first = got
    for t in range(T):
        want = od.attention(q[t].float().numpy().reshape(Hq, D), K[:, : n0 + t + 1].float().numpy(),
                            V[:, : n0 + t + 1].float().numpy(), scale)
        g_ = got[t].float().cpu().numpy().reshape(Hq, D)
        worst = np.abs(g_ - want).max() / np.abs(want).max()
        assert worst <= 2.0**-7, worst


@pytest.mark.parametrize("Hq,Hk", [(8, 8), (8, 4), (16, 4), (8, 1)])
@pytest.mark.parametrize("n0,T,S", [(700, 1, 1), (700, 1, 2), (2400, 1, 19), (2559, 1, 20), (2600, 3, 21), (300, 2, 20),
                                     (4990, 1, 39), (5000, 2, 40), (5200, 1, 41), (90, 1, 40), (8000, 1, 63),
                                     (8100, 2, 64), (8300, 1, 65), (300, 1, 64)])
def test_the_fold_of_a_few_spans_gives_the_general_folds_bits(card, n0, T, Hq, Hk, S):
    """up to 64 spans are folded by a kernel that shares nothing between its waves (built for 20, 40 and 64); the knob attn_merge_few = 0 sends
    every count through the general fold: the same output bits, at the counts on both sides of each limit, with spans
    past the row's keys (no maximum, no sum) and for every number of query heads a kv head"""
    D = 128
    cap = n0 + T + 3
    g = gen(7000 + n0 + S + Hq)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    q = torch.randn(T, Hq * D, generator=g).to(torch.bfloat16).cuda()
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    outs = []
    try:
        for knob in (0, -1):
            card.set_tuning("attn_merge_few", knob)
            att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
            card.attn_decode(q, K, V, att, n0t, Hq, Hk, D, 1.0 / np.sqrt(D), S, scratch)
            torch.cuda.synchronize()
            outs.append(att)
    finally:
        card.set_tuning("attn_merge_few", -1)
    assert torch.equal(outs[0], outs[1])
    assert bool(outs[0].float().abs().sum() > 0)


@pytest.mark.parametrize("n0,T,Hq,Hk,S,seed", [(300, 8, 32, 8, 5, 0), (0, 5, 8, 2, 1, 1), (63, 32, 16, 2, 7, 2),
                                                (1000, 16, 8, 1, 16, 3)])
def test_attn_decode_over_a_tree_of_rows(card, n0, T, Hq, Hk, S, seed):
    """a verify pass's tree (the reference's TREE form, native/cuda/btb_attn_flash.cuh:284-286): row t sees the cache's
    n0 keys and, of the pass's own rows, its ancestors and itself - against f64 attention over exactly those keys; a
    tree that is a chain gives the chain form's bits"""
    D = 128
    cap = n0 + T + 3
    g = gen(650 + seed)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    q = torch.randn(T, Hq * D, generator=g).to(torch.bfloat16)
    par = [-1] + [int(torch.randint(-1, t, (1,), generator=g)) for t in range(1, T)]   # any earlier row, or a new root
    part = torch.tensor(par, dtype=torch.int32, device="cuda")
    att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    card.attn_decode(q.cuda(), K.cuda(), V.cuda(), att, n0t, Hq, Hk, D, scale, S, scratch, par=part)
    got = att.float().cpu().numpy()
    for t in range(T):
        seen, p_ = [], t
        while p_ >= 0:
            seen.append(n0 + p_)
            p_ = par[p_]
        keys = list(range(n0)) + sorted(seen)
        want = od.attention(q[t].float().numpy().reshape(Hq, D), K[:, keys].float().numpy(), V[:, keys].float().numpy(),
                            scale)
        worst = np.abs(got[t].reshape(Hq, D) - want).max() / np.abs(want).max()
        assert worst <= 2.0**-7, (t, worst)
    chain = torch.arange(-1, T - 1, dtype=torch.int32, device="cuda")
    a = torch.zeros_like(att)
    b = torch.zeros_like(att)
    card.attn_decode(q.cuda(), K.cuda(), V.cuda(), a, n0t, Hq, Hk, D, scale, S, scratch, par=chain)
    card.attn_decode(q.cuda(), K.cuda(), V.cuda(), b, n0t, Hq, Hk, D, scale, S, scratch)
    assert torch.equal(a, b)
    with pytest.raises(Exception):
        card.attn_decode(torch.zeros(33, Hq * D, dtype=torch.bfloat16, device="cuda"), K.cuda(), V.cuda(),
                         torch.zeros(33, Hq * D, dtype=torch.bfloat16, device="cuda"), n0t, Hq, Hk, D, scale, 1,
                         card.attn_scratch(33, Hq, Hk, D, 1), par=torch.zeros(33, dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("n0,T,Hq,Hk,S,tree,win", [(1000, 8, 32, 8, 9, False, 0), (1000, 8, 32, 8, 5, False, 0),
                                                    (300, 5, 8, 2, 3, True, 0), (120, 16, 8, 4, 1, False, 0),
                                                    (700, 6, 16, 4, 6, True, 200), (0, 3, 8, 2, 1, False, 0),
                                                    (500, 2, 32, 8, 4, False, 37)])
def test_attn_short_spans_kept_in_registers(card, n0, T, Hq, Hk, S, tree, win):
    """a pass of several rows whose spans are one or two batches of keys (128 / 256) takes the kernel that asks for a
    span's keys at once: against f64 attention over the keys each row sees, the bits of the general kernel at the same
    span count"""
    D = 128
    cap = n0 + T + 3
    span = -(-(-(-cap // S)) // 128) * 128
    assert span in (128, 256)
    g = gen(690 + n0 + T)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    q = torch.randn(T, Hq * D, generator=g).to(torch.bfloat16)
    par = [-1] + [int(torch.randint(-1, t, (1,), generator=g)) for t in range(1, T)] if tree else None
    part = None if par is None else torch.tensor(par, dtype=torch.int32, device="cuda")
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    card.set_tuning("attn_mfma", 0)  # the vector-ALU kernels: the matrix-core form has a test of its own below
    try:
        att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        card.attn_decode(q.cuda(), K.cuda(), V.cuda(), att, n0t, Hq, Hk, D, scale, S, scratch, par=part, win=win)
    finally:
        card.set_tuning("attn_mfma", -1)
    # the general kernel at the same span count (what a launch by the reference's kernel name takes): the same bits
    pm = torch.zeros(S * T * Hq, dtype=torch.float32, device="cuda")
    pl, pa = torch.zeros_like(pm), torch.zeros(S * T * Hq * D, dtype=torch.float32, device="cuda")
    general = torch.zeros_like(att)
    Kc, Vc = K.cuda(), V.cuda()
    p_ = lambda t: None if t is None else t.data_ptr()
    assert card.lib.btb_hip_attn_decode_parts(p_(q.cuda().contiguous()), p_(Kc), p_(Vc), p_(general), p_(n0t), p_(part), T,
                                              Hq, Hk, D, int(Kc.stride(0)), int(Kc.stride(1)), float(scale), span, S,
                                              int(win), None, p_(pm), p_(pl), p_(pa), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(att, general)
    got = att.float().cpu().numpy()
    for t in range(T):
        if par is None:
            slots = list(range(n0 + t + 1))            # slot = position in a chain
            pos = slots
        else:
            path, p_ = [], t
            while p_ >= 0:
                path.append(p_)
                p_ = par[p_]
            path = path[::-1]                            # root first: depth d at position n0 + d
            slots = list(range(n0)) + [n0 + p for p in path]
            pos = list(range(n0)) + [n0 + d for d in range(len(path))]
        keep = [s_ for s_, ps in zip(slots, pos) if win == 0 or ps >= pos[-1] + 1 - win]
        want = od.attention(q[t].float().numpy().reshape(Hq, D), K[:, keep].float().numpy(), V[:, keep].float().numpy(),
                            scale)
        worst = np.abs(got[t].reshape(Hq, D) - want).max() / np.abs(want).max()
        assert worst <= 2.0**-7, (t, worst)


@pytest.mark.parametrize("n0,T,Hq,Hk,tree,win", [(4000, 8, 32, 8, False, 0), (1000, 16, 32, 8, False, 0),
                                                  (300, 5, 8, 2, True, 0), (120, 2, 8, 4, False, 0),
                                                  (700, 6, 16, 4, True, 200), (0, 3, 8, 2, False, 0),
                                                  (500, 2, 32, 8, False, 37), (250, 21, 16, 4, False, 0),
                                                  (380, 32, 8, 2, True, 0), (127, 9, 32, 8, False, 0),
                                                  (1, 13, 8, 4, True, 5)])
def test_attn_rows_on_the_matrix_cores(card, n0, T, Hq, Hk, tree, win):
    """a pass of several rows with spans of 128 keys takes the matrix-core kernel (every row that shares a kv head in one
    workgroup; more than 64 (row, head) pairs a kv head are several workgroups): against f64 attention over the keys
    each row sees - chain, tree, window, the pass's own rows straddling a span's end, a span with nothing to see -
    within the bar of the vector-ALU kernel it replaces (knob attn_mfma = 0; the two differ in f32 summation order),
    the same bits on a second call, and a tree that is a chain gives the chain's bits"""
    D = 128
    cap = n0 + T + 3
    S = -(-cap // 128)
    g = gen(700 + n0 + T)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    # slots the pass has not written hold whatever was there: NaN bits must not leak through weight 0
    K[:, n0 + T:] = float("nan")
    V[:, n0 + T:] = float("nan")
    q = torch.randn(T, Hq * D, generator=g).to(torch.bfloat16)
    par = [-1] + [int(torch.randint(-1, t, (1,), generator=g)) for t in range(1, T)] if tree else None
    part = None if par is None else torch.tensor(par, dtype=torch.int32, device="cuda")
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)

    def run(p_=part):
        att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        card.attn_decode(q.cuda(), K.cuda(), V.cuda(), att, n0t, Hq, Hk, D, scale, S, scratch, par=p_, win=win)
        return att.clone()

    y = run()
    assert torch.equal(run(), y)
    card.set_tuning("attn_mfma", 0)
    try:
        vec = run()
    finally:
        card.set_tuning("attn_mfma", -1)
    peak = float(vec.float().abs().max())
    assert float((vec.float() - y.float()).abs().max()) <= peak * 2.0**-7
    if not tree:
        chain = torch.arange(-1, T - 1, dtype=torch.int32, device="cuda")
        if T <= 32:
            assert torch.equal(run(chain), y)
    got = y.float().cpu().numpy()
    assert np.isfinite(got).all()
    for t in range(T):
        if par is None:
            slots = list(range(n0 + t + 1))
            pos = slots
        else:
            path, p_ = [], t
            while p_ >= 0:
                path.append(p_)
                p_ = par[p_]
            path = path[::-1]
            slots = list(range(n0)) + [n0 + p for p in path]
            pos = list(range(n0)) + [n0 + d for d in range(len(path))]
        keep = [s_ for s_, ps in zip(slots, pos) if win == 0 or ps >= pos[-1] + 1 - win]
        want = od.attention(q[t].float().numpy().reshape(Hq, D), K[:, keep].float().numpy(), V[:, keep].float().numpy(),
                            scale)
        worst = np.abs(got[t].reshape(Hq, D) - want).max() / np.abs(want).max()
        assert worst <= 2.0**-7, (t, worst)


@pytest.mark.parametrize("n0,Hq,Hk,S", [(4096, 32, 8, 36), (100, 32, 8, 4), (0, 8, 8, 1), (63, 16, 2, 7), (64, 16, 2, 2),
                                         (500, 8, 1, 16), (31, 4, 2, 3), (300, 8, 1, 40), (200, 4, 4, 5)])
@pytest.mark.parametrize("with_norm", [True, False])
def test_attn_decode_qkv_is_the_two_kernels_in_one(card, n0, Hq, Hk, S, with_norm):
    """the step's own attention from the fused qkv row against norm_rope_kv followed by attn_decode: the same output
    bits, the same cache row, nothing else in the cache touched - with slot n0 first, last and inside its span"""
    from btb_amd.decode import StackConfig, rope_tables

    D = 128
    cap = n0 + 6
    g = gen(640 + n0 + Hq)
    K0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    qkv = torch.randn(1, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
    wq = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda() if with_norm else None
    wk = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda() if with_norm else None
    cfg = StackConfig(layers=1, hidden=256, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=256, vocab=256)
    cos, sin = rope_tables(cfg, cap, "cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    scratch = card.attn_scratch(1, Hq, Hk, D, S)
    Ka, Va = K0.clone(), V0.clone()
    q = torch.zeros(1, Hq * D, dtype=torch.bfloat16, device="cuda")
    want = torch.zeros(1, Hq * D, dtype=torch.bfloat16, device="cuda")
    card.norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, n0t, Ka, Va, q, Hq, Hk, D)
    card.attn_decode(q, Ka, Va, want, n0t, Hq, Hk, D, scale, S, scratch)
    # whatever the scratch holds, and again over what the first call left there
    scratch.fill_(float("nan"))
    for rep in range(2):
        Kb, Vb = K0.clone(), V0.clone()
        got = torch.zeros_like(want)
        card.attn_decode_qkv(qkv, wq, wk, 1e-6, cos, sin, n0t, Kb, Vb, got, Hq, Hk, D, scale, S, scratch)
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep
        assert torch.equal(Ka, Kb) and torch.equal(Va, Vb)
        assert not torch.equal(Kb[:, n0], K0[:, n0])  # the row was written


@pytest.mark.parametrize("n0,T,Hq,Hk,tree", [(4000, 8, 32, 8, False), (4000, 7, 32, 8, False), (125, 8, 32, 8, False),
                                              (120, 16, 8, 4, True), (0, 2, 8, 2, False), (127, 3, 8, 4, False),
                                              (255, 16, 8, 4, True), (300, 5, 8, 2, True), (128, 4, 32, 8, False),
                                              (250, 9, 16, 8, True), (1, 13, 4, 2, False), (383, 2, 32, 8, False),
                                              (4000, 16, 32, 8, False), (120, 16, 16, 4, True), (255, 32, 8, 4, True),
                                              (100, 12, 32, 8, False), (126, 9, 8, 2, True), (300, 20, 4, 2, False)])
@pytest.mark.parametrize("with_norm", [True, False])
def test_attn_rows_from_the_fused_qkv_rows(card, n0, T, Hq, Hk, tree, with_norm):
    """a pass's attention from its fused qkv rows (up to 32 (row, head) pairs a kv head in one workgroup, up to 64 in
    two) against norm_rope_kv followed by attn_decode: the same output bits,
    the same cache rows, nothing else in the cache touched - chain and tree (rows at their depths), the pass's own slots
    at a span's start, across its end, and past the written part of the cache (which holds NaN bits)"""
    from btb_amd.decode import StackConfig, rope_tables

    D = 128
    cap = n0 + T + 5
    S = -(-cap // 128)
    assert card.attn_rows_fused(T, Hq, Hk, D, cap, S)
    g = gen(660 + n0 + T + Hq)
    K0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    V0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    K0[:, n0:] = float("nan")
    V0[:, n0:] = float("nan")
    K0, V0 = K0.cuda(), V0.cuda()
    qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
    wq = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda() if with_norm else None
    wk = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda() if with_norm else None
    cfg = StackConfig(layers=1, hidden=256, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=256, vocab=256)
    cos, sin = rope_tables(cfg, cap, "cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    par = depth = None
    if tree:
        pl = [-1] + [int(torch.randint(-1, t, (1,), generator=g)) for t in range(1, T)]
        dl = []
        for t in range(T):
            dl.append(0 if pl[t] < 0 else dl[pl[t]] + 1)
        par = torch.tensor(pl, dtype=torch.int32, device="cuda")
        depth = torch.tensor(dl, dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    Ka, Va = K0.clone(), V0.clone()
    q = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    want = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    card.norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, n0t, Ka, Va, q, Hq, Hk, D, depth=depth)
    card.attn_decode(q, Ka, Va, want, n0t, Hq, Hk, D, scale, S, scratch, par=par)
    assert bool(torch.isfinite(want.float()).all())
    scratch.fill_(float("nan"))
    for rep in range(2):
        Kb, Vb = K0.clone(), V0.clone()
        got = torch.zeros_like(want)
        card.attn_decode_qkv_rows(qkv, wq, wk, 1e-6, cos, sin, n0t, Kb, Vb, got, Hq, Hk, D, scale, S, scratch,
                                  depth=depth, par=par)
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep
        same = lambda a, b: torch.equal(a.view(torch.int16), b.view(torch.int16))
        assert same(Ka, Kb) and same(Va, Vb)
        assert bool(torch.isfinite(Kb[:, n0:n0 + T].float()).all())  # the rows were written


@pytest.mark.parametrize("centered,positions", [(True, False), (False, True), (True, True)])
def test_attn_rows_from_the_fused_qkv_rows_centered_weights_and_given_positions(card, centered, positions):
    """the same equality with norm weights stored around zero (`centered`: the factor is 1 + w) and with a chain whose
    rows stand at given depths"""
    from btb_amd.decode import StackConfig, rope_tables

    D, Hq, Hk, T, n0 = 128, 16, 4, 6, 200
    cap = n0 + 24
    S = -(-cap // 128)
    g = gen(690)
    K0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
    wq = (0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    wk = (0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    cfg = StackConfig(layers=1, hidden=256, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=256, vocab=256)
    cos, sin = rope_tables(cfg, cap, "cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    depth = torch.tensor([0, 3, 4, 9, 10, 17], dtype=torch.int32, device="cuda") if positions else None
    scale = 1.0 / np.sqrt(D)
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    Ka, Va, Kb, Vb = K0.clone(), V0.clone(), K0.clone(), V0.clone()
    q = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    want, got = torch.zeros_like(q), torch.zeros_like(q)
    card.norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, n0t, Ka, Va, q, Hq, Hk, D, depth=depth, centered=centered)
    card.attn_decode(q, Ka, Va, want, n0t, Hq, Hk, D, scale, S, scratch)
    card.attn_decode_qkv_rows(qkv, wq, wk, 1e-6, cos, sin, n0t, Kb, Vb, got, Hq, Hk, D, scale, S, scratch, depth=depth,
                              centered=centered)
    assert torch.equal(got, want)
    assert torch.equal(Ka, Kb) and torch.equal(Va, Vb)


def test_attn_rows_from_the_fused_qkv_rows_over_drawn_shapes(card):
    """the same equality over a hundred drawn passes: 2 or 4 query heads a kv head, 1 to 8 kv heads, 2 rows up to 64
    pairs, cache lengths 0 .. 700 with any amount of room behind, chain or tree, with or without (centered) norm
    weights"""
    from btb_amd.decode import StackConfig, rope_tables

    rng = np.random.default_rng(20251)
    D, done = 128, 0
    same = lambda a, b: torch.equal(a.view(torch.int16), b.view(torch.int16))
    while done < 100:
        G = int(rng.choice([2, 4]))
        Hk = int(rng.choice([1, 2, 4, 8]))
        Hq = Hk * G
        T = int(rng.integers(2, 64 // G + 1))
        n0, pad = int(rng.integers(0, 700)), int(rng.integers(0, 40))
        cap = n0 + T + pad
        S = -(-cap // 128)
        assert card.attn_rows_fused(T, Hq, Hk, D, cap, S)
        g = gen(int(rng.integers(1 << 30)))
        K0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
        V0 = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
        K0[:, n0:] = float("nan")
        V0[:, n0:] = float("nan")
        K0, V0 = K0.cuda(), V0.cuda()
        qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
        with_norm, centered = bool(rng.integers(2)), bool(rng.integers(2))
        mk = lambda: (0.1 * torch.randn(D, generator=g) + (0.0 if centered else 1.0)).to(torch.bfloat16).cuda()
        wq, wk = (mk(), mk()) if with_norm else (None, None)
        cfg = StackConfig(layers=1, hidden=256, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=256, vocab=256)
        cos, sin = rope_tables(cfg, cap, "cuda")
        n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
        par = depth = None
        if rng.integers(2):
            pl = [-1] + [int(rng.integers(-1, t)) for t in range(1, T)]
            dl = []
            for t in range(T):
                dl.append(0 if pl[t] < 0 else dl[pl[t]] + 1)
            par = torch.tensor(pl, dtype=torch.int32, device="cuda")
            depth = torch.tensor(dl, dtype=torch.int32, device="cuda")
        scale = 1.0 / np.sqrt(D)
        scratch = card.attn_scratch(T, Hq, Hk, D, S)
        Ka, Va, Kb, Vb = K0.clone(), V0.clone(), K0.clone(), V0.clone()
        q = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        want, got = torch.zeros_like(q), torch.zeros_like(q)
        card.norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, n0t, Ka, Va, q, Hq, Hk, D, depth=depth, centered=centered)
        card.attn_decode(q, Ka, Va, want, n0t, Hq, Hk, D, scale, S, scratch, par=par)
        card.attn_decode_qkv_rows(qkv, wq, wk, 1e-6, cos, sin, n0t, Kb, Vb, got, Hq, Hk, D, scale, S, scratch,
                                  depth=depth, par=par, centered=centered)
        torch.cuda.synchronize()
        what = dict(G=G, Hk=Hk, T=T, n0=n0, cap=cap, norm=with_norm, centered=centered, tree=par is not None)
        assert same(got, want) and same(Ka, Kb) and same(Va, Vb), what
        assert bool(torch.isfinite(want.float()).all()), what
        done += 1


def test_attn_rows_from_the_fused_qkv_rows_only_where_it_fits(card):
    """shapes the fused pass does not take are named by the query and refused by the call: one row, more than 64
    (row, head) pairs a kv head, spans of 256 keys, 8 query heads a kv head"""
    D = 128
    assert card.attn_rows_fused(8, 32, 8, D, 4608, 36)
    for T, Hq, Hk, cap, S in ((1, 32, 8, 4608, 36), (17, 32, 8, 4608, 36), (8, 32, 8, 4608, 18), (4, 16, 2, 512, 4)):
        assert not card.attn_rows_fused(T, Hq, Hk, D, cap, S)
        qkv = torch.zeros(T, (Hq + 2 * Hk) * D, dtype=torch.bfloat16, device="cuda")
        K = torch.zeros(Hk, cap, D, dtype=torch.bfloat16, device="cuda")
        att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        tab = torch.zeros(cap, D, dtype=torch.bfloat16, device="cuda")
        n0t = torch.zeros(1, dtype=torch.int32, device="cuda")
        with pytest.raises(Exception, match="attn_decode_qkv_rows"):
            card.attn_decode_qkv_rows(qkv, None, None, 1e-6, tab, tab, n0t, K, K.clone(), att, Hq, Hk, D, 0.1, S,
                                      card.attn_scratch(T, Hq, Hk, D, S))


def test_silu_mul_and_argmax_and_embed(card):
    gu = acts_bf16(3, 2 * 768, seed=630)
    m = torch.empty(3, 768, dtype=torch.bfloat16, device="cuda")
    card.silu_mul(gu.cuda(), m)
    ulp_close(m, od.silu_mul(gu.float().numpy()), 2.0)
    logits = acts_bf16(2, 151936, seed=631)
    logits[0, 777] = logits[0, 99999] = 30.0   # a tie: the lower index wins
    logits[1, 151935] = 31.0
    out = torch.zeros(2, dtype=torch.int32, device="cuda")
    card.argmax(logits.cuda(), out)
    assert out.tolist() == [777, 151935]
    # the reference's scan (native/src/sample.rs:53-67): a NaN never wins, a row with nothing above -inf gives 0,
    # and a width that is no multiple of 8 takes the element-wise path
    odd = acts_bf16(4, 1003, seed=633)
    odd[0, 0] = float("nan")
    odd[0, 500] = odd[0, 1002] = 9.0
    odd[1, :] = float("-inf")
    odd[2, :] = float("nan")
    odd[3, 1002] = 50.0
    out4 = torch.zeros(4, dtype=torch.int32, device="cuda")
    card.argmax(odd.cuda(), out4)
    assert out4.tolist() == [500, 0, 0, 1002]
    wide = acts_bf16(2, 4096, seed=634)
    wide[0, 8] = float("nan")
    wide[0, 4095] = wide[0, 9] = 12.0
    wide[1, :] = float("-inf")
    wide[1, 3000] = -1e30
    out2 = torch.zeros(2, dtype=torch.int32, device="cuda")
    card.argmax(wide.cuda(), out2)
    assert out2.tolist() == [9, 3000]
    table = weights_bf16(1000, 64, seed=632).cuda()
    ids = torch.tensor([5, 999, 0], dtype=torch.int32, device="cuda")
    h = torch.zeros(3, 64, dtype=torch.bfloat16, device="cuda")
    card.embed(table, ids, h)
    assert torch.equal(h, table[ids.long()])


def test_publish(card):
    n0 = torch.tensor([41], dtype=torch.int32, device="cuda")
    picked = torch.tensor([1234], dtype=torch.int32, device="cuda")
    nxt = torch.zeros(1, dtype=torch.int32, device="cuda")
    tok = torch.zeros(1, dtype=torch.int32).pin_memory()
    ln = torch.zeros(1, dtype=torch.int32).pin_memory()
    ts = torch.zeros(1, dtype=torch.int64).pin_memory()
    card.publish(n0, picked, nxt, tok, ln, ts)
    torch.cuda.synchronize()
    assert int(tok[0]) == 1234 and int(ln[0]) == 42 and int(n0[0]) == 42 and int(nxt[0]) == 1234 and int(ts[0]) != 0


@pytest.mark.parametrize("n0,T,Hq,Hk,S,win,tree", [(300, 1, 32, 8, 3, 128, False), (300, 6, 8, 2, 2, 17, False),
                                                    (40, 8, 16, 2, 1, 3, True), (700, 8, 32, 8, 5, 500, True),
                                                    (5, 4, 8, 8, 1, 64, False)])
def test_attn_decode_under_a_window(card, n0, T, Hq, Hk, S, win, tree):
    """the reference's window (native/cuda/btb_attn_flash.cuh:437: first = last + 1 - win): a row at logical position
    `last` - n0 + t in a chain, n0 + its depth in a tree - sees positions first .. last only; against f64 attention
    over exactly those keys"""
    D = 128
    cap = n0 + T + 3
    g = gen(680 + n0 + win)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    q = torch.randn(T, Hq * D, generator=g).to(torch.bfloat16)
    par = [-1, 0, 1, 2, 1, 4, 0, 6][:T] if tree else None
    part = None if par is None else torch.tensor(par, dtype=torch.int32, device="cuda")
    att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    card.attn_decode(q.cuda(), K.cuda(), V.cuda(), att, n0t, Hq, Hk, D, scale, S, card.attn_scratch(T, Hq, Hk, D, S),
                     par=part, win=win)
    got = att.float().cpu().numpy()
    for t in range(T):
        if par is None:
            slots = list(range(n0 + t + 1))            # slot = position in a chain
            pos = slots
        else:
            path, p_ = [], t
            while p_ >= 0:
                path.append(p_)
                p_ = par[p_]
            path = path[::-1]                            # root first: depth d at position n0 + d
            slots = list(range(n0)) + [n0 + p for p in path]
            pos = list(range(n0)) + [n0 + d for d in range(len(path))]
        last = pos[-1]
        keep = [s for s, ps in zip(slots, pos) if ps >= last + 1 - win]
        want = od.attention(q[t].float().numpy().reshape(Hq, D), K[:, keep].float().numpy(), V[:, keep].float().numpy(),
                            scale)
        worst = np.abs(got[t].reshape(Hq, D) - want).max() / np.abs(want).max()
        assert worst <= 2.0**-7, (t, worst)


def test_attn_and_rope_through_the_caches_row_map(card):
    """`tbl` maps a logical slot to its cache row - an address, never a bit (native/cuda/btb_attn_flash.cuh:34): the
    pass over a cache whose rows were shuffled by the map gives the unshuffled cache's bits, and norm_rope_kv with the
    map writes the pass's rows where the map says"""
    D, Hq, Hk, T, n0, S = 128, 16, 4, 5, 200, 3
    cap = 256
    cfg = StackConfig(layers=1, hidden=64, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=64, vocab=8)
    g = gen(690)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
    wq = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    wk = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    cos, sin = rope_tables(cfg, cap, "cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    perm = torch.randperm(cap, generator=g).to(torch.int32)
    tbl = perm.cuda()
    Kp, Vp = torch.zeros_like(K), torch.zeros_like(V)
    Kp[:, perm.long()] = K                              # logical slot j lives in row perm[j]
    Vp[:, perm.long()] = V
    scale = 1.0 / np.sqrt(D)
    scratch = card.attn_scratch(T, Hq, Hk, D, S)
    par = torch.tensor([-1, 0, 0, 2, 3], dtype=torch.int32, device="cuda")
    outs = []
    for Kc, Vc, m in ((K.clone(), V.clone(), None), (Kp, Vp, tbl)):
        q = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        card.norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, n0t, Kc, Vc, q, Hq, Hk, D, tbl=m)
        att = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
        card.attn_decode(q, Kc, Vc, att, n0t, Hq, Hk, D, scale, S, scratch, par=par, win=150, tbl=m)
        outs.append((q, att, Kc, Vc))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    # the pass's rows landed in their mapped cache rows
    for t in range(T):
        assert torch.equal(outs[1][2][:, int(perm[n0 + t])], outs[0][2][:, n0 + t])
        assert torch.equal(outs[1][3][:, int(perm[n0 + t])], outs[0][3][:, n0 + t])
    assert bool(outs[0][1].float().abs().sum() > 0)


def test_attn_span_count_limit(card):
    """spans * (query heads per kv head) is at most 1024 - the states the span fold turns into factors: the maximum
    is taken and right, one more span is refused (nothing is launched)"""
    D, Hq, Hk, n0 = 128, 8, 2, 2100
    G = Hq // Hk
    cap = n0 + 8
    g = gen(695)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16)
    q = torch.randn(1, Hq * D, generator=g).to(torch.bfloat16)
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    S = 1024 // G
    att = torch.zeros(1, Hq * D, dtype=torch.bfloat16, device="cuda")
    card.attn_decode(q.cuda(), K.cuda(), V.cuda(), att, n0t, Hq, Hk, D, scale, S, card.attn_scratch(1, Hq, Hk, D, S))
    want = od.attention(q[0].float().numpy().reshape(Hq, D), K[:, : n0 + 1].float().numpy(),
                        V[:, : n0 + 1].float().numpy(), scale)
    got = att[0].float().cpu().numpy().reshape(Hq, D)
    assert np.abs(got - want).max() / np.abs(want).max() <= 2.0**-7
    att.fill_(3.0)
    with pytest.raises(Exception):
        card.attn_decode(q.cuda(), K.cuda(), V.cuda(), att, n0t, Hq, Hk, D, scale, S + 1,
                         card.attn_scratch(1, Hq, Hk, D, S + 1))
    torch.cuda.synchronize()
    assert bool((att == 3.0).all())
