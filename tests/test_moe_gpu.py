"""The routed MoE decode layer on the GPU (Qwen3-30B-A3B shape: hidden 2048, 128 experts, top-8, intermediate 768)
against the CPU path restated in oracle/moe.py, on the same seeded inputs.

Bars: the top-k picks, as ordered lists, are bit-exact; the router's f32 logits are
bit-exact (they are made in the CPU's order); the routing weights agree to one bf16 ulp (the two sides' expf may
differ in the last bit); the layer output agrees within max relative error 1e-2 of the largest output (bf16 rows; the
expert matvecs accumulate in f32 in a different order than the CPU's, which can flip a bf16 rounding of gu, h or d)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from btb_amd.moe import Experts, Router
from oracle import codecs
from oracle import moe as omoe

from .helpers import acts_bf16, bits16, f32_bits, gen, weights_bf16

pytestmark = pytest.mark.gpu

E, K, H, I = 128, 8, 2048, 768


@pytest.fixture(scope="module")
def layer_weights():
    g = gen(500)
    wr = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
    gu = (torch.randn(E, 2 * I, H, generator=g) * 0.02).to(torch.bfloat16)
    dn = (torch.randn(E, H, I, generator=g) * 0.02).to(torch.bfloat16)
    return wr, gu, dn


@pytest.mark.parametrize("T", [1, 4, 8])
def test_moe_layer_matches_cpu_path(card, layer_weights, T):
    wr, gu, dn = layer_weights
    x = acts_bf16(T, H, seed=510 + T)
    router = Router(card, wr.cuda(), K)
    experts = Experts(card, gu.cuda(), dn.cuda())
    logits, weights, picks = router(x.cuda())
    y = experts(x.cuda(), picks, weights)
    torch.cuda.synchronize()

    want, ologits, ow, opicks = omoe.layer(bits16(wr), bits16(gu), bits16(dn), x.float().numpy(), K, "bf16")
    raw = card.gemv_lane16(wr.cuda(), x.float().cuda()).cpu().numpy()
    assert np.array_equal(f32_bits(raw), f32_bits(ologits))                       # logits: the CPU's bits
    assert np.array_equal(picks.cpu().numpy().astype(np.int64), opicks)           # picks: bit-exact, in rank order
    dw = np.abs(weights.float().cpu().numpy() - ow)
    assert np.all(dw <= np.abs(ow) * 2.0**-7)                                     # weights: within a bf16 ulp
    got = y.float().cpu().numpy()
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 1e-2, err


def test_experts_with_the_cpu_picks(card, layer_weights):
    """the expert stage on its own, fed the oracle's picks and weights: only the matvecs' summation order differs"""
    wr, gu, dn = layer_weights
    T = 4
    x = acts_bf16(T, H, seed=520)
    _, ow, opicks = omoe.router(bits16(wr), x.float().numpy(), K, "bf16")
    want = omoe.experts(bits16(gu), bits16(dn), x.float().numpy(), opicks, ow, "bf16")
    experts = Experts(card, gu.cuda(), dn.cuda())
    y = experts(x.cuda(), torch.from_numpy(opicks).to(torch.int32).cuda(),
                torch.from_numpy(ow).to(torch.bfloat16).cuda())
    got = y.float().cpu().numpy()
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()


def test_route_tie_rule_and_bf16_logits(card):
    """equal logits: the lower index wins (native/cuda/btb_kernels.cu:848-851, 900, 912); bf16 logits as the
    reference's kernel takes them"""
    logits = torch.zeros(2, 16)
    logits[0, [3, 7, 11]] = 2.0      # three equal maxima, then thirteen equal zeros
    logits[1] = torch.arange(16, 0, -1).float()
    idx, w, w32 = card.moe_route(logits.cuda(), 5)
    assert idx[0].tolist() == [3, 7, 11, 0, 1]
    assert idx[1].tolist() == [0, 1, 2, 3, 4]
    assert abs(float(w32[0].sum()) - 1.0) < 1e-6
    idxb, wb, _ = card.moe_route(logits.to(torch.bfloat16).cuda(), 5)
    assert torch.equal(idxb, idx) and torch.equal(wb, w)
    # torch's own routing on distinct values agrees
    g = torch.randn(6, 128, generator=gen(530))
    p = torch.softmax(g, dim=-1)
    top, ids = torch.topk(p, 8, dim=-1)
    idx, w, w32 = card.moe_route(g.cuda(), 8)
    assert torch.equal(idx.cpu().long(), ids)
    assert torch.allclose(w32.cpu(), top / top.sum(-1, keepdim=True), rtol=1e-5, atol=0)
    with pytest.raises(Exception):
        card.moe_route(g.cuda(), 33)


def test_route_in_registers_and_through_lds_agree(card):
    """up to 256 experts the row stays in registers, beyond that it goes through LDS: a 300-wide row whose upper
    experts are far below the rest must route as its first 128, 200 and 256 do, ties, zeros of probability and a row
    of NaN included"""
    g = torch.randn(9, 300, generator=gen(531))
    g[:, 128:] -= 200.0                       # exp underflows to +0: live, never picked before a real one
    g[1, :128] = g[1, :128].round()           # many exact ties
    g[2, 5] = float("nan")                    # every probability NaN: the first k experts
    g[3, :128] = 1.5                          # all equal: index order
    g[4, 17] = float("inf")                   # inf - inf: NaN again
    wide = card.moe_route(g.cuda(), 8)
    for E in (64, 100, 128, 200, 256):
        head = card.moe_route(g.cuda(), 8, E=E)
        if E >= 128:
            assert torch.equal(head[0], wide[0]), E
            ok = ~torch.isnan(wide[2])
            assert torch.equal(head[2][ok], wide[2][ok]) and torch.equal(torch.isnan(head[2]), ~ok), E
        ref = torch.softmax(g[:, :E], dim=-1)
        top, ids = torch.topk(ref[[0, 5, 6, 7, 8]], 8, dim=-1)
        assert torch.equal(head[0].cpu().long()[[0, 5, 6, 7, 8]], ids), E
    assert wide[0][2].tolist() == list(range(8)) and wide[0][4].tolist() == list(range(8))
    # k = 32 of 40: the zero-probability tail is taken in index order
    z = torch.full((1, 40), -300.0)
    z[0, [9, 4, 30]] = torch.tensor([3.0, 2.0, 1.0])
    idx, _, _ = card.moe_route(z.cuda(), 32)
    assert idx[0].tolist() == [9, 4, 30] + [i for i in range(40) if i not in (9, 4, 30)][:29]


@pytest.mark.parametrize("T,E,H", [(1, 128, 2048), (5, 128, 2048), (3, 60, 520), (2, 384, 256), (9, 128, 2048),
                                   (64, 256, 1024), (3, 200, 384), (7, 40, 128)])
def test_router_in_two_launches_is_the_three_step_form(card, T, E, H):
    """bf16 rows straight into the host-order matvec, the logits rounded inside the routing kernel: the same bits as
    widening the rows first, routing the f32 logits and rounding them afterwards, and the same on a second call"""
    g = gen(540 + T)
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).cuda()
    x = acts_bf16(T, H, seed=545 + T).cuda()
    logits, logits16, idx, w, w32 = card.moe_router(wr, x, 8)
    again = card.moe_router(wr, x, 8)
    raw = card.gemv_lane16(wr, x.float())
    ridx, rw, rw32 = card.moe_route(raw, 8)
    assert torch.equal(logits.view(torch.int32), raw.view(torch.int32))
    assert torch.equal(logits16.view(torch.int16), raw.to(torch.bfloat16).view(torch.int16))
    assert torch.equal(idx, ridx) and torch.equal(w.view(torch.int16), rw.view(torch.int16))
    assert torch.equal(w32.view(torch.int32), rw32.view(torch.int32))
    want, ow, opicks = omoe.router(bits16(wr.cpu()), x.float().cpu().numpy(), 8, "bf16")
    assert np.array_equal(f32_bits(logits.cpu().numpy()), f32_bits(want))
    assert np.array_equal(idx.cpu().numpy().astype(np.int64), opicks)
    for a, b in zip((logits, logits16, idx, w, w32), again):
        bits = torch.int16 if a.dtype == torch.bfloat16 else torch.int32
        assert torch.equal(a.view(bits), b.view(bits))


@pytest.mark.parametrize("T,k,n_experts", [(1, 8, 128), (8, 8, 128), (13, 4, 60), (64, 8, 128), (5, 3, 700), (200, 8, 16)])
def test_group_picks_is_the_stable_sort(card, T, k, n_experts):
    """`group_picks` (btb/engine/host.py:283-296) on the device against the oracle's stable argsort, entry for entry:
    few experts with many rows each, more experts than one workgroup's threads, experts nobody picked"""
    g = gen(560 + T)
    picks = torch.stack([torch.randperm(n_experts, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    slot, token, offs, counts = card.moe_group_picks(picks.cuda(), n_experts)
    wslot, wtoken, woffs, wcounts = omoe.group_picks(picks.numpy(), n_experts)
    assert np.array_equal(counts.cpu().numpy(), wcounts)
    assert np.array_equal(offs.cpu().numpy(), woffs)
    assert np.array_equal(slot.cpu().numpy(), wslot)
    assert np.array_equal(token.cpu().numpy(), wtoken)


@pytest.mark.parametrize("T,share", [(4, 2), (8, 3), (12, 1), (9, 40)])
def test_rows_that_share_an_expert_go_through_it_together(card, layer_weights, T, share):
    """the gate/up kernel that streams an expert once for all the rows that picked it writes the bits of the kernel
    that streams it once a pair (knob moe_grouped = 0), with picks drawn from `share` + k - 1 experts so that rows
    share many (an expert picked by more than four rows takes more than one pass), and from all 128"""
    wr, gu, dn = layer_weights
    g = gen(570 + T)
    pool = min(E, share + K - 1)
    picks = torch.stack([torch.randperm(pool, generator=g)[:K] * (E // pool) for _ in range(T)]).to(torch.int32).cuda()
    w = torch.rand(T, K, generator=g).to(torch.bfloat16).cuda()
    x = acts_bf16(T, H, seed=580 + T).cuda()
    experts = Experts(card, gu.cuda(), dn.cuda())
    try:
        card.set_tuning("moe_grouped", 1)  # from eight rows on it is the default; here for every T
        y = experts(x, picks, w).clone()
        card.set_tuning("moe_grouped", 0)
        by_pair = experts(x, picks, w).clone()
    finally:
        card.set_tuning("moe_grouped", -1)
    assert torch.equal(y.view(torch.int16), by_pair.view(torch.int16))
    want = omoe.experts(bits16(gu), bits16(dn), x.float().cpu().numpy(), picks.cpu().numpy().astype(np.int64),
                        w.float().cpu().numpy(), "bf16")
    assert np.abs(y.float().cpu().numpy() - want).max() <= 1e-2 * np.abs(want).max()


# -- MXFP4 expert stacks: the stored bytes through the same two kernels ------------------------------------------------


def mx_stacks(seed: int, E_: int, I_: int, H_: int):
    """N(0, 0.02) expert stacks quantised to MXFP4 (the repository's own encoder; what is checked is the layer over the
    stored bytes, whatever made them)"""
    from btb_amd import mxfp4
    from btb_amd.load import MxExperts

    g = gen(seed)
    gu = torch.randn(E_ * 2 * I_, H_, generator=g) * 0.02
    dn = torch.randn(E_ * H_, I_, generator=g) * 0.02
    gb, gs = mxfp4.quantize(gu)
    db, ds = mxfp4.quantize(dn)
    return MxExperts(gb.reshape(E_, 2 * I_, H_ // 32, 16), gs.reshape(E_, 2 * I_, H_ // 32),
                     db.reshape(E_, H_, I_ // 32, 16), ds.reshape(E_, H_, I_ // 32))


def to_gpu(ex):
    from btb_amd.load import MxExperts

    mv = lambda t: None if t is None else t.cuda()
    return MxExperts(ex.gate_up_blocks.cuda(), ex.gate_up_scales.cuda(), ex.down_blocks.cuda(), ex.down_scales.cuda(),
                     mv(ex.gate_up_bias), mv(ex.down_bias))


def oracle_mx(ex, x, picks, w, **kw):
    f = lambda t: None if t is None else t.float().numpy()
    return omoe.experts_mx4(ex.gate_up_blocks.numpy(), ex.gate_up_scales.numpy(), ex.down_blocks.numpy(),
                            ex.down_scales.numpy(), x.float().numpy(), picks, w, dt="bf16", gu_bias=f(ex.gate_up_bias),
                            dn_bias=f(ex.down_bias), **kw)


@pytest.mark.parametrize("T", [1, 4, 8, 16])
def test_mxfp4_moe_layer_matches_cpu_path(card, layer_weights, T):
    """C4's layer with its experts stored as MXFP4 (concatenated halves, SiLU): the router's picks are the CPU's bit for
    bit, the layer within 1e-2 of the CPU path over the same stored bytes (btb_gemv_mxfp4_rows per expert, the rows'
    dtype chain of _Experts); 8 and 16 rows take the grouped gate/up kernel"""
    from btb_amd.moe import MxExpertsLayer

    wr = layer_weights[0]
    ex = mx_stacks(540, E, I, H)
    x = acts_bf16(T, H, seed=541 + T)
    router = Router(card, wr.cuda(), K)
    layer = MxExpertsLayer(card, to_gpu(ex), oss=False)
    _, weights, picks = router(x.cuda())
    y = layer(x.cuda(), picks, weights)
    torch.cuda.synchronize()
    _, ow, opicks = omoe.router(bits16(wr), x.float().numpy(), K, "bf16")
    assert np.array_equal(picks.cpu().numpy().astype(np.int64), opicks)
    want = oracle_mx(ex, x, opicks, weights.float().cpu().numpy(), oss=False)
    got = y.float().cpu().numpy()
    assert np.abs(want).max() > 0
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()
    # the grouped gate/up kernel and the pair kernel: the same bits
    card.set_tuning("moe_grouped", 0)
    y0 = layer(x.cuda(), picks, weights).clone()
    card.set_tuning("moe_grouped", 1)
    y1 = layer(x.cuda(), picks, weights).clone()
    card.set_tuning("moe_grouped", -1)
    assert torch.equal(y0, y1) and torch.equal(y0, y)


@pytest.mark.parametrize("layer,T", [(0, 1), (1, 3), (2, 8), (3, 16)])
def test_gpt_oss_experts_on_the_reference_fixture(card, layer, T):
    """the reference's tiny gpt-oss expert tensors as stored (interleaved gate / up rows, biases): the gpt-oss middle on
    the GPU against the CPU path restated in oracle/moe.py (itself held to transformers' GptOssExperts in
    tests/test_oracle_moe.py), picks drawn, weights a softmax over them; within 1e-2 of the largest output"""
    import os

    from btb_amd.load import load_mx_experts
    from btb_amd.moe import MxExpertsLayer

    from .helpers import GOLDEN

    ex = load_mx_experts(os.path.join(GOLDEN, "tiny_gpt_oss"), layer, device="cpu")
    assert ex.gate_up_bias is not None and ex.down_bias is not None and (ex.experts, ex.hidden, ex.intermediate) == (8, 64, 64)
    g = gen(560 + layer)
    k = 4
    x = torch.randn(T, ex.hidden, generator=g).to(torch.bfloat16)
    picks = torch.stack([torch.randperm(ex.experts, generator=g)[:k] for _ in range(T)])
    w = torch.softmax(torch.randn(T, k, generator=g), dim=-1).to(torch.bfloat16)
    y = MxExpertsLayer(card, to_gpu(ex))(x.cuda(), picks.to(torch.int32).cuda(), w.cuda())
    want = oracle_mx(ex, x, picks.numpy(), w.float().numpy(), oss=True)
    got = y.float().cpu().numpy()
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()
    # the biases and the interleaving matter at this size: without them the result is far off
    bare = oracle_mx(ex, x, picks.numpy(), w.float().numpy(), oss=False)
    assert np.abs(bare - want).max() > 5e-2 * np.abs(want).max()


def test_gpt_oss_experts_at_its_real_row_lengths(card):
    """gpt-oss's 2880-wide rows (90 blocks: no power of two, a span's last units guarded), the clamps exercised by
    large activations"""
    from btb_amd.load import MxExperts
    from btb_amd.moe import MxExpertsLayer

    E_, H_, I_, k, T = 6, 2880, 2880, 4, 3
    ex = mx_stacks(570, E_, I_, H_)
    g = gen(571)
    ex = MxExperts(ex.gate_up_blocks, ex.gate_up_scales, ex.down_blocks, ex.down_scales,
                   (torch.randn(E_, 2 * I_, generator=g) * 0.5).to(torch.bfloat16),
                   (torch.randn(E_, H_, generator=g) * 0.1).to(torch.bfloat16))
    x = (torch.randn(T, H_, generator=g) * 6.0).to(torch.bfloat16)      # gate / up values past the limit of 7
    picks = torch.stack([torch.randperm(E_, generator=g)[:k] for _ in range(T)])
    w = torch.softmax(torch.randn(T, k, generator=g), dim=-1).to(torch.bfloat16)
    y = MxExpertsLayer(card, to_gpu(ex))(x.cuda(), picks.to(torch.int32).cuda(), w.cuda())
    want = oracle_mx(ex, x, picks.numpy(), w.float().numpy(), oss=True)
    got = y.float().cpu().numpy()
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()


def test_mxfp4_experts_refusals(card):
    from btb_amd.load import MxExperts
    from btb_amd.moe import MxExpertsLayer

    ex = to_gpu(mx_stacks(580, 4, 64, 64))
    x = torch.zeros(2, 64, dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros(2, 2, dtype=torch.int32, device="cuda")
    w = torch.ones(2, 2, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        card.moe_experts_mx4(ex, x[:, :32], idx, w)
    with pytest.raises(ValueError):
        card.moe_experts_mx4(ex, x, idx, w[:, :1])
    biased = MxExperts(ex.gate_up_blocks, ex.gate_up_scales, ex.down_blocks, ex.down_scales,
                       torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda"), None)
    with pytest.raises(ValueError):
        MxExpertsLayer(card, biased, oss=False)
    L = card.lib
    p = lambda t: t.data_ptr()
    h = torch.zeros(2, 2, 64, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(2, 64, dtype=torch.bfloat16, device="cuda")
    a = (p(ex.gate_up_blocks), p(ex.gate_up_scales), p(ex.down_blocks), p(ex.down_scales))
    assert L.btb_hip_moe_experts_mxfp4(None, a[1], a[2], a[3], None, None, p(x), p(idx), p(w), p(h), p(y), 2, 2, 4, 64, 64,
                                       0, 0.0, 0.0, None) == -1
    assert L.btb_hip_moe_experts_mxfp4(*a, None, None, p(x), p(idx), p(w), p(h), p(y), 2, 2, 4, 48, 64, 0, 0.0, 0.0,
                                       None) == -6          # H % 32
    assert L.btb_hip_moe_experts_mxfp4(*a, p(y), None, p(x), p(idx), p(w), p(h), p(y), 2, 2, 4, 64, 64, 0, 0.0, 0.0,
                                       None) == -6          # a bias without the gpt-oss form
    assert bool((y == 0).all())
