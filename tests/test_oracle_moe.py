"""Pins oracle/moe.py on the CPU against statements it was not written from.

* the whole f32 layer against a plain-torch layer: `softmax -> torch.topk -> / sum -> sum_e w_e * W_dn(silu(g) * u)`,
  every token a dense loop over its own picks, torch matmuls - another summation order, another top-k, so the two
  agree to rounding (1e-5 of the largest output) and a structural mistake in either cannot pass;
* hand cases whose answers are worked out below, chosen so that one plausible mistake each fails: the gate / up halves
  swapped, the renormalisation dropped, the expert sum taken in descending instead of ascending order (bf16 rows,
  values where the order of three additions shows), ties going to the higher index;
* `group_picks` against the one-hot / `torch.where` listing the reference's docstring names (host.py:283-296).

The reference: btb/engine/families/qwen4/router.py:43-51, btb/engine/host.py:508-569 (one row), :906-967 (several).
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import codecs
from oracle import moe as omoe

from .helpers import bits16, gen


def stacks(E, I, H, seed, std=0.02):
    g = gen(seed)
    wr = (torch.randn(E, H, generator=g) * std).to(torch.bfloat16)
    gu = (torch.randn(E, 2 * I, H, generator=g) * std).to(torch.bfloat16)
    dn = (torch.randn(E, H, I, generator=g) * std).to(torch.bfloat16)
    return wr, gu, dn


def torch_layer(wr, gu, dn, x, k):
    """the textbook layer in f32 torch, token by token over its own picks"""
    wr, gu, dn, x = wr.float(), gu.float(), dn.float(), x.float()
    I = dn.shape[2]
    logits = x @ wr.T
    probs = torch.softmax(logits, dim=-1)
    top, idx = torch.topk(probs, k, dim=-1)
    top = top / top.sum(dim=-1, keepdim=True)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(k):
            e = int(idx[t, j])
            a = gu[e] @ x[t]
            h = torch.nn.functional.silu(a[:I]) * a[I:]
            out[t] += top[t, j] * (dn[e] @ h)
    return out.numpy(), logits.numpy(), top.numpy(), idx.numpy()


@pytest.mark.parametrize("T,E,k,I,H", [(1, 16, 4, 32, 64), (5, 32, 8, 48, 96), (8, 128, 8, 24, 128)])
def test_the_f32_layer_agrees_with_a_plain_torch_layer(T, E, k, I, H):
    wr, gu, dn = stacks(E, I, H, seed=T * 7 + E, std=0.2)   # std 0.2: outputs far above f32 noise
    x = torch.randn(T, H, generator=gen(900 + T)).to(torch.bfloat16)
    got, logits, w, picks = omoe.layer(bits16(wr), bits16(gu), bits16(dn), x.float().numpy(), k, dt="f32")
    want, wlogits, wtop, widx = torch_layer(wr, gu, dn, x, k)
    assert np.array_equal(picks, widx)                      # ordered: value descending
    assert np.abs(logits - wlogits).max() <= 1e-5 * np.abs(wlogits).max()
    assert np.abs(w - wtop).max() <= 1e-6
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


def test_the_bf16_layer_stays_close_to_the_f32_one():
    wr, gu, dn = stacks(32, 48, 96, seed=3, std=0.2)
    x = torch.randn(4, 96, generator=gen(77)).to(torch.bfloat16)
    a, *_ = omoe.layer(bits16(wr), bits16(gu), bits16(dn), x.float().numpy(), 8, dt="bf16")
    b, *_ = omoe.layer(bits16(wr), bits16(gu), bits16(dn), x.float().numpy(), 8, dt="f32")
    assert np.array_equal(a, codecs.round_bf16(a))          # every output is a bf16
    assert np.abs(a - b).max() <= 2e-2 * np.abs(b).max()


# ---- hand cases ---------------------------------------------------------------------------------------------------


def bf(a):
    return bits16(torch.tensor(a, dtype=torch.float32).to(torch.bfloat16))


def test_router_by_hand_renormalises_and_orders_by_value():
    # H = 1, x = 1: logits are the router column. softmax(ln 1, ln 2, ln 4, ln 1) = (1, 2, 4, 1) / 8
    wr = bf([[0.0], [np.log(2.0)], [np.log(4.0)], [0.0]])
    x = np.ones((1, 1), np.float32)
    _, w, picks = omoe.router(wr, x, 2, dt="f32")
    assert picks.tolist() == [[2, 1]]                       # value descending, not index order
    lg = codecs.bf16_bits_to_f32(wr)[:, 0].astype(np.float64)
    p = np.exp(lg) / np.exp(lg).sum()
    assert np.allclose(w, [[p[2] / (p[2] + p[1]), p[1] / (p[2] + p[1])]], atol=1e-6)
    assert abs(float(w.sum()) - 1.0) < 1e-6                 # dropped renormalisation: the sum would be ~0.75
    _, w_raw, _ = omoe.router(wr, x, 2, dt="f32", norm_topk=False)
    assert np.allclose(w_raw, [[p[2], p[1]]], atol=1e-6) and float(w_raw.sum()) < 0.8


def test_router_ties_go_to_the_lower_index():
    """equal probabilities: the lower expert index first (btb_kernels.cu:848-851; torch.topk's CPU rule as well)"""
    wr = bf([[1.0], [2.0], [2.0], [1.0], [2.0]])
    _, w, picks = omoe.router(wr, np.ones((1, 1), np.float32), 2, dt="f32")
    assert picks.tolist() == [[1, 2]] and w.tolist() == [[0.5, 0.5]]
    _, _, picks = omoe.router(wr, np.ones((1, 1), np.float32), 4, dt="f32")
    assert picks.tolist() == [[1, 2, 4, 0]]


def test_experts_by_hand_gate_is_the_first_half():
    """one expert, H = 1, I = 1: gate row = 2, up row = 3, down = 1, x = 1 -> silu(2) * 3. Swapped halves: silu(3) * 2"""
    gu = bf([[[2.0], [3.0]]])        # [E=1, 2I=2, H=1]: gate row first, then up
    dn = bf([[[1.0]]])
    x = np.ones((1, 1), np.float32)
    out = omoe.experts(gu, dn, x, np.array([[0]]), np.ones((1, 1), np.float32), dt="f32")
    silu = lambda v: v / (1.0 + np.exp(-v))
    assert abs(out[0, 0] - silu(2.0) * 3.0) < 1e-6
    assert abs(silu(2.0) * 3.0 - silu(3.0) * 2.0) > 0.4     # the two readings are far apart


def test_experts_apply_the_picks_weight_by_position():
    """token 0 picks (1, 0) with weights (0.75, 0.25): expert 1 gets 0.75, not 0.25"""
    gu = bf([[[1.0], [1.0]], [[1.0], [2.0]]])               # expert 0: up 1, expert 1: up 2
    dn = bf([[[1.0]], [[1.0]]])
    x = np.ones((1, 1), np.float32)
    s = 1.0 / (1.0 + np.exp(-1.0))
    out = omoe.experts(gu, dn, x, np.array([[1, 0]]), np.array([[0.75, 0.25]], np.float32), dt="f32")
    assert abs(out[0, 0] - (0.75 * s * 2.0 + 0.25 * s * 1.0)) < 1e-6


def test_expert_sum_runs_in_ascending_expert_order_in_bf16():
    """three experts whose weighted outputs are 256, 1, 1 (as experts 0, 1, 2). bf16 has 8 bits: 256 + 1 = 257 rounds
    to 256 (tie to even), then + 1 again 256: ascending order gives 256. Descending gives (1 + 1) + 256 = 258.
    The picks arrive in value order (2, 1, 0), so summing in pick order would also give 258."""
    big = 256.0
    # every expert computes the same thing, bf16(bf16(silu(8)) * 1) = 8 (silu(8) = 7.9973 rounds to 8.0); the picks'
    # weights (exact powers of two) carry the three values
    gu = bf([[[8.0], [1.0]]] * 3)
    dn = bf([[[1.0]]] * 3)
    x = np.ones((1, 1), np.float32)
    base = omoe.experts(gu[:1], dn[:1], x, np.array([[0]]), np.ones((1, 1), np.float32), dt="bf16")[0, 0]
    assert base == 8.0
    wts = np.array([[1.0 / 8.0, 1.0 / 8.0, big / 8.0]], np.float32)        # for picks (2, 1, 0)
    out = omoe.experts(gu, dn, x, np.array([[2, 1, 0]]), wts, dt="bf16")
    assert out[0, 0] == 256.0
    # the same numbers with the big value on the highest expert: ascending order adds 1 + 1 first -> 258
    wts2 = np.array([[big / 8.0, 1.0 / 8.0, 1.0 / 8.0]], np.float32)       # picks (2, 1, 0): expert 2 is the big one
    out2 = omoe.experts(gu, dn, x, np.array([[2, 1, 0]]), wts2, dt="bf16")
    assert out2[0, 0] == 258.0
    # in f32 rows nothing is lost either way
    assert omoe.experts(gu, dn, x, np.array([[2, 1, 0]]), wts, dt="f32")[0, 0] == pytest.approx(
        258.0 * omoe.silu(np.float32(8.0)) / 8.0, rel=1e-6)


def test_experts_round_at_each_step_of_the_dtype_chain():
    """bf16 rows: gu -> bf16, silu -> bf16, product -> bf16, down -> bf16, times weight -> bf16 (host.py:547-569)"""
    rng = np.random.default_rng(5)
    H, I = 16, 8
    gu_f = codecs.round_bf16(rng.standard_normal((1, 2 * I, H)).astype(np.float32) * 0.3)
    dn_f = codecs.round_bf16(rng.standard_normal((1, H, I)).astype(np.float32) * 0.3)
    x = codecs.round_bf16(rng.standard_normal((1, H)).astype(np.float32))
    w = codecs.round_bf16(np.array([[0.37]], np.float32))
    gu_b = bits16(torch.from_numpy(gu_f).to(torch.bfloat16))
    dn_b = bits16(torch.from_numpy(dn_f).to(torch.bfloat16))
    got = omoe.experts(gu_b, dn_b, x, np.array([[0]]), w, dt="bf16")[0]
    R = codecs.round_bf16
    a = R((gu_f[0].astype(np.float64) @ x[0].astype(np.float64)).astype(np.float32))
    s = R((a[:I].astype(np.float64) / (1.0 + np.exp(-a[:I].astype(np.float64)))).astype(np.float32))
    h = R(s * a[I:])
    d = R((dn_f[0].astype(np.float64) @ h.astype(np.float64)).astype(np.float32))
    want = R(d * w[0, 0])
    # f64 matvecs against the oracle's f32 lane order: at most one bf16 step apart, and mostly equal
    ulp = np.abs(want) * 2.0 ** -7 + 1e-30
    assert np.all(np.abs(got - want) <= ulp)
    assert np.mean(got == want) >= 0.75


def test_group_picks_lists_an_experts_pairs_pick_major_then_row():
    g = gen(41)
    T, k, E = 6, 4, 10
    picks = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    pos, row, offs, counts = omoe.group_picks(picks.numpy(), E)
    mask = torch.nn.functional.one_hot(picks, E).permute(2, 1, 0)          # [E, k, T]
    for e in range(E):
        p, r = torch.where(mask[e])
        a, n = int(offs[e]), int(counts[e])
        assert n == len(p)
        assert pos[a : a + n].tolist() == p.tolist() and row[a : a + n].tolist() == r.tolist()
    assert int(counts.sum()) == T * k and offs[0] == 0


# -- MXFP4 expert stacks, gpt-oss's middle ---------------------------------------------------------------------------


def oss_fixture(layer: int = 0):
    """the reference's tiny gpt-oss expert tensors (tests/golden/tiny_gpt_oss, copied as data): blocks, scales, biases"""
    import os

    from safetensors import safe_open

    from .helpers import GOLDEN

    base = f"model.layers.{layer}.mlp.experts."
    with safe_open(os.path.join(GOLDEN, "tiny_gpt_oss", "experts-00001-of-00001.safetensors"), framework="pt") as f:
        return {n: f.get_tensor(base + n) for n in ("gate_up_proj_blocks", "gate_up_proj_scales", "gate_up_proj_bias",
                                                    "down_proj_blocks", "down_proj_scales", "down_proj_bias")}


def oss_inputs(T, E, k, H, seed):
    g = gen(seed)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    picks = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).numpy()
    w = torch.softmax(torch.randn(T, k, generator=g), dim=-1).to(torch.bfloat16)
    return x, picks, w


def run_oracle_oss(t, x, picks, w, dt, **kw):
    kw.setdefault("gu_bias", t["gate_up_proj_bias"].float().numpy())
    kw.setdefault("dn_bias", t["down_proj_bias"].float().numpy())
    return omoe.experts_mx4(t["gate_up_proj_blocks"].numpy(), t["gate_up_proj_scales"].numpy(),
                            t["down_proj_blocks"].numpy(), t["down_proj_scales"].numpy(), x.float().numpy(), picks,
                            w.float().numpy(), dt=dt, **kw)


@pytest.mark.parametrize("layer,T", [(0, 1), (1, 5), (3, 8)])
def test_gpt_oss_experts_agree_with_transformers_over_the_dequantised_stacks(layer, T):
    """the f32 chain against transformers' GptOssExperts (a library here, not the reference) holding the same stacks
    dequantised: interleaved halves, biases, clamps, (up + 1) * gate * sigmoid(alpha gate), the down bias before the
    weight, the experts summed per row"""
    tm = pytest.importorskip("transformers.models.gpt_oss.modeling_gpt_oss")
    t = oss_fixture(layer)
    E, I2, gh = t["gate_up_proj_scales"].shape
    H, I, k = gh * 32, I2 // 2, 4
    x, picks, w = oss_inputs(T, E, k, H, seed=950 + layer)
    got = run_oracle_oss(t, x, picks, w, "f32")

    from transformers import GptOssConfig

    m = tm.GptOssExperts(GptOssConfig(intermediate_size=I, num_local_experts=E, hidden_size=H))
    gu = torch.from_numpy(codecs.mxfp4_dequantize(t["gate_up_proj_blocks"].numpy(), t["gate_up_proj_scales"].numpy()))
    dn = torch.from_numpy(codecs.mxfp4_dequantize(t["down_proj_blocks"].numpy(), t["down_proj_scales"].numpy()))
    with torch.no_grad():
        m.gate_up_proj.copy_(gu.reshape(E, 2 * I, H).transpose(1, 2))
        m.down_proj.copy_(dn.reshape(E, H, I).transpose(1, 2))
        m.gate_up_proj_bias.copy_(t["gate_up_proj_bias"].float())
        m.down_proj_bias.copy_(t["down_proj_bias"].float())
        want = m(x.float(), router_indices=torch.from_numpy(picks), routing_weights=w.float()).numpy()
    assert np.abs(want).max() > 1e-3
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    # planted mistakes, each far past the bar: the halves concatenated, no clamp (limit huge moves nothing here, so a
    # tiny limit stands in for "the clamp is applied"), up without its + 1 (alpha = 0 and the bias dropped differ too)
    for wrong in (dict(oss=False, gu_bias=None, dn_bias=None), dict(limit=0.01), dict(alpha=0.0), dict(gu_bias=None),
                  dict(dn_bias=None)):
        bad = run_oracle_oss(t, x, picks, w, "f32", **wrong)
        assert np.abs(bad - want).max() > 1e-3 * np.abs(want).max(), wrong


def test_gpt_oss_gate_rounds_where_torch_rounds_it():
    """the bf16 chain's rounding points: the same expression evaluated by torch on bf16 tensors, bit for bit, on
    values that cross both clamps"""
    g = gen(960)
    gu = (torch.randn(64, 256, generator=g) * 4.0).to(torch.bfloat16)
    alpha, limit = 1.702, 7.0
    gate, up = gu[..., ::2], gu[..., 1::2]
    gate = gate.clamp(min=None, max=limit)
    up = up.clamp(min=-limit, max=limit)
    want = (up + 1) * (gate * torch.sigmoid(gate * alpha))
    assert want.dtype == torch.bfloat16 and bool((gu.float().abs() > limit).any())
    got = omoe.gpt_oss_gate(gu.float().numpy(), alpha, limit, "bf16")
    # torch's bf16 sigmoid and this one may differ in the last f32 bit before the rounding: a handful of bf16 flips
    flips = np.count_nonzero(bits16(want) != bits16(torch.from_numpy(got).to(torch.bfloat16)))
    assert flips <= want.numel() // 500, flips
    assert np.abs(got - want.float().numpy()).max() <= 2.0**-7 * np.abs(want.float().numpy()).max()
