"""Pins oracle/decode.py on the CPU, with nothing from the GPU code in the loop.

* `od.step` over the reference's tiny Qwen3 store against the receipts the reference banked for it
  (tests/fixtures/receipts_qwen3.pt, written by tests/make_fixtures.py:1230-1264 with the f32 host engine): with f32
  rows the logits after the 16-token prompt and the cached K / V rows agree to 1e-4, the ten greedy tokens are equal;
  with bf16 rows (the card's rounding points) they stay within the bars the GPU path is held to (3e-2 / 2e-2).
* each piece against something it was not written from: attention against a brute-force f64 softmax spelled out key by
  key, norm + rope against the textbook rotate-half on hand cases where a wrong sign or a swapped half shows, the
  residual norm and SwiGLU against closed forms, the greedy pick's tie rule.
* mutation checks: the step with one plausible mistake planted (gate / up halves swapped, rope sign flipped, kv head
  mapping transposed, a dropped residual) must FAIL the f32 bar by a factor of ten or more - the receipts
  can tell these apart (the tiny model's weights are small, so some mistakes move its logits by a percent only: it is
  the 1e-4 bar on the f32 form that pins the structure, the piece tests below that pin the rounding points).
"""

from __future__ import annotations

import math
import os

import numpy as np
import pytest
import torch

from btb_amd.load import Store, read_config
from oracle import codecs
from oracle import decode as od

from .helpers import GOLDEN, bits16

PROMPT = [3, 17, 42, 5, 99, 120, 7, 7, 200, 12, 45, 8, 3, 17, 60, 61]  # tests/helpers.py:256 of the reference
CAP = 32


@pytest.fixture(scope="module")
def receipts():
    return torch.load(os.path.join(GOLDEN, "receipts_qwen3.pt"), weights_only=True)


@pytest.fixture(scope="module")
def tiny():
    """(cfg, W): the reference's tiny Qwen3 store as the bit patterns od.step takes, q/k/v and gate/up stacked by rows"""
    path = os.path.join(GOLDEN, "tiny_qwen3")
    cfg, raw = read_config(path)
    store = Store(path)
    g = lambda n: bits16(store.get(n).to(torch.bfloat16))
    W = {}
    for i in range(cfg.layers):
        s, d = f"model.layers.{i}.", f"layers.{i}."
        W[d + "qkv"] = np.concatenate([g(s + f"self_attn.{p}_proj.weight") for p in "qkv"], axis=0)
        W[d + "o"] = g(s + "self_attn.o_proj.weight")
        W[d + "gu"] = np.concatenate([g(s + "mlp.gate_proj.weight"), g(s + "mlp.up_proj.weight")], axis=0)
        W[d + "down"] = g(s + "mlp.down_proj.weight")
        W[d + "ln1"] = g(s + "input_layernorm.weight")
        W[d + "ln2"] = g(s + "post_attention_layernorm.weight")
        W[d + "wq"] = g(s + "self_attn.q_norm.weight")
        W[d + "wk"] = g(s + "self_attn.k_norm.weight")
    W["embed"] = g("model.embed_tokens.weight")
    W["norm"] = g("model.norm.weight")
    assert raw["tie_word_embeddings"] is True
    W["head"] = W["embed"]
    return cfg, W


def run_prompt(cfg, W, dt, greedy=10, step=od.step):
    kv = np.zeros((cfg.layers, 2, cfg.kv_heads, CAP, cfg.head_dim), np.float32)
    n0 = 0
    for tok in PROMPT:
        logits, nxt = step(cfg, W, tok, kv, n0, dt)
        n0 += 1
    prompt_logits, keys = logits.copy(), kv[:, :, :, : len(PROMPT)].copy()
    toks = [nxt]
    for _ in range(greedy - 1):
        logits, nxt = step(cfg, W, toks[-1], kv, n0, dt)
        n0 += 1
        toks.append(nxt)
    return prompt_logits, keys, toks


def rb(v) -> float:
    """one value rounded to bf16"""
    return float(np.asarray(codecs.round_bf16(np.asarray([v], np.float32))).reshape(-1)[0])


def worst(got, want):
    want = want.float().numpy() if isinstance(want, torch.Tensor) else want
    return float(np.abs(got - want).max() / np.abs(want).max())


@pytest.mark.parametrize("dt,logit_bar,kv_bar", [("f32", 1e-4, 1e-4), ("bf16", 3e-2, 2e-2)])
def test_step_reproduces_the_reference_receipts(tiny, receipts, dt, logit_bar, kv_bar):
    cfg, W = tiny
    logits, keys, toks = run_prompt(cfg, W, dt)
    r = receipts["bf16"]
    assert worst(logits, r["prompt_logits"]) <= logit_bar
    assert toks == r["greedy"] == receipts["ref"]["greedy"]
    for i in range(cfg.layers):
        k_want, v_want = (t[0, :, : len(PROMPT)] for t in r["keys"][i])
        assert worst(keys[i, 0], k_want) <= kv_bar
        assert worst(keys[i, 1], v_want) <= kv_bar


CHUNK = [9, 33, 14, 71, 33, 5, 90, 2]       # tests/helpers.py:257-260 of the reference: the receipts' verify tree
PARENTS = [-1, 0, 1, 2, 1, 4, 0, 6]
PATH = [0, 1, 4, 5]


def test_step_reproduces_the_tree_pass_and_the_step_after_it(tiny, receipts):
    """`chunk_logits[t]` are the logits of tree row t, i.e. of the chain prompt + (root .. t); `next` those after the
    accepted path and its last token once more (tests/make_fixtures.py:1244-1249; tests/helpers.py:263-278 of the
    reference); `keys` hold the prompt, the accepted path and that step: 21 rows"""
    cfg, W = tiny
    kv0 = np.zeros((cfg.layers, 2, cfg.kv_heads, CAP, cfg.head_dim), np.float32)
    for n0, tok in enumerate(PROMPT):
        od.step(cfg, W, tok, kv0, n0, "f32")
    r = receipts["bf16"]
    for t in range(len(CHUNK)):
        chain, j = [], t
        while j >= 0:
            chain.append(CHUNK[j])
            j = PARENTS[j]
        kv = kv0.copy()
        for d, tok in enumerate(reversed(chain)):
            logits, _ = od.step(cfg, W, tok, kv, len(PROMPT) + d, "f32")
        assert worst(logits, r["chunk_logits"][t]) <= 1e-4, t
    kv = kv0.copy()
    seq = [CHUNK[j] for j in PATH] + [CHUNK[PATH[-1]]]
    for d, tok in enumerate(seq):
        logits, _ = od.step(cfg, W, tok, kv, len(PROMPT) + d, "f32")
    assert worst(logits, r["next"]) <= 1e-4
    n = len(PROMPT) + len(seq)
    for i in range(cfg.layers):
        assert tuple(r["keys"][i][0].shape) == (1, cfg.kv_heads, n, cfg.head_dim)
        assert worst(kv[i, 0, :, :n], r["keys"][i][0][0]) <= 1e-4
        assert worst(kv[i, 1, :, :n], r["keys"][i][1][0]) <= 1e-4


# ---- planted mistakes must fail the receipts ---------------------------------------------------------------------


def _mutant(kind):
    def step(cfg, W, token, kv, n0, dt):
        Hq, Hk, D = cfg.q_heads, cfg.kv_heads, cfg.head_dim
        if kind == "halves":   # gate and up rows swapped: silu on the wrong half
            W = dict(W)
            for i in range(cfg.layers):
                gu = W[f"layers.{i}.gu"]
                W[f"layers.{i}.gu"] = np.concatenate([gu[cfg.intermediate:], gu[: cfg.intermediate]], axis=0)
            return od.step(cfg, W, token, kv, n0, dt)
        if kind == "no_qnorm":  # the q / k norms dropped
            W = {k: v for k, v in W.items() if not k.endswith((".wq", ".wk"))}
            return od.step(cfg, W, token, kv, n0, dt)
        saved = {}
        try:
            if kind == "rope_sign":
                saved["norm_rope"] = od.norm_rope

                def bad(v, wn, eps, cos, sin, dt="bf16"):
                    return saved["norm_rope"](v, wn, eps, cos, -sin, dt)

                od.norm_rope = bad
            elif kind == "kv_map":   # query head j reads kv head j % Hk instead of j // G
                saved["attention"] = od.attention

                def bad(q, K, V, scale, dt="bf16"):
                    G = q.shape[0] // K.shape[0]
                    perm = [(j % K.shape[0]) * G + j // K.shape[0] for j in range(q.shape[0])]
                    out = saved["attention"](q[perm], K, V, scale, dt)
                    inv = np.argsort(perm)
                    return out[inv]

                od.attention = bad
            elif kind == "scale":    # 1/D instead of 1/sqrt(D)
                saved["attention"] = od.attention
                od.attention = lambda q, K, V, scale, dt="bf16": saved["attention"](q, K, V, scale * scale, dt)
            elif kind == "eps":      # eps inside the mean dropped to the outside of the root
                saved["add_rmsnorm"] = od.add_rmsnorm
                od.add_rmsnorm = lambda h, y, w, eps, dt="bf16": saved["add_rmsnorm"](h, y, w, 1e-2, dt)
            return od.step(cfg, W, token, kv, n0, dt)
        finally:
            for k, v in saved.items():
                setattr(od, k, v)

    return step


@pytest.mark.parametrize("kind", ["halves", "no_qnorm", "rope_sign", "kv_map", "scale", "eps"])
def test_a_planted_mistake_fails_the_receipts(tiny, receipts, kind):
    cfg, W = tiny
    logits, keys, _ = run_prompt(cfg, W, "f32", greedy=1, step=_mutant(kind))
    r = receipts["bf16"]
    off = worst(logits, r["prompt_logits"])
    koff = max(worst(keys[i, 0], r["keys"][i][0][0, :, : len(PROMPT)]) for i in range(cfg.layers))
    assert max(off, koff) > 1e-3, (kind, off, koff)   # ten times the 1e-4 the f32 form is held to, at the least


# ---- the pieces, each against an independent statement --------------------------------------------------------------


def test_attention_against_a_brute_force_softmax():
    rng = np.random.default_rng(7)
    Hq, Hk, D, n = 8, 2, 16, 37
    q = codecs.round_bf16(rng.standard_normal((Hq, D)).astype(np.float32))
    K = codecs.round_bf16(rng.standard_normal((Hk, n, D)).astype(np.float32))
    V = codecs.round_bf16(rng.standard_normal((Hk, n, D)).astype(np.float32))
    scale = 1.0 / math.sqrt(D)
    got = od.attention(q, K, V, scale, "f32")
    G = Hq // Hk
    for j in range(Hq):
        g = j // G
        s = [scale * sum(float(q[j, d]) * float(K[g, t, d]) for d in range(D)) for t in range(n)]
        z = sum(math.exp(v) for v in s)
        for d in range(D):
            want = sum(math.exp(s[t]) / z * float(V[g, t, d]) for t in range(n))
            assert abs(got[j, d] - want) <= 1e-6 * max(1.0, abs(want))
    # the bf16 form is that, rounded once
    assert np.array_equal(od.attention(q, K, V, scale, "bf16"), codecs.round_bf16(got))


def test_attention_head_mapping_is_by_blocks_of_G():
    """with one key the output is that kv head's V row: query heads 0..G-1 read kv head 0, the next G kv head 1"""
    Hq, Hk, D = 4, 2, 8
    q = np.ones((Hq, D), np.float32)
    K = np.ones((Hk, 1, D), np.float32)
    V = np.stack([np.full((1, D), 1.0, np.float32), np.full((1, D), 2.0, np.float32)])
    out = od.attention(q, K, V, 0.5)
    assert out[:, 0].tolist() == [1.0, 1.0, 2.0, 2.0]


def test_norm_rope_hand_cases():
    D = 4
    one = bits16(torch.ones(D, dtype=torch.bfloat16))
    # no rotation at angle 0: only the norm acts. v = (3, 4, 0, 0): mean square 25/4, rstd = 2/5
    v = np.array([[3.0, 4.0, 0.0, 0.0]], np.float32)
    out = od.norm_rope(v, one, 0.0, np.ones(D, np.float32), np.zeros(D, np.float32), "f32")
    assert np.allclose(out, [[1.2, 1.6, 0.0, 0.0]], atol=1e-6)
    # a quarter turn (cos 0, sin 1), no norm weight: out = rotate_half(v) = (-v2, -v3, v0, v1)
    v = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    out = od.norm_rope(v, None, 0.0, np.zeros(D, np.float32), np.ones(D, np.float32), "f32")
    assert out.tolist() == [[-3.0, -4.0, 1.0, 2.0]]
    # a general angle per pair against complex multiplication: (v_i + i v_{i+D/2}) * e^{i a_i}
    a = np.array([0.3, 1.1], np.float64)
    cos, sin = np.cos(np.concatenate([a, a])).astype(np.float32), np.sin(np.concatenate([a, a])).astype(np.float32)
    out = od.norm_rope(v, None, 0.0, cos, sin, "f32")[0]
    z = (v[0, :2] + 1j * v[0, 2:]) * np.exp(1j * a)
    assert np.allclose(out, np.concatenate([z.real, z.imag]), atol=1e-6)
    # the norm weight multiplies after the scaling, per dim
    w = bits16(torch.tensor([1.0, 2.0, 0.5, 4.0], dtype=torch.bfloat16))
    v = np.array([[2.0, 2.0, 2.0, 2.0]], np.float32)
    out = od.norm_rope(v, w, 0.0, np.ones(D, np.float32), np.zeros(D, np.float32), "f32")
    assert np.allclose(out, [[1.0, 2.0, 0.5, 4.0]], atol=1e-6)


def test_norm_rope_rounding_points():
    """bf16 rows: the normed value, q*cos and the final sum are each rounded once (btb_kernels.cu:296-326)"""
    rng = np.random.default_rng(3)
    D = 8
    v = codecs.round_bf16(rng.standard_normal((2, D)).astype(np.float32))
    w = bits16(torch.from_numpy(1.0 + 0.1 * rng.standard_normal(D).astype(np.float32)).to(torch.bfloat16))
    cos = codecs.round_bf16(np.cos(rng.standard_normal(D)).astype(np.float32))
    sin = codecs.round_bf16(np.sin(rng.standard_normal(D)).astype(np.float32))
    got = od.norm_rope(v, w, 1e-6, cos, sin, "bf16")
    wf = codecs.bf16_bits_to_f32(w)
    for r in range(2):
        rstd = 1.0 / math.sqrt(sum(float(t) ** 2 for t in v[r]) / D + 1e-6)
        nv = [rb(np.float32(v[r, i] * np.float32(rstd)) * wf[i]) for i in range(D)]
        for i in range(D):
            rot = -nv[i + D // 2] if i < D // 2 else nv[i - D // 2]
            qc = rb(nv[i] * float(cos[i]))
            want = rb(rot * float(sin[i]) + qc)
            assert got[r, i] == want


def test_add_rmsnorm_closed_form_and_rounding():
    one = bits16(torch.ones(4, dtype=torch.bfloat16))
    h = np.array([[1.0, 1.0, 1.0, 1.0]], np.float32)
    y = np.array([[2.0, 3.0, -1.0, -1.0]], np.float32)       # h + y = (3, 4, 0, 0)
    h2, x = od.add_rmsnorm(h, y, one, 0.0, "f32")
    assert h2.tolist() == [[3.0, 4.0, 0.0, 0.0]] and np.allclose(x, [[1.2, 1.6, 0.0, 0.0]], atol=1e-6)
    h2b, xb = od.add_rmsnorm(h, y, one, 0.0, "bf16")
    assert np.array_equal(xb, codecs.round_bf16(np.array([[1.2, 1.6, 0.0, 0.0]], np.float32)))
    # the sum is rounded to bf16 before the norm reads it: 1 + 2^-9 is not a bf16
    h = np.array([[1.0, 0.0, 0.0, 0.0]], np.float32)
    y = np.array([[2.0 ** -9, 0.0, 0.0, 0.0]], np.float32)
    h2b, _ = od.add_rmsnorm(h, y, one, 0.0, "bf16")
    assert h2b[0, 0] == 1.0
    # eps sits inside the root with the mean
    _, x = od.add_rmsnorm(np.zeros((1, 4), np.float32), None, one, 0.25, "f32")
    assert np.all(x == 0.0)
    _, x = od.add_rmsnorm(np.full((1, 4), 0.5, np.float32), None, one, 0.75, "f32")   # mean 0.25 + 0.75 = 1
    assert np.allclose(x, 0.5)


def test_silu_mul_halves_and_rounding():
    gu = np.array([[0.0, 2.0, 5.0, 7.0]], np.float32)         # gate (0, 2), up (5, 7)
    out = od.silu_mul(gu, "f32")
    assert out[0, 0] == 0.0 and abs(out[0, 1] - 7.0 * 2.0 / (1.0 + math.exp(-2.0))) < 1e-5
    b = od.silu_mul(gu, "bf16")
    assert b[0, 1] == rb(rb(2.0 / (1.0 + math.exp(-2.0))) * 7.0)


def test_greedy_pick_takes_the_lowest_index_on_ties(tiny):
    """native/src/sample.rs:53-67: strict > from the left; np.argmax, which `step` uses, has the same rule"""
    assert int(np.argmax(np.array([1.0, 3.0, 3.0, 2.0], np.float32))) == 1


def test_rope_tables_are_the_default_rope():
    cos, sin = od.rope_tables(8, 10000.0, 5, "f32")
    for p in range(5):
        for i in range(4):
            a = p * 10000.0 ** (-2.0 * i / 8)
            assert abs(cos[p, i] - math.cos(a)) < 1e-6 and abs(sin[p, i + 4] - math.sin(a)) < 1e-6
    cb, _ = od.rope_tables(8, 10000.0, 5, "bf16")
    assert np.array_equal(cb, codecs.round_bf16(cos))
