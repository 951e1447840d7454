"""The whole decode step on the GPU - eager and as a captured, replayed hipGraph - against the CPU restatement
(oracle/decode.py) at a reduced Qwen3 shape, in bf16 and with every linear in the 12-bit packed form.

Bars: the two sides share every rounding point and differ in the order of the f32 additions inside matvecs, norms and
attention, so a bf16 rounding can flip here and there and travel through the layers: logits are held to 3e-2 of the
largest logit, and the greedy token must agree whenever the oracle's top-2 margin exceeds that bar. The packed stack
must reproduce the bf16 stack's GPU logits to the same bar (on the CPU the pair is bit-equal: native/tests/gemv.rs:297-299)
and a replayed graph must reproduce the eager step bit for bit, replay after replay."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from btb_amd.decode import DecodeStep, Linear, StackConfig
from btb_amd.pack12 import P12Weight
from oracle import decode as od

from .helpers import bits16, gen

pytestmark = pytest.mark.gpu

CFG = StackConfig(layers=3, hidden=256, q_heads=4, kv_heads=2, head_dim=128, intermediate=512, vocab=1000)
CAP, N0, TOKEN = 96, 40, 17


def make_weights(card, packed: bool, CFG: StackConfig = CFG):
    g = gen(700)
    W, dev = {}, {}

    def mat(name, rows, cols):
        t = (torch.randn(rows, cols, generator=g) * 0.05).to(torch.bfloat16)
        W[name] = bits16(t)
        dev[name] = Linear(card, P12Weight.pack(t.cuda(), card) if packed else t.cuda())

    def vec(name, n):
        t = (1.0 + 0.1 * torch.randn(n, generator=g)).to(torch.bfloat16)
        W[name] = bits16(t)
        dev[name] = t.cuda()

    H, I = CFG.hidden, CFG.intermediate
    for i in range(CFG.layers):
        L = f"layers.{i}."
        mat(L + "qkv", CFG.qkv_rows, H)
        mat(L + "o", H, CFG.q_heads * CFG.head_dim)
        mat(L + "gu", 2 * I, H)
        mat(L + "down", H, I)
        for n_, ln in (("ln1", H), ("ln2", H), ("wq", CFG.head_dim), ("wk", CFG.head_dim)):
            vec(L + n_, ln)
    emb = (torch.randn(CFG.vocab, H, generator=g)).to(torch.bfloat16)
    W["embed"], dev["embed"] = bits16(emb), emb.cuda()
    vec("norm", H)
    mat("head", CFG.vocab, H)
    kv = torch.randn(CFG.layers, 2, CFG.kv_heads, CAP, CFG.head_dim, generator=g).to(torch.bfloat16)
    return W, dev, kv


def run_gpu(card, dev, kv, graph: bool, fold: bool = True, fused: bool = True):
    step = DecodeStep(card, CFG, dev, CAP, fold_silu=fold, fused=fused)
    step.kv.copy_(kv.cuda())
    step.reset(N0, TOKEN)
    if graph:
        step.capture(warmup=1)
        step.kv.copy_(kv.cuda())
        step.reset(N0, TOKEN)
        step.replay()
    else:
        step.body()
    torch.cuda.synchronize()
    return step


@pytest.mark.parametrize("packed", [False, True])
def test_decode_step_matches_cpu_path(card, packed):
    W, dev, kv = make_weights(card, packed)
    step = run_gpu(card, dev, kv, graph=False)
    okv = kv.float().numpy().copy()
    want, tok = od.step(CFG, W, TOKEN, okv, N0)
    got = step.logits[0].float().cpu().numpy()
    bar = 3e-2 * np.abs(want).max()
    assert np.abs(got - want).max() <= bar
    top2 = np.sort(want)[-2:]
    if top2[1] - top2[0] > 2 * bar:
        assert step.token() == tok
    # the step wrote its K / V row at slot N0, advanced the cache and fed its token forward
    assert int(step.n0[0]) == N0 + 1 and int(step.host_n0[0]) == N0 + 1 and int(step.ids[0]) == step.token()
    krow = step.kv[:, 0, :, N0].float().cpu().numpy()
    assert np.abs(krow - okv[:, 0, :, N0]).max() <= 3e-2 * np.abs(okv[:, 0, :, N0]).max()


def test_packed_stack_tracks_the_bf16_stack(card):
    _, dev_b, kv = make_weights(card, False)
    _, dev_p, _ = make_weights(card, True)
    a = run_gpu(card, dev_b, kv, graph=False, fold=False).logits.float()
    b = run_gpu(card, dev_p, kv, graph=False).logits.float()
    assert (a - b).abs().max() <= 3e-2 * a.abs().max()
    c = run_gpu(card, dev_b, kv, graph=False, fold=True).logits.float()
    assert (a - c).abs().max() <= 3e-2 * a.abs().max()   # the SwiGLU fold and the two-kernel form agree


@pytest.mark.parametrize("packed", [False, True])
def test_fused_launches_change_no_bit(card, packed):
    """the six-launch layer (norms folded into the matvecs' x loads, gate / up / activation in one kernel) against the
    one-launch-per-operator sequence: the same bits in the logits, the residual stream and the cache row"""
    _, dev, kv = make_weights(card, packed)
    a = run_gpu(card, dev, kv, graph=False, fold=False, fused=False)
    b = run_gpu(card, dev, kv, graph=False, fused=True)
    assert torch.equal(a.logits, b.logits) and a.token() == b.token()
    assert torch.equal(a.kv[:, :, :, N0], b.kv[:, :, :, N0])


def test_graph_replays_equal_the_eager_step(card):
    """several replays, with eager work and synchronisations between them, each checked against the eager result"""
    W, dev, kv = make_weights(card, False)
    eager = run_gpu(card, dev, kv, graph=False)
    want_logits, want_tok = eager.logits.clone(), eager.token()
    step = DecodeStep(card, CFG, dev, CAP)
    step.kv.copy_(kv.cuda())
    step.reset(N0, TOKEN)
    step.capture(warmup=1)
    for rep in range(4):
        step.kv.copy_(kv.cuda())
        step.reset(N0, TOKEN)
        step.replay()
        torch.cuda.synchronize()
        assert torch.equal(step.logits, want_logits), rep
        assert step.token() == want_tok and int(step.host_n0[0]) == N0 + 1
        junk = torch.randn(1 << 16, device="cuda").sum()   # unrelated eager work between the replays
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
    # consecutive replays decode a sequence: each step feeds its token and cache row to the next
    step.kv.copy_(kv.cuda())
    step.reset(N0, TOKEN)
    toks = []
    for _ in range(3):
        step.replay()
        torch.cuda.synchronize()
        toks.append(step.token())
    assert int(step.n0[0]) == N0 + 3 and toks[0] == want_tok



@pytest.mark.parametrize("fused", [False, True])
def test_verify_pass_over_a_tree(card, fused):
    """a pass of several rows as a tree (speculative verify): the rows on a root-to-leaf path see exactly what they see
    as a chain pass of that path's tokens, so their logits agree with that pass's - to the step's bar, not to the bit:
    the attention folds the same keys in batches cut elsewhere - and a tree that is a chain is the chain pass bit for
    bit"""
    _, dev, kv = make_weights(card, False)
    par, toks = [-1, 0, 0, 2, 2], [17, 5, 901, 33, 4]

    def run(T, tokens, tree):
        step = DecodeStep(card, CFG, dev, CAP, T=T, fused=fused, fold_silu=fused)
        step.kv.copy_(kv.cuda())
        step.reset(N0, tokens[0])
        step.ids.copy_(torch.tensor(tokens, dtype=torch.int32))
        if tree is not None:
            step.set_tree(tree)
        step.body()
        torch.cuda.synchronize()
        return step.logits.float().clone()

    tree = run(5, toks, par)
    for path in ([0, 1], [0, 2, 3], [0, 2, 4]):
        chain = run(len(path), [toks[t] for t in path], None)
        for i, t in enumerate(path):
            assert float((tree[t] - chain[i]).abs().max()) <= 3e-2 * float(chain[i].abs().max()), (path, t)
    a = run(4, toks[:4], [-1, 0, 1, 2])
    b = run(4, toks[:4], None)
    assert torch.equal(a, b)


def test_sequence_by_width(card):
    """the sequence a step takes when none is asked for - fused launches up to three rows, one launch per operator (its
    matvecs on the matrix cores) from four - and that a pass of eight rows gives the same logits either way, to the
    step's bar"""
    _, dev, kv = make_weights(card, False)
    assert DecodeStep(card, CFG, dev, CAP).fused and DecodeStep(card, CFG, dev, CAP, T=3).fused
    toks = [17, 5, 901, 33, 4, 250, 7, 12]
    out = []
    for fused in (None, True):
        step = DecodeStep(card, CFG, dev, CAP, T=8, fused=fused)
        assert step.fused == bool(fused) and step.fold_silu == bool(fused)
        step.kv.copy_(kv.cuda())
        step.reset(N0, toks[0])
        step.ids.copy_(torch.tensor(toks, dtype=torch.int32))
        step.body()
        torch.cuda.synchronize()
        out.append(step.logits.float().clone())
    assert float((out[0] - out[1]).abs().max()) <= 3e-2 * float(out[1].abs().max())
    assert torch.equal(out[0].argmax(dim=1), out[1].argmax(dim=1))


def test_a_step_past_the_cache_is_refused(card):
    """the kernels write the pass's rows at n0 + t without looking; the host counts the cache's rows from the last reset
    and refuses the step - eager or replayed - that would write past the end"""
    _, dev, kv = make_weights(card, False)
    step = DecodeStep(card, CFG, dev, CAP, T=2)
    step.reset(CAP - 3, 5)
    step.body()          # rows CAP-3, CAP-2
    step.body()          # rows CAP-2, CAP-1
    with pytest.raises(RuntimeError, match="cache is full"):
        step.body()
    torch.cuda.synchronize()
    step.reset(CAP - 3, 5)
    step.capture(warmup=1)
    step.replay()
    with pytest.raises(RuntimeError, match="cache is full"):
        step.replay()
    torch.cuda.synchronize()
