"""The decode step at the full shape the benchmark times - the Qwen3-4B-shaped stack (36 layers, hidden 2560, 32 / 8
heads of 128, intermediate 9728, vocab 151936), 4096 keys of context, captured and replayed as a hipGraph - against
the CPU restatement (oracle/decode.py) on the same weights and cache.

Bars. The two sides share every rounding point and differ in the order of f32 additions; a flipped bf16 rounding then
travels through the random-init layers, and the difference grows with depth - measured on MI355X against the oracle,
root mean square of the logits' error over that of the logits (the worst logit over the largest is the same size):
0.4 % after 1 layer, 1.0 % after 4, 2.1 % after 12, 3.1 % after 24, 4.0 % after 36; the GPU's own bf16 and 12-bit
stacks (the same weights, another summation order) part by 2.8 % at 36. So the stack cut to its first layer and to
its first four is held to the 3-layer test's bar (3e-2 of the largest logit on every logit, and 1.5e-2 rms), which is
what pins the full-width kernels, and the full 36 layers to 6e-2 rms and 8e-2 on the worst logit, with the greedy
token equal whenever the oracle's top-2 margin exceeds twice that. The exact pins at full size are the
size-independent properties: the six-launch fused step equals the one-launch-per-operator step bit for bit (each of
those operators is held to the oracle at these very shapes in tests/test_gemv_gpu.py and tests/test_glue_gpu.py), a
replayed graph equals the eager step bit for bit, and the stack stored at 12 bits a weight (a lossless form) stays
within the same bars of the bf16 stack."""

from __future__ import annotations

import dataclasses

import numpy as np
import pytest
import torch

from btb_amd.decode import QWEN3_4B, DecodeStep, random_stack
from oracle import decode as od

from .helpers import bits16

pytestmark = pytest.mark.gpu

CAP, N0, TOKEN = 4104, 4095, 1234


def _rel(got: np.ndarray, want: np.ndarray) -> tuple[float, float]:
    """(worst error over the largest value, rms error over rms value)"""
    return (float(np.abs(got - want).max() / np.abs(want).max()),
            float(np.sqrt(np.mean((got - want) ** 2)) / np.sqrt(np.mean(want**2))))


def _run(card, w, kv, graph: bool, fused: bool = True, cfg=QWEN3_4B):
    step = DecodeStep(card, cfg, w, CAP, fold_silu=fused, fused=fused)
    step.kv.copy_(kv)
    step.reset(N0, TOKEN)
    if graph:
        step.capture(warmup=1)
        step.kv.copy_(kv)
        step.reset(N0, TOKEN)
        step.replay()
    else:
        step.body()
    torch.cuda.synchronize()
    return step


def test_full_shape_step_against_the_cpu_path(card):
    cfg = QWEN3_4B
    w = random_stack(card, cfg)
    g = torch.Generator(device="cuda").manual_seed(0x0B7B0909)
    kv = torch.randn(cfg.layers, 2, cfg.kv_heads, CAP, cfg.head_dim, generator=g, device="cuda").to(torch.bfloat16)
    eager = _run(card, w, kv, graph=False)
    graph = _run(card, w, kv, graph=True)
    assert torch.equal(eager.logits, graph.logits) and eager.token() == graph.token()
    assert torch.equal(eager.kv[:, :, :, N0], graph.kv[:, :, :, N0])
    plain = _run(card, w, kv, graph=False, fused=False)
    assert torch.equal(plain.logits, graph.logits) and torch.equal(plain.kv[:, :, :, N0], graph.kv[:, :, :, N0])
    del plain, eager

    W = {k: bits16(v.w if hasattr(v, "w") else v) for k, v in w.items()}
    okv = kv.float().cpu().numpy()
    want, tok = od.step(cfg, W, TOKEN, okv, N0)
    got = graph.logits[0].float().cpu().numpy()
    worst, rms = _rel(got, want)
    assert worst <= 8e-2 and rms <= 6e-2, (worst, rms)
    bar = 8e-2 * np.abs(want).max()
    top2 = np.sort(want)[-2:]
    if top2[1] - top2[0] > 2 * bar:
        assert graph.token() == tok
    krow = graph.kv[:, 0, :, N0].float().cpu().numpy()
    peak = np.abs(okv[:, 0, :, N0]).max()
    assert np.abs(krow[0] - okv[0, 0, :, N0]).max() <= 3e-2 * peak   # the first layer's new key row
    assert np.abs(krow - okv[:, 0, :, N0]).max() <= 8e-2 * peak      # every layer's, the drift included
    # the first layer alone and the first four, at the reduced-shape test's bar
    for nl in (1, 4):
        cut = dataclasses.replace(cfg, layers=nl)
        short = _run(card, w, kv[:nl], graph=False, cfg=cut)
        ref, _ = od.step(cut, W, TOKEN, kv[:nl].float().cpu().numpy(), N0)
        worst, rms = _rel(short.logits[0].float().cpu().numpy(), ref)
        assert worst <= 3e-2 and rms <= 1.5e-2, (nl, worst, rms)
    del W, okv

    packed = _run(card, random_stack(card, cfg, packed=True), kv, graph=True)
    worst, rms = _rel(packed.logits[0].float().cpu().numpy(), got)
    assert worst <= 8e-2 and rms <= 6e-2, (worst, rms)


@pytest.mark.parametrize("packed", [False, True])
def test_each_full_shape_layer_alone_against_the_cpu_path(card, packed):
    """Every one of the 36 full-shape layers on its own, at the tight bar: the layer is handed the CPU path's own
    input - the residual and the pending block output as the oracle's step had them at that depth (teacher forcing) -
    runs the step's launches (add + norm + qkv, attention over the 4096-key cache, o, add + norm + gate/up + SwiGLU,
    down) and must leave the oracle's residual and block output within 1e-2 of the largest value (measured: 7e-3 at worst), with no drift from
    the layers before it to lean on. Both stored forms: bf16, and the same weights at 12 bits a weight."""
    cfg = QWEN3_4B
    Hq, Hk, D, H, I = cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.hidden, cfg.intermediate
    w16 = random_stack(card, cfg)
    W = {k: bits16(v.w if hasattr(v, "w") else v) for k, v in w16.items()}
    w = random_stack(card, cfg, packed=True) if packed else w16
    g = torch.Generator(device="cuda").manual_seed(0x0B7B0909)
    kv = torch.randn(cfg.layers, 2, cfg.kv_heads, CAP, cfg.head_dim, generator=g, device="cuda").to(torch.bfloat16)
    okv = kv.float().cpu().numpy()
    trace: list = []
    od.step(cfg, W, TOKEN, okv, N0, trace=trace)
    assert len(trace) == cfg.layers + 1
    del W

    step = DecodeStep(card, cfg, w, CAP)          # its buffers, rope tables and attention scratch; the body is not run
    step.kv.copy_(kv)
    step.reset(N0, TOKEN)
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).cuda()
    worst_h = worst_y = 0.0
    for i in range(cfg.layers):
        L = f"layers.{i}."
        h_in, y_in = trace[i]
        h_want, y_want = trace[i + 1]
        h0 = bf(h_in)
        hb, ha = torch.zeros_like(h0), torch.zeros_like(h0)
        card.gemv_norm(w[L + "qkv"].w, h0, None if y_in is None else bf(y_in), w[L + "ln1"], cfg.eps, hb, step.qkv)
        card.attn_decode_qkv(step.qkv, w.get(L + "wq"), w.get(L + "wk"), cfg.eps, step.cos, step.sin, step.n0,
                             step.kv[i, 0], step.kv[i, 1], step.att, Hq, Hk, D, step.scale, step.S, step.scratch)
        w[L + "o"].matvec(step.att, step.y)
        card.gemv_norm(w[L + "gu"].w, hb, step.y, w[L + "ln2"], cfg.eps, ha, step.m, glu=True)
        w[L + "down"].matvec(step.m, step.y)
        torch.cuda.synchronize()
        eh = _rel(ha.float().cpu().numpy(), h_want)[0]
        ey = _rel(step.y.float().cpu().numpy(), y_want)[0]
        worst_h, worst_y = max(worst_h, eh), max(worst_y, ey)
        assert eh <= 1e-2 and ey <= 1e-2, (i, eh, ey)
        # the layer's new key and value rows are the oracle's too
        krow = step.kv[i, :, :, N0].float().cpu().numpy()
        assert np.abs(krow - okv[i, :, :, N0]).max() <= 1e-2 * np.abs(okv[i, :, :, N0]).max(), i
    print(f"teacher-forced layers ({'pack12' if packed else 'bf16'}): worst residual {worst_h:.2e}, worst block output {worst_y:.2e}")
