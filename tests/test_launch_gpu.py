"""The reference's launcher surface over this library: kernels launched by the reference's kernel names with the
reference's own parameter lists (btb/engine/card_launch.py:428-440; the `extern "C"` signatures of
native/cuda/btb_kernels.cu and btb_gemv_mma.cuh) give the results of the typed wrappers, bit for bit."""

from __future__ import annotations

import ctypes

import pytest
import torch

from btb_amd import mxfp4

from .helpers import acts_bf16, gen, weights_bf16

pytestmark = pytest.mark.gpu

P, I, F, LL = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong


def p(t):
    return P(t.data_ptr()) if t is not None else P(None)


def test_matvec_kernels_by_name(card):
    R, C = 2560, 4096
    w = weights_bf16(R, C, seed=800).cuda()
    for M in (1, 4, 16):
        x = acts_bf16(M, C, seed=801).cuda()
        want = card.gemv(w, x)
        y = torch.zeros(M, R, dtype=torch.bfloat16, device="cuda")
        card.launch(f"btb_gemv_bf16_m{M}", ((R + 3) // 4, 1, 1), (128, 1, 1), [p(w), p(x), p(y), I(R), I(C)])
        assert torch.equal(y.view(torch.int16), want.view(torch.int16))
        y.zero_()
        card.launch("btb_gemv_mma_bf16", (64, 1, 1), (256, 1, 1), [p(w), p(x), p(y), I(R), I(C), I(M)], shared=4096)
        assert torch.equal(y.view(torch.int16), want.view(torch.int16))
        f = torch.zeros(M, R, dtype=torch.float32, device="cuda")
        card.launch(f"btb_gemv_lane16_f32_m{M}", (R // 4, 1, 1), (128, 1, 1), [p(w), p(x.float()), p(f), I(R), I(C)])
        assert torch.equal(f.view(torch.int32), card.gemv_lane16(w, x.float()).view(torch.int32))
    Iw = 1024
    wg = weights_bf16(2 * Iw, C, seed=802).cuda()
    x = acts_bf16(2, C, seed=803).cuda()
    m = torch.zeros(2, Iw, dtype=torch.bfloat16, device="cuda")
    card.launch("btb_gemv_mma_glu_silu", (32, 1, 1), (256, 1, 1), [p(wg), p(x), p(m), I(Iw), I(C), I(2)])
    assert torch.equal(m.view(torch.int16), card.gemv_glu_silu(wg, x).view(torch.int16))
    gu = card.gemv(wg, x)
    m2 = torch.zeros_like(m)
    card.launch("btb_silu_mul", (8, 1, 1), (256, 1, 1), [p(gu), p(m2), I(2), I(Iw)])
    assert torch.equal(m2.view(torch.int16), m.view(torch.int16))
    wd = weights_bf16(512, Iw, seed=804).cuda()
    yd = torch.zeros(2, 512, dtype=torch.bfloat16, device="cuda")
    card.launch("btb_gemv_silu_bf16_m2", (128, 1, 1), (128, 1, 1), [p(wd), p(gu), p(yd), I(512), I(Iw)])
    assert torch.equal(yd.view(torch.int16), card.gemv_silu(wd, gu).view(torch.int16))


def test_glue_and_routing_kernels_by_name(card):
    T, H = 3, 2560
    h = acts_bf16(T, H, seed=810).cuda()
    y = acts_bf16(T, H, seed=811).cuda()
    w = (1.0 + 0.1 * torch.randn(H, generator=gen(812))).to(torch.bfloat16).cuda()
    h1, x1 = h.clone(), torch.zeros_like(h)
    card.add_rmsnorm(h1, y, w, 1e-6, x1)
    h2, x2 = h.clone(), torch.zeros_like(h)
    card.launch("btb_add_rmsnorm", (T, 1, 1), (256, 1, 1), [p(h2), p(y), p(w), F(1e-6), p(x2), I(H), I(0)])
    assert torch.equal(h1, h2) and torch.equal(x1, x2)

    logits = torch.randn(5, 128, generator=gen(813)).to(torch.bfloat16).cuda()
    idx, wt, _ = card.moe_route(logits, 8)
    idx2 = torch.zeros_like(idx)
    wt2 = torch.zeros_like(wt)
    card.launch("btb_moe_route", (5, 1, 1), (128, 1, 1),
                [p(logits), I(128), I(128), I(8), p(idx2), p(wt2), P(None), P(None), P(None), P(None), P(None)], shared=512)
    assert torch.equal(idx, idx2) and torch.equal(wt.view(torch.int16), wt2.view(torch.int16))

    src = weights_bf16(64, 256, seed=814).float()
    blocks, scales = mxfp4.quantize(src)
    b, s = blocks.reshape(-1).cuda(), scales.reshape(-1).cuda()
    groups = 64 * 256 // 32 // 4                      # four seats of a quarter of the blocks each
    seats = torch.tensor([2, 0, 3], dtype=torch.int32, device="cuda")
    out = torch.zeros(3, groups * 32, dtype=torch.bfloat16, device="cuda")
    card.launch("btb_mx4_widen", ((groups + 255) // 256, 3, 1), (256, 1, 1), [p(b), p(s), p(seats), LL(groups), p(out)])
    wide = mxfp4.dequantize(blocks, scales).reshape(4, groups * 32).to(torch.bfloat16)
    assert torch.equal(out.cpu().view(torch.int16), wide[[2, 0, 3]].view(torch.int16))


def test_launcher_refusals(card):
    with pytest.raises(KeyError):
        card.launch("btb_gemm_mma_bf16", (1, 1, 1), (1, 1, 1), [])
    with pytest.raises(ValueError):
        card.launch("btb_gemv_bf16_m1", (1, 1, 1), (128, 1, 1), [P(None)] * 4)
    with pytest.raises(RuntimeError):      # the library's own refusal: a null weight pointer, nothing launched
        card.launch("btb_gemv_bf16_m1", (1, 1, 1), (128, 1, 1), [P(None), P(None), P(None), I(8), I(8)])
    assert "btb_gemv_bf16_m32" in card.fn and "btb_moe_route" in card.fn
    card.close()
    card.close()


def test_attention_rope_and_publish_kernels_by_name(card):
    """btb_norm_rope_kv_tbl_d128, btb_attn_flash_d128 and btb_publish with the reference's own parameter lists
    (btb/engine/card_launch.py:469-523, 2152-2212, 2334-2347): the typed wrappers' bits. The attention's partial-state
    arrays are the caller's, at the reference's sizes, and hold the key groups' states; its arrival counter is not
    needed (a second launch folds the groups) and is left at zero."""
    import numpy as np

    from btb_amd.decode import StackConfig, rope_tables

    D, Hq, Hk, T, n0 = 128, 16, 4, 4, 700
    G = Hq // Hk
    S = 2                                              # key groups of 512: the graph's capacity is 1024 slots
    cap = S * 512
    cfg = StackConfig(layers=1, hidden=64, q_heads=Hq, kv_heads=Hk, head_dim=D, intermediate=64, vocab=8)
    g = gen(820)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(torch.bfloat16).cuda()
    wq = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    wk = (1.0 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).cuda()
    cos, sin = rope_tables(cfg, cap, "cuda")
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    par = torch.tensor([-1, 0, 1, 0], dtype=torch.int32, device="cuda")
    depth = torch.tensor([0, 1, 2, 1], dtype=torch.int32, device="cuda")
    tbl = torch.randperm(cap, generator=g).to(torch.int32).cuda()
    scale = 1.0 / np.sqrt(D)
    hs, rs = int(K.stride(0)), int(K.stride(1))

    K1, V1, K2, V2 = K.clone(), V.clone(), K.clone(), V.clone()
    q1 = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    q2 = torch.zeros_like(q1)
    card.norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, n0t, K1, V1, q1, Hq, Hk, D, depth=depth, tbl=tbl)
    card.launch("btb_norm_rope_kv_tbl_d128", (Hq + 2 * Hk, T, 1), (32, 1, 1),
                [p(qkv), p(wq), p(wk), F(1e-6), p(cos), p(sin), p(n0t), p(depth), p(K2), p(V2), p(q2), I(T), I(Hq), I(Hk),
                 I(hs), I(rs), I(0), p(tbl)])
    assert torch.equal(q1, q2) and torch.equal(K1, K2) and torch.equal(V1, V2)

    a1 = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    a2 = torch.zeros_like(a1)
    card.attn_decode(q1, K1, V1, a1, n0t, Hq, Hk, D, scale, S, card.attn_scratch(T, Hq, Hk, D, S), par=par, win=300, tbl=tbl)
    part_m = torch.zeros(S * T * Hq, dtype=torch.float32, device="cuda")
    part_l = torch.zeros(S * T * Hq, dtype=torch.float32, device="cuda")
    part_acc = torch.zeros(S * T * Hq * D, dtype=torch.float32, device="cuda")
    cnt = torch.zeros(T * Hq, dtype=torch.int32, device="cuda")
    card.launch("btb_attn_flash_d128", ((T * G + 7) // 8, S, Hk), (256, 1, 1),
                [p(q1), p(K1), p(V1), p(a2), p(n0t), p(par), I(T), I(Hq), I(Hk), I(hs), I(rs), F(scale), p(part_m),
                 p(part_l), p(part_acc), p(cnt), I(300), p(tbl)], shared=8192)
    assert torch.equal(a1, a2) and bool(a1.float().abs().sum() > 0)
    assert int(cnt.abs().sum()) == 0 and bool(part_l.abs().sum() > 0)   # the states went into the caller's arrays

    ids = torch.tensor([4242], dtype=torch.int32, device="cuda")
    out_tok = torch.zeros(1, dtype=torch.int32).pin_memory()
    out_n0 = torch.zeros(1, dtype=torch.int32).pin_memory()
    out_ts = torch.zeros(1, dtype=torch.int64).pin_memory()
    card.launch("btb_publish", (1, 1, 1), (32, 1, 1), [p(n0t), p(ids), p(out_tok), p(out_n0), p(out_ts)])
    torch.cuda.synchronize()
    assert int(out_tok[0]) == 4242 and int(out_n0[0]) == n0 and int(out_ts[0]) > 0 and int(n0t[0]) == n0
    for name in ("btb_attn_flash_d128", "btb_publish", "btb_norm_rope_kv_tbl_d64"):
        assert name in card.fn
