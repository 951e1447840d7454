"""The attention entry point that allocates nothing (btb_hip_attn_decode_noalloc) against the one that takes a
workspace (btb_hip_attn_decode): the same kernels over the library's own static array, so the outputs are equal bit for
bit - on two calls in a row, the second smaller (the array keeps the first call's states), then a tree pass, the size
limit's refusal, and raw through ctypes with no torch allocation between the calls."""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from btb_amd import native

from .helpers import gen

pytestmark = pytest.mark.gpu

D = 128


def inputs(n0, T, Hq, Hk, seed):
    cap = n0 + T + 5
    g = gen(7700 + seed)
    K = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    V = torch.randn(Hk, cap, D, generator=g).to(torch.bfloat16).cuda()
    q = torch.randn(T, Hq * D, generator=g).to(torch.bfloat16).cuda()
    n0t = torch.tensor([n0], dtype=torch.int32, device="cuda")
    return q, K, V, n0t


def both(card, n0, T, Hq, Hk, S, seed, par=None):
    q, K, V, n0t = inputs(n0, T, Hq, Hk, seed)
    scale = 1.0 / np.sqrt(D)
    want = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device="cuda")
    got = torch.full_like(want, 7.0)
    card.attn_decode(q, K, V, want, n0t, Hq, Hk, D, scale, S, card.attn_scratch(T, Hq, Hk, D, S), par=par)
    card.attn_decode_noalloc(q, K, V, got, n0t, Hq, Hk, D, scale, S, par=par)
    torch.cuda.synchronize()
    return got, want


def test_two_calls_in_a_row_the_second_smaller(card):
    # the first call fills most of the array (8 rows x 32 heads x 31 spans x 130 floats = 1 031 680 of 1 048 576)
    got, want = both(card, 3000, 8, 32, 8, 31, seed=0)
    assert torch.equal(got, want) and bool(want.float().abs().sum() > 0)
    # the second, smaller one finds the first call's states still there and must not read any of them
    got, want = both(card, 100, 1, 32, 8, 4, seed=1)
    assert torch.equal(got, want)
    got, want = both(card, 0, 1, 8, 8, 1, seed=2)
    assert torch.equal(got, want)
    # and a larger one again
    got, want = both(card, 4096, 1, 32, 8, 32, seed=3)
    assert torch.equal(got, want)


def test_tree_pass(card):
    T = 8
    par = torch.tensor([-1, 0, 1, 2, 1, 4, 0, 6], dtype=torch.int32, device="cuda")
    got, want = both(card, 300, T, 32, 8, 5, seed=4, par=par)
    assert torch.equal(got, want)


def test_sizes_beyond_the_array_are_refused_and_write_nothing(card):
    q, K, V, n0t = inputs(64, 8, 32, 8, seed=5)
    att = torch.full((8, 32 * D), 3.0, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(native.HipError) as e:
        card.attn_decode_noalloc(q, K, V, att, n0t, 32, 8, D, 0.1, 32)      # 8 * 32 * 32 * 130 floats > 2^20
    assert "ERR_DOMAIN" in str(e.value) or "-6" in str(e.value)
    torch.cuda.synchronize()
    assert bool((att == 3.0).all())


def test_raw_c_abi_with_no_allocation_between_the_calls(card):
    """through ctypes, every buffer made beforehand: the two calls themselves allocate nothing (torch's allocator
    counters do not move, and the library has no hipMalloc on this path)"""
    lib = card.lib
    q, K, V, n0t = inputs(500, 2, 16, 2, seed=6)
    q2, K2, V2, n02 = inputs(40, 1, 16, 2, seed=7)
    Hq, Hk, S = 16, 2, 7
    scale = 1.0 / np.sqrt(D)
    outs = [torch.zeros(2, Hq * D, dtype=torch.bfloat16, device="cuda"), torch.zeros(1, Hq * D, dtype=torch.bfloat16, device="cuda")]
    refs = [torch.zeros_like(o) for o in outs]
    work = [card.attn_scratch(2, Hq, Hk, D, S), card.attn_scratch(1, Hq, Hk, D, S)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    for (qq, KK, VV, nn, T), out in zip(((q, K, V, n0t, 2), (q2, K2, V2, n02, 1)), outs):
        rc = lib.btb_hip_attn_decode_noalloc(p(qq), p(KK), p(VV), p(out), p(nn), None, T, Hq, Hk, D,
                                             int(KK.stride(0)), int(KK.stride(1)), ctypes.c_float(scale),
                                             int(KK.shape[1]), S, stream)
        assert rc == native.OK, lib.btb_hip_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    for (qq, KK, VV, nn, T), ref, w in zip(((q, K, V, n0t, 2), (q2, K2, V2, n02, 1)), refs, work):
        rc = lib.btb_hip_attn_decode(p(qq), p(KK), p(VV), p(ref), p(nn), None, T, Hq, Hk, D, int(KK.stride(0)),
                                     int(KK.stride(1)), ctypes.c_float(scale), int(KK.shape[1]), S, p(w), stream)
        assert rc == native.OK
    torch.cuda.synchronize()
    assert torch.equal(outs[0], refs[0]) and torch.equal(outs[1], refs[1])
    assert lib.btb_hip_attn_decode_noalloc(None, p(K), p(V), p(outs[0]), p(n0t), None, 2, Hq, Hk, D, 1, 1,
                                           ctypes.c_float(scale), 10, S, stream) == native.ERR_NULL
