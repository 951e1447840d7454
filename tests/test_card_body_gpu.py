"""The reference's card pass run ONLY through `launch(name, grid, block, args)`: `card_body` below restates the kernel
sequence of `_card_body` (btb/engine/cuda.py:1601-1837) for a dense Qwen3 stack - the same typed launchers
(`k.btb_add_rmsnorm(grid, block, ...)`, `k.btb_gemv_bf16(M, grid, block, ...)`, ...), the same argument lists, grids and
blocks, `k.ptr(Role, tensor)` for every address, the buffers of `_card_buffers` (:1491-1562) and the attention states
of `_card_parts` (:1563-1583) - over `HipCard`, the object a maintainer hands the reference in place of `_Cuda`. Nothing
here calls a typed wrapper of this library (`card.gemv`, `card.attn_decode`, ...): every kernel goes by its reference
name through the launcher.

What it is held to is not this library but the reference's own end-to-end receipts for its tiny Qwen3 fixture
(tests/fixtures/receipts_qwen3.pt, copied as data; made by the reference's f32 host engine): the logits after the
16-token prompt, every layer's K / V rows, the ten greedy tokens, the logits of every row of the receipts' verify tree
and of the step after the accepted path. Bars: the card path rounds activations to bf16 where the reference's card
kernels do, so logits are held to 3e-2 of the largest logit, cache rows to 2e-2 of the largest entry (the bars of
tests/test_load_gpu.py; the CPU restatement of the same rounding points sits at the same distance from the receipts,
tests/test_oracle_decode.py) and the greedy tokens must be the receipts'.
"""

from __future__ import annotations

import functools
import os

import numpy as np
import pytest
import torch

from btb_amd import card_launch as cl
from btb_amd.decode import recording, rope_tables
from btb_amd.load import load_stack

from .helpers import GOLDEN

pytestmark = pytest.mark.gpu

PROMPT = [3, 17, 42, 5, 99, 120, 7, 7, 200, 12, 45, 8, 3, 17, 60, 61]  # tests/helpers.py:256 of the reference
CHUNK = [9, 33, 14, 71, 33, 5, 90, 2]                                  # :257-260, the receipts' verify tree
PARENTS = [-1, 0, 1, 2, 1, 4, 0, 6]
PATH = [0, 1, 4, 5]
CAP = 1024          # two key groups of 512: the second never holds a live key
MMA_WARPS = 4       # btb/engine/cuda.py: the tensor-core matvec's warps a block
CARD_ROWS = (1, 2, 4, 8, 16, 32)


def card_m(T: int) -> int:
    """the row count a pass of T rows is padded to (the reference's `_card_m`: the next of 1, 2, 4, 8, 16, 32)"""
    return next(m for m in CARD_ROWS if m >= T)


def buffers(cfg, T: int, mma: bool, tail: bool = True) -> dict:
    """`_card_buffers` + `_card_parts` for one graph of T rows: the matvec-facing buffers at the padded row count, the
    attention's per-group states at S = ceil(cap / 512) groups, the tree as a chain until a pass says otherwise"""
    H, Hq, Hk, D, I = cfg.hidden, cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.intermediate
    M = 32 if mma else card_m(T)
    S = (CAP + 511) // 512
    n = S * T * Hq
    z = lambda *shape, dt=torch.bfloat16: torch.zeros(*shape, dtype=dt, device="cuda")
    return {
        "T": T, "M": M, "S": S, "mma": mma, "tail": tail,
        "m": z(M, I), "h": z(M, H), "x": z(M, H), "y": z(M, H), "qkv": z(M, (Hq + 2 * Hk) * D), "q": z(M, Hq, D),
        "att": z(M, Hq * D), "gu": z(M, 2 * I), "logits": z(M, cfg.vocab),
        "part_m": z(n, dt=torch.float32), "part_l": z(n, dt=torch.float32), "part_acc": z(n * D, dt=torch.float32),
        "cnt": z(T * Hq, dt=torch.int32), "n0": z(1, dt=torch.int32),
        "depth": torch.arange(T, dtype=torch.int32, device="cuda"),
        "par": torch.arange(-1, T - 1, dtype=torch.int32, device="cuda"),
    }


def card_body(k, cfg, W, g, arena, tables, row_map=None, fused=False, rows=None):
    """one pass over `g`'s buffers: every layer and the tail, each kernel by its reference name. `rows`: the pass's
    rows are sequences of their own, laid out by that int32 array (the reference's `rows` mode, cuda.py:1736-1756)"""
    T, M, mma = g["T"], g["M"], g["mma"]
    H, Hq, Hk, D, I = cfg.hidden, cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.intermediate
    G, S = Hq // Hk, g["S"]
    paged = row_map is not None
    attn_grid, attn_block = ((T * G + 7) // 8, S, Hk), (8 * 32, 1, 1)
    n0p, depth, par = k.ptr(cl.PrefixLen, g["n0"]), k.ptr(cl.Depths, g["depth"]), k.ptr(cl.TreeParents, g["par"])
    part_m, part_l = k.ptr(cl.PartMax, g["part_m"]), k.ptr(cl.PartSum, g["part_l"])
    part_acc, cnt = k.ptr(cl.PartAcc, g["part_acc"]), k.ptr(cl.Arrivals, g["cnt"])
    q, att = k.ptr(cl.Query, g["q"]), k.ptr(cl.AttnOut, g["att"])
    tbl = k.ptr(cl.RowMap, row_map)
    layout = k.ptr(cl.RowsLayout, rows)
    t_rows, q_heads, kv_heads = cl.Rows(T), cl.QHeads(Hq), cl.KvHeads(Hk)
    cen = cl.NormCentered(0)
    h, x, hidden, row = k.ptr(cl.Residual, g["h"]), k.ptr(cl.Normed, g["x"]), cl.Hidden(H), (T, 1, 1)
    cos_t, sin_t = tables
    cos, sin = k.ptr(cl.RopeCos, cos_t), k.ptr(cl.RopeSin, sin_t)
    eps = cl.NormEps(cfg.eps)
    scale, win = cl.AttnScale(1.0 / np.sqrt(D)), cl.Window(0)

    def matvec(Wm, xin, yout, R, C):
        w, mi, mo = k.ptr(cl.Weight, Wm), k.ptr(cl.MatIn, xin), k.ptr(cl.MatOut, yout)
        if mma:  # the tensor-core form takes the pass's true row count
            grid, block = ((R + 16 * MMA_WARPS - 1) // (16 * MMA_WARPS), 1, 1), (32 * MMA_WARPS, 1, 1)
            k.btb_gemv_mma_bf16(grid, block, w, mi, mo, cl.OutDim(R), cl.InDim(C), t_rows)
        else:
            k.btb_gemv_bf16(M, ((R + 3) // 4, 1, 1), (128, 1, 1), w, mi, mo, cl.OutDim(R), cl.InDim(C))

    y_prev = None
    for i in range(cfg.layers):
        L = f"layers.{i}."
        kb, vb = arena[i, 0], arena[i, 1]                      # [Hk, cap, D] views of the position-major arena
        K, V = k.ptr(cl.KCache, kb), k.ptr(cl.VCache, vb)
        hs, rs = cl.CacheHeadStride(int(kb.stride(0))), cl.CacheRowStride(int(kb.stride(1)))
        k.btb_add_rmsnorm(row, (256, 1, 1), h, k.ptr(cl.BlockOut, y_prev), k.ptr(cl.NormWeight, W[L + "ln1"]), eps, x,
                          hidden, cen)
        matvec(W[L + "qkv"].w, g["x"], g["qkv"], (Hq + 2 * Hk) * D, H)
        qkv, wq, wk = k.ptr(cl.Qkv, g["qkv"]), k.ptr(cl.QNorm, W[L + "wq"]), k.ptr(cl.KNorm, W[L + "wk"])
        nrk_grid = (Hq + 2 * Hk, T, 1)
        if rows is not None:
            k.btb_norm_rope_kv_rows(D, nrk_grid, (32, 1, 1), qkv, wq, wk, eps, cos, sin, layout, K, V, q, t_rows,
                                    q_heads, kv_heads, hs, rs, cen)
        elif paged:
            k.btb_norm_rope_kv_tbl(D, nrk_grid, (32, 1, 1), qkv, wq, wk, eps, cos, sin, n0p, depth, K, V, q, t_rows,
                                   q_heads, kv_heads, hs, rs, cen, tbl)
        else:
            k.btb_norm_rope_kv(D, nrk_grid, (32, 1, 1), qkv, wq, wk, eps, cos, sin, n0p, depth, K, V, q, t_rows,
                               q_heads, kv_heads, hs, rs, cen)
        if rows is not None:
            k.btb_attn_flash_rows(D, (T * ((G + 7) // 8), S, Hk), attn_block, q, K, V, att, layout, t_rows, q_heads,
                                  kv_heads, hs, rs, scale, part_m, part_l, part_acc, cnt, win)
        else:
            k.btb_attn_flash(D, attn_grid, attn_block, q, K, V, att, n0p, par, t_rows, q_heads, kv_heads, hs, rs,
                             scale, part_m, part_l, part_acc, cnt, win, tbl)
        matvec(W[L + "o"].w, g["att"], g["y"], H, Hq * D)
        k.btb_add_rmsnorm(row, (256, 1, 1), h, k.ptr(cl.BlockOut, g["y"]), k.ptr(cl.NormWeight, W[L + "ln2"]), eps, x,
                          hidden, cen)
        glu = fused and mma
        if glu:  # gate, up and the activation in one kernel
            k.btb_gemv_mma_glu_silu(((I + 16 * MMA_WARPS - 1) // (16 * MMA_WARPS), 1, 1), (32 * MMA_WARPS, 1, 1),
                                    k.ptr(cl.Weight, W[L + "gu"].w), k.ptr(cl.MatIn, g["x"]), k.ptr(cl.MlpAct, g["m"]),
                                    cl.Intermediate(I), cl.InDim(H), cl.Rows(T))
        else:
            matvec(W[L + "gu"].w, g["x"], g["gu"], 2 * I, H)
        if mma:
            if not glu:
                k.btb_silu_mul((min(4096, (M * I + 255) // 256), 1, 1), (256, 1, 1), k.ptr(cl.GateUp, g["gu"]),
                               k.ptr(cl.MlpAct, g["m"]), cl.Rows(M), cl.Intermediate(I))
            matvec(W[L + "down"].w, g["m"], g["y"], H, I)
        else:  # the activation folded into the down projection's x load
            k.btb_gemv_silu_bf16(M, ((H + 3) // 4, 1, 1), (128, 1, 1), k.ptr(cl.Weight, W[L + "down"].w),
                                 k.ptr(cl.GateUp, g["gu"]), k.ptr(cl.MatOut, g["y"]), cl.OutDim(H), cl.InDim(I))
        y_prev = g["y"]
    k.btb_add_rmsnorm(row, (256, 1, 1), h, k.ptr(cl.BlockOut, y_prev), k.ptr(cl.NormWeight, W["norm"]), eps, x, hidden,
                      cen)
    matvec(W["head"].w, g["x"], g["logits"], cfg.vocab, H)


class Pass:
    """a pass graph as the reference keeps it: buffers made once, the body run eagerly as a warm-up, then captured; a
    pass = the inputs written into the static buffers, then a replay"""

    def __init__(self, k, cfg, W, arena, tables, T, mma, row_map=None, fused=False, capture=True, rows=None):
        self.k, self.cfg, self.W, self.g = k, cfg, W, buffers(cfg, T, mma)
        self.run = functools.partial(card_body, k, cfg, W, self.g, arena, tables, row_map, fused, rows)
        self.graph = None
        if capture:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self.g["h"][:T] = W["embed"][torch.zeros(T, dtype=torch.long, device="cuda")]
                self.run()                                      # the warm-up writes slot 0 .. T - 1: overwritten later
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with recording(self.graph):
                self.run()

    def __call__(self, tokens, n0, par=None):
        g, T = self.g, self.g["T"]
        ids = torch.tensor(tokens, dtype=torch.long, device="cuda")
        g["h"][:T] = self.W["embed"][ids]                        # the reference gathers the rows with torch too
        g["n0"].fill_(n0)
        if par is not None:
            depth = []
            for p in par:
                depth.append(0 if p < 0 else depth[p] + 1)
            g["par"].copy_(torch.tensor(par, dtype=torch.int32))
            g["depth"].copy_(torch.tensor(depth, dtype=torch.int32))
        if self.graph is not None:
            self.graph.replay()
        else:
            self.run()
        torch.cuda.synchronize()
        return g["logits"][:T].float().cpu().numpy()


@pytest.fixture(scope="module")
def receipts():
    return torch.load(os.path.join(GOLDEN, "receipts_qwen3.pt"), weights_only=True)


@pytest.fixture(scope="module")
def tiny(card):
    cfg, W = load_stack(card, os.path.join(GOLDEN, "tiny_qwen3"))
    assert all(isinstance(W[f"layers.{i}.{n}"].w, torch.Tensor) for i in range(cfg.layers) for n in ("qkv", "o", "gu", "down"))
    return cfg, W


def new_arena(cfg):
    """the card graph's arena: position-major [layer, K/V, rows, Hk, D], handed to the kernels as [Hk, cap, D] views
    (head stride D, row stride Hk D), as the reference lays it out (btb/engine/arena.py; cuda.py:1725-1726)"""
    A = torch.zeros(cfg.layers, 2, CAP, cfg.kv_heads, cfg.head_dim, dtype=torch.bfloat16, device="cuda")
    return A, A.permute(0, 1, 3, 2, 4)


def worst(got, want):
    want = want.float().numpy() if isinstance(want, torch.Tensor) else want
    return float(np.abs(got - want).max() / np.abs(want).max())


@pytest.mark.parametrize("capture", [True, False])
def test_the_step_by_kernel_names_reproduces_the_receipts(card, tiny, receipts, capture):
    cfg, W = tiny
    assert isinstance(card, cl.CardLaunch)
    A, arena = new_arena(cfg)
    tables = rope_tables(cfg, CAP, "cuda")
    step = Pass(card, cfg, W, arena, tables, T=1, mma=False, capture=capture)
    A.zero_()
    r = receipts["bf16"]
    for n0, tok in enumerate(PROMPT):
        logits = step([tok], n0)
    assert worst(logits[0], r["prompt_logits"]) <= 3e-2
    n = len(PROMPT)
    for i in range(cfg.layers):
        k_want, v_want = (t[0, :, :n] for t in r["keys"][i])
        assert worst(arena[i, 0, :, :n].float().cpu().numpy(), k_want) <= 2e-2, i
        assert worst(arena[i, 1, :, :n].float().cpu().numpy(), v_want) <= 2e-2, i
    toks = [int(np.argmax(logits[0]))]
    out_tok = torch.zeros(1, dtype=torch.int32).pin_memory()
    out_n0 = torch.zeros(1, dtype=torch.int32).pin_memory()
    out_ts = torch.zeros(1, dtype=torch.int64).pin_memory()
    ids = torch.zeros(1, dtype=torch.int32, device="cuda")
    for j in range(9):
        logits = step([toks[-1]], n + j)
        toks.append(int(np.argmax(logits[0])))
        ids.fill_(toks[-1])
        card.btb_publish((1, 1, 1), (32, 1, 1), card.ptr(cl.PrefixLen, step.g["n0"]), card.ptr(cl.StepToken, ids),
                         card.ptr(cl.HostToken, out_tok), card.ptr(cl.HostLen, out_n0), card.ptr(cl.HostClock, out_ts))
        torch.cuda.synchronize()
        assert (int(out_tok[0]), int(out_n0[0])) == (toks[-1], n + j) and int(out_ts[0]) > 0
    assert toks == r["greedy"] == receipts["ref"]["greedy"]


@pytest.mark.parametrize("fused,paged", [(False, False), (True, False), (False, True)])
def test_the_verify_pass_by_kernel_names_reproduces_the_receipts(card, tiny, receipts, fused, paged):
    """the receipts' verify tree as one pass of 8 rows on the tensor-core matvec names (32-row buffers, the pass's
    true row count an argument), with and without the fused gate/up kernel, and through the cache's row map"""
    cfg, W = tiny
    A, arena = new_arena(cfg)
    tables = rope_tables(cfg, CAP, "cuda")
    row_map = None
    if paged:  # logical slot -> cache row: a fixed permutation of the arena's rows
        row_map = torch.randperm(CAP, generator=torch.Generator().manual_seed(5)).to(torch.int32).cuda()
    step = Pass(card, cfg, W, arena, tables, T=1, mma=False, row_map=row_map)
    tree = Pass(card, cfg, W, arena, tables, T=len(CHUNK), mma=True, row_map=row_map, fused=fused)
    A.zero_()
    for n0, tok in enumerate(PROMPT):
        step([tok], n0)
    r = receipts["bf16"]
    n = len(PROMPT)
    logits = tree(CHUNK, n, PARENTS)
    for t in range(len(CHUNK)):
        assert worst(logits[t], r["chunk_logits"][t]) <= 3e-2, t
    # the accepted path and its last token once more, as steps: `next`, and the 21 cached rows
    seq = [CHUNK[j] for j in PATH] + [CHUNK[PATH[-1]]]
    for d, tok in enumerate(seq):
        logits = step([tok], n + d)
    assert worst(logits[0], r["next"]) <= 3e-2
    rows = n + len(seq)
    at = (lambda t: t) if row_map is None else (lambda t: t[:, row_map.long()])
    for i in range(cfg.layers):
        assert worst(at(arena[i, 0])[:, :rows].float().cpu().numpy(), r["keys"][i][0][0]) <= 2e-2, i
        assert worst(at(arena[i, 1])[:, :rows].float().cpu().numpy(), r["keys"][i][1][0]) <= 2e-2, i


def test_a_pass_of_forked_rows_by_kernel_names(card, tiny, receipts):
    """the reference's rows mode: four forks of the prompt, a token each, stepped twice as one captured pass of four
    rows (`btb_norm_rope_kv_rows`, `btb_attn_flash_rows`; the layout array rewritten between the replays, as the
    reference rewrites it, cuda.py:3457-3464; a fifth, padding row behind them). Every fork's logits are the bits of
    that sequence stepped alone through the one-row graph over a cache of its own, and the fork that follows the
    receipts' greedy path picks the receipts' tokens"""
    cfg, W = tiny
    r = receipts["bf16"]
    tables = rope_tables(cfg, CAP, "cuda")
    n, B, T, base, Wd = len(PROMPT), 4, 5, 512, 4
    forks = [[r["greedy"][0], r["greedy"][1]], [9, 33], [r["greedy"][0], 71], [200, 200]]
    # each fork alone: the prompt, then its two tokens, through the one-row step
    alone = []
    A1, arena1 = new_arena(cfg)
    step = Pass(card, cfg, W, arena1, tables, T=1, mma=False)
    for toks in forks:
        A1.zero_()
        for n0, tok in enumerate(PROMPT):
            step([tok], n0)
        alone.append([step([tok], n + d)[0].copy() for d, tok in enumerate(toks)])
    # the forks as rows of one pass over one arena: the prompt's rows once, every fork's steps in stretches of Wd slots
    A, arena = new_arena(cfg)
    rw = torch.zeros(3 + 3 * T, dtype=torch.int32, device="cuda")
    rows = Pass(card, cfg, W, arena, tables, T=T, mma=False, rows=rw)
    A.zero_()
    A[:, :, :n] = A1[:, :, :n]                                   # the shared prefix (any fork's: the prompt's rows)
    for d in range(2):
        rw.copy_(card.rows_layout(base, d, Wd, [(c, 0, n) for c in range(B)], pad_to=T))
        logits = rows([f[d] for f in forks] + [0], 0)
        for t in range(B):
            assert np.array_equal(logits[t], alone[t][d]), (d, t)
        assert int(np.argmax(logits[0])) == r["greedy"][d + 1]
    # the forks' rows lie where the layout says, and nowhere else
    live = torch.zeros(CAP, dtype=torch.bool, device="cuda")
    live[:n] = True
    live[base : base + 2 * Wd] = True
    assert not bool(A[:, :, ~live].any()) and bool(A[:, :, base : base + 2 * Wd].any())


def test_card_launch_surface(card):
    """what `_card_body` asks of its `k`: `ptr(role, tensor)`, `fn` holding every kernel name it looks up, `sms`,
    `GEMV_ROWS`, and a typed launcher per kernel family of this path"""
    t = torch.zeros(4, device="cuda")
    assert card.ptr(cl.Weight, t) == t.data_ptr() and card.ptr(cl.RowMap, None) == 0
    assert set(card.fn) == set(cl.KERNELS)
    assert card.GEMV_ROWS == (1, 2, 4, 8, 16, 32) and card.sms > 0
    for fam in cl.SPEC:
        assert callable(getattr(card, fam))
    with pytest.raises(TypeError):
        card.btb_silu_mul((1, 1, 1), (256, 1, 1), 0, 0, 1)              # a parameter short
    with pytest.raises(ValueError):
        card.btb_gemv_bf16(3, (1, 1, 1), (128, 1, 1), 0, 0, 0, 8, 8)    # no kernel of 3 rows
