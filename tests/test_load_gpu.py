"""Stores on disk -> VRAM -> the decode step, against the end-to-end receipts the reference banked for its tiny Qwen3
fixture (tests/fixtures/receipts_qwen3.pt, copied as data; written by tests/make_fixtures.py:1230-1264 with the
reference's f32 host engine, itself held within 1e-4 of transformers): the logits after the 16-token prompt, the prompt's
K / V rows per layer and the ten greedy tokens. The same model is loaded from its three stores - bf16 shards, the 12-bit
store (`layers.*` packed, the rest from its parent) and the FP8 e4m3 store (16 x 16 scale blocks) - each kept in its
stored form in VRAM.

Bars. The receipts are f32 activations; the card path rounds activations to bf16 at the reference card kernels'
rounding points, so logits are held to 3e-2 of the largest logit (the bar of the step's own parity test), the cache
rows to 2e-2 of the largest entry, and the greedy tokens must be the receipts' (their top-2 margin is far above the
bar). FP8 stores quantised weights: its logits are held to the FP8 store's own f32 evaluation, not to the receipts."""

from __future__ import annotations

import os

import numpy as np
import pytest
import torch

from btb_amd import fp8
from btb_amd.decode import DecodeStep
from btb_amd.fp8 import F8Weight
from btb_amd.load import Parts, Store, load_stack, read_config
from btb_amd.pack12 import P12Weight

from .helpers import GOLDEN, reference_logits

pytestmark = pytest.mark.gpu

PROMPT = [3, 17, 42, 5, 99, 120, 7, 7, 200, 12, 45, 8, 3, 17, 60, 61]  # tests/helpers.py:256 of the reference
CAP = 64


@pytest.fixture(scope="module")
def receipts():
    return torch.load(os.path.join(GOLDEN, "receipts_qwen3.pt"), weights_only=True)


def run_prompt(card, cfg, w, greedy: int = 10, **kw):
    step = DecodeStep(card, cfg, w, CAP, **kw)
    step.reset(0, PROMPT[0])
    for tok in PROMPT:
        step.ids.fill_(tok)
        step.body()
    torch.cuda.synchronize()
    logits = step.logits[0].float().cpu().numpy().copy()
    kv = step.kv[:, :, :, : len(PROMPT)].float().cpu().numpy().copy()
    toks = [step.token()]
    for _ in range(greedy - 1):
        step.body()
        torch.cuda.synchronize()
        toks.append(step.token())
    assert int(step.n0[0]) == len(PROMPT) + greedy - 1
    return logits, kv, toks


def check_receipt(got, want, bar):
    want = want.float().numpy() if isinstance(want, torch.Tensor) else want
    worst = np.abs(got - want).max() / np.abs(want).max()
    assert worst <= bar, worst


@pytest.mark.parametrize("store,kind,kw", [("tiny_qwen3", "bf16", {}), ("tiny_qwen3", "bf16", {"fused": False}),
                                           ("tiny_qwen3-pack12", "p12", {}),
                                           ("tiny_qwen3-pack12", "p12", {"fuse": False})])
def test_loaded_store_reproduces_the_receipts(card, receipts, store, kind, kw):
    fuse = kw.pop("fuse", True)
    cfg, w = load_stack(card, os.path.join(GOLDEN, store), fuse=fuse)
    assert (cfg.layers, cfg.hidden, cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.vocab) == (4, 64, 4, 2, 128, 256)
    qkv = w["layers.0.qkv"]
    if kind == "p12":
        assert isinstance(qkv, Parts) if not fuse else isinstance(qkv.w, P12Weight)
        assert isinstance(w["layers.3.down"].w, P12Weight) and w["head"].w.dtype == torch.bfloat16
    logits, kv, toks = run_prompt(card, cfg, w, **kw)
    r = receipts[kind]
    check_receipt(logits, r["prompt_logits"], 3e-2)
    assert toks == r["greedy"] == receipts["ref"]["greedy"]
    for i in range(cfg.layers):
        k_want, v_want = (t[0, :, : len(PROMPT)].float().numpy() for t in r["keys"][i])
        check_receipt(kv[i, 0], k_want, 2e-2)
        check_receipt(kv[i, 1], v_want, 2e-2)


def test_fp8_store_loads_as_stored_and_tracks_its_own_f32_evaluation(card, receipts):
    path = os.path.join(GOLDEN, "tiny_qwen3-f8_e4m3")
    cfg, w = load_stack(card, path)
    gu = w["layers.1.gu"].w
    assert isinstance(gu, F8Weight) and gu.shape == (2 * cfg.intermediate, cfg.hidden) and gu.grid == (16, 4)
    logits, _, toks = run_prompt(card, cfg, w)
    # the same store evaluated in f32 on the CPU: held weights bf16(e4m3 * scale), f32 activations, plain torch (the
    # forward pass tests/test_load.py pins against the receipts)
    store = Store(path)
    cfg2, _ = read_config(path)

    def held(name):
        t = store.get(name)
        if t.dtype == fp8.E4M3:
            return fp8.held(t, store.get(name + "_scale_inv")).float()
        return t.float()

    want = reference_logits(cfg2, held, PROMPT)
    check_receipt(logits, want, 3e-2)
    assert toks[0] == int(np.argmax(want))
    # quantisation moves the logits a little off the receipts, not far
    check_receipt(logits, receipts["bf16"]["prompt_logits"], 0.25)


def test_mxfp4_expert_store_widens_bit_exact_on_the_gpu(card):
    """every layer of the reference's tiny gpt-oss store: its MXFP4 expert stacks go to VRAM as stored and
    btb_hip_mx4_widen makes of them, bit for bit, what transformers' convert_moe_packed_tensors does (a library already
    here, not the reference), whole stacks and picked seats; an expert's matvec over the stored bytes equals the
    matvec over the widened matrix within the bf16-output bar"""
    from btb_amd.load import load_mx_experts

    tm = pytest.importorskip("transformers.integrations.mxfp4")
    path = os.path.join(GOLDEN, "tiny_gpt_oss")
    for layer in range(4):
        ex = load_mx_experts(path, layer)
        for which, blocks, scales in (("gate_up", ex.gate_up_blocks, ex.gate_up_scales),
                                      ("down", ex.down_blocks, ex.down_scales)):
            want = tm.convert_moe_packed_tensors(blocks.cpu(), scales.cpu(), dtype=torch.bfloat16).transpose(1, 2)
            got = ex.widen(card, which)
            assert torch.equal(got.cpu().view(torch.int16), want.contiguous().view(torch.int16)), (layer, which)
            seats = torch.tensor([6, 1, 1, 4], dtype=torch.int32, device="cuda")
            picked = ex.widen(card, which, seats)
            assert torch.equal(picked.cpu().view(torch.int16), want[[6, 1, 1, 4]].contiguous().view(torch.int16))
        x = torch.randn(2, ex.hidden, generator=torch.Generator().manual_seed(layer)).to(torch.bfloat16).cuda()
        y = card.gemv_mx4(ex.gate_up(2), x).float().cpu().numpy()
        ref = (x.float().cpu() @ ex.widen(card, "gate_up", dtype=torch.float32)[2].cpu().T).numpy()
        assert np.abs(y - ref).max() <= 2.0**-7 * np.abs(ref).max()
