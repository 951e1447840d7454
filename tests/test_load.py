"""The store readers on the CPU: config parsing, shard lookup, the 12-bit store's fall-through to its parent - and the
pin of the f32 forward pass (tests/helpers.py: reference_logits) the GPU loader test measures the FP8 store with: on
the bf16 store it must give the logits the reference banked in receipts_qwen3.pt."""

from __future__ import annotations

import os

import numpy as np
import pytest
import torch

from btb_amd.load import Store, read_config

from .helpers import GOLDEN, reference_logits

PROMPT = [3, 17, 42, 5, 99, 120, 7, 7, 200, 12, 45, 8, 3, 17, 60, 61]  # tests/helpers.py:256 of the reference


def test_config_and_store_lookup():
    cfg, raw = read_config(os.path.join(GOLDEN, "tiny_qwen3"))
    assert (cfg.layers, cfg.hidden, cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.intermediate, cfg.vocab) == \
        (4, 64, 4, 2, 128, 128, 256)
    assert cfg.eps == 1e-6 and cfg.rope_theta == 1_000_000.0 and raw["tie_word_embeddings"] is True
    store = Store(os.path.join(GOLDEN, "tiny_qwen3"))
    assert store.has("model.layers.3.mlp.down_proj.weight") and not store.has("lm_head.weight")
    assert tuple(store.get("model.embed_tokens.weight").shape) == (256, 64)


def test_packed_store_falls_through_to_its_parent():
    store = Store(os.path.join(GOLDEN, "tiny_qwen3-pack12"))
    assert store.parent is not None and store.parent.path.endswith("tiny_qwen3")
    assert store.has("model.layers.0.self_attn.q_proj.weight.pack12")
    assert store.has("model.embed_tokens.weight")  # held by the parent only
    assert store.get("model.embed_tokens.weight").dtype == torch.bfloat16
    meta = store.get("model.layers.0.self_attn.q_proj.weight.pack12.meta")
    assert meta.dtype == torch.uint8 and meta.numel() >= 24 + 16


def test_fp8_store_holds_bytes_and_inverse_scales():
    store = Store(os.path.join(GOLDEN, "tiny_qwen3-f8_e4m3"))
    w = store.get("model.layers.2.mlp.gate_proj.weight")
    s = store.get("model.layers.2.mlp.gate_proj.weight_scale_inv")
    assert w.dtype == torch.float8_e4m3fn and tuple(w.shape) == (128, 64) and tuple(s.shape) == (8, 4)
    assert store.get("model.embed_tokens.weight").dtype == torch.bfloat16  # not converted


def test_the_f32_forward_reproduces_the_bf16_receipts():
    path = os.path.join(GOLDEN, "tiny_qwen3")
    store = Store(path)
    cfg, _ = read_config(path)
    want = torch.load(os.path.join(GOLDEN, "receipts_qwen3.pt"), weights_only=True)["bf16"]["prompt_logits"].numpy()
    got = reference_logits(cfg, lambda n: store.get(n).float(), PROMPT)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max() + 1e-4


def test_mxfp4_expert_store_reads_as_stored():
    """the reference's tiny gpt-oss fixture (its MXFP4 expert tensors, copied as data): shapes, views, refusals"""
    from btb_amd.load import MxExperts, load_mx_experts

    path = os.path.join(GOLDEN, "tiny_gpt_oss")
    ex = load_mx_experts(path, 1, device="cpu")
    assert (ex.experts, ex.hidden, ex.intermediate) == (8, 64, 64)
    assert tuple(ex.gate_up_blocks.shape) == (8, 128, 2, 16) and tuple(ex.down_scales.shape) == (8, 64, 2)
    w = ex.gate_up(3)
    assert w.shape == (128, 64) and w.blocks.data_ptr() == ex.gate_up_blocks[3].data_ptr()      # a view, not a copy
    assert ex.down(7).shape == (64, 64) and ex.nbytes == 8 * (128 + 64) * 2 * 17
    # the views dequantise to what transformers makes of the same bytes
    tm = pytest.importorskip("transformers.integrations.mxfp4")
    want = tm.convert_moe_packed_tensors(ex.down_blocks, ex.down_scales, dtype=torch.float32).transpose(1, 2)
    assert torch.equal(ex.down(5).dequantize().view(torch.int32), want[5].contiguous().view(torch.int32))
    with pytest.raises(KeyError):
        load_mx_experts(path, 9, device="cpu")
    with pytest.raises(ValueError):
        MxExperts(ex.gate_up_blocks, ex.gate_up_scales, ex.gate_up_blocks, ex.gate_up_scales)
