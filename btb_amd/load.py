"""Checkpoints on disk to weights in VRAM, in the form they are stored in: the loaders behind the decode step.

A store is a directory of `*.safetensors` shards with `config.json` (and `model.safetensors.index.json` when sharded),
as the reference reads it (btb/engine/tiers.py:513-527, 595-626; btb/pack12.py:113-133; btb/fp8.py:29-62). Three
stored forms are taken as they are, none widened to bf16 in memory:

  bf16        `<name>.weight` bf16                                     -> a bf16 tensor on the GPU
  pack12      `<name>.weight.pack12` (u8 blob) + `.pack12.meta`        -> `P12Weight` (low bytes, codes, table, escapes;
              a 12-bit store holds only `layers.*` and names its       the per-row escape index is built on the GPU at
              parent under `config.json: btb.source`)                   load)
  fp8 e4m3    `<name>.weight` float8_e4m3fn + `<name>.weight_scale_inv` -> `F8Weight` (bytes + the f32 scale grid)
  mxfp4       `<name>_blocks` u8 [E, rows, K/32, 16] + `<name>_scales`  -> `MxExperts`: a layer's expert stacks as stored
              u8 [E, rows, K/32] (gpt-oss's routed experts,              (17 bytes per 32 weights), an expert's matrix an
              btb/mxfp4.py:4-29, 127-168)                               `MxWeight` view into them

The card's step multiplies q/k/v as one matrix and gate/up as one (btb/engine/cuda.py:1722-1834), so the loader
stacks them by rows: bf16 rows are concatenated; FP8 bytes and their scale grids are concatenated (every part holds a
whole number of scale blocks); 12-bit parts have a table each, so they are widened on the GPU, stacked and packed
again as one matrix - still 12 bits a weight in VRAM, the widened copy is dropped (`fuse=False` keeps each part as
stored and multiplies them one after another instead).
"""

from __future__ import annotations

import glob
import json
import os
from typing import Any

import torch
from safetensors import safe_open

from . import pack12
from .decode import Linear, StackConfig
from .fp8 import E4M3, F8Weight, scale_grid
from .mxfp4 import BLOCK, BLOCK_BYTES, MxWeight
from .pack12 import P12Weight


def read_config(path: str) -> tuple[StackConfig, dict[str, Any]]:
    """the stack's shape from a store's config.json (Qwen3-style dense decoder), and the raw config"""
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    rope = raw.get("rope_parameters") or {}
    heads = int(raw["num_attention_heads"])
    cfg = StackConfig(
        layers=int(raw["num_hidden_layers"]),
        hidden=int(raw["hidden_size"]),
        q_heads=heads,
        kv_heads=int(raw.get("num_key_value_heads", heads)),
        head_dim=int(raw.get("head_dim") or int(raw["hidden_size"]) // heads),
        intermediate=int(raw["intermediate_size"]),
        vocab=int(raw["vocab_size"]),
        eps=float(raw.get("rms_norm_eps", 1e-6)),
        rope_theta=float(rope.get("rope_theta", raw.get("rope_theta", 1_000_000.0))),
    )
    return cfg, raw


class Store:
    """name -> tensor over a directory's shards, opened on demand (nothing is read until a tensor is asked for);
    a 12-bit store falls through to its parent for the tensors it does not hold"""

    def __init__(self, path: str) -> None:
        self.path = path
        self.where: dict[str, str] = {}
        index = os.path.join(path, "model.safetensors.index.json")
        if os.path.exists(index):
            with open(index) as f:
                self.where = {k: os.path.join(path, v) for k, v in json.load(f)["weight_map"].items()}
        else:
            for shard in sorted(glob.glob(os.path.join(path, "*.safetensors"))):
                with safe_open(shard, framework="pt") as f:
                    for k in f.keys():
                        self.where[k] = shard
        if not self.where:
            raise FileNotFoundError(f"[load] no safetensors tensors under {path}")
        self.parent: Store | None = None
        cfg_path = os.path.join(path, "config.json")
        if os.path.exists(cfg_path):
            with open(cfg_path) as f:
                src = (json.load(f).get("btb") or {}).get("source")
            if src:
                self.parent = Store(os.path.normpath(os.path.join(path, src)))

    def has(self, name: str) -> bool:
        return name in self.where or (self.parent is not None and self.parent.has(name))

    def get(self, name: str) -> torch.Tensor:
        if name in self.where:
            with safe_open(self.where[name], framework="pt") as f:
                return f.get_tensor(name)
        if self.parent is not None:
            return self.parent.get(name)
        raise KeyError(f"[load] {name} is in neither {self.path} nor its parent")


def _vector(store: Store, name: str, dev: Any) -> torch.Tensor | None:
    """a norm weight as bf16 on the GPU (a 12-bit store packs these too: unpacked here, they are a few hundred bytes)"""
    if store.has(name + ".pack12"):
        lo, hi4, table, ei, ev, shape = pack12.split(store.get(name + ".pack12"), store.get(name + ".pack12.meta"))
        n = 1
        for d in shape:
            n *= d
        return pack12.unpack_bf16(lo, hi4, table, n, shape, ei, ev).to(dev)
    if store.has(name):
        return store.get(name).to(torch.bfloat16).to(dev)
    return None


def _matrix(store: Store, card: Any, name: str, dev: Any) -> Any:
    """one stored matrix on the GPU in its stored form"""
    if store.has(name + ".pack12"):
        body = store.get(name + ".pack12").to(dev)
        lo, hi4, table, ei, ev, shape = pack12.split(body, store.get(name + ".pack12.meta"))
        if len(shape) != 2:
            raise ValueError(f"[load] {name}: a packed matrix has two dims, got {shape}")
        return P12Weight(lo, hi4, table, ei, ev, shape[0], shape[1], card)
    t = store.get(name)
    if t.dtype == E4M3:
        s = scale_grid(store.get(name + "_scale_inv"))
        return F8Weight(t.view(torch.uint8).to(dev), s.to(dev), int(t.shape[0]), int(t.shape[1]))
    return t.to(torch.bfloat16).to(dev).contiguous()


def _stack_rows(card: Any, parts: list[Any]) -> Any:
    """the parts as one matrix, rows stacked, in their common stored form"""
    if all(isinstance(p, torch.Tensor) for p in parts):
        return torch.cat(parts, dim=0).contiguous()
    if all(isinstance(p, F8Weight) for p in parts):
        cols = parts[0].shape[1]
        bm = {p.shape[0] // p.grid[0] for p in parts}
        sc = {p.grid[1] for p in parts}
        if len(bm) != 1 or len(sc) != 1 or any(p.shape[1] != cols for p in parts):
            raise ValueError("[load] FP8 parts with different scale blocks do not stack")
        rows = sum(p.shape[0] for p in parts)
        return F8Weight(torch.cat([p.w.reshape(p.shape) for p in parts], dim=0).reshape(-1),
                        torch.cat([p.scales for p in parts], dim=0), rows, cols)
    if all(isinstance(p, P12Weight) for p in parts):
        wide = [card.p12_widen(p.lo, p.hi4, p.table, p.esc_idx, p.esc_val, p.shape[0] * p.shape[1], p.shape)
                for p in parts]
        return P12Weight.pack(torch.cat(wide, dim=0).contiguous(), card)
    raise ValueError("[load] the parts of a stacked matrix are stored in different forms")


class Parts:
    """several stored matrices that share their input and write consecutive slices of one output: what q/k/v (or gate
    and up) are when a 12-bit store's parts are kept exactly as stored"""

    def __init__(self, card: Any, parts: list[Any]) -> None:
        self.card, self.parts = card, [Linear(card, p) for p in parts]
        self.shape = (sum(p.shape[0] for p in self.parts), self.parts[0].shape[1])

    @property
    def nbytes(self) -> int:
        return sum(p.nbytes for p in self.parts)

    def matvec(self, x: torch.Tensor, y: torch.Tensor) -> None:
        if x.shape[0] != 1:
            raise ValueError("[load] kept-as-stored parts multiply one row at a time")
        r0 = 0
        for p in self.parts:
            p.matvec(x, y[:, r0 : r0 + p.shape[0]])
            r0 += p.shape[0]


def load_stack(card: Any, path: str, fuse: bool = True, device: Any = "cuda") -> tuple[StackConfig, dict[str, Any]]:
    """(config, weights) of a dense Qwen3-style store for `DecodeStep`: `layers.{i}.{qkv,o,gu,down}` and `head` as
    `Linear` (bf16 tensor, `P12Weight` or `F8Weight` inside), the norm vectors and `embed` as bf16 tensors"""
    cfg, raw = read_config(path)
    store = Store(path)
    dev = torch.device(device)
    w: dict[str, Any] = {}

    def lin(parts: list[Any]) -> Any:
        if len(parts) == 1:
            return Linear(card, parts[0])
        if fuse or not all(isinstance(p, P12Weight) for p in parts):
            return Linear(card, _stack_rows(card, parts))
        return Parts(card, parts)

    for i in range(cfg.layers):
        src, dst = f"model.layers.{i}.", f"layers.{i}."
        mat = lambda n: _matrix(store, card, src + n + ".weight", dev)
        w[dst + "qkv"] = lin([mat("self_attn.q_proj"), mat("self_attn.k_proj"), mat("self_attn.v_proj")])
        w[dst + "o"] = lin([mat("self_attn.o_proj")])
        w[dst + "gu"] = lin([mat("mlp.gate_proj"), mat("mlp.up_proj")])
        w[dst + "down"] = lin([mat("mlp.down_proj")])
        w[dst + "ln1"] = _vector(store, src + "input_layernorm.weight", dev)
        w[dst + "ln2"] = _vector(store, src + "post_attention_layernorm.weight", dev)
        for ours, theirs in (("wq", "self_attn.q_norm.weight"), ("wk", "self_attn.k_norm.weight")):
            v = _vector(store, src + theirs, dev)
            if v is not None:
                w[dst + ours] = v
    w["embed"] = store.get("model.embed_tokens.weight").to(torch.bfloat16).to(dev).contiguous()
    w["norm"] = _vector(store, "model.norm.weight", dev)
    tied = bool(raw.get("tie_word_embeddings", False)) or not store.has("lm_head.weight")
    w["head"] = Linear(card, w["embed"] if tied else _matrix(store, card, "lm_head.weight", dev))
    return cfg, w


class MxExperts:
    """One layer's routed experts as an MXFP4 checkpoint stores them, in VRAM unchanged: `gate_up_blocks` u8
    [E, 2I, H/32, 16] with `gate_up_scales` u8 [E, 2I, H/32], `down_blocks` u8 [E, H, I/32, 16] with `down_scales`
    (btb/mxfp4.py:4-29: 32 weights along K share 16 bytes and one e8m0 exponent; the slot order of an expert is
    gate_up blocks, gate_up scales, down blocks, down scales). gpt-oss interleaves its gate and up rows (gate at the
    even rows); the rows are kept as stored. `gate_up(e)` / `down(e)` are expert e's matrices as `MxWeight` views
    (no copy) for `HipCard.gemv_mx4`; `widen` is `HipCard.mx4_widen` over a whole stack or the experts at `seats`."""

    __slots__ = ("down_bias", "down_blocks", "down_scales", "experts", "gate_up_bias", "gate_up_blocks", "gate_up_scales",
                 "hidden", "intermediate")

    def __init__(self, gate_up_blocks: torch.Tensor, gate_up_scales: torch.Tensor, down_blocks: torch.Tensor,
                 down_scales: torch.Tensor, gate_up_bias: torch.Tensor | None = None,
                 down_bias: torch.Tensor | None = None) -> None:
        for b, sc, what in ((gate_up_blocks, gate_up_scales, "gate_up"), (down_blocks, down_scales, "down")):
            if b.dtype != torch.uint8 or sc.dtype != torch.uint8 or b.dim() != 4 or b.shape[-1] != BLOCK_BYTES \
                    or tuple(b.shape[:-1]) != tuple(sc.shape):
                raise ValueError(f"[load] {what}: MXFP4 stacks are uint8 blocks [E, rows, K/32, {BLOCK_BYTES}] with "
                                 f"scales [E, rows, K/32], got {tuple(b.shape)} {b.dtype} and {tuple(sc.shape)} {sc.dtype}")
        E, rows_gu, g_h = (int(v) for v in gate_up_scales.shape)
        E2, rows_dn, g_i = (int(v) for v in down_scales.shape)
        H, I = g_h * BLOCK, g_i * BLOCK
        if E != E2 or rows_dn != H or rows_gu != 2 * I:
            raise ValueError(f"[load] gate_up [{E}, {rows_gu}, {H}] and down [{E2}, {rows_dn}, {I}] are not one layer's "
                             f"experts")
        self.gate_up_blocks, self.gate_up_scales = gate_up_blocks.contiguous(), gate_up_scales.contiguous()
        self.down_blocks, self.down_scales = down_blocks.contiguous(), down_scales.contiguous()
        self.experts, self.hidden, self.intermediate = E, H, I
        # gpt-oss's expert biases, bf16 as the checkpoint holds them: [E, 2I] (interleaved like the rows) and [E, H]
        for b, shape, what in ((gate_up_bias, (E, 2 * I), "gate_up_bias"), (down_bias, (E, H), "down_bias")):
            if b is not None and (tuple(b.shape) != shape or b.dtype != torch.bfloat16):
                raise ValueError(f"[load] {what} is bf16 {shape}, got {tuple(b.shape)} {b.dtype}")
        self.gate_up_bias = None if gate_up_bias is None else gate_up_bias.contiguous()
        self.down_bias = None if down_bias is None else down_bias.contiguous()

    def gate_up(self, e: int) -> MxWeight:
        return MxWeight(self.gate_up_blocks[e].reshape(-1), self.gate_up_scales[e].reshape(-1), 2 * self.intermediate,
                        self.hidden)

    def down(self, e: int) -> MxWeight:
        return MxWeight(self.down_blocks[e].reshape(-1), self.down_scales[e].reshape(-1), self.hidden, self.intermediate)

    @property
    def nbytes(self) -> int:
        return sum(int(t.numel()) for t in (self.gate_up_blocks, self.gate_up_scales, self.down_blocks, self.down_scales))

    def widen(self, card: Any, which: str, seats: torch.Tensor | None = None,
              dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        """the `which` ("gate_up" or "down") matrices of every expert, or of those at `seats`, widened on the GPU:
        [n, rows, K] in `dtype`"""
        if which not in ("gate_up", "down"):
            raise ValueError("[load] which is 'gate_up' or 'down'")
        blocks = self.gate_up_blocks if which == "gate_up" else self.down_blocks
        scales = self.gate_up_scales if which == "gate_up" else self.down_scales
        flat = card.mx4_widen(blocks, scales, seats, dtype=dtype)
        return flat.reshape(flat.shape[0], int(scales.shape[1]), int(scales.shape[2]) * BLOCK)


def load_mx_experts(path: str | Store, layer: int, device: Any = "cuda",
                    prefix: str = "model.layers.{i}.mlp.experts.") -> MxExperts:
    """layer `layer`'s MXFP4 expert stacks of a store, uploaded as stored (`<prefix>{gate_up,down}_proj_{blocks,scales}`,
    and `<prefix>{gate_up,down}_proj_bias` where the store holds them)"""
    store = path if isinstance(path, Store) else Store(path)
    base = prefix.format(i=int(layer))
    names = [base + n for n in ("gate_up_proj_blocks", "gate_up_proj_scales", "down_proj_blocks", "down_proj_scales")]
    missing = [n for n in names if not store.has(n)]
    if missing:
        raise KeyError(f"[load] not an MXFP4 expert layer: {missing[0]} is not in {store.path}")
    dev = torch.device(device)
    biases = [store.get(base + n).to(torch.bfloat16).to(dev) if store.has(base + n) else None
              for n in ("gate_up_proj_bias", "down_proj_bias")]
    return MxExperts(*(store.get(n).to(dev) for n in names), *biases)
