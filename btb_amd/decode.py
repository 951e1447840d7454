"""The dense decode step on the GPU as one hipGraph: the counterpart of the reference's card graph
(`_card_buffers` btb/engine/cuda.py:1491-1562, `_card_body` :1601-1837, `_capture` :988-999, `_card_step_graph` :2101)
for a Qwen3-shaped stack with every weight resident in VRAM, in bf16 or in the 12-bit packed form.

Per layer, as the reference sequences it: add_rmsnorm -> qkv matvec -> q/k norm + rope + cache write -> decode
attention -> o matvec -> add_rmsnorm -> gate_up matvec -> activation -> down matvec; then the final norm, the head
matvec, the greedy pick and the publish. The default (`fused`) form issues the same arithmetic in six launches a
layer instead of eight: every add_rmsnorm rides in the following matvec's x load and gate / up / activation are one
kernel; passes of four rows and more (a speculative verify) take the plain sequence, whose matvecs run on the matrix
cores. `DecodeStep.capture()` records the whole step with
torch's graph capture (a hipGraph on ROCm); afterwards the host only replays it and reads the token from pinned
memory.
"""

from __future__ import annotations

import contextlib
import gc
import math
from dataclasses import dataclass
from typing import Any

import torch

from .fp8 import F8Weight
from .mxfp4 import MxWeight
from .pack12 import P12Weight


@contextlib.contextmanager
def recording(graph: torch.cuda.CUDAGraph):
    """`torch.cuda.graph(graph)` with Python's cyclic collector held off while the stream records. A collection that
    runs in the middle of a recording can drop an older graph or device tensors that a dead reference cycle still
    held, and the runtime does not take a graph destroyed or device memory released while a stream records: the
    process aborts. So what is already dead is collected before the recording starts, and nothing is while it runs."""
    gc.collect()
    was_on = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            yield graph
    finally:
        if was_on:
            gc.enable()


@dataclass(frozen=True)
class StackConfig:
    """the shape of a dense decoder stack (Qwen3-4B: 36, 2560, 32, 8, 128, 9728, 151936)"""

    layers: int = 36
    hidden: int = 2560
    q_heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    intermediate: int = 9728
    vocab: int = 151936
    eps: float = 1e-6
    rope_theta: float = 1_000_000.0

    @property
    def qkv_rows(self) -> int:
        return (self.q_heads + 2 * self.kv_heads) * self.head_dim

    def weight_elements(self) -> int:
        """the linear weights' element count per step: 4 matrices a layer and the head"""
        per = (self.qkv_rows * self.hidden + self.hidden * self.q_heads * self.head_dim
               + 2 * self.intermediate * self.hidden + self.hidden * self.intermediate)
        return self.layers * per + self.vocab * self.hidden


QWEN3_4B = StackConfig()


def rope_tables(cfg: StackConfig, positions: int, device: Any) -> tuple[torch.Tensor, torch.Tensor]:
    """the model's rotary tables as the card kernels read them: cos / sin [positions, D] bf16 (the default rope:
    angles pos * theta^(-2i/D) over the first half of the dims, repeated over the second)"""
    half = cfg.head_dim // 2
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, half, dtype=torch.float32, device=device) * 2.0 / cfg.head_dim))
    ang = torch.arange(positions, dtype=torch.float32, device=device)[:, None] * inv[None, :]
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos().to(torch.bfloat16).contiguous(), emb.sin().to(torch.bfloat16).contiguous()


class Linear:
    """one linear's weight on the GPU in its stored form, multiplied as stored: a bf16 tensor or a `P12Weight`"""

    __slots__ = ("card", "w")

    def __init__(self, card: Any, w: Any) -> None:
        self.card = card
        self.w = w

    @property
    def shape(self) -> tuple[int, int]:
        return (int(self.w.shape[0]), int(self.w.shape[1]))

    @property
    def nbytes(self) -> int:
        return int(self.w.numel()) * 2 if isinstance(self.w, torch.Tensor) else int(self.w.nbytes)

    @property
    def fusable(self) -> bool:
        """whether the residual add + norm and the gate/up activation can ride in this matrix's matvec (bf16, pack12)"""
        return isinstance(self.w, (torch.Tensor, P12Weight))

    def matvec(self, x: torch.Tensor, y: torch.Tensor) -> None:
        if isinstance(self.w, P12Weight):
            self.card.gemv_p12(self.w, x, y)
        elif isinstance(self.w, F8Weight):
            self.card.gemv_fp8(self.w, x, y)
        elif isinstance(self.w, MxWeight):
            self.card.gemv_mx4(self.w, x, y)
        else:
            self.card.gemv(self.w, x, y)


class DecodeStep:
    """Buffers, caches and the kernel sequence of one decode step over `T` rows (1: the step; more: a chain of rows
    verified in one pass). `weights` maps `layers.{i}.{ln1,ln2,wq,wk}` (bf16 vectors), `layers.{i}.{qkv,o,gu,down}`
    (`Linear`), `embed` (bf16 [V, H]), `norm` and `head` (`Linear`)."""

    def __init__(self, card: Any, cfg: StackConfig, weights: dict[str, Any], cap: int, T: int = 1,
                 attn_spans: int | None = None, fold_silu: bool | None = None, fused: bool | None = None) -> None:
        dev = torch.device("cuda")
        self.card, self.cfg, self.w, self.cap, self.T = card, cfg, weights, int(cap), int(T)
        H, D, Hq, Hk, I = cfg.hidden, cfg.head_dim, cfg.q_heads, cfg.kv_heads, cfg.intermediate
        bf = dict(dtype=torch.bfloat16, device=dev)
        self.h = torch.zeros(T, H, **bf)
        self.h2 = torch.zeros(T, H, **bf)
        self.x = torch.zeros(T, H, **bf)
        self.y = torch.zeros(T, H, **bf)
        self.qkv = torch.zeros(T, cfg.qkv_rows, **bf)
        self.q = torch.zeros(T, Hq * D, **bf)
        self.att = torch.zeros(T, Hq * D, **bf)
        self.gu = torch.zeros(T, 2 * I, **bf)
        self.m = torch.zeros(T, I, **bf)
        self.logits = torch.zeros(T, cfg.vocab, **bf)
        self.ids = torch.zeros(T, dtype=torch.int32, device=dev)
        self.picked = torch.zeros(T, dtype=torch.int32, device=dev)
        self.n0 = torch.zeros(1, dtype=torch.int32, device=dev)
        # the caches: [layer, K/V, kv head, slot, dim], head-major so a key's row is one contiguous run
        self.kv = torch.zeros(cfg.layers, 2, Hk, self.cap, D, **bf)
        self.cos, self.sin = rope_tables(cfg, self.cap, dev)
        self.scale = 1.0 / math.sqrt(D)
        # key spans: enough workgroups (kv heads x spans) to cover the CUs once, a span at least 64 keys; a pass of T
        # rows launches T times the workgroups, so it takes longer spans - two workgroups a CU in all (measured on
        # the [2560 / 9728] stack at 4096 keys: 8 rows 4.32 ms a pass with 32 spans, 3.83 with 8; 16 rows 5.6 / 4.7)
        if attn_spans is None:
            attn_spans = max(1, min(self.cap // 64, (card.sms + Hk - 1) // Hk, (2 * card.sms) // (Hk * self.T)))
            if self.T == 1 and D == 128 and Hq // Hk >= 4:
                # the step's own attention kernel splits a kv head's query heads over workgroups of two heads, and a
                # workgroup folds its span 128 keys at a time: about a CU's worth of (kv head, head pair, span)
                # triples, each span a whole number of those batches (the library rounds a span up to one)
                per = max(128, self.cap // max(1, card.sms // (Hk * (Hq // Hk // 2))) // 128 * 128)
                attn_spans = max(1, -(-self.cap // per))
            elif 2 <= self.T <= 16 and D == 128 and Hq // Hk in (2, 4) and self.cap <= 128 * (1024 // (Hq // Hk)):
                # a pass of a few rows: spans of 128 keys, one batch of the attention's sixteen streams, which a
                # workgroup asks for at once and keeps in registers (measured at 4096 keys, ms a pass with this
                # against the best span count of the general kernel: 2 rows 2.95 / 3.12, 4 rows 3.51 / 3.68, 8 rows
                # 3.67 / 3.83, 16 rows 4.64 / 4.83)
                attn_spans = -(-self.cap // 128)
        self.S = int(attn_spans)
        self.scratch = card.attn_scratch(T, Hq, Hk, D, self.S, dev)
        # Which sequence: up to three rows the fused launches win (fewer launches, every matvec on the streaming
        # kernel); from four rows on the sequence with the residual add + norm as launches of their own does. From
        # five rows its matvecs take the matrix cores; a matvec with the add + norm folded in does too (every
        # workgroup then makes the pass's normed rows for itself ahead of its first tile), but what that adds to each
        # workgroup is more than the launch it saves (measured on the 36-layer [2560 / 9728] stack, bf16: 3.03
        # against 2.97 ms at 5 rows, 3.28 against 3.12 at 8, 4.30 against 3.87 at 16; at 4 rows, vector kernels
        # both ways, 4.3 against 4.0).
        chosen = fused is None
        if fused is None:
            fused = T <= 3
        if fold_silu is None:
            fold_silu = fused
        self.fold_silu = bool(fold_silu)
        # the fused launches exist for bf16 and 12-bit matrices; any other stored form takes one launch per operator
        lins = [weights[f"layers.{i}.{k}"] for i in range(cfg.layers) for k in ("qkv", "o", "gu", "down")] + [weights["head"]]
        self.fused = bool(fused) and all(getattr(m, "fusable", False) for m in lins)
        # a pass's q / k norm, rope and cache write ride in its attention kernel where that kernel takes the pass's
        # shape - in the fused sequence, and in the other one too unless the caller asked for a launch per operator
        # ... and the activation in the gate / up matvec's epilogue (bf16 matrices)
        self.glu_fold = (chosen or bool(fused)) and T > 1
        self.rows_attn_fused = (chosen or bool(fused)) and T > 1 and bool(
            card.attn_rows_fused(T, cfg.q_heads, cfg.kv_heads, cfg.head_dim, self.cap, self.S))
        # the handoff to the host: token, cache length and the GPU's clock in pinned memory
        self.host_tok = torch.zeros(1, dtype=torch.int32).pin_memory()
        self.host_n0 = torch.zeros(1, dtype=torch.int32).pin_memory()
        self.host_ts = torch.zeros(1, dtype=torch.int64).pin_memory()
        self.graph: torch.cuda.CUDAGraph | None = None
        # a pass of several rows is a chain unless `set_tree` says otherwise: each row's parent among the pass's rows
        # and its depth (the rope position past the cache), read by the kernels from these two device tensors
        self.par = torch.arange(-1, self.T - 1, dtype=torch.int32, device=dev) if self.T > 1 else None
        self.depth = torch.arange(self.T, dtype=torch.int32, device=dev) if self.T > 1 else None
        self._rows = 0  # the host's count of the cache's rows (n0 starts at 0 on the device too); reset() sets both

    # -- state ---------------------------------------------------------------------------------------------------

    def reset(self, n0: int, token: int) -> None:
        """the cache holds `n0` rows; `token` is the step's input"""
        if not 0 <= n0 + self.T <= self.cap:
            raise ValueError(f"[decode] {n0} cached rows and a pass of {self.T} do not fit a cache of {self.cap}")
        self.n0.fill_(int(n0))
        self.ids.fill_(int(token))
        self._rows = int(n0)  # the host's count of the cache's rows: every step run or replayed adds one

    def set_tree(self, par: list[int] | None) -> None:
        """the pass's rows as a tree (a speculative verify pass: the reference's `par` / `depth` arguments,
        native/cuda/btb_attn_flash.cuh:284-286, btb_kernels.cu:330-335): par[t] is row t's parent among the pass's
        rows, -1 for a root (a child of the cache's last row); a row attends to the cache, its ancestors and itself
        and takes the rope position n0 + its depth. None: a chain. Written into the tensors a captured graph reads."""
        if self.T == 1:
            raise ValueError("[decode] a pass of one row has no tree")
        if par is None:
            par = list(range(-1, self.T - 1))
        if len(par) != self.T or self.T > 32 or any(not -1 <= p < t for t, p in enumerate(par)):
            raise ValueError("[decode] par names, for each of at most 32 rows, an earlier row of the pass or -1")
        depth = []
        for p in par:
            depth.append(0 if p < 0 else depth[p] + 1)
        self.par.copy_(torch.tensor(par, dtype=torch.int32))
        self.depth.copy_(torch.tensor(depth, dtype=torch.int32))

    def weight_bytes(self) -> int:
        """bytes of linear weights one step streams"""
        n = sum(self.w[f"layers.{i}.{k}"].nbytes for i in range(self.cfg.layers) for k in ("qkv", "o", "gu", "down"))
        return n + self.w["head"].nbytes

    def kv_bytes(self, n: int) -> int:
        """bytes of cache one step reads with `n` keys a head"""
        return self.cfg.layers * 2 * self.cfg.kv_heads * n * self.cfg.head_dim * 2

    # -- the kernel sequence ---------------------------------------------------------------------------------------

    def _advance(self) -> None:
        """refuse a step whose rows would be written past the cache's end (the kernels do not look: the slot is
        n0 + t on the device), counting from the last `reset`"""
        if self._rows + self.T > self.cap:
            raise RuntimeError(f"[decode] the cache is full: {self._rows} rows of {self.cap}, and the step writes {self.T}")
        self._rows += 1

    def body(self) -> None:
        if not torch.cuda.is_current_stream_capturing():  # a step being recorded runs nothing
            self._advance()
        if self.fused:
            self._body_fused()
        else:
            self._body_plain()

    def _body_plain(self) -> None:
        """one launch per operator, in the reference's order (btb/engine/cuda.py:1722-1834) - but for a pass's q / k
        norm and rope, which ride in its attention kernel unless the step was built with `fused=False`"""
        k, cfg, w = self.card, self.cfg, self.w
        Hq, Hk, D = cfg.q_heads, cfg.kv_heads, cfg.head_dim
        k.embed(w["embed"], self.ids, self.h)
        y_prev = None
        for i in range(cfg.layers):
            L = f"layers.{i}."
            K, V = self.kv[i, 0], self.kv[i, 1]
            k.add_rmsnorm(self.h, y_prev, w[L + "ln1"], cfg.eps, self.x)
            w[L + "qkv"].matvec(self.x, self.qkv)
            if self.rows_attn_fused:
                k.attn_decode_qkv_rows(self.qkv, w.get(L + "wq"), w.get(L + "wk"), cfg.eps, self.cos, self.sin,
                                       self.n0, K, V, self.att, Hq, Hk, D, self.scale, self.S, self.scratch,
                                       depth=self.depth, par=self.par)
            else:
                k.norm_rope_kv(self.qkv, w.get(L + "wq"), w.get(L + "wk"), cfg.eps, self.cos, self.sin, self.n0, K, V,
                               self.q, Hq, Hk, D, depth=self.depth)
                k.attn_decode(self.q, K, V, self.att, self.n0, Hq, Hk, D, self.scale, self.S, self.scratch,
                              par=self.par)
            w[L + "o"].matvec(self.att, self.y)
            k.add_rmsnorm(self.h, self.y, w[L + "ln2"], cfg.eps, self.x)
            down = w[L + "down"]
            if self.glu_fold and isinstance(w[L + "gu"].w, torch.Tensor):
                k.gemv_glu_silu(w[L + "gu"].w, self.x, self.m)
                down.matvec(self.m, self.y)
                y_prev = self.y
                continue
            w[L + "gu"].matvec(self.x, self.gu)
            if self.fold_silu and isinstance(down.w, torch.Tensor):
                k.gemv_silu(down.w, self.gu, self.y)
            else:
                k.silu_mul(self.gu, self.m)
                down.matvec(self.m, self.y)
            y_prev = self.y
        k.add_rmsnorm(self.h, y_prev, w["norm"], cfg.eps, self.x)
        w["head"].matvec(self.x, self.logits)
        k.argmax(self.logits, self.picked)
        k.publish(self.n0, self.picked, self.ids, self.host_tok, self.host_n0, self.host_ts)

    def _body_fused(self) -> None:
        """the same arithmetic in fewer launches: each residual add + norm rides in the x load of the matvec that
        follows it (the residual ping-pongs between two buffers), gate / up / activation are one kernel, the q / k norm
        and rope ride in the attention kernel. Bit for bit
        the plain sequence's result."""
        k, cfg, w = self.card, self.cfg, self.w
        Hq, Hk, D = cfg.q_heads, cfg.kv_heads, cfg.head_dim
        ha, hb = self.h, self.h2
        y_prev = None
        for i in range(cfg.layers):
            L = f"layers.{i}."
            K, V = self.kv[i, 0], self.kv[i, 1]
            if i == 0:  # the residual starts as the tokens' embedding rows, gathered by the first matvec itself
                k.gemv_embed_norm(w[L + "qkv"].w, w["embed"], self.ids, w[L + "ln1"], cfg.eps, hb, self.qkv)
            else:
                k.gemv_norm(w[L + "qkv"].w, ha, y_prev, w[L + "ln1"], cfg.eps, hb, self.qkv)
            if self.T == 1 and D == 128:
                k.attn_decode_qkv(self.qkv, w.get(L + "wq"), w.get(L + "wk"), cfg.eps, self.cos, self.sin, self.n0, K,
                                  V, self.att, Hq, Hk, D, self.scale, self.S, self.scratch)
            elif self.rows_attn_fused:
                k.attn_decode_qkv_rows(self.qkv, w.get(L + "wq"), w.get(L + "wk"), cfg.eps, self.cos, self.sin,
                                       self.n0, K, V, self.att, Hq, Hk, D, self.scale, self.S, self.scratch,
                                       depth=self.depth, par=self.par)
            else:
                k.norm_rope_kv(self.qkv, w.get(L + "wq"), w.get(L + "wk"), cfg.eps, self.cos, self.sin, self.n0, K, V,
                               self.q, Hq, Hk, D, depth=self.depth)
                k.attn_decode(self.q, K, V, self.att, self.n0, Hq, Hk, D, self.scale, self.S, self.scratch,
                              par=self.par)
            w[L + "o"].matvec(self.att, self.y)
            k.gemv_norm(w[L + "gu"].w, hb, self.y, w[L + "ln2"], cfg.eps, ha, self.m, glu=True)
            w[L + "down"].matvec(self.m, self.y)
            y_prev = self.y
        k.gemv_norm(w["head"].w, ha, y_prev, w["norm"], cfg.eps, None, self.logits)
        if self.T == 1:
            k.argmax_publish(self.logits, self.picked, self.n0, self.ids, self.host_tok, self.host_n0, self.host_ts)
        else:
            k.argmax(self.logits, self.picked)
            k.publish(self.n0, self.picked, self.ids, self.host_tok, self.host_n0, self.host_ts)

    def capture(self, warmup: int = 2) -> torch.cuda.CUDAGraph:
        """run the step eagerly (on a side stream, as a capture requires), then record it: the hipGraph the host
        replays. The warm-up steps advance the cache; `reset` before the first replay."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                self.body()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with recording(g):
            self.body()
        self.graph = g
        return g

    def replay(self) -> None:
        if self.graph is None:
            raise RuntimeError("[decode] capture() the step before replaying it")
        self._advance()
        self.graph.replay()

    def token(self) -> int:
        """the last step's token as the host sees it (after a synchronize, or once host_n0 shows the new length)"""
        return int(self.host_tok[0])


def random_stack(card: Any, cfg: StackConfig, seed: int = 0x0B7B0000, packed: bool = False,
                 std: float = 0.02) -> dict[str, Any]:
    """random-init weights of the stack's shape on the GPU: linears ~ N(0, std) rounded to bf16 (drawn with the
    device's generator, one seed per tensor), norm weights one. `packed`: every linear stored in the 12-bit form."""
    dev = torch.device("cuda")
    H, I = cfg.hidden, cfg.intermediate
    n = [0]

    def mat(rows: int, cols: int) -> Linear:
        g = torch.Generator(device=dev).manual_seed(seed + n[0])
        n[0] += 1
        t = (torch.randn(rows, cols, generator=g, device=dev, dtype=torch.float32) * std).to(torch.bfloat16)
        return Linear(card, P12Weight.pack(t, card) if packed else t)

    w: dict[str, Any] = {}
    for i in range(cfg.layers):
        L = f"layers.{i}."
        w[L + "qkv"] = mat(cfg.qkv_rows, H)
        w[L + "o"] = mat(H, cfg.q_heads * cfg.head_dim)
        w[L + "gu"] = mat(2 * I, H)
        w[L + "down"] = mat(H, I)
        for name, length in (("ln1", H), ("ln2", H), ("wq", cfg.head_dim), ("wk", cfg.head_dim)):
            w[L + name] = torch.ones(length, dtype=torch.bfloat16, device=dev)
    g = torch.Generator(device=dev).manual_seed(seed + 100_000)
    w["embed"] = (torch.randn(cfg.vocab, H, generator=g, device=dev, dtype=torch.float32) * std).to(torch.bfloat16)
    w["norm"] = torch.ones(H, dtype=torch.bfloat16, device=dev)
    w["head"] = mat(cfg.vocab, H)
    return w
