"""The routed MoE decode layer on the GPU: the counterparts of the reference's `Qwen4Router`
(btb/engine/families/qwen4/router.py:21-51) and `_Experts` (btb/engine/host.py:310-1107, its arithmetic only: every
expert is resident in VRAM here, so there is no store, no wave and no host round trip).

    router = Router(card, w_router, top_k)           # w_router bf16 [E, H]
    experts = Experts(card, gate_up, down)           # bf16 stacks [E, 2I, H], [E, H, I]
    logits, weights, picks = router(x)               # x bf16 [T, H]
    y = experts(x, picks, weights)                   # bf16 [T, H], summed in ascending expert order

MXFP4 expert stacks (gpt-oss's checkpoints, or any stack quantised the same way) stay as stored and go through the same
two kernels with the widening in their registers:

    experts = MxExpertsLayer(card, load_mx_experts(path, layer))          # gpt-oss: interleaved rows, biases, clamped gate
    experts = MxExpertsLayer(card, MxExperts(...), oss=False)             # concatenated halves, SiLU
"""

from __future__ import annotations

from typing import Any

import torch


class Router:
    """f32 logits by the host's own matvec order on the card (so the picks are the CPU path's, bit for bit), then the
    card's softmax / top-k / renormalise. Returns (logits in x's dtype, weights in x's dtype, picks int32)."""

    def __init__(self, card: Any, weight: torch.Tensor, top_k: int, norm_topk_prob: bool = True) -> None:
        if weight.dtype != torch.bfloat16 or weight.dim() != 2 or not weight.is_cuda:
            raise ValueError("[moe] the router's weight is a bf16 [E, H] matrix on the GPU")
        if not norm_topk_prob:
            raise ValueError("[moe] the card's router renormalises the picked weights (norm_topk_prob)")
        self.card = card
        self.weight = weight.contiguous()
        self.top_k = int(top_k)
        self.num_experts, self.hidden_dim = (int(s) for s in weight.shape)

    def __call__(self, hidden_states: torch.Tensor):
        x = hidden_states.reshape(-1, self.hidden_dim)
        if x.dtype == torch.bfloat16:  # the rows as held: logits and routing in two launches, nothing between them
            _, logits16, picks, weights, _ = self.card.moe_router(self.weight, x.contiguous(), self.top_k)
            return logits16, weights, picks
        logits = self.card.gemv_lane16(self.weight, x.float().contiguous())
        picks, weights, _ = self.card.moe_route(logits, self.top_k)
        return logits.to(hidden_states.dtype), weights.to(hidden_states.dtype), picks


class Experts:
    """The layer's experts as two bf16 stacks on the GPU. `__call__(x, picks, weights)` is `_Experts.forward`'s
    result: [T, H] in the rows' dtype (bf16), every pick's product times its weight, summed in ascending expert
    order with each step rounded to bf16."""

    def __init__(self, card: Any, gate_up: torch.Tensor, down: torch.Tensor) -> None:
        E, I2, H = (int(s) for s in gate_up.shape)
        if tuple(down.shape) != (E, H, I2 // 2):
            raise ValueError(f"[moe] gate_up {tuple(gate_up.shape)} and down {tuple(down.shape)} are not one layer's")
        self.card = card
        self.gate_up = gate_up.contiguous()
        self.down = down.contiguous()
        self.num_experts, self.hidden_dim, self.intermediate_dim = E, H, I2 // 2
        self._gu: torch.Tensor | None = None

    def __call__(self, hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor,
                 out: torch.Tensor | None = None) -> torch.Tensor:
        x = hidden_states.reshape(-1, self.hidden_dim)
        if x.dtype != torch.bfloat16:
            raise ValueError("[moe] the card's experts take bf16 rows")
        T, k = (int(s) for s in top_k_index.shape)
        if self._gu is None or self._gu.shape[0] < T or self._gu.shape[1] != k:
            self._gu = torch.empty(T, k, 2 * self.intermediate_dim, dtype=torch.bfloat16, device=x.device)
        return self.card.moe_experts(self.gate_up, self.down, x.contiguous(), top_k_index.to(torch.int32).contiguous(),
                                     top_k_weights.to(torch.bfloat16).contiguous(), out, self._gu[:T])


class MxExpertsLayer:
    """The layer's experts as MXFP4 stacks on the GPU, as the checkpoint stores them (`btb_amd.load.MxExperts`): the
    reference's `_Experts` over `Native.gemv_mx4_group` (btb/engine/host.py:459-461, 508-569) with every expert
    resident. `oss` (the default): gpt-oss's experts - gate and up rows interleaved, the experts' biases, the clamped
    gate `(up + 1) * gate * sigmoid(alpha * gate)` (host.py:443-451); `oss=False`: concatenated halves and SiLU. Same
    call and result as `Experts`."""

    def __init__(self, card: Any, stacks: Any, oss: bool = True, alpha: float = 1.702, limit: float = 7.0) -> None:
        if not oss and (stacks.gate_up_bias is not None or stacks.down_bias is not None):
            raise ValueError("[moe] expert biases belong to the gpt-oss form")
        self.card, self.stacks, self.oss, self.alpha, self.limit = card, stacks, bool(oss), float(alpha), float(limit)
        self.num_experts, self.hidden_dim, self.intermediate_dim = stacks.experts, stacks.hidden, stacks.intermediate
        self._h: torch.Tensor | None = None

    def __call__(self, hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor,
                 out: torch.Tensor | None = None) -> torch.Tensor:
        x = hidden_states.reshape(-1, self.hidden_dim)
        if x.dtype != torch.bfloat16:
            raise ValueError("[moe] the card's experts take bf16 rows")
        T, k = (int(s) for s in top_k_index.shape)
        if self._h is None or self._h.shape[0] < T or self._h.shape[1] != k:
            self._h = torch.empty(T, k, self.intermediate_dim, dtype=torch.bfloat16, device=x.device)
        return self.card.moe_experts_mx4(self.stacks, x.contiguous(), top_k_index.to(torch.int32).contiguous(),
                                         top_k_weights.to(torch.bfloat16).contiguous(), out, self._h[:T], oss=self.oss,
                                         alpha=self.alpha, limit=self.limit)
