"""Routed feed-forward: a router picks ``top`` of several small gated feed-forwards per token.

The router's logits are a 32-bit product of the part's input with a matrix [R, hidden], R = experts with weights +
identity experts.  The scores are the softmax over all R; the choice goes by score + a learned correction per
output (``correction``), the weights by the chosen outputs' scores alone, divided by their sum (+ 1e-20).  The last
``identity`` router outputs stand for experts without tensors whose output is their input.  Every expert is
``down(act(gate(x), up(x)))`` without biases, with the clamped gated unit
``act(g, u) = g' * sigmoid(alpha * g') * (u' + 1)``, ``g' = min(g, limit)``, ``u' = clamp(u, -limit, limit)``.
A shared expert of the same form (sizes and limit of its own) may run for every token and is added.
Two more forms, each a parameter: ``routing="top_logits"`` picks the ``top`` largest of logits + a learned bias per
output (the ``correction`` tensor, then a bias on the logits) and weighs them by the softmax over the picked ones
alone; ``routing="sigmoid"`` scores every output by the sigmoid of its own logit, chooses by score + correction and
weighs by the chosen scores over their sum (+ 1e-20); ``weight_scale`` multiplies every weight; ``limit=None`` makes
every expert the plain gated unit ``silu(g) * u``.

The experts' matrices are stacked ([experts, 2 ff, hidden] with gate rows, then up rows, per expert, and
[experts, hidden, ff]); the loader puts the checkpoint's per-expert tensors into their rows.  A step groups
its (token, expert) pairs by expert on the device and runs the two products over the grouped rows
(``ops.moe_sort``, ``ops.moe_rows``); launches are sized by the step's token count alone, so a step of single
tokens can be replayed from a graph.  The result is 32-bit: ``forward_onto`` adds it onto another branch of
the same block (and that branch's bias) in the kernel that sums the experts.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import FeedForward, PartEnv, StepContext, WeightDecl, register_part
from .linear import gate_up, linear

DEFAULT_NAMES = {"router": "router", "correction": "correction", "expert": "e{index}", "gate": "gate", "up": "up",
                 "down": "down", "shared": "shared"}


def tile_rows_for(tokens: int, top: int, experts: int) -> int:
    """Grouped rows a block of the expert products takes, from the rows an expert gets on average: a function of
    the step's size alone."""
    mean = tokens * top / max(1, experts)
    if mean >= 96:
        return 128
    if mean >= 48:
        return 64
    return 32 if mean >= 24 else 16


@register_part("ffn", "routed_experts")
class RoutedExperts(FeedForward):
    def __init__(self, hidden_size: int, experts: int, intermediate_size: int, top: int, limit: Optional[float],
                 prefix: str, identity: int = 0, alpha: float = 1.702, correction: bool = True,
                 shared_size: int = 0, shared_limit: Optional[float] = None, names: Optional[Dict[str, str]] = None,
                 routing: str = "softmax_all", weight_scale: float = 1.0):
        modes = {"softmax_all": ops.ROUTE_SOFTMAX_ALL, "top_logits": ops.ROUTE_TOP_LOGITS, "sigmoid": ops.ROUTE_SIGMOID}
        if routing not in modes:
            raise ValueError(f"routing={routing!r}: one of {sorted(modes)}")
        self.mode, self.weight_scale = modes[routing], float(weight_scale)
        limit = 0.0 if limit is None else limit            # the kernels read a limit of 0 as the plain unit
        if experts < 0 or identity < 0 or experts + identity < 1:
            raise ValueError(f"{experts} experts and {identity} identity experts: a router needs at least one output")
        if not 1 <= top <= experts + identity:
            raise ValueError(f"top={top} of {experts + identity} router outputs")
        if experts + identity > ops.MOE_MAX_ROUTER or top > ops.MOE_MAX_TOP:
            raise ValueError(f"at most {ops.MOE_MAX_ROUTER} router outputs and a top of {ops.MOE_MAX_TOP}")
        self.hidden_size, self.experts, self.identity, self.top = hidden_size, int(experts), int(identity), int(top)
        self.ff, self.limit, self.alpha = int(intermediate_size), float(limit), float(alpha)
        self.shared_ff = int(shared_size)
        self.shared_limit = float(shared_limit) if shared_limit is not None else self.limit
        self.has_correction = bool(correction)
        self.prefix = prefix
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_router = self.correction = self.w_gate_up = self.w_down = self.w_shared_gate_up = self.w_shared_down = None

    # ------------------------------------------------------------------ weights
    def _expert(self, index: int, role: str) -> str:
        return f"{self.prefix}.{self.names['expert'].format(index=index)}.{self.names[role]}"

    def _shared(self, role: str) -> str:
        return f"{self.prefix}.{self.names['shared']}.{self.names[role]}"

    def weights(self) -> List[WeightDecl]:
        p, H, I, R = self.prefix, self.hidden_size, self.ff, self.experts + self.identity
        out = [WeightDecl(f"{p}.{self.names['router']}", (R, H), keep_fp32=True)]
        if self.has_correction:
            out.append(WeightDecl(f"{p}.{self.names['correction']}", (R,), keep_fp32=True))
        for e in range(self.experts):
            out += [WeightDecl(self._expert(e, "gate"), (I, H), merged_into=f"{p}.experts.gate_up", row_offset=2 * I * e),
                    WeightDecl(self._expert(e, "up"), (I, H), merged_into=f"{p}.experts.gate_up", row_offset=2 * I * e + I),
                    WeightDecl(self._expert(e, "down"), (H, I), merged_into=f"{p}.experts.down", row_offset=H * e)]
        if self.shared_ff:
            S = self.shared_ff
            out += [WeightDecl(self._shared("gate"), (S, H), merged_into=f"{p}.shared.gate_up", row_offset=0),
                    WeightDecl(self._shared("up"), (S, H), merged_into=f"{p}.shared.gate_up", row_offset=S),
                    WeightDecl(self._shared("down"), (H, S))]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        p, H, I = self.prefix, self.hidden_size, self.ff
        self.w_router = tensors[f"{p}.{self.names['router']}"].contiguous()
        self.correction = tensors[f"{p}.{self.names['correction']}"].contiguous() if self.has_correction else None
        if self.experts:
            self.w_gate_up = tensors[f"{p}.experts.gate_up"].contiguous().view(self.experts, 2 * I, H)
            self.w_down = tensors[f"{p}.experts.down"].contiguous().view(self.experts, H, I)
        if self.shared_ff:
            self.w_shared_gate_up = tensors[f"{p}.shared.gate_up"].contiguous()
            self.w_shared_down = tensors[self._shared("down")].contiguous()

    # ------------------------------------------------------------------ the step
    def route(self, x: torch.Tensor):
        """(ids int32 [T, top], weights float32 [T, top]) of the rows of x."""
        if self.hidden_size <= ops.MOE_ROUTER_MAX_WIDTH:
            return ops.moe_router(x, self.w_router, self.correction, self.top, self.mode, self.weight_scale)     # the product and the routing in one
        logits = ops.gemm_simple(x, self.w_router, out_dtype=torch.float32)       # 32-bit sums in a fixed order
        return ops.moe_route(logits, self.correction, self.top, self.mode, self.weight_scale)

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return self.forward_onto(x, ctx, None, None)

    def forward_onto(self, x: torch.Tensor, ctx: StepContext, base: Optional[torch.Tensor],
                     bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """float32 [T, hidden]: ``base`` (another branch's output, or None) + ``bias`` + this feed-forward of x."""
        T = x.shape[0]
        ids, weights = self.route(x)
        y = None
        tile_rows = tile_rows_for(T, self.top, self.experts)
        slot_of_pair = ids.view(-1)               # read for experts with weights only
        if self.experts:
            slot_of_pair, token_of_slot, tiles, _ = ops.moe_sort(ids, self.experts, tile_rows)
            act = ops.moe_rows(x, token_of_slot, self.w_gate_up, tiles, tile_rows, T * self.top, gated=True,
                               limit=self.limit, alpha=self.alpha)
            y = ops.moe_rows(act, None, self.w_down, tiles, tile_rows, T * self.top, gated=False)
        shared = None
        if self.shared_ff:
            # gate | up with the unit on store where the few-rows kernels take the step, as the dense feed-forward's
            act = gate_up(x, self.w_shared_gate_up, self.shared_limit, self.alpha)
            shared = linear(act, self.w_shared_down)
        return ops.moe_combine(y, x, ids, weights, slot_of_pair, self.experts, base=base, bias=bias, shared=shared)
