"""Dense gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(ullm/models/qwen3.py:23-46, ullm/layers/activation.py:16-18).  gate and up are one fused
projection with rows gate | up (qwen3.py:307-308).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import FeedForward, PartEnv, StepContext, WeightDecl, register_part
from .linear import add_into_stream, can_fuse, gate_up, linear, linear_into_stream, linear_of_norm


@register_part("ffn", "swiglu")
class SwiGLU(FeedForward):
    folds_norm = True
    hands_norm_ahead = True

    def __init__(self, hidden_size: int, intermediate_size: int, prefix: str, names: Optional[Dict[str, str]] = None):
        self.hidden_size, self.intermediate_size, self.prefix = hidden_size, intermediate_size, prefix
        # tensor names behind the prefix; "gate_up" is the merged matrix's (a checkpoint may hold it whole)
        self.names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight",
                      "gate_up": "gate_up_proj.weight", **(names or {})}
        self.w_gate_up = self.w_down = None

    def weights(self) -> List[WeightDecl]:
        p, H, I, n = self.prefix, self.hidden_size, self.intermediate_size, self.names
        merged = f"{p}.{n['gate_up']}"               # rows gate | up, put together by the loader
        return [WeightDecl(f"{p}.{n['gate']}", (I, H), merged_into=merged, row_offset=0),
                WeightDecl(f"{p}.{n['up']}", (I, H), merged_into=merged, row_offset=I),
                WeightDecl(f"{p}.{n['down']}", (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        p, n = self.prefix, self.names
        self.w_gate_up = tensors[f"{p}.{n['gate_up']}"].contiguous()
        self.w_down = tensors[f"{p}.{n['down']}"].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        act = gate_up(x, self.w_gate_up)
        return linear_into_stream(act, self.w_down, ctx)

    def fusable(self, residual, ctx: StepContext) -> bool:
        return can_fuse(residual, ctx.dtype, self.w_gate_up, self.w_down)

    def forward_fused(self, x, residual, ctx: StepContext, then=None):
        act = linear_of_norm(x, self.w_gate_up, silu=True)     # the norm before, silu(gate) * up behind the first product
        return add_into_stream(act, self.w_down, residual, then, ctx.dtype)   # residual add (and the next norm's part) behind the second


ACTIVATIONS = {"relu2": ops.ACT_RELU2, "gelu_tanh": ops.ACT_GELU_TANH}


@register_part("ffn", "mlp")
class MLP(FeedForward):
    """Dense feed-forward without a gate: down(act(up(x))), no biases; ``activation`` is "relu2" (the square of
    relu) or "gelu_tanh".  The activation is applied in 32-bit: to the product's 32-bit sums on store where the
    few-rows and rows kernels run, to the stored product (bfloat16 or float32) behind the library's and the 32-bit
    product."""

    def __init__(self, hidden_size: int, intermediate_size: int, prefix: str, activation: str = "relu2",
                 names: Optional[Dict[str, str]] = None):
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation={activation!r}; known: {sorted(ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.prefix = hidden_size, intermediate_size, prefix
        self.act = ACTIVATIONS[activation]
        self.names = {"up": "up_proj.weight", "down": "down_proj.weight", **(names or {})}
        self.w_up = self.w_down = None

    def weights(self) -> List[WeightDecl]:
        p, H, I, n = self.prefix, self.hidden_size, self.intermediate_size, self.names
        return [WeightDecl(f"{p}.{n['up']}", (I, H)), WeightDecl(f"{p}.{n['down']}", (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.w_up = tensors[f"{self.prefix}.{self.names['up']}"].contiguous()
        self.w_down = tensors[f"{self.prefix}.{self.names['down']}"].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return linear_into_stream(linear(x, self.w_up, act=self.act), self.w_down, ctx)
