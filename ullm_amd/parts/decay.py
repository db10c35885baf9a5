"""Mixers whose memory is a matrix state per head that decays per key channel (linear attention with decays).

All three share one recurrence (``ops.decay_scan``): per head S_t = diag(d_t) S_(t-1) + k_t v_t^T with S [key_dim,
value_dim], and o_t = S_t^T q_t, or with a bonus for the current token o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t.
They differ in where q, k, v and the decays d come from and in what stands behind the outputs:

``gated_linear_attention``  q = W_q h * key_dim^(-1/2), k = W_k h, v = W_v h; d = sigmoid(z)^(1/tau) with
    z = W_a2 (W_a1 h) + b (a low-rank product); every head's o over its root mean square times a gain shared by the
    heads, times silu(W_g h), then W_o.
``lightning_attention``  q, k, v = silu of their projections; one constant decay per head; all heads' outputs
    normed together times a gain, times sigmoid(W_g h), then W_o.
``time_mix``  every projection reads its own blend h + (h' - h) * mu of the token's input h and the previous
    token's h' (zeros before the first token; the last h is part of the state); d = exp(-exp(W_w2 tanh(W_w1 .) +
    w0)); the bonus u; every head's o over its root mean square, times a gain per column, times silu(W_g .), then W_o.

What a request keeps between steps is one float32 row per slot: the heads' states (for ``time_mix`` the last input
row ahead of them).  The projections leave float32 rows also where the model computes in bfloat16, so everything
that enters the recurrence is 32-bit; the recurrence walks an entry's tokens in order whatever the batch holds.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..kernels import ops
from .base import LayerCache, Mixer, PartEnv, StateNeed, StepContext, WeightDecl, register_part
from .linear import linear, linear_into_stream


class _DecayMixer(Mixer):
    """What the three have in common: sizes, the state row, names."""
    DEFAULT_NAMES: Dict[str, str] = {}

    def __init__(self, hidden_size: int, heads: int, key_dim: int, value_dim: int, norm_eps: float, prefix: str,
                 names: Optional[Dict[str, str]] = None):
        if heads < 1 or key_dim < 1 or value_dim < 1:
            raise ValueError("heads and sizes must be positive")
        if key_dim > ops.DECAY_SCAN_MAX_KEYS:
            raise ValueError(f"{key_dim} key channels a head: the recurrence takes at most {ops.DECAY_SCAN_MAX_KEYS}")
        self.hidden_size, self.heads, self.key_dim, self.value_dim = hidden_size, heads, key_dim, value_dim
        self.norm_eps, self.prefix = float(norm_eps), prefix
        self.names = {**self.DEFAULT_NAMES, **(names or {})}
        self.qk, self.inner = heads * key_dim, heads * value_dim
        self.carry = 0                                   # values of the state row ahead of the heads' states

    def _name(self, role: str) -> str:
        return f"{self.prefix}.{self.names[role]}"

    def cache_need(self):
        return StateNeed((self.carry + self.heads * self.key_dim * self.value_dim,), torch.float32, graph_safe=True)

    @staticmethod
    def _rows(cache: LayerCache) -> torch.Tensor:
        return cache.state.view(cache.state.shape[0], -1)

    @staticmethod
    def _ahead(x: torch.Tensor, ctx: StepContext) -> bool:
        """Whether a pass of its own applies the inputs' functions ahead of the recurrence: in steps of many tokens
        with portions of prompts (the recurrence's blocks, one per slice of value channels, would each apply them to a
        whole chunk again); a step of single tokens leaves them to the recurrence, a launch fewer."""
        return x.shape[0] >= ops.DECAY_PREPARE_FROM and ctx.max_q_len > 1


@register_part("mixer", "gated_linear_attention")
class GatedLinearAttention(_DecayMixer):
    DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a2_bias": "a2.b"}

    def __init__(self, hidden_size: int, heads: int, key_dim: int, value_dim: int, tau: float, norm_eps: float,
                 prefix: str, rank: int = 16, names: Optional[Dict[str, str]] = None):
        super().__init__(hidden_size, heads, key_dim, value_dim, norm_eps, prefix, names)
        if tau <= 0:
            raise ValueError("tau must be positive")
        self.tau, self.rank = float(tau), int(rank)

    def weights(self) -> List[WeightDecl]:
        H, p = self.hidden_size, f"{self.prefix}.in"
        # one matrix q | k | v | g | a1: the loader puts the tensors into its rows; the low-rank product's inner size
        # is whatever the checkpoint's tensors have
        rows = (("q", self.qk), ("k", self.qk), ("v", self.inner), ("g", self.inner))
        out, off = [], 0
        for role, n in rows:
            out.append(WeightDecl(self._name(role), (n, H), merged_into=p, row_offset=off))
            off += n
        out += [WeightDecl(self._name("a1"), (self.rank, H), free_dims=(0,)),
                WeightDecl(self._name("a2"), (self.qk, self.rank), free_dims=(1,)),
                WeightDecl(self._name("a2_bias"), (self.qk,), keep_fp32=True),
                WeightDecl(self._name("norm"), (self.value_dim,), init="gain", keep_fp32=True),
                WeightDecl(self._name("o"), (H, self.inner))]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.w_in = tensors[f"{self.prefix}.in"].contiguous()
        self.w_a1, self.w_a2 = tensors[self._name("a1")].contiguous(), tensors[self._name("a2")].contiguous()
        self.b_a2, self.gain = tensors[self._name("a2_bias")].contiguous(), tensors[self._name("norm")].contiguous()
        self.w_o = tensors[self._name("o")].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        proj = linear(x, self.w_in, out_dtype=torch.float32)                        # q | k | v | g
        z = linear(linear(x, self.w_a1, out_dtype=torch.float32), self.w_a2, self.b_a2, out_dtype=torch.float32)
        qk, inner = self.qk, self.inner
        kind = ops.DECAY_SIGMOID_ROOT
        if self._ahead(x, ctx):
            # many tokens: the decays' function is applied once per value ahead of the recurrence, not by each of its blocks
            ops.decay_prepare(None, z, kind, self.tau)
            kind = ops.DECAY_READY
        o = ops.decay_scan(proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + inner], z, kind,
                           self._rows(cache), 0, ctx.q_start, ctx.entry_slot, ctx.num_entries, self.heads, self.key_dim,
                           self.value_dim, tau=self.tau, q_scale=self.key_dim ** -0.5, write_state=cache.owner,
                           max_len=ctx.max_q_len)
        y = ops.gated_unit_norm(o, proj[:, 2 * qk + inner:], self.gain, self.norm_eps, self.heads, ops.GATE_SILU, ctx.dtype)
        return linear_into_stream(y, self.w_o, ctx)


@register_part("mixer", "lightning_attention")
class LightningAttention(_DecayMixer):
    DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm"}

    def __init__(self, hidden_size: int, heads: int, key_dim: int, value_dim: int, decay: Sequence[float],
                 norm_eps: float, prefix: str, names: Optional[Dict[str, str]] = None):
        super().__init__(hidden_size, heads, key_dim, value_dim, norm_eps, prefix, names)
        if len(decay) != heads:
            raise ValueError(f"{len(decay)} decays for {heads} heads")
        self.decay_values = tuple(float(d) for d in decay)

    def weights(self) -> List[WeightDecl]:
        H, p = self.hidden_size, f"{self.prefix}.in"
        out, off = [], 0
        for role, n in (("q", self.qk), ("k", self.qk), ("v", self.inner), ("g", self.inner)):
            out.append(WeightDecl(self._name(role), (n, H), merged_into=p, row_offset=off))
            off += n
        out += [WeightDecl(self._name("norm"), (self.inner,), init="gain", keep_fp32=True),
                WeightDecl(self._name("o"), (H, self.inner))]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.w_in = tensors[f"{self.prefix}.in"].contiguous()
        self.gain, self.w_o = tensors[self._name("norm")].contiguous(), tensors[self._name("o")].contiguous()
        # the constants are rounded to 32-bit once, from the 64-bit numbers of the configuration
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(env.device)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        proj = linear(x, self.w_in, out_dtype=torch.float32)                        # q | k | v | g
        qk, inner = self.qk, self.inner
        ahead = self._ahead(x, ctx)
        if ahead:
            ops.decay_prepare(proj[:, :2 * qk + inner])              # silu of q | k | v once per value
        o = ops.decay_scan(proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + inner], self.decay, ops.DECAY_PER_HEAD,
                           self._rows(cache), 0, ctx.q_start, ctx.entry_slot, ctx.num_entries, self.heads, self.key_dim,
                           self.value_dim, silu_inputs=not ahead, write_state=cache.owner, max_len=ctx.max_q_len)
        y = ops.gated_unit_norm(o, proj[:, 2 * qk + inner:], self.gain, self.norm_eps, 1, ops.GATE_SIGMOID, ctx.dtype)
        return linear_into_stream(y, self.w_o, ctx)


@register_part("mixer", "time_mix")
class TimeMix(_DecayMixer):
    DEFAULT_NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "w1": "w1", "w2": "w2", "w0": "w0",
                     "u": "u", "mu": "mu.{which}"}
    BLENDS = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, heads: int, head_dim: int, norm_eps: float, prefix: str, rank: int = 16,
                 names: Optional[Dict[str, str]] = None):
        super().__init__(hidden_size, heads, head_dim, head_dim, norm_eps, prefix, names)
        self.rank = int(rank)
        self.carry = hidden_size                          # the previous token's input row leads the state row

    def _mu(self, which: str) -> str:
        return f"{self.prefix}.{self.names['mu'].format(which=which)}"

    def weights(self) -> List[WeightDecl]:
        H, n = self.hidden_size, self.qk
        out = [WeightDecl(self._mu(s), (H,), keep_fp32=True, merged_into=f"{self.prefix}.mu", row_offset=i * H)
               for i, s in enumerate(self.BLENDS)]
        out += [WeightDecl(self._name(role), (n, H)) for role in ("r", "k", "v", "g")]
        out += [WeightDecl(self._name("w1"), (self.rank, H), free_dims=(0,)),
                WeightDecl(self._name("w2"), (n, self.rank), free_dims=(1,)),
                WeightDecl(self._name("w0"), (n,), keep_fp32=True),
                WeightDecl(self._name("u"), (self.heads, self.key_dim), keep_fp32=True),
                WeightDecl(self._name("norm"), (n,), init="gain", keep_fp32=True),
                WeightDecl(self._name("o"), (H, n))]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        get = lambda role: tensors[self._name(role)].contiguous()       # noqa: E731
        self.mu = tensors[f"{self.prefix}.mu"].contiguous().view(len(self.BLENDS), self.hidden_size)
        self.w_r, self.w_k, self.w_v, self.w_g, self.w_o = get("r"), get("k"), get("v"), get("g"), get("o")
        self.w_w1, self.w_w2, self.w0, self.bonus, self.gain = get("w1"), get("w2"), get("w0"), get("u"), get("norm")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        rows = self._rows(cache)
        blends = ops.token_shift(x, self.mu, rows, 0, ctx.token_entry, ctx.q_start, ctx.entry_slot, ctx.num_entries,
                                 write_state=cache.owner)                            # [r, k, v, g, w][T, hidden]
        f32 = torch.float32
        r, k, v = (linear(blends[i], w, out_dtype=f32) for i, w in enumerate((self.w_r, self.w_k, self.w_v)))
        g = linear(blends[3], self.w_g, out_dtype=f32)
        z = linear(linear(blends[4], self.w_w1, out_dtype=f32, act=ops.ACT_TANH), self.w_w2, self.w0, out_dtype=f32)
        kind = ops.DECAY_EXP_EXP
        if self._ahead(x, ctx):
            ops.decay_prepare(None, z, kind)
            kind = ops.DECAY_READY
        o = ops.decay_scan(r, k, v, z, kind, rows, self.carry, ctx.q_start, ctx.entry_slot, ctx.num_entries,
                           self.heads, self.key_dim, self.value_dim, bonus=self.bonus, write_state=cache.owner,
                           max_len=ctx.max_q_len)
        y = ops.gated_unit_norm(o, g, self.gain, self.norm_eps, self.heads, ops.GATE_SILU, ctx.dtype)
        return linear_into_stream(y, self.w_o, ctx)


@register_part("mixer", "side_by_side")
class SideBySide(Mixer):
    """Two mixers that read the same input; the result is ``left_scale * left + right_scale * right`` in 32-bit.
    Each keeps what it keeps: the block sees the needs of both, in this order, and hands each its own view.  A
    block that can add two weighted branches itself asks for them with ``forward_pair``."""

    def __init__(self, left: Mixer, right: Mixer, left_scale: float = 1.0, right_scale: float = 1.0):
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.step_planners = {**left.step_planners, **right.step_planners}
        self._needs = [(m, m.cache_need()) for m in (left, right)]

    def children(self):
        return [self.left, self.right]

    def cache_need(self):
        needs = []
        for _, need in self._needs:
            if need is not None:
                needs.extend(need if isinstance(need, (list, tuple)) else [need])
        return needs or None

    def _views(self, cache: LayerCache):
        parts = cache.parts if cache.parts else [cache]
        out, at = [], 0
        for _, need in self._needs:
            n = 0 if need is None else (len(need) if isinstance(need, (list, tuple)) else 1)
            out.append(LayerCache() if n == 0 else parts[at] if n == 1 else LayerCache.of_parts(parts[at:at + n]))
            at += n
        return out

    def forward_pair(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache):
        """(left, left_scale, right, right_scale): the two branches, not yet added."""
        left_cache, right_cache = self._views(cache)
        return (_plain(self.left.forward(x, ctx, left_cache)), self.left_scale,
                _plain(self.right.forward(x, ctx, right_cache)), self.right_scale)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        left, a, right, b = self.forward_pair(x, ctx, cache)
        return ops.weighted_sum(left, right, a, b)


def _plain(y: torch.Tensor) -> torch.Tensor:
    """A stack of partial sums added up."""
    return ops.branch_sum(y) if y.dim() == 3 else y
