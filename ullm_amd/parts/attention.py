"""Grouped-query attention over the paged cache, as a mixer.

Reference: ullm/models/qwen3.py:49-130 (projection, per-head q/k norm, rotation, attention, output
projection) and ullm/layers/attention.py:279-313 (write k, v to the cache, then attend over it).
Head size is a parameter of its own (qwen3.py:78: not hidden/heads), the q/k norms and the position
encoding are optional parts, and a window bounds how far back a query looks (0 = everything; the
reference never windows).

Beyond that form the same mixer takes, each as a parameter of its own: a value size that differs from the
query/key size (``value_dim``), the q/k norm taken over the whole projection instead of per head
(``qk_norm="whole"``, gains of the projections' full sizes), a bias on the scores by distance (a position part
with ``score_bias()``), a gate per head on the heads' outputs (``head_gate``: sigmoid of one more projection of
the mixer's input), no key/value projections of its own (``own_kv=False``: the layer reads the cache another
layer writes), values that are the keys as projected, before rotation (``values="keys"``: no value projection),
a sink per head in the softmax's denominator (``sink``: a learned number with no key and no value; ``sink_value``:
the same number for every head, a constant of the design without a tensor), a per-head norm without gains
(``qk_norm_gain=False``: queries and keys are only divided by their root mean square), biases on the
projections also there (``bias`` on q, k and v, ``out_bias`` on the output) and other tensor names (``names``).
Any of these takes the general path below: one projection
q | k | v | gate, heads padded with zeros to a size the attention kernels take (zero key dims add nothing to a
score, zero value dims give zero outputs that meet zero columns of the output projection).
"""
from __future__ import annotations

import math

from typing import Dict, List, Optional

import numpy as np
import torch

from ..kernels import ops
from .base import (KVNeed, LayerCache, Mixer, PartEnv, PositionEncoding, StepContext, StepPlan, StepShape, WeightDecl,
                   register_part)
from .linear import add_into_stream, can_fuse, linear, linear_into_stream, linear_of_norm


# Up to this many single new tokens a step, the attention kernel norms, rotates and writes the new keys itself.
# With more, its waves fill the chip and the extra work at each wave's start is no longer hidden behind the
# others' loads: the kernel of its own, which does it for all tokens at once, is then the faster way.
FUSED_DECODE_MAX_TOKENS = 64

DEFAULT_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                 "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "gate": "gate_proj.weight",
                 "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
                 "sink": "sinks"}
KERNEL_HEAD_SIZES = (32, 64, 96, 128, 256)      # what the matrix-core attention kernels take


def padded_head_size(*sizes: int) -> int:
    """The size heads are stored with in the cache: the smallest the matrix-core kernels take that holds
    every given size, or the largest given size (made even) where none does."""
    need = max(sizes)
    for size in KERNEL_HEAD_SIZES:
        if size >= need:
            return size
    return need + need % 2


def plan_attention_step(shape: StepShape) -> StepPlan:
    """How the attention kernels split a batch: the tokens of one-token entries (``decode_tokens``, longest
    context first: the short ones fill the tail of the launch), and tiles of up to ``ops.PREFILL_TILE``
    consecutive tokens (first token, count) of the longer entries by rising number of keys (``tiles``), with
    the numbers the launches are shaped by.  Padding entries of a captured batch are one-token entries."""
    dec, tiles, max_decode_kv, t0 = [], [], 0, 0
    for n, start in zip(shape.lens, shape.starts):
        if n == 1:
            dec.append((-start, t0))
            max_decode_kv = max(max_decode_kv, start + 1)
        else:
            for first in range(0, n, ops.PREFILL_TILE):
                count = min(ops.PREFILL_TILE, n - first)
                tiles.append((start + first + count, t0 + first, count))
        t0 += n
    tiles.sort()
    dec.sort()
    decode_tokens = [t for _, t in dec] + list(range(t0, t0 + shape.pad_entries))
    if shape.kv_bucket is not None:
        max_decode_kv = shape.kv_bucket                   # a captured launch: the split of the keys is fixed
    return StepPlan(
        arrays={"decode_tokens": np.asarray(decode_tokens, dtype=np.int32),
                "tiles": np.asarray([x for _, first, count in tiles for x in (first, count)], dtype=np.int32)},
        facts={"num_decode": len(decode_tokens), "max_decode_kv": max_decode_kv, "num_tiles": len(tiles),
               "tile_keys_total": sum(k for k, _, _ in tiles), "tile_keys_max": tiles[-1][0] if tiles else 0})


@register_part("mixer", "gqa_attention")
class GQAttention(Mixer):
    folds_norm = True
    hands_norm_ahead = True
    step_planners = {"attention": plan_attention_step}

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, prefix: str,
                 position: Optional[PositionEncoding] = None, qk_norm_eps: Optional[float] = None,
                 bias: bool = False, window: int = 0, scale: Optional[float] = None,
                 value_dim: Optional[int] = None, qk_norm: str = "head", head_gate: bool = False,
                 own_kv: bool = True, names: Optional[Dict[str, str]] = None, values: str = "own",
                 sink: bool = False, out_bias: bool = False, sink_value: Optional[float] = None,
                 qk_norm_gain: bool = True):
        if qk_norm not in ("head", "whole"):
            raise ValueError(f"qk_norm={qk_norm!r}: 'head' (per head) or 'whole' (over the whole projection)")
        if values not in ("own", "keys"):
            raise ValueError(f"values={values!r}: 'own' (a value projection) or 'keys' (the keys as projected)")
        self.dim, self.vdim = head_dim, head_dim if value_dim is None else int(value_dim)
        self.qk_norm, self.head_gate, self.own_kv = qk_norm, bool(head_gate), bool(own_kv)
        self.values_are_keys, self.sink, self.out_bias = values == "keys", bool(sink), bool(out_bias)
        self.sink_value = None if sink_value is None else float(sink_value)
        self.norm_has_gain = bool(qk_norm_gain)
        if self.sink and self.sink_value is not None:
            raise ValueError("a sink is a learned tensor (sink) or one constant (sink_value), not both")
        if not self.norm_has_gain and (qk_norm != "head" or qk_norm_eps is None):
            raise ValueError("a norm without gains is the per-head norm (qk_norm='head' with an eps)")
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.general = (self.vdim != head_dim or qk_norm == "whole" or self.head_gate or not self.own_kv
                        or names is not None or self.values_are_keys or self.sink or self.out_bias
                        or self.sink_value is not None or not self.norm_has_gain
                        or (position is not None and type(position).score_bias is not PositionEncoding.score_bias))
        if self.general:
            if self.values_are_keys and (self.vdim != head_dim or qk_norm == "whole" or not self.own_kv):
                raise ValueError("values that are the keys need keys of the layer's own, of the values' size, "
                                 "and no norm over the whole projection")
            head_dim = padded_head_size(head_dim, self.vdim)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim % 2 or head_dim > 512:
            raise ValueError(f"head_dim={head_dim} must be even and at most 512")
        self.hidden_size, self.nq, self.nkv, self.hd = hidden_size, num_heads, num_kv_heads, head_dim
        self.prefix = prefix
        self.position = position
        self.qk_norm_eps = qk_norm_eps          # None: no per-head norm
        self.bias = bias
        self.window = int(window)
        self.scale = float(scale) if scale is not None else self.dim ** -0.5   # qwen3.py:81
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = self.q_gain = self.k_gain = None
        self.sinks = self.sinks_log2 = None

    def children(self):
        return [self.position] if self.position is not None else []

    def cache_need(self):
        return KVNeed(self.nkv, self.hd, self.window)

    def weights(self) -> List[WeightDecl]:
        if self.general:
            return self._general_weights()
        p, H, hd = self.prefix, self.hidden_size, self.hd
        # q, k and v are used as one matrix with rows q | k | v, as the reference merges them
        # (ullm/layers/linear.py:381-389); the loader puts the three tensors into its rows
        rows = (("q", self.nq * hd, 0), ("k", self.nkv * hd, self.nq * hd), ("v", self.nkv * hd, (self.nq + self.nkv) * hd))
        out = [WeightDecl(f"{p}.{n}_proj.weight", (r, H), merged_into=f"{p}.qkv_proj.weight", row_offset=off)
               for n, r, off in rows]
        out.append(WeightDecl(f"{p}.o_proj.weight", (H, self.nq * hd)))
        if self.bias:   # qwen3.py:146 (attention_bias): on q, k, v only; o_proj never has one (qwen3.py:94)
            out += [WeightDecl(f"{p}.{n}_proj.bias", (r,), keep_fp32=True, merged_into=f"{p}.qkv_proj.bias", row_offset=off)
                    for n, r, off in rows]
        if self.qk_norm_eps is not None:
            out += [WeightDecl(f"{p}.q_norm.weight", (hd,), init="gain", keep_fp32=True),
                    WeightDecl(f"{p}.k_norm.weight", (hd,), init="gain", keep_fp32=True)]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        if self.general:
            return self._general_bind(tensors, env)
        p = self.prefix
        self.w_qkv = tensors[f"{p}.qkv_proj.weight"].contiguous()
        self.w_o = tensors[f"{p}.o_proj.weight"].contiguous()
        if self.bias:
            self.b_qkv = tensors[f"{p}.qkv_proj.bias"].contiguous()
        if self.qk_norm_eps is not None:
            self.q_gain = tensors[f"{p}.q_norm.weight"].contiguous()
            self.k_gain = tensors[f"{p}.k_norm.weight"].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if self.general:
            return self._general_forward(x, ctx, cache)
        return linear_into_stream(self._attend(linear(x, self.w_qkv, self.b_qkv), ctx, cache), self.w_o, ctx)

    def fusable(self, residual, ctx: StepContext) -> bool:
        if self.general:
            return False
        return can_fuse(residual, ctx.dtype, self.w_qkv, self.w_o)

    def forward_fused(self, x, residual, ctx: StepContext, cache: LayerCache, then=None):
        qkv = linear_of_norm(x, self.w_qkv, self.b_qkv)                               # the norm before folded in
        # the residual add, and the next norm's share of the work, folded behind
        return add_into_stream(self._attend(qkv, ctx, cache), self.w_o, residual, then, ctx.dtype)

    def _attend(self, qkv: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        """Per-head norm, rotation, cache write and attention for a fused projection [T, (nq+2nkv)*hd];
        returns the heads' outputs [T, nq*hd]."""
        T = qkv.shape[0]
        x = qkv
        group = ctx.groups[cache.group]
        table, rot, style = self.position.kernel_args() if self.position is not None else (None, 0, 0)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        plan = ctx.plans["attention"]
        work = plan.facts
        if (work["num_decode"] == T and not work["num_tiles"] and T <= FUSED_DECODE_MAX_TOKENS
                and ops.attention_decode_fused_supports(x.dtype, self.hd, group.page_size, self.nq, self.nkv, rot, style)):
            # a step of single new tokens: norm, rotation and cache write happen inside the attention kernel
            out = torch.empty((T, self.nq * self.hd), dtype=x.dtype, device=x.device)
            ops.attention_decode_fused(
                qkv, out, self.q_gain, self.k_gain, eps, table, rot, style, cache.k_pool, cache.v_pool,
                plan.arrays["decode_tokens"], work["num_decode"], ctx.positions, ctx.token_entry, group.block_table,
                group.page_size, self.nq, self.nkv, self.hd, self.scale, self.window, work["max_decode_kv"],
                write_kv=cache.owner)
            return out
        q = torch.empty((T, self.nq * self.hd), dtype=x.dtype, device=x.device)
        ops.qk_norm_rope_write(
            qkv, q, self.q_gain, self.k_gain, eps,
            table, rot, style, ctx.positions, ctx.token_entry, group.block_table,
            cache.k_pool, cache.v_pool, group.page_size, self.nq, self.nkv, self.hd, write_kv=cache.owner)
        return ops.paged_attention(q, cache.k_pool, cache.v_pool, ctx, group, self.nq, self.nkv, self.hd,
                                   self.scale, self.window, plan)

    # ------------------------------------------------------------------ the general path
    def _name(self, role: str) -> str:
        return f"{self.prefix}.{self.names[role]}"

    def _general_weights(self) -> List[WeightDecl]:
        H, nq, nkv, d, dv = self.hidden_size, self.nq, self.nkv, self.dim, self.vdim
        out = [WeightDecl(self._name("q"), (nq * d, H)), WeightDecl(self._name("o"), (H, nq * dv))]
        if self.own_kv:
            out.append(WeightDecl(self._name("k"), (nkv * d, H)))
            if not self.values_are_keys:
                out.append(WeightDecl(self._name("v"), (nkv * dv, H)))
        if self.bias:
            out.append(WeightDecl(self._name("q_bias"), (nq * d,), keep_fp32=True))
            if self.own_kv:
                out.append(WeightDecl(self._name("k_bias"), (nkv * d,), keep_fp32=True))
                if not self.values_are_keys:
                    out.append(WeightDecl(self._name("v_bias"), (nkv * dv,), keep_fp32=True))
        if self.out_bias:
            out.append(WeightDecl(self._name("o_bias"), (H,), keep_fp32=True))
        if self.sink:
            out.append(WeightDecl(self._name("sink"), (nq,), keep_fp32=True))
        if self.qk_norm_eps is not None and self.norm_has_gain:
            per = d if self.qk_norm == "head" else None
            out.append(WeightDecl(self._name("q_norm"), (per or nq * d,), init="gain", keep_fp32=True))
            if self.own_kv:
                out.append(WeightDecl(self._name("k_norm"), (per or nkv * d,), init="gain", keep_fp32=True))
        if self.head_gate:
            out.append(WeightDecl(self._name("gate"), (nq, H)))
        return out

    def _general_bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        """One input matrix with rows q | k | v | gate (a reader of another layer's cache: q | gate), every head
        padded with zero rows to the stored head size, the gate's rows to a multiple of eight; the output
        matrix with zero columns where the values are padded; gains padded alike."""
        H, nq, nkv, d, dv, hd = self.hidden_size, self.nq, self.nkv, self.dim, self.vdim, self.hd

        def heads_padded(t: torch.Tensor, heads: int, size: int) -> torch.Tensor:      # [heads*size, ...] -> [heads*hd, ...]
            if size == hd:
                return t
            out = torch.zeros((heads, hd) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
            out[:, :size] = t.view((heads, size) + tuple(t.shape[1:]))
            return out.view((heads * hd,) + tuple(t.shape[1:]))

        pieces = [heads_padded(tensors[self._name("q")], nq, d)]
        biases = [heads_padded(tensors[self._name("q_bias")], nq, d)] if self.bias else []
        self.q_off, self.k_off, self.v_off = 0, nq * hd, (nq + nkv) * hd
        if self.own_kv:
            pieces.append(heads_padded(tensors[self._name("k")], nkv, d))
            if self.bias:
                biases.append(heads_padded(tensors[self._name("k_bias")], nkv, d))
            if not self.values_are_keys:
                pieces.append(heads_padded(tensors[self._name("v")], nkv, dv))
                if self.bias:
                    biases.append(heads_padded(tensors[self._name("v_bias")], nkv, dv))
        self.gate_off = sum(p.shape[0] for p in pieces)
        if self.head_gate:
            gate = tensors[self._name("gate")]
            pieces.append(torch.cat((gate, gate.new_zeros((-nq % 8, H))), dim=0))
            if self.bias:
                biases.append(biases[0].new_zeros((pieces[-1].shape[0],)))
        self.w_qkv = torch.cat(pieces, dim=0).contiguous()
        self.b_qkv = torch.cat(biases, dim=0).contiguous() if self.bias else None
        self.b_o = tensors[self._name("o_bias")].contiguous() if self.out_bias else None
        if self.sink or self.sink_value is not None:
            self.sinks = (tensors[self._name("sink")].to(torch.float32).contiguous() if self.sink else
                          torch.full((nq,), self.sink_value, dtype=torch.float32, device=env.device))
            self.sinks_log2 = (self.sinks * math.log2(math.e)).contiguous()
        w_o = tensors[self._name("o")]
        if dv != hd:
            wide = w_o.new_zeros((H, nq, hd))
            wide[:, :, :dv] = w_o.view(H, nq, dv)
            w_o = wide.view(H, nq * hd)
        self.w_o = w_o.contiguous()
        if self.qk_norm_eps is not None:
            if self.qk_norm == "head":
                # a head's gains, padded like the head (the padded values are zeros whatever they are multiplied by)
                def head_gain(role):
                    g = (tensors[self._name(role)].to(torch.float32) if self.norm_has_gain
                         else torch.ones((d,), dtype=torch.float32, device=env.device))
                    return torch.cat((g, g.new_ones((hd - d,)))).contiguous()
                self.q_gain = head_gain("q_norm")
                self.k_gain = head_gain("k_norm") if self.own_kv else None
            else:
                self.q_gain = heads_padded(tensors[self._name("q_norm")], nq, d).contiguous()
                self.k_gain = heads_padded(tensors[self._name("k_norm")], nkv, d).contiguous() if self.own_kv else None

    def _general_forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if cache.owner != self.own_kv:
            raise RuntimeError(f"{self.prefix}: a layer " + ("with keys and values of its own must write its cache"
                               if self.own_kv else "without keys and values of its own cannot own a cache"))
        nq, nkv, hd = self.nq, self.nkv, self.hd
        T = x.shape[0]
        group = ctx.groups[cache.group]
        proj = linear(x, self.w_qkv, self.b_qkv)
        q = torch.empty((T, nq * hd), dtype=proj.dtype, device=proj.device)
        table, rot, style = self.position.kernel_args() if self.position is not None else (None, 0, 0)
        if self.qk_norm == "head" and self.own_kv:
            kv_heads = nkv if self.values_are_keys else 2 * nkv
            ops.qk_norm_rope_write(proj[:, :(nq + kv_heads) * hd], q, self.q_gain, self.k_gain, self.qk_norm_eps or 0.0,
                                   table, rot, style, ctx.positions, ctx.token_entry, group.block_table, cache.k_pool,
                                   cache.v_pool, group.page_size, nq, nkv, hd, write_kv=True,
                                   values_from_keys=self.values_are_keys, norm_dim=self.dim)
        else:
            if style != 0 and rot > 0 or (self.qk_norm == "head" and self.qk_norm_eps is not None):
                raise NotImplementedError("rotation or a per-head norm without keys of the layer's own: not built")
            ops.qk_whole_norm_write(proj, self.q_off, self.k_off, self.v_off, q, self.q_gain, self.k_gain,
                                    self.qk_norm_eps or 0.0, nq * self.dim, nkv * self.dim, ctx.positions,
                                    ctx.token_entry, group.block_table, cache.k_pool, cache.v_pool, group.page_size,
                                    nq, nkv, hd, has_kv=self.own_kv)
        bias = self.position.score_bias() if self.position is not None else None
        # the bias joins the scores and the gate the heads' outputs inside the attention kernels
        out = ops.paged_attention(q, cache.k_pool, cache.v_pool, ctx, group, nq, nkv, hd, self.scale, self.window,
                                  ctx.plans["attention"], bias=bias,
                                  bias_log2=self.position.score_bias_log2() if bias is not None else None,
                                  gate=proj[:, self.gate_off:] if self.head_gate else None,
                                  sink=self.sinks, sink_log2=self.sinks_log2)
        if self.b_o is not None:
            # the bias joins the 32-bit sums of the product, which stay 32-bit on their way to the stream
            return linear(out, self.w_o, self.b_o, out_dtype=torch.float32)
        return linear_into_stream(out, self.w_o, ctx)
