"""Latent attention as a mixer: queries and keys/values that go through small latents, over the paged cache.

With h the mixer's input:  c_q = rmsnorm(W_dq h) * g_q,  q = W_uq c_q, laid out per head as ``dim`` plain dims and
then ``rot_dim`` dims that are turned by the position;  W_dkv h = [kv latent | one rotated key part for all heads],
c = rmsnorm(kv latent) * g_kv;  per head the plain key is W_uk[h] c and the value W_uv[h] c;  score =
(q_plain . k_plain + q_rot . k_rot) * scale over the keys up to the token itself, softmax, a head's output times the
sigmoid of its gate (one more projection of h), then W_o.

Only c and the rotated key part are kept per token: since q_plain[h] . (W_uk[h] c) = (W_uk[h]^T q_plain[h]) . c, the
layer runs as grouped-query attention with ONE key/value head whose key row is [c | k_rot] and whose value row is c;
the queries are [W_uk[h]^T q_plain[h] | q_rot[h]] and a head's output  sum_j p_j c_j  goes through W_uv[h].  Prompt
portions and single tokens take the same path, whatever is in the cache.  The cache group is the paged one of any
attention layer (one head of size kv_rank + rot_dim, padded to a size the matrix-core kernels take), with the
normed latent stored a second time as the value pool in those kernels' transposed layout.

The position part is any rotation by a table (:class:`~ullm_amd.parts.position.Rotary`, half-split pairs over all
``rot_dim`` dims); sizes, scale, eps and tensor names are parameters.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .attention import padded_head_size, plan_attention_step
from .base import KVNeed, LayerCache, Mixer, PartEnv, PositionEncoding, StepContext, WeightDecl, register_part
from .linear import linear, linear_into_stream

DEFAULT_NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
                 "uv": "uv", "gate": "g", "o": "o"}


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    step_planners = {"attention": plan_attention_step}

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int,
                 kv_rank: int, scale: float, norm_eps: float, prefix: str, position: Optional[PositionEncoding] = None,
                 head_gate: bool = True, names: Optional[Dict[str, str]] = None):
        if rot_dim % 2 or rot_dim < 0 or head_dim < 1:
            raise ValueError(f"{head_dim} plain and {rot_dim} rotated dims: the rotated dims come in pairs, and a head has plain dims")
        if (rot_dim > 0) != (position is not None):
            raise ValueError("rotated dims need a position part, and a position part rotated dims")
        self.hidden_size, self.nq, self.dim, self.rot, self.vdim = hidden_size, num_heads, head_dim, rot_dim, value_dim
        self.q_rank, self.kv_rank, self.scale, self.eps = q_rank, kv_rank, float(scale), float(norm_eps)
        self.hd = padded_head_size(kv_rank + rot_dim)        # the size of the one cached head
        if self.hd > 1024:
            raise ValueError(f"a latent of {kv_rank} and {rot_dim} rotated dims: the cached head is at most 1024")
        self.prefix, self.position, self.head_gate = prefix, position, bool(head_gate)
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_down = self.w_uq = self.w_uk = self.w_uvT = self.w_o = self.q_gain = self.kv_gain = None

    def children(self):
        return [self.position] if self.position is not None else []

    def cache_need(self):
        return KVNeed(1, self.hd, 0)

    def _name(self, role: str) -> str:
        return f"{self.prefix}.{self.names[role]}"

    def weights(self) -> List[WeightDecl]:
        H, nq, d, r, dv, qr, kr = self.hidden_size, self.nq, self.dim, self.rot, self.vdim, self.q_rank, self.kv_rank
        merged = f"{self.prefix}.down"                    # rows: q latent | kv latent and rotated key part | gates
        out = [WeightDecl(self._name("dq"), (qr, H), merged_into=merged, row_offset=0),
               WeightDecl(self._name("dkv"), (kr + r, H), merged_into=merged, row_offset=qr)]
        if self.head_gate:
            out.append(WeightDecl(self._name("gate"), (nq, H), merged_into=merged, row_offset=qr + kr + r))
        out += [WeightDecl(self._name("dq_norm"), (qr,), init="gain", keep_fp32=True),
                WeightDecl(self._name("dkv_norm"), (kr,), init="gain", keep_fp32=True),
                WeightDecl(self._name("uq"), (nq * (d + r), qr)), WeightDecl(self._name("uk"), (nq * d, kr)),
                WeightDecl(self._name("uv"), (nq * dv, kr)), WeightDecl(self._name("o"), (H, nq * dv))]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        nq, d, dv, kr = self.nq, self.dim, self.vdim, self.kv_rank
        self.w_down = tensors[f"{self.prefix}.down"].contiguous()
        self.w_uq = tensors[self._name("uq")].contiguous()
        # a matrix per head, stored [heads, inputs, outputs]: W_uk[h] as it is takes the plain query dims to the
        # latent (q' = W_uk[h]^T q_plain), W_uv[h] transposed takes a latent to the head's values
        self.w_uk = tensors[self._name("uk")].contiguous().view(nq, d, kr)
        self.w_uvT = tensors[self._name("uv")].view(nq, dv, kr).transpose(1, 2).contiguous()
        self.w_o = tensors[self._name("o")].contiguous()
        self.q_gain = tensors[self._name("dq_norm")].contiguous()
        self.kv_gain = tensors[self._name("dkv_norm")].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        nq, d, r, kr, hd = self.nq, self.dim, self.rot, self.kv_rank, self.hd
        T = x.shape[0]
        group = ctx.groups[cache.group]
        table = self.position.kernel_args()[0] if self.position is not None else None
        # the latents, the rotated key part and the gates in one product whose 32-bit sums the norms read
        proj = linear(x, self.w_down, out_dtype=torch.float32)
        cq, gate = ops.latent_prepare(
            proj, 0, self.q_rank, self.q_rank, kr, self.q_rank + kr, r, self.q_rank + kr + r, nq if self.head_gate else 0,
            self.q_gain, self.kv_gain, self.eps, table, ctx.positions, ctx.token_entry, group.block_table,
            cache.k_pool, cache.v_pool, group.page_size, hd, cache.owner, ctx.dtype)
        q = linear(cq, self.w_uq)                                                   # [T, nq * (d + r)]
        into_latent = ops.head_linear(q.view(T, nq, d + r)[:, :, :d], self.w_uk)    # [T, nq, kr]
        queries = ops.latent_query(into_latent, q, d, r, hd, table, ctx.positions)  # [T, nq * hd]
        out = ops.paged_attention(queries, cache.k_pool, cache.v_pool, ctx, group, nq, 1, hd, self.scale, 0,
                                  ctx.plans["attention"], gate=gate)
        values = torch.empty((T, nq, self.vdim), dtype=out.dtype, device=out.device)
        ops.head_linear(out.view(T, nq, hd)[:, :, :kr], self.w_uvT, out=values)     # [T, nq, dv]
        return linear_into_stream(values.view(T, nq * self.vdim), self.w_o, ctx)
