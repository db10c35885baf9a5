"""Pre-norm residual block: h += mixer(norm1(h)); h += ffn(norm2(h)).

The reference carries (branch output, residual) between layers and lets the next norm do the add
(ullm/models/qwen3.py:159-178, ullm/layers/layernorm.py:24-26).  The same trick is kept: a branch
output is left ``pending`` and added inside the next fused add+norm kernel, which saves one pass
over the residual stream per branch.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import (Block, FeedForward, LayerCache, Mixer, Norm, NormedBranch, PartEnv, PendingNorm, StepContext, StreamsBranch,
                   WeightDecl, register_part)


@register_part("block", "prenorm")
class PreNormBlock(Block):
    hands_norm_ahead = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def cache_need(self):
        return self.mixer.cache_need()

    def entry_norm(self):
        return self.mixer_norm

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache, next_norm: Optional[Norm] = None):
        # Each half: the norm kernel adds the pending branch into the stream and normalises; the
        # part then either adds its result into the stream itself (folded into its last kernel,
        # where it offers that for this batch) or returns it as the next pending branch.
        # Where nothing is left to add, a part that folds the norm into its first projection gets
        # the norm as a record instead of its result: then a half is two or three kernels.  A part
        # whose last kernel can also prepare the norm that follows is told which one that is, and
        # what it returns is the record for the part behind that norm.
        if self.mixer.fusable(residual, ctx):
            x = self._normed(self.mixer_norm, self.mixer, pending, residual, ctx)
            if self.mixer.hands_norm_ahead:
                pending = self.mixer.forward_fused(x, residual, ctx, cache, then=self.ffn_norm)
            else:
                pending = self.mixer.forward_fused(x, residual, ctx, cache)
        else:
            pending = self.mixer.forward(self._normed(self.mixer_norm, None, pending, residual, ctx), ctx, cache)
        if self.ffn.fusable(residual, ctx):
            x = self._normed(self.ffn_norm, self.ffn, pending, residual, ctx)
            if self.ffn.hands_norm_ahead:
                return residual, self.ffn.forward_fused(x, residual, ctx, then=next_norm)
            return residual, self.ffn.forward_fused(x, residual, ctx)
        return residual, self.ffn.forward(self._normed(self.ffn_norm, None, pending, residual, ctx), ctx)

    @staticmethod
    def _normed(norm: Norm, part, pending, residual, ctx: StepContext):
        """The input of the part behind ``norm``: the normed stream, or the norm as a record where nothing is
        left to add and ``part`` (None: a part that wants its input computed) folds it into its first product."""
        if isinstance(pending, PendingNorm):
            # the stream is complete and a product has prepared a norm: this one, by the way it was asked for
            if part is not None and part.folds_norm and pending.norm is norm:
                return pending
            pending = None
        if pending is None and part is not None and part.folds_norm:
            record = norm.pending(residual, ctx.dtype)
            if record is not None:
                return record
        return norm.add_norm(pending, residual, out_dtype=ctx.dtype)


@register_part("block", "sandwich")
class SandwichBlock(Block):
    """Norms on both sides of each sublayer and a multiplier on what joins the stream:
    h += mult * mixer_post(mixer(mixer_norm(h))); h += mult * ffn_post(ffn(ffn_norm(h))).  A block without a
    feed-forward (``ffn`` None) has the first sublayer only.  The norm behind a sublayer is not a kernel of
    its own: the branch is handed on as a :class:`NormedBranch`, and the next norm of the stream applies it,
    the multiplier, the add and itself in one pass."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, mixer_post: Norm, mult: float = 1.0,
                 ffn_norm: Optional[Norm] = None, ffn: Optional[FeedForward] = None, ffn_post: Optional[Norm] = None):
        if (ffn is None) != (ffn_norm is None) or (ffn is None) != (ffn_post is None):
            raise ValueError("a feed-forward comes with the norms on both of its sides, or not at all")
        self.mixer_norm, self.mixer, self.mixer_post = mixer_norm, mixer, mixer_post
        self.ffn_norm, self.ffn, self.ffn_post = ffn_norm, ffn, ffn_post
        self.mult = float(mult)

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post)
                if p is not None]

    def cache_need(self):
        return self.mixer.cache_need()

    def entry_norm(self):
        return self.mixer_norm

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache):
        if isinstance(pending, PendingNorm):
            pending = None                               # the stream is complete; this block norms it itself
        x = self.mixer_norm.add_norm(pending, residual, out_dtype=ctx.dtype)
        pending = NormedBranch(_one_branch(self.mixer.forward(x, ctx, cache)), self.mixer_post, self.mult)
        if self.ffn is None:
            return residual, pending
        x = self.ffn_norm.add_norm(pending, residual, out_dtype=ctx.dtype)
        return residual, NormedBranch(_one_branch(self.ffn.forward(x, ctx)), self.ffn_post, self.mult)


def _one_branch(y):
    """A stack of partial sums [S, T, hidden] added up: a norm behind the branch needs the whole rows."""
    return ops.branch_sum(y) if y.dim() == 3 else y


@register_part("block", "parallel")
class ParallelBlock(Block):
    """One norm whose output both sublayers read, and a multiplier on their sum:
    h = norm(x); x += mult * (mixer(h) + ffn(h)).  A block without a feed-forward (``ffn`` None) adds the mixer
    alone.  The sum of the two branches is 32-bit and travels on as the pending branch; the next norm of the
    stream multiplies, adds and norms in one pass.  A feed-forward that offers ``forward_onto(x, ctx, base)`` adds
    its result onto the mixer's in its own last kernel."""

    def __init__(self, norm: Norm, mixer: Mixer, ffn: Optional[FeedForward] = None, mult: float = 1.0):
        self.norm, self.mixer, self.ffn, self.mult = norm, mixer, ffn, float(mult)

    def children(self):
        return [p for p in (self.norm, self.mixer, self.ffn) if p is not None]

    def cache_need(self):
        return self.mixer.cache_need()

    def entry_norm(self):
        return self.norm

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache):
        if isinstance(pending, PendingNorm):
            pending = None                               # the stream is complete; this block norms it itself
        h = self.norm.add_norm(pending, residual, out_dtype=ctx.dtype)
        mixed = self.mixer.forward(h, ctx, cache)
        if self.ffn is None:
            return residual, NormedBranch(_one_branch(mixed), None, self.mult)
        if hasattr(self.ffn, "forward_onto"):
            return residual, NormedBranch(self.ffn.forward_onto(h, ctx, _one_branch(mixed)), None, self.mult)
        # one kernel adds the two branches, whichever of them are stacks of partial sums
        return residual, NormedBranch(ops.branch_sum(mixed, self.ffn.forward(h, ctx)), None, self.mult)


@register_part("block", "mix_in_embedding")
class MixInEmbedding(Block):
    """Not a layer of sublayers but a step between layers: the stream is replaced by a product of itself and the
    embedding output side by side, x <- W [x ; e] with W [hidden, 2 hidden] (the stream's columns first).  A model
    that passes a run of layers several times puts it ahead of every pass.  It keeps nothing between steps.  The
    model hands every block the embedding output as ``ctx.embedded`` if one of its blocks says ``needs_embedding``.
    What is pending joins the stream in the kernel that lays the two rows side by side; the product's 32-bit
    sums are the new stream."""
    needs_embedding = True

    def __init__(self, hidden_size: int, weight_name: str):
        self.hidden_size, self.weight_name = int(hidden_size), weight_name
        self.w: Optional[torch.Tensor] = None

    def weights(self):
        from .base import WeightDecl
        return [WeightDecl(self.weight_name, (self.hidden_size, 2 * self.hidden_size))]

    def bind(self, tensors, env) -> None:
        self.w = tensors[self.weight_name].contiguous()

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache):
        from .linear import linear
        if ctx.embedded is None:
            raise RuntimeError("mix_in_embedding: the model did not keep the embedding output")
        branch, mult = None, 1.0
        if isinstance(pending, NormedBranch):
            if pending.post is not None:
                # a norm stands behind the branch: the general add kernel applies it; no norm of the stream is asked for
                ops.add_norm_general(pending.branch, residual, None, 0.0, ops.NORM_RMS, None,
                                     post_gain=pending.post.kernel_form()[0], post_eps=pending.post.kernel_form()[1],
                                     post_kind=pending.post.kernel_form()[2], mult=pending.mult)
            else:
                branch, mult = _one_branch(pending.branch), pending.mult
        elif pending is not None and not isinstance(pending, PendingNorm):
            branch = _one_branch(pending)
        both = ops.stream_pair(branch, mult, residual, ctx.embedded, ctx.dtype)
        return linear(both, self.w, out_dtype=torch.float32), None


@register_part("block", "hyper_prenorm")
class HyperPreNormBlock(Block):
    """A pre-norm block of a model that keeps ``streams`` copies x_1 .. x_S of its residual stream (float32
    [S, T, hidden], all equal to the embedding output at the start; the model sums them at the end).  Sublayer q
    (the mixer, then the feed-forward if there is one) reads u = sum_s in_q[s] x_s, computes y = sublayer(norm_q(u)),
    and then every copy at once, from the old ones, becomes x_t <- sum_s mix_q[s, t] x_s + mult * out_q[t] * y.
    Per sublayer three small tensors: ``in`` [S], ``out`` [S], ``mix`` [S, S] (indexed [from, to]), under
    ``<prefix>.<names[0]>`` and ``<prefix>.<names[1]>``.  With one copy and no such tensors in the checkpoint they are
    ones: the plain pre-norm block with a multiplier.

    The write-back of a sublayer and the read and norm of the next are one kernel (``ops.streams_step``): what a
    sublayer returns travels on as a :class:`StreamsBranch` and is settled by whoever norms the streams next, the
    next block of this kind or the model's last norm."""

    def __init__(self, hidden_size: int, streams: int, mixer_norm: Norm, mixer: Mixer, prefix: str, mult: float = 1.0,
                 ffn_norm: Optional[Norm] = None, ffn: Optional[FeedForward] = None, names=("hc1", "hc2")):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward comes with its norm, or not at all")
        if not 1 <= streams <= ops.STREAMS_MAX:
            raise ValueError(f"{streams} copies of the stream: 1 to {ops.STREAMS_MAX}")
        for norm in (mixer_norm, ffn_norm):
            if norm is not None and type(norm).kernel_form is Norm.kernel_form:
                raise TypeError(f"{type(norm).__name__} has no kernel form: it cannot norm a mix of streams")
        self.hidden_size, self.streams, self.mult, self.prefix, self.names = hidden_size, int(streams), float(mult), prefix, tuple(names)
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.coeffs = []                                  # per sublayer (in, out, mix)

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def cache_need(self):
        return self.mixer.cache_need()

    def entry_norm(self):
        return self.mixer_norm

    def _sublayers(self):
        return self.names[:1] if self.ffn is None else self.names[:2]

    def weights(self):
        S = self.streams
        fill = 1.0 if S == 1 else None                    # one copy: a checkpoint may leave the coefficients out
        out = []
        for name in self._sublayers():
            p = f"{self.prefix}.{name}"
            out += [WeightDecl(f"{p}.in", (S,), init="gain", keep_fp32=True, default=fill),
                    WeightDecl(f"{p}.out", (S,), init="gain", keep_fp32=True, default=fill),
                    WeightDecl(f"{p}.mix", (S, S), init="gain", keep_fp32=True, default=fill)]
        return out

    def bind(self, tensors, env: PartEnv) -> None:
        self.coeffs = [tuple(tensors[f"{self.prefix}.{name}.{k}"].contiguous() for k in ("in", "out", "mix"))
                       for name in self._sublayers()]

    def _read(self, streams, pending, norm: Norm, in_w, ctx: StepContext):
        """Settle what is pending and return the norm of the mix the next sublayer reads."""
        gain, eps, kind = norm.kernel_form()
        if pending is None or isinstance(pending, PendingNorm):
            return ops.streams_step(streams, in_w=in_w, gain=gain, eps=eps, kind=kind, out_dtype=ctx.dtype)
        if not isinstance(pending, StreamsBranch):
            raise TypeError("a block over several streams takes what a block of its kind left pending")
        return ops.streams_step(streams, pending.branch, pending.mix, pending.out_w, pending.mult, in_w, gain, eps, kind,
                                ctx.dtype, second=pending.second, a=pending.a, b=pending.b)

    def _branch(self, y, coeffs) -> "StreamsBranch":
        _, out_w, mix = coeffs
        if isinstance(y, tuple):                          # two weighted branches, added where the streams are written
            first, a, second, b = y
            if first.dtype == second.dtype:
                return StreamsBranch(first, mix, out_w, self.mult, second, a, b)
            y = ops.weighted_sum(first, second, a, b)
        return StreamsBranch(_one_branch(y), mix, out_w, self.mult)

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache):
        if residual.dim() != 3 or residual.shape[0] != self.streams:
            raise RuntimeError(f"{self.prefix}: the model does not carry {self.streams} copies of its stream")
        x = self._read(residual, pending, self.mixer_norm, self.coeffs[0][0], ctx)
        if hasattr(self.mixer, "forward_pair"):
            y = self.mixer.forward_pair(x, ctx, cache)
        else:
            y = self.mixer.forward(x, ctx, cache)
        pending = self._branch(y, self.coeffs[0])
        if self.ffn is None:
            return residual, pending
        x = self._read(residual, pending, self.ffn_norm, self.coeffs[1][0], ctx)
        return residual, self._branch(self.ffn.forward(x, ctx), self.coeffs[1])


def join_streams(streams, pending, norm: Norm, rows, out_dtype):
    """The last norm of a model over several copies of its stream: what is pending is settled, the copies are added
    and the sum is normed, for the tokens ``rows`` lists only (nothing is written back)."""
    form = norm.kernel_form()
    if form is None:
        raise TypeError(f"{type(norm).__name__} has no kernel form: it cannot norm a sum of streams")
    gain, eps, kind = form
    ones = torch.ones((streams.shape[0],), dtype=torch.float32, device=streams.device)
    if isinstance(pending, StreamsBranch):
        return ops.streams_step(streams, pending.branch, pending.mix, pending.out_w, pending.mult, ones, gain, eps, kind,
                                out_dtype, rows=rows, second=pending.second, a=pending.a, b=pending.b)
    return ops.streams_step(streams, in_w=ones, gain=gain, eps=eps, kind=kind, out_dtype=out_dtype, rows=rows)
