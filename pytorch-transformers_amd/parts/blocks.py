"""How norm, mixer and feed-forward stand in a block, and how the residual is summed.

The two arrangements of ``FalconDecoderLayer.forward``
(src/transformers/models/falcon/modeling_falcon.py:614-683):

parallel    ``x + (ffn(norm_ffn(x)) + mixer(norm_mixer(x)))``; with one norm both branches read
            the same normed input (:630-634, :648-676).  The sum is formed in that order:
            feed-forward plus mixer first (:673-674), then the residual (:676).
sequential  ``r = x + mixer(norm_in(x))``; ``r + ffn(norm_post(r))`` (:652-659, :676).

The additions ride in the last matrix product's epilogue of each branch, or, in steps of few tokens,
the products stay unreduced and the next norm forms the sum while it reads it (``ResidualSum``).
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..engine.spec import INIT_ZERO_NOISE, VECTOR, TensorSpec
from .base import Part, PendingNormSum, ResidualSum, StepContext, WideResidual, WideSum, as_tensor, register_part
from .linear import Linear, PendingProjection


def _can_defer(part: Part) -> bool:
    return bool(getattr(part, "can_defer", False))


def _normed(x, norm: Part, other: Optional[Part] = None):
    """``(x as a tensor, norm(x), other(x) or None)`` for a block input that may be a sum not formed yet."""
    if isinstance(x, ResidualSum):
        if hasattr(norm, "forward_sum"):
            return norm.forward_sum(x, other=other)
        x = x.tensor()
    if other is None:
        return x, norm.forward(x), None
    if hasattr(norm, "forward_pair"):  # two norms of one input in one pass, where the norm offers it
        a, m = norm.forward_pair(x, other)
    else:
        a, m = norm.forward(x), other.forward(x)
    return x, a, m


def _sum_parallel(ffn_out: PendingProjection, mixer_out: PendingProjection, x: torch.Tensor):
    """feed-forward + mixer + residual, in that order, formed now or left to the next norm."""
    both = PendingProjection.partial_pair(ffn_out, mixer_out)
    if both is not None:
        return ResidualSum([both[0], both[1], x])
    p = ffn_out.partial()
    if p is not None:
        return ResidualSum([p, mixer_out.partial() or mixer_out.run(), x])
    if ffn_out.additions_cost_a_pass():  # prompts: the next norm adds the three while it reads them
        return ResidualSum([ffn_out.run(), mixer_out.run(), x])
    return ffn_out.run(add1=mixer_out.run(), add2=x)


def _sum_sequential(out: PendingProjection, residual: torch.Tensor):
    p = out.partial()
    if p is not None:
        return ResidualSum([p, residual])
    if out.additions_cost_a_pass():
        return ResidualSum([out.run(), residual])
    return out.run(add1=residual)


class ParallelBlock(Part):
    accepts_sum = True

    def __init__(self, mixer: Part, feed_forward: Part, norm_mixer: Part, norm_ffn: Optional[Part] = None):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_mixer = norm_mixer
        self.norm_ffn = norm_ffn

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.norm_mixer, self.norm_ffn, self.mixer, self.feed_forward) if p is not None)

    def after_load(self) -> None:
        """With one norm both branches start from the same input: their first matrices are laid out side by
        side, so that prompts can run them as one product."""
        if self.norm_ffn is None and hasattr(self.mixer, "input_projection") and hasattr(self.feed_forward, "input_projection"):
            Linear.join(self.mixer.input_projection()[0], self.feed_forward.input_projection()[0])

    def forward(self, x, ctx: StepContext, call):
        x, a, m = _normed(x, self.norm_mixer, self.norm_ffn)
        if m is None:
            m = a
        kw_mixer, kw_ffn = {}, {}
        # both branches start with a product of the norm's output: one launch for the two in small steps
        if hasattr(self.mixer, "input_projection") and hasattr(self.feed_forward, "input_projection"):
            (lin_a, kw_a), (lin_m, kw_m) = self.mixer.input_projection(), self.feed_forward.input_projection()
            tail = self.mixer.projection_tail(ctx, call) if hasattr(self.mixer, "projection_tail") else None
            both = Linear.pair(lin_a, a, kw_a, lin_m, m, kw_m, tail=tail)
            if both is not None:
                kw_mixer["projected"], kw_ffn["projected"] = both
        if _can_defer(self.feed_forward) and _can_defer(self.mixer):
            # the branches' last products: one launch of partial sums where that pays, which the
            # next norm adds to the residual while it reads them
            out_a = self.mixer.forward(a, ctx, call, defer=True, **kw_mixer)
            out_m = self.feed_forward.forward(m, ctx, defer=True, **kw_ffn)
            return _sum_parallel(out_m, out_a, x)
        mixed = self.mixer.forward(a, ctx, call, **kw_mixer)
        return self.feed_forward.forward(m, ctx, add1=mixed, add2=x, **kw_ffn)


class SequentialBlock(Part):
    accepts_sum = True

    def __init__(self, mixer: Part, feed_forward: Part, norm_in: Part, norm_post: Part):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in = norm_in
        self.norm_post = norm_post

    def children(self) -> Sequence[Part]:
        return (self.norm_in, self.norm_post, self.mixer, self.feed_forward)

    def forward(self, x, ctx: StepContext, call):
        x, a, _ = _normed(x, self.norm_in)
        if _can_defer(self.mixer):
            r = _sum_sequential(self.mixer.forward(a, ctx, call, defer=True), x)
        else:
            r = self.mixer.forward(a, ctx, call, residual=x)
        r, m, _ = _normed(r, self.norm_post)
        if _can_defer(self.feed_forward):
            return _sum_sequential(self.feed_forward.forward(m, ctx, defer=True), r)
        return self.feed_forward.forward(m, ctx, add1=r)


class PostNormBlock(Part):
    """``x <- x + m * norm_mixer(mixer(x))``, then ``x <- x + m * norm_ffn(ffn(x))``: the sublayers read the stream
    itself and the norm stands on each sublayer's output; ``m`` is a constant.  The stream is kept in 32-bit
    whatever the compute type (``WideResidual``): a sublayer reads its copy in the compute type, the norm, the
    scaling and the addition are one 32-bit launch that also writes that copy for the next sublayer.
    ``feed_forward`` may be None (a layer of the mixer alone).  With ``depth_mix`` (``parts.depth.DepthMix``) the
    block's result is kept as the next of the step's streams and what goes on is their weighted sum.  ``hand_on_unformed``
    (for a model's last block, with LayerNorms): the last sublayer's output goes on not yet normed and added
    (``PendingNormSum``), and the final norm's launch does both on its way, for the rows whose logits are wanted alone."""

    accepts_sum = False
    accepts_wide = True

    def __init__(self, mixer: Part, feed_forward: Optional[Part], norm_mixer: Part, norm_ffn: Optional[Part],
                 residual_mult: float = 1.0, depth_mix: Optional[Part] = None, hand_on_unformed: bool = False):
        if (feed_forward is None) != (norm_ffn is None):
            raise ValueError("a feed-forward and its norm come together or not at all")
        self.mixer, self.feed_forward, self.norm_mixer, self.norm_ffn = mixer, feed_forward, norm_mixer, norm_ffn
        self.residual_mult = float(residual_mult)
        self.depth_mix = depth_mix
        last_norm = norm_mixer if norm_ffn is None else norm_ffn
        self.hand_on_unformed = bool(hand_on_unformed) and depth_mix is None and hasattr(last_norm, "affine")

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.norm_mixer, self.norm_ffn, self.mixer, self.feed_forward, self.depth_mix)
                     if p is not None)

    def after_load(self) -> None:
        for part in (self.mixer, self.feed_forward):
            if part is not None and hasattr(part, "after_load"):
                part.after_load()

    def _enter(self, x, ctx: StepContext) -> WideResidual:
        """The stream as this block wants it; the first block of a model is given the embedding's plain tensor."""
        from .. import ops

        if isinstance(x, WideResidual):
            return x
        x = as_tensor(x)
        history = None
        if self.depth_mix is not None:
            history = self.depth_mix.new_history(x.shape[0], x.shape[1], x.device)
            wide = ops.widen(x, history.next_plane())
        else:
            wide = x if x.dtype == torch.float32 else ops.widen(x)
        return WideResidual(wide, x if x.dtype == ctx.dtype else wide, history)

    def forward(self, x, ctx: StepContext, call):
        x = self._enter(x, ctx)
        last = self.feed_forward is None
        history = x.history
        keep = history.next_plane() if (history is not None and self.depth_mix is not None) else None
        # the launch that forms the block's result also keeps it as a stream and goes on to the streams' weighted sum
        mix = self.depth_mix.fused(history) if keep is not None else None
        mixed = self.mixer.forward(x.narrow, ctx, call)
        if last and self.hand_on_unformed:
            return PendingNormSum(x.wide, mixed, self.norm_mixer.affine(), self.residual_mult, self.norm_mixer.eps, ctx.dtype)
        narrow, wide = self.norm_mixer.apply(mixed, ctx.dtype, residual=x.wide, mult=self.residual_mult, want_wide=True,
                                             out_wide=keep if last else None, mix=mix if last else None)
        if not last:
            out = self.feed_forward.forward(narrow, ctx)
            if self.hand_on_unformed:
                return PendingNormSum(wide, out, self.norm_ffn.affine(), self.residual_mult, self.norm_ffn.eps, ctx.dtype)
            narrow, wide = self.norm_ffn.apply(out, ctx.dtype, residual=wide, mult=self.residual_mult, want_wide=True,
                                               out_wide=keep, mix=mix)
        return WideResidual(wide, narrow, history)


class ShiftedParallelBlock(Part):
    """``x <- x + (mixer(shift(norm_mixer(x))) + ffn(norm_ffn(x)))`` over a stream kept in 32-bit: both branches read
    norms of the same x.  ``shift``: what the mixer reads, ``h = norm_mixer(x)``, is replaced by ``h + (h' - h) * mu``
    with h' the h of the token before (zeros at a sequence's first token) and ``mu`` a learned vector (``shift_name``
    in the file).  The h of a sequence's last token is part of its state: a row of the state table that the run
    order's entry names as ``also("shift")``.  ``feed_forward`` may be None (a layer of the mixer alone).

    The block hands on ``x`` and its branches' results as a sum that is not formed (``WideSum``); the next block's
    first launch forms it, norms it twice and shifts (``ops.shift_norm``)."""

    accepts_sum = False
    accepts_wide = True

    def __init__(self, mixer: Part, feed_forward: Optional[Part], norm_mixer: Part, norm_ffn: Optional[Part],
                 shift_name: str, hidden_size: int):
        if (feed_forward is None) != (norm_ffn is None):
            raise ValueError("a feed-forward and its norm come together or not at all")
        if getattr(norm_mixer, "offset", 0.0) or getattr(norm_mixer, "groups", 1) != 1 or (
                norm_ffn is not None and (norm_ffn.offset or norm_ffn.groups != 1 or norm_ffn.eps != norm_mixer.eps)):
            raise ValueError("the shifted block's launch takes plain RMS norms with one eps")
        self.mixer, self.feed_forward, self.norm_mixer, self.norm_ffn = mixer, feed_forward, norm_mixer, norm_ffn
        self.shift_name, self.hidden_size = shift_name, int(hidden_size)
        self.mu: Optional[torch.Tensor] = None

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.norm_mixer, self.norm_ffn, self.mixer, self.feed_forward) if p is not None)

    def tensor_specs(self):
        return [TensorSpec(self.shift_name, (self.hidden_size,), VECTOR, INIT_ZERO_NOISE)]

    def load(self, tensors) -> None:
        self.mu = tensors[self.shift_name]

    def after_load(self) -> None:
        for part in (self.mixer, self.feed_forward):
            if part is not None and hasattr(part, "after_load"):
                part.after_load()

    def forward(self, x, ctx: StepContext, call):
        from .. import ops

        if isinstance(x, WideSum):
            base, terms = x.base, x.terms
        elif isinstance(x, WideResidual):
            base, terms = x.wide, []
        else:
            x = as_tensor(x)
            base, terms = (x if x.dtype == torch.float32 else ops.widen(x)), []
        group, layer = call.also("shift")
        state = ctx.cache.state_layer(group, layer)
        stream, a, m = ops.shift_norm(base, terms, self.norm_mixer.weight, None if self.norm_ffn is None else self.norm_ffn.weight,
                                      self.mu, self.norm_mixer.eps, state, ctx, ctx.dtype)
        kw_mixer, kw_ffn = {}, {}
        # both branches start with a product of a norm of x: one launch for the two in small steps
        if hasattr(self.mixer, "input_projection") and hasattr(self.feed_forward, "input_projection"):
            (lin_a, kw_a), (lin_m, kw_m) = self.mixer.input_projection(), self.feed_forward.input_projection()
            both = Linear.pair(lin_a, a, kw_a, lin_m, m, kw_m) if lin_a is not None and lin_m is not None else None
            if both is not None:
                kw_mixer["projected"], kw_ffn["projected"] = both
        mixed = self.mixer.forward(a, ctx, call, **kw_mixer)
        ff = self.feed_forward.forward(m, ctx, **kw_ffn) if self.feed_forward is not None else None
        return WideSum(stream, [mixed, ff], ctx.dtype)


class SandwichBlock(Part):
    """A norm in front of and behind each sublayer, over a stream kept in 32-bit:

        x <- x + m * norm_mixer_out(mixer(norm_mixer(x)));   x <- x + m * norm_ffn_out(ffn(norm_ffn(x)))

    with ``m`` a constant and the four norms LayerNorms with weight and bias and one eps (``ops.layernorm_stream``: the
    norm behind a sublayer, the addition and the norm in front of the next sublayer are one launch, across the
    block's end too: the block hands its last sublayer on not yet added, ``PendingNormSum``).  ``feed_forward`` may be
    None (a layer of the mixer alone).  ``loop_entry`` (``parts.depth.LoopEntry``): where the run order's entry says
    that a pass of a loop starts with this block (``call.loop_pass``), the terms that the loop adds to the stream in
    front of the pass ride in the block's first launch."""

    accepts_sum = False
    accepts_wide = True

    def __init__(self, mixer: Part, feed_forward: Optional[Part], norm_mixer: Part, norm_mixer_out: Part,
                 norm_ffn: Optional[Part], norm_ffn_out: Optional[Part], residual_mult: float = 1.0,
                 loop_entry: Optional[Part] = None):
        if not ((feed_forward is None) == (norm_ffn is None) == (norm_ffn_out is None)):
            raise ValueError("a feed-forward and its two norms come together or not at all")
        norms = [n for n in (norm_mixer, norm_mixer_out, norm_ffn, norm_ffn_out) if n is not None]
        if any(not hasattr(n, "affine") for n in norms) or len({n.eps for n in norms}) != 1:
            raise ValueError("the block's launches take LayerNorms with weight and bias and one eps")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.norm_mixer, self.norm_mixer_out, self.norm_ffn, self.norm_ffn_out = norm_mixer, norm_mixer_out, norm_ffn, norm_ffn_out
        self.residual_mult, self.eps = float(residual_mult), norm_mixer.eps
        self.loop_entry = loop_entry

    def children(self) -> Sequence[Part]:
        return tuple(p for p in (self.norm_mixer, self.norm_mixer_out, self.norm_ffn, self.norm_ffn_out, self.mixer,
                                 self.feed_forward, self.loop_entry) if p is not None)

    def after_load(self) -> None:
        for part in (self.mixer, self.feed_forward):
            if part is not None and hasattr(part, "after_load"):
                part.after_load()

    def forward(self, x, ctx: StepContext, call):
        from .. import ops

        dtype, eps, m = ctx.dtype, self.eps, self.residual_mult
        if isinstance(x, PendingNormSum) and not x.formed and x.eps == eps:
            terms = x.launch_terms()
        elif isinstance(x, WideResidual):
            terms = {"x": x.wide}
        else:
            x = as_tensor(x)
            terms = {"x": x if x.dtype == torch.float32 else ops.widen(x)}
        if self.loop_entry is not None and getattr(call, "loop_pass", None) is not None:
            add, vec = self.loop_entry.terms(call.loop_pass, ctx)
            terms.update(add=add, vec=vec)
        changed = len(terms) > 1  # the launch forms a stream that is not in memory yet
        h, wide = ops.layernorm_stream(dtype, pre=self.norm_mixer.affine(), eps=eps, want_wide=changed, **terms)
        if not changed:
            wide = terms["x"]
        mixed = self.mixer.forward(h, ctx, call)
        if self.feed_forward is None:
            return PendingNormSum(wide, mixed, self.norm_mixer_out.affine(), m, eps, dtype)
        h, wide = ops.layernorm_stream(dtype, x=wide, y=mixed, post=self.norm_mixer_out.affine(), mult=m,
                                       pre=self.norm_ffn.affine(), eps=eps)
        out = self.feed_forward.forward(h, ctx)
        return PendingNormSum(wide, out, self.norm_ffn_out.affine(), m, eps, dtype)


register_part("block", "sandwich", SandwichBlock)
register_part("block", "shifted_parallel", ShiftedParallelBlock)
register_part("block", "post_norm", PostNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "sequential", SequentialBlock)
