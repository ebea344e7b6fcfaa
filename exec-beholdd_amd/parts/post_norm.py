"""A layer whose norms stand behind the sums ("post-norm"):

    x <- norm1(alpha x + mixer(x));   x <- norm2(alpha x + feed_forward(x))   where the layer has a feed-forward

The sublayers read the residual x itself (rounded to the activation type where that is narrower); `alpha` weighs the
residual against the sublayer's result.  The residual stays float32: the weighted sum, the norm's statistics and its
result are float32 and written back over the residual, and the same kernel writes the rounded copy that the next
sublayer's products read (`norm.sum_forward`), so a sublayer costs one pass over the rows beside its products.  A
sublayer that can write its result instead of adding it (`writes_fresh`) gets an empty matrix; any other registered
mixer or feed-forward gets a zeroed one to add into, so the block takes every part the pre-norm block takes.  The
norm is any registered one that offers `sum_forward`.
"""

from __future__ import annotations

import torch

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, graph_rows_allowed


class PostNormBlock:
    def __init__(self, width: int, alpha: float, mixer, mixer_norm, feed_forward=None, feed_forward_norm=None):
        for norm in (mixer_norm, feed_forward_norm):
            if norm is not None and not hasattr(norm, "sum_forward"):
                raise TypeError(f"{type(norm).__name__} cannot norm a weighted sum in place (no sum_forward)")
        self.width, self.alpha = int(width), float(alpha)
        self.mixer, self.mixer_norm = mixer, mixer_norm
        self.feed_forward, self.feed_forward_norm = feed_forward, feed_forward_norm

    def parts(self):
        sublayer = [self.feed_forward, self.feed_forward_norm] if self.feed_forward is not None else []
        return [self.mixer, self.mixer_norm, *sublayer]

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    @property
    def graph_safe_rows(self):
        return graph_rows_allowed(self.parts())

    def tensor_specs(self):
        return [spec for part in self.parts() for spec in part.tensor_specs()]

    def load(self, get):
        for part in self.parts():
            part.load(get)

    def prepare(self, kernels):
        for part in self.parts():
            if hasattr(part, "prepare"):
                part.prepare(kernels)

    def working_bytes(self, step) -> int:
        # a sublayer's result kept apart from the residual, and the rounded copy of the residual that the next one reads
        total = step.matrix(step.rows, self.width, 4) + 2 * step.matrix(step.rows, self.width)
        return total + sum(part.working_bytes(step) for part in (self.mixer, self.feed_forward) if hasattr(part, "working_bytes"))

    def unaccounted_parts(self) -> list:
        return [type(part).__name__ for part in (self.mixer, self.feed_forward) if part is not None and not hasattr(part, "working_bytes")]

    def cache_need(self):
        return self.mixer.cache_need()

    def entry_reader(self):
        """The product that alone reads this block's first input, if its mixer says so."""
        return getattr(self.mixer, "input_reader", None)

    def _input(self, ctx, hidden, part):
        """The residual as a sublayer reads it when nothing before has written that form."""
        if ctx.act_dtype == torch.float32:
            return hidden
        x = ctx.new_activations(hidden.shape[0], self.width, reader=getattr(part, "input_reader", None))
        ctx.kernels.cast_concat(hidden, None, x)
        return x

    def _run(self, ctx, hidden, x, part, *cache):
        result = ctx.new_f32(hidden.shape[0], self.width)
        if getattr(part, "writes_fresh", False):
            part.forward(ctx, x, result, *cache, fresh=True)
        else:
            result.zero_()
            part.forward(ctx, x, result, *cache)
        return result

    def forward(self, ctx, hidden, cache, prepared=None, next_block=None):
        """`hidden` [rows, width] float32, updated in place.  `prepared`: the mixer's input, if the block before wrote it
        with its last norm; returns the next block's, if that block reads one."""
        after = next_block.entry_reader() if isinstance(next_block, PostNormBlock) else None
        wanted_after = isinstance(next_block, PostNormBlock)
        x = prepared if prepared is not None else self._input(ctx, hidden, self.mixer)
        result = self._run(ctx, hidden, x, self.mixer, cache)
        if self.feed_forward is None:
            return self.mixer_norm.sum_forward(ctx, hidden, result, self.alpha, reader=after, rounded=wanted_after)
        x = self.mixer_norm.sum_forward(ctx, hidden, result, self.alpha, reader=getattr(self.feed_forward, "input_reader", None))
        result = self._run(ctx, hidden, x, self.feed_forward)
        return self.feed_forward_norm.sum_forward(ctx, hidden, result, self.alpha, reader=after, rounded=wanted_after)


@BLOCKS.register("post_norm")
def _build_post_norm(config, layer_index, prefix, kinds, shared):
    """Tensor names: <prefix>norm1 / norm2 (with the norm's own suffixes); `config.postln_alpha` weighs the residual."""
    norm = NORMS.get(kinds.norm)
    feed_forward = FEED_FORWARDS.get(kinds.feed_forward)(config, layer_index, prefix, shared)
    return PostNormBlock(
        config.hidden, getattr(config, "postln_alpha", 1.0), MIXERS.get(kinds.mixer)(config, layer_index, prefix, shared),
        norm(config, config.hidden, prefix + "norm1", shared), feed_forward,
        norm(config, config.hidden, prefix + "norm2", shared) if feed_forward is not None else None)
