"""Arrangements of norm, mixer and feed-forward in a layer. GPT-2's is pre-norm: a norm before
the mixer and one before the feed-forward, each branch added to the residual stream
(engine/src/transformer_block.c:49-71)."""

from __future__ import annotations

from .base import Block, FeedForward, LayerContext, Mixer, Norm, register_part


class PreNormBlock(Block):
    def __init__(self, norm_1: Norm, mixer: Mixer, norm_2: Norm, feed_forward: FeedForward, compute_dtype,
                 names=("ln_1.", "attn.", "ln_2.", "mlp.")):
        self.norm_1, self.mixer, self.norm_2, self.feed_forward = norm_1, mixer, norm_2, feed_forward
        self.compute_dtype = compute_dtype
        self._names = names

    def children(self):
        return dict(zip(self._names, (self.norm_1, self.mixer, self.norm_2, self.feed_forward)))

    def mixer_part(self):
        return self.mixer

    takes_pending = True

    def forward(self, hidden, ctx: LayerContext):
        hidden = self.mixer.forward_normed(hidden, self.norm_1, self.compute_dtype, ctx)
        return self.feed_forward.forward_normed(hidden, self.norm_2, self.compute_dtype, ctx)


class PostNormBlock(Block):
    """Norm after the sum: x <- norm_1(alpha * x + mixer(x)), then x <- norm_2(alpha * x + feed_forward(x)); the branches
    read x itself. ``alpha`` scales the stream in both sums. ``feed_forward`` None: the layer ends behind its mixer. The norms
    have ``forward_sum`` (RMSNorm), and mixer and feed-forward return their branch alone when given no residual."""

    takes_pending = True   # takes plain rows, pending rows or a norm's NormedRows, and returns NormedRows

    def __init__(self, norm_1: Norm, mixer: Mixer, norm_2: Norm | None, feed_forward: FeedForward | None, alpha: float, compute_dtype,
                 names=("norm1", "mix.", "norm2", "mlp.")):
        if (norm_2 is None) != (feed_forward is None):
            raise ValueError("the second norm goes with the feed-forward")
        self.norm_1, self.mixer, self.norm_2, self.feed_forward = norm_1, mixer, norm_2, feed_forward
        self.alpha, self.compute_dtype = float(alpha), compute_dtype
        self._names = names

    def children(self):
        parts = dict(zip(self._names, (self.norm_1, self.mixer, self.norm_2, self.feed_forward)))
        return {name: part for name, part in parts.items() if part is not None}

    def mixer_part(self):
        return self.mixer

    def forward(self, hidden, ctx: LayerContext):
        from ..ops import kernels

        if not isinstance(hidden, kernels.NormedRows):
            stream = kernels.settle(hidden)
            hidden = kernels.NormedRows(stream, stream if self.compute_dtype == stream.dtype else kernels.convert(stream, self.compute_dtype))
        hidden = self.norm_1.forward_sum(hidden.stream, self.mixer.forward(hidden.rows, None, ctx), self.alpha, self.compute_dtype)
        if self.feed_forward is None:
            return hidden
        return self.norm_2.forward_sum(hidden.stream, self.feed_forward.forward(hidden.rows, None), self.alpha, self.compute_dtype)


class BranchNormBlock(Block):
    """Norm on each branch's output: x <- x + norm_1(mixer(x)), then x <- x + norm_2(feed_forward(x)); the branches read the
    stream itself. ``feed_forward`` None: the layer ends behind its mixer. The norms have ``forward_onto`` (RMSNorm), and mixer and
    feed-forward return their branch alone when given no residual. The stream travels as kernels.NormedRows: in float32 and, the
    same numbers, in the compute type that the next branch's products read."""

    takes_pending = True

    def __init__(self, norm_1: Norm, mixer: Mixer, norm_2: Norm | None, feed_forward: FeedForward | None, compute_dtype,
                 names=("norm1", "mix.", "norm2", "mlp.")):
        if (norm_2 is None) != (feed_forward is None):
            raise ValueError("the second norm goes with the feed-forward")
        self.norm_1, self.mixer, self.norm_2, self.feed_forward = norm_1, mixer, norm_2, feed_forward
        self.compute_dtype = compute_dtype
        self._names = names

    def children(self):
        parts = dict(zip(self._names, (self.norm_1, self.mixer, self.norm_2, self.feed_forward)))
        return {name: part for name, part in parts.items() if part is not None}

    def mixer_part(self):
        return self.mixer

    def forward(self, hidden, ctx: LayerContext):
        from ..ops import kernels

        if not isinstance(hidden, kernels.NormedRows):
            stream = kernels.settle(hidden)
            hidden = kernels.NormedRows(stream, stream if self.compute_dtype == stream.dtype else kernels.convert(stream, self.compute_dtype))
        hidden = self.norm_1.forward_onto(hidden.stream, self.mixer.forward(hidden.rows, None, ctx), self.compute_dtype)
        if self.feed_forward is None:
            return hidden
        return self.norm_2.forward_onto(hidden.stream, self.feed_forward.forward(hidden.rows, None), self.compute_dtype)


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "post_norm", PostNormBlock)
register_part("block", "branch_norm", BranchNormBlock)
