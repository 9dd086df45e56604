"""How norm, mixer and feed-forward are arranged in a layer (reference models/qwen3.py:55-74)."""
from __future__ import annotations

from ..kernels import ops
from .base import FeedForward, Mixer, Norm, ParamSpec, Part, PendingNorm, ScaledSum, Settled, few_tokens, register_part, side_branch


def one_tensor(x):
    """A sublayer's output as one tensor: a tuple of outputs (`FeedForward.forward`) becomes their float32 sum."""
    if not isinstance(x, (tuple, list)):
        return x
    total = None
    for t in x:
        v = t.float().sum(0) if t.dim() == 3 else t.float()
        total = v if total is None else total + v
    return total


def settled(h, residual):
    """(h, residual) with a `ScaledSum` in place of h turned into a `Settled` stream."""
    if isinstance(h, ScaledSum):
        return Settled(None), h.settle(residual)
    return h, residual


def norm_of(norm: Norm, x, residual):
    """Run a norm on x, which may be float32 partial sums [P, T, n] of a split product; a norm
    that does not declare `accepts_partials` gets their sum."""
    x = one_tensor(x)
    if x.dim() == 3 and not getattr(norm, "accepts_partials", False):
        x = x.sum(0)
    return norm.forward(x, residual)


@register_part("block", "pre_norm")
class PreNormBlock(Part):
    """residual += input; x = norm1(residual); a = mixer(x); residual += a; x = norm2(residual);
    return feed_forward(x), residual.

    The layer's output is added to the residual by whoever runs next: the next block's first
    norm or the model's final norm (reference models/qwen3.py:65-74: the add lives inside the
    norm call). The residual stream is float32.
    """

    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm | None, feed_forward: FeedForward | None):
        """Without a feed-forward (and its norm) the layer is its first half: the mixer's output is what is left to add."""
        super().__init__()
        if (norm2 is None) != (feed_forward is None):
            raise ValueError("a feed-forward and its norm come together")
        self.add_child("norm1", norm1)
        self.add_child("mixer", mixer)
        if feed_forward is not None:
            self.add_child("norm2", norm2)
            self.add_child("feed_forward", feed_forward)
        else:
            self.norm2 = self.feed_forward = None

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need()

    def forward(self, h, residual, step, cache, state):
        h, residual = settled(h, residual)
        if isinstance(h, Settled):          # the layer before has added its output already: the stream starts anew here
            h, residual = residual, None
        # a part that takes it gets the norm before it as a `PendingNorm` and may run it inside its first product
        if getattr(self.mixer, "takes_pending_norm", False):
            x = PendingNorm(self.norm1, h, residual)
            a = self.mixer.forward(x, step, cache, state)
            residual = x.new_residual()
        else:
            x, residual = norm_of(self.norm1, h, residual)
            a = self.mixer.forward(x, step, cache, state)
        if self.feed_forward is None:
            return a, residual
        if getattr(self.feed_forward, "takes_pending_norm", False):
            x = PendingNorm(self.norm2, a, residual)
            out = self.feed_forward.forward(x)
            return one_tensor(out), x.new_residual()
        x, residual = norm_of(self.norm2, a, residual)
        return one_tensor(self.feed_forward.forward(x)), residual


@register_part("block", "output_norm")
class OutputNormBlock(Part):
    """stream += norm1(mixer(stream)); stream += norm2(feed_forward(stream)): the norms sit on the sublayers'
    outputs only, and the sublayers read the stream itself (rounded to the compute dtype). Without a
    feed-forward the layer is its first half. The stream is float32; each sum and each norm is one kernel
    that also hands on the rounded stream."""

    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm | None = None, feed_forward: FeedForward | None = None):
        super().__init__()
        if (norm2 is None) != (feed_forward is None):
            raise ValueError("a feed-forward and its norm come together")
        self.add_child("norm1", norm1)
        self.add_child("mixer", mixer)
        if feed_forward is not None:
            self.add_child("norm2", norm2)
            self.add_child("feed_forward", feed_forward)
        else:
            self.norm2 = self.feed_forward = None

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need()

    def forward(self, h, residual, step, cache, state):
        h, residual = settled(h, residual)
        if isinstance(h, Settled):
            x, stream = (h.rounded if h.rounded is not None else residual.to(self.norm1.out_dtype)), residual
        elif residual is None:               # the first layer: the embedding's rows are the stream
            x, stream = h, h.float()
        else:                                # behind a layer that leaves its output to be added
            stream = residual + (h.sum(0) if h.dim() == 3 else h).float()
            x = stream.to(h.dtype if h.dim() == 2 else self.norm1.out_dtype)
        if getattr(self.mixer, "returns_terms", False) and hasattr(self.norm1, "add_terms"):
            # a mixer that is a weighted sum of several outputs: sum, norm and residual sum as one kernel
            x, stream = self.norm1.add_terms(self.mixer.forward(x, step, cache, state, terms=True), stream)
        else:
            x, stream = self.norm1.add_to(self.mixer.forward(x, step, cache, state), stream)
        if self.feed_forward is not None:
            x, stream = self.norm2.add_to(one_tensor(self.feed_forward.forward(x)), stream)
        return Settled(x), stream


def _ones(shape, generator, device):
    import torch
    return 1.0 + 0.2 * (torch.rand(shape, generator=generator, dtype=torch.float32, device=device) - 0.5)


@register_part("block", "parallel")
class ParallelBlock(Part):
    """stream += mult * (scale1 * mixer(norm1(stream)) + scale2 * feed_forward(norm2(stream))): both sublayers read
    the same stream, each through a norm of its own, and each output is multiplied element by element by a learned
    scale before the sum (`layer_scale`; without it the scales are 1). Without a feed-forward the layer is its first
    half. The two norms share the stream's root mean square and are one kernel; that kernel also forms the sum the
    layer before has left (`ScaledSum`), so a stack of such layers costs one pass over the stream per layer. The
    stream is float32.

    In steps of few tokens (`base.SIDE_BRANCH_MAX_TOKENS`), where a layer is a chain of short launches, the feed-forward
    runs on a second stream beside the mixer (`base.side_branch`): the two meet again before the layer returns, so a
    captured step holds them as two branches of its graph. What the second stream allocates is read on the first only
    behind that meeting, and written again only behind the next layer's parting, which follows the kernel that read it."""

    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm | None = None, feed_forward: FeedForward | None = None,
                 residual_mult: float = 1.0, layer_scale: bool = False):
        super().__init__()
        if (norm2 is None) != (feed_forward is None):
            raise ValueError("a feed-forward and its norm come together")
        for norm in (norm1, norm2):
            if norm is not None and (not hasattr(norm, "weight") or not hasattr(norm, "eps") or getattr(norm, "one_plus", False)):
                raise ValueError("the parallel block runs plain RMS norms (weight and eps) inside its own kernel")
        if norm2 is not None and (norm2.eps != norm1.eps or norm2.size != norm1.size):
            raise ValueError("the two norms of a parallel block share one eps and one width")
        self.residual_mult = float(residual_mult)
        self.layer_scale = bool(layer_scale)
        self.add_child("norm1", norm1)
        self.add_child("mixer", mixer)
        if feed_forward is not None:
            self.add_child("norm2", norm2)
            self.add_child("feed_forward", feed_forward)
        else:
            self.norm2 = self.feed_forward = None
        if layer_scale:
            self.add_param("scale1", ParamSpec((norm1.size,), init=_ones, dtype="float32"))
            if feed_forward is not None:
                self.add_param("scale2", ParamSpec((norm1.size,), init=_ones, dtype="float32"))
        else:
            self.scale1 = self.scale2 = None

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need()

    def forward(self, h, residual, step, cache, state):
        if isinstance(h, ScaledSum):
            stream, terms, mult = residual, h.terms, h.mult
        elif isinstance(h, Settled):
            stream, terms, mult = residual, [], 1.0
        elif residual is None:               # the first layer: the embedding's rows are the stream
            stream, terms, mult = h, [], 1.0
        else:                                # behind a layer that leaves its output to be added
            stream, terms, mult = residual, [(one_tensor(h), None)], 1.0
        w2 = self.norm2.weight if self.feed_forward is not None else None
        stream, x1, x2 = ops.scaled_sum_norm(stream, terms, mult, self.norm1.weight, w2, self.norm1.eps, self.norm1.out_dtype)
        b = None
        if self.feed_forward is not None and few_tokens(x1):
            with side_branch(x1.device, 1) as branch:
                b = self.feed_forward.forward(x2)
            out = [(self.mixer.forward(x1, step, cache, state), self.scale1)]
            branch.join()
        else:
            out = [(self.mixer.forward(x1, step, cache, state), self.scale1)]
            if self.feed_forward is not None:
                b = self.feed_forward.forward(x2)
        if b is not None:
            out += [(t, self.scale2 if self.layer_scale else None) for t in (b if isinstance(b, (tuple, list)) else (b,))]
        return ScaledSum(out, self.residual_mult), stream
