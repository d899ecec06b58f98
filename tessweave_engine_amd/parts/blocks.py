"""How a layer's parts are arranged. Pre-norm with two residuals (flow_engine/model.py:179-202):

    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed
from ..kernels import ops
from ..weights.spec import AVERAGE, ONE_PLUS_NORMAL, VECTOR, TensorSpec
from .base import ROUNDED_STREAM, Block, fold_pending


class PreNormBlock(Block):
    def __init__(self, mixer_norm, mixer, ffn_norm, ffn):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype, device):
        for p in self.parts():
            p.bind(tensors, dtype, device)

    def forward(self, ctx, run, x, pending=None):
        h = normalise(self.mixer_norm, ctx, x, pending)
        pending = self.mixer.forward(ctx, run, h, x)
        h = normalise(self.ffn_norm, ctx, x, pending)
        return self.ffn.forward(ctx, h, x)


def normalise(norm, ctx, x, pending=None, rows=None):
    """NORM of X; PENDING partial sums go to a norm that folds them, and are folded here for one that does not
    (which only happens when parts are driven by hand: a model defers sums only if all its norms fold them)."""
    if pending is not None and not norm.folds_pending:
        pending = fold_pending(x, pending)
    if pending is not None:
        return norm.forward(ctx, x, rows=rows, add=pending)
    return norm.forward(ctx, x, rows=rows)


class ParallelBlock(Block):
    """Mixer and feed-forward side by side, each behind a norm of its own, both of the same stream:

        x <- x + mixer(norm1(x)) + ff(norm2(x))

    mixer_norm, ffn_norm: `RMSNorm` parts (weights and eps; both norms are one kernel: the row is read and its
    statistic formed once). ffn / ffn_norm may be None: the layer then has only the mixer. Both sublayers add into
    the stream after both norms have read it. The sublayers' sums are complete when the block returns (a model of
    such blocks is built with `defer_sums=False`)."""

    def __init__(self, hidden, mixer_norm, mixer, ffn_norm=None, ffn=None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        if ffn_norm is not None and ffn_norm.eps != mixer_norm.eps:
            raise ValueError("the two norms of a parallel block share their eps")
        self.hidden = int(hidden)
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype, device):
        for p in self.parts():
            p.bind(tensors, dtype, device)

    def forward(self, ctx, run, x, pending=None):
        pending = fold_pending(x, pending)
        n = ctx.n_tokens
        h1 = ctx.scratch("norm.out", (n, self.hidden))
        h2 = ctx.scratch("norm.out.second", (n, self.hidden)) if self.ffn is not None else None
        ops.rmsnorm_pair(x, self.mixer_norm.weight, self.mixer_norm.eps, h1,
                         self.ffn_norm.weight if self.ffn is not None else None, h2)
        left = self.mixer.forward(ctx, run, h1, x)
        if left is not None:
            raise RuntimeError("a parallel block's mixer must add into the stream itself")
        if self.ffn is not None:
            left = self.ffn.forward(ctx, h2, x)
            if left is not None:
                raise RuntimeError("a parallel block's feed-forward must add into the stream itself")
        return None


class PostNormBlock(Block):
    """Norm after the sum, with an optional scale per channel on each sublayer's result:

        x <- norm1(alpha * x + scale1 * mixer(x));  x <- norm2(alpha * x + scale2 * ff(x))

    The sublayers read the stream x itself (rounded to the compute type). mixer_norm, ffn_norm: `RMSNorm` parts
    (weight and eps; sum, scale, norm and the rounding for the next sublayer are one kernel, which also adds up
    split-K partial sums a sublayer leaves pending). ffn / ffn_norm may be None: the layer then has only the
    first sublayer. scale names: float32 [hidden] checkpoint tensors, or None. The mixer and the feed-forward
    must take `accumulate=False` (their result alone, not added into the stream)."""

    def __init__(self, hidden, mixer, mixer_norm, ffn=None, ffn_norm=None, alpha=1.0, mixer_scale_name=None,
                 ffn_scale_name=None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.hidden, self.alpha = int(hidden), float(alpha)
        self.mixer, self.mixer_norm, self.ffn, self.ffn_norm = mixer, mixer_norm, ffn, ffn_norm
        self.mixer_scale_name = mixer_scale_name
        self.ffn_scale_name = ffn_scale_name if ffn is not None else None
        self.mixer_scale = self.ffn_scale = None

    def parts(self):
        return [p for p in (self.mixer, self.mixer_norm, self.ffn, self.ffn_norm) if p is not None]

    def tensor_specs(self):
        specs = [s for p in self.parts() for s in p.tensor_specs()]
        for name in (self.mixer_scale_name, self.ffn_scale_name):
            if name:
                specs.append(TensorSpec(name, (self.hidden,), VECTOR, ONE_PLUS_NORMAL))
        return specs

    def bind(self, tensors, dtype, device):
        for p in self.parts():
            p.bind(tensors, dtype, device)
        self.mixer_scale = tensors.pop(self.mixer_scale_name).contiguous() if self.mixer_scale_name else None
        self.ffn_scale = tensors.pop(self.ffn_scale_name).contiguous() if self.ffn_scale_name else None

    def weight_tensors(self):
        return [t for t in (self.mixer_scale, self.ffn_scale) if t is not None]

    def _rounded(self, ctx, x):
        """The stream in the compute type: what the part before left, else rounded now (float32 runs read x itself)."""
        h = ctx.shared.get(ROUNDED_STREAM)
        if h is None:
            if ctx.dtype == torch.float32:
                return x
            h = ops.round_rows(x, ctx.scratch("stream.rounded", (ctx.n_tokens, self.hidden)))
        return h

    def _sublayer(self, ctx, x, norm, scale, result, pending):
        rounded = ctx.scratch("stream.rounded", (ctx.n_tokens, self.hidden)) if ctx.dtype != torch.float32 else None
        ops.residual_norm(x, norm.weight, norm.eps, out=rounded, y=result if pending is None else None, add=pending,
                          scale=scale, alpha=self.alpha)
        ctx.shared[ROUNDED_STREAM] = rounded if rounded is not None else x

    def forward(self, ctx, run, x, pending=None):
        pending = fold_pending(x, pending)
        n = ctx.n_tokens
        result = ctx.scratch("sublayer.result", (n, self.hidden), torch.float32)
        left = self.mixer.forward(ctx, run, self._rounded(ctx, x), result, accumulate=False)
        self._sublayer(ctx, x, self.mixer_norm, self.mixer_scale, result, left)
        if self.ffn is not None:
            left = self.ffn.forward(ctx, self._rounded(ctx, x), result, accumulate=False)
            self._sublayer(ctx, x, self.ffn_norm, self.ffn_scale, result, left)
        return None


class ResultNormBlock(Block):
    """A norm on each sublayer's RESULT, scaled into the stream:

        x <- x + mult * norm1(mixer(x));  x <- x + mult * norm2(ff(x))

    The sublayers read the stream x itself (rounded to the compute type). mixer_norm, ffn_norm: `RMSNorm` parts (weight
    and eps; norm, scaling, sum and the rounding for the next sublayer are one kernel, which also adds up split-K
    partial sums a sublayer leaves pending). ffn / ffn_norm may be None: the layer then has only the first sublayer.
    The mixer and the feed-forward must take `accumulate=False` (their result alone, not added into the stream)."""

    def __init__(self, hidden, mixer, mixer_norm, ffn=None, ffn_norm=None, mult=1.0, unused_names=()):
        """unused_names: tensors a checkpoint may hold for this layer that nothing reads (the norm of a feed-forward the
        layer does not have): accepted if present, never required."""
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.hidden, self.mult = int(hidden), float(mult)
        self.mixer, self.mixer_norm, self.ffn, self.ffn_norm = mixer, mixer_norm, ffn, ffn_norm
        self.unused_names = tuple(unused_names)

    def parts(self):
        return [p for p in (self.mixer, self.mixer_norm, self.ffn, self.ffn_norm) if p is not None]

    def tensor_specs(self):
        specs = [s for p in self.parts() for s in p.tensor_specs()]
        return specs + [TensorSpec(name, (1,), VECTOR, optional_alias_of="(unused)") for name in self.unused_names]

    def bind(self, tensors, dtype, device):
        for p in self.parts():
            p.bind(tensors, dtype, device)

    def _rounded(self, ctx, x):
        """The stream in the compute type: what the part before left, else rounded now (float32 runs read x itself)."""
        h = ctx.shared.get(ROUNDED_STREAM)
        if h is None:
            if ctx.dtype == torch.float32:
                return x
            h = ops.round_rows(x, ctx.scratch("stream.rounded", (ctx.n_tokens, self.hidden)))
        return h

    def _sublayer(self, ctx, x, norm, result, pending):
        rounded = ctx.scratch("stream.rounded", (ctx.n_tokens, self.hidden)) if ctx.dtype != torch.float32 else None
        ops.add_normed(x, norm.weight, norm.eps, mult=self.mult, y=result if pending is None else None, add=pending,
                       out=rounded)
        ctx.shared[ROUNDED_STREAM] = rounded if rounded is not None else x

    def forward(self, ctx, run, x, pending=None):
        pending = fold_pending(x, pending)
        result = ctx.scratch("sublayer.result", (ctx.n_tokens, self.hidden), torch.float32)
        left = self.mixer.forward(ctx, run, self._rounded(ctx, x), result, accumulate=False)
        self._sublayer(ctx, x, self.mixer_norm, result, left)
        if self.ffn is not None:
            left = self.ffn.forward(ctx, self._rounded(ctx, x), result, accumulate=False)
            self._sublayer(ctx, x, self.ffn_norm, result, left)
        return None


class DepthMixedBlock(Block):
    """Pre-norm block whose sublayers read their normed input through a short causal convolution, with an
    optional per-layer token input, and whose output is a learned mix of every layer's result so far:

        x <- x + mixer(conv1(norm1(x)));  x <- x + ff(conv2(norm2(x)))        (the residual multiplier is the
        x <- x + mult * side(x) / rms(side(x)) * w                              mixer's and feed-forward's own)
        X_(layer + 1) = x;  x <- sum_{j <= layer + 1} mix[j] * X_j             (X_0 the embedding output)

    mixer_in, ffn_in: `CausalConv` parts with a norm (norm, convolution and rounding are one kernel); their last
    inputs are state of the block's cache slot beside the mixer's own. ffn / ffn_in / side / mix_name may be None.
    The results X_j of a step live in one float32 scratch buffer [layers + 1, largest step's rows, hidden]
    (`HISTORY_TAG`); X_0 is written there by the embedding (`PositionedEmbedding(keep=(HISTORY_TAG, layers + 1))`).
    """

    HISTORY_TAG = "depth.history"

    def __init__(self, layer, n_layers, hidden, mixer_in, mixer, ffn_in=None, ffn=None, side=None, side_mult=1.0,
                 mix_name=None, unused_names=()):
        """unused_names: tensors a checkpoint may hold for this layer that nothing reads (the norm and convolution
        of a feed-forward the layer does not have): accepted if present, never required."""
        self.unused_names = tuple(unused_names)
        self.layer, self.n_layers, self.hidden = int(layer), int(n_layers), int(hidden)
        self.mixer_in, self.mixer, self.ffn_in, self.ffn, self.side = mixer_in, mixer, ffn_in, ffn, side
        self.side_mult, self.mix_name = float(side_mult), mix_name
        self.mix = None

    def parts(self):
        return [p for p in (self.mixer_in, self.mixer, self.ffn_in, self.ffn, self.side) if p is not None]

    def tensor_specs(self):
        specs = [s for p in self.parts() for s in p.tensor_specs()]
        if self.mix_name:
            specs.append(TensorSpec(self.mix_name, (self.layer + 2,), VECTOR, AVERAGE))
        specs += [TensorSpec(name, (1,), VECTOR, optional_alias_of="(unused)") for name in self.unused_names]
        return specs

    def bind(self, tensors, dtype, device):
        for p in self.parts():
            p.bind(tensors, dtype, device)
        if self.mix_name:
            self.mix = tensors.pop(self.mix_name).contiguous()

    def weight_tensors(self):
        return [self.mix] if self.mix is not None else []

    def cache_need(self):
        need = self.mixer.cache_need() or CacheNeed()
        own = tuple(p.state_need() for p in (self.mixer_in, self.ffn_in) if p is not None)
        return need.merged(CacheNeed(states=own))

    def forward(self, ctx, run, x, pending=None):
        pending = fold_pending(x, pending)
        n = ctx.n_tokens
        h = ctx.scratch("norm.out", (n, self.hidden))
        self.mixer_in.forward(ctx, run, x, out=h)
        self.mixer.forward(ctx, run, h, x)
        if self.ffn is not None:
            self.ffn_in.forward(ctx, run, x, out=h)
            self.ffn.forward(ctx, h, x)
        y = self.side.forward(ctx, x) if self.side is not None else None
        history = None
        if self.mix is not None:
            history = ctx.workspace.get(self.HISTORY_TAG, (self.n_layers + 1, ctx.max_tokens, self.hidden), torch.float32)
        if y is not None or history is not None:
            ops.layer_end(x, self.layer, branch=y, branch_weight=self.side.weight if self.side is not None else None,
                          eps=self.side.eps if self.side is not None else 0.0, mult=self.side_mult, history=history,
                          mix=self.mix)
        return None
