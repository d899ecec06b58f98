"""SwiGLU feed-forward: x += down( silu(gate(h)) * up(h) ), no biases (flow_engine/model.py:68-85); the same with
another activation (`GatedFeedForward`); and one without a gate, down( relu(up(h))^2 ) (`ReluSquaredFeedForward`).

`accumulate=False` asks for the result alone (written to x, or left as pending partial sums of the result alone),
for arrangements that scale it or norm the sum."""
from __future__ import annotations

from ..kernels import ops
from .base import FeedForward
from .linear import Linear


class SwiGLU(FeedForward):
    def __init__(self, prefix, hidden, intermediate, packed=True):
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.gate_up = Linear([prefix + "gate_proj", prefix + "up_proj"], hidden, [intermediate, intermediate],
                              packed=packed, glu=True)
        self.down = Linear([prefix + "down_proj"], intermediate, [hidden])

    def parts(self):
        return [self.gate_up, self.down]

    def tensor_specs(self):
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def bind(self, tensors, dtype, device):
        self.gate_up.bind(tensors, dtype, device)
        self.down.bind(tensors, dtype, device)

    def forward(self, ctx, h, x, accumulate=True):
        n = h.shape[0]
        act = ctx.scratch("ffn.act", (n, self.intermediate))
        if self.gate_up.gated:
            # silu(gate) * up is formed in the projection's epilogue; [n, 2 * intermediate] is never stored
            self.gate_up.forward_glu(ctx, h, act)
        else:
            gu = ctx.scratch("ffn.gate_up", (n, 2 * self.intermediate))
            self.gate_up.forward(ctx, h, gu)
            ops.silu_mul(gu, act)
        if ctx.defer_sums and not self.down.biases and self.down.deferrable(n):
            # where the down projection splits K (few rows; many rows against its long K), the sums are left to the next norm
            return self.down.forward_partials(ctx, act, "down")
        self.down.forward(ctx, act, x, residual=x if accumulate else None)
        return None


class GatedFeedForward(FeedForward):
    """x += out_scale * down( act(gate(h)) * up(h) ) with a choice of activation and of tensor names.

    activation "silu" is `SwiGLU`'s arithmetic; "gelu_tanh" is 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
    Gate and up rows are interleaved so that the matrix kernels' gated epilogue forms act(gate) * up (where the
    intermediate size is no multiple of 16 a kernel of its own multiplies after one packed product); out_scale is
    folded into that multiplication, before the rounding to the compute type, so the down projection adds straight
    into the residual stream.
    """

    def __init__(self, names, hidden, intermediate, activation="gelu_tanh", out_scale=1.0, suffix=".weight", limit=None):
        """activation: "gelu_tanh", "silu", or "swish_limited", which needs `limit` L and computes
        g' * sigmoid(1.702 g') * (u' + 1) with g' = min(gate, L), u' = clamp(up, -L, L) (and takes no out_scale)."""
        if activation not in ("gelu_tanh", "silu", "swish_limited"):
            raise ValueError("GatedFeedForward computes gelu_tanh, silu or swish_limited")
        if activation == "swish_limited" and (limit is None or not float(limit) > 0 or float(out_scale) != 1.0):
            raise ValueError("swish_limited needs a positive limit and takes no out_scale")
        gate, up, down = names
        self.hidden, self.intermediate, self.out_scale = int(hidden), int(intermediate), float(out_scale)
        self.activation = activation
        self.limit = float(limit) if limit is not None else None
        self.gate_up = Linear([gate, up], hidden, [intermediate, intermediate], glu=True, suffixes=(suffix, ".bias"))
        self.down = Linear([down], intermediate, [hidden], suffixes=(suffix, ".bias"))

    def parts(self):
        return [self.gate_up, self.down]

    def tensor_specs(self):
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def bind(self, tensors, dtype, device):
        self.gate_up.bind(tensors, dtype, device)
        self.down.bind(tensors, dtype, device)

    def forward(self, ctx, h, x, accumulate=True):
        n = h.shape[0]
        act = ctx.scratch("ffn.act", (n, self.intermediate))
        limited = self.activation == "swish_limited"
        if self.gate_up.gated:
            self.gate_up.forward_glu(ctx, h, act, activation=self.activation, factor=self.limit if limited else self.out_scale)
        else:
            gu = ctx.scratch("ffn.gate_up", (n, 2 * self.intermediate))
            self.gate_up.forward(ctx, h, gu)
            if limited:
                ops.swish_limited_mul(gu, act, self.limit)
            elif self.activation == "silu" and self.out_scale == 1.0:
                ops.silu_mul(gu, act)
            elif self.activation == "silu":
                raise ValueError("silu with an output scale needs an intermediate size that is a multiple of 16")
            else:
                ops.gelu_mul(gu, act, self.out_scale)
        self.down.forward(ctx, act, x, residual=x if accumulate else None)
        return None


class PlainFeedForward(FeedForward):
    """x += down( act(up(h)) ): no gate, no biases; act "relu_squared" (max(z, 0)^2) or "gelu" (the exact one, z Phi(z)).
    names = (up, down), the checkpoint prefixes of the two matrices. defer=False: the down projection always finishes
    its sums itself (for a part that adds more to the same result)."""

    def __init__(self, names, hidden, intermediate, suffix=".weight", activation="relu_squared", defer=True):
        up, down = names
        if activation not in ops.LINEAR_ACTIVATIONS:
            raise ValueError("a plain feed-forward computes relu_squared or gelu")
        self.activation, self.defer = activation, bool(defer)
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.up = Linear([up], hidden, [intermediate], suffixes=(suffix, ".bias"))
        self.down = Linear([down], intermediate, [hidden], suffixes=(suffix, ".bias"))

    def parts(self):
        return [self.up, self.down]

    def tensor_specs(self):
        return self.up.tensor_specs() + self.down.tensor_specs()

    def bind(self, tensors, dtype, device):
        self.up.bind(tensors, dtype, device)
        self.down.bind(tensors, dtype, device)

    def forward(self, ctx, h, x, accumulate=True):
        n = h.shape[0]
        act = ctx.scratch("ffn.act", (n, self.intermediate))
        if n <= 64 and self.up.deferrable(n):
            # few rows: the product leaves its split-K sums, and the activation's kernel adds them up
            ops.activation(act, self.activation, partial=self.up.forward_partials(ctx, h, "up"))
        elif not self.up.forward_act(ctx, h, act, self.activation):       # many rows: in the product's epilogue
            self.up.forward(ctx, h, act)
            ops.activation(act, self.activation)
        if self.defer and ctx.defer_sums and self.down.deferrable(n):
            return self.down.forward_partials(ctx, act, "down")          # whoever norms next adds them up
        self.down.forward(ctx, act, x, residual=x if accumulate else None)
        return None


class ReluSquaredFeedForward(PlainFeedForward):
    """x += down( relu(up(h))^2 )."""

    def __init__(self, names, hidden, intermediate, suffix=".weight"):
        super().__init__(names, hidden, intermediate, suffix=suffix, activation="relu_squared")
