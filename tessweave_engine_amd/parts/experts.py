"""A feed-forward of routed experts, optionally beside a shared expert that every token runs.

    z = W_router h (float32),  s = sigmoid(z);  a token runs the `top` experts with the largest scores
    x += sum over its experts e of expert_e(s_e * h)  (+ shared(h))       the score multiplies the expert's INPUT and
                                                                           is not renormalised
    expert(y) = down( g' * sigmoid(1.702 g') * (u' + 1) ),  g' = min(gate y, L),  u' = clamp(up y, -L, L)

Experts have no biases. The experts' matrices are stacked on the device ([experts, inner, width] and [experts, width,
inner], the reduction sizes padded to multiples of 32 with zeros, in the order the matrix unit's fragments are read:
`ops.moe_blocked`) and all experts of a step run in two grouped
products on the matrix unit, whose launch shapes depend on the step's rows only: nothing waits for the host.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import MATRIX, NORMAL, VECTOR, TensorSpec
from .base import FeedForward


class RoutedExperts(FeedForward):
    def __init__(self, prefix, hidden, experts, top, intermediate, limit, shared=None, router_name="router",
                 expert_names=("e{}.gate", "e{}.up", "e{}.down")):
        """shared: a `FeedForward` part that every token runs as well (or None). expert_names: the checkpoint's
        names, behind the prefix, of expert number {}'s three matrices."""
        self.prefix, self.hidden, self.experts, self.top = prefix, int(hidden), int(experts), int(top)
        self.intermediate, self.limit, self.shared = int(intermediate), float(limit), shared
        if not 0 < self.top <= self.experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"1 to {ops.MOE_MAX_EXPERTS} experts, of which `top` are chosen")
        if not self.limit > 0:
            raise ValueError("the experts' limit must be positive")
        self.router_name, self.expert_names = router_name, tuple(expert_names)
        self.router = self.gate = self.up = self.down = None

    def parts(self):
        return [self.shared] if self.shared is not None else []

    def _names(self, e):
        return [self.prefix + n.format(e) for n in self.expert_names]

    def tensor_specs(self):
        C, F = self.hidden, self.intermediate
        specs = [TensorSpec(self.prefix + self.router_name, (self.experts, C), VECTOR, NORMAL)]
        for e in range(self.experts):
            gate, up, down = self._names(e)
            specs += [TensorSpec(gate, (F, C), MATRIX, NORMAL), TensorSpec(up, (F, C), MATRIX, NORMAL),
                      TensorSpec(down, (C, F), MATRIX, NORMAL)]
        return specs + (self.shared.tensor_specs() if self.shared is not None else [])

    def bind(self, tensors, dtype, device):
        C, F, X = self.hidden, self.intermediate, self.experts
        Cd, Fd = ops.moe_pad(C), ops.moe_pad(F)
        self.router = tensors.pop(self.prefix + self.router_name).contiguous()        # float32: the router's precision
        gate = torch.zeros(X, Fd, Cd, dtype=dtype, device=device)
        up = torch.zeros(X, Fd, Cd, dtype=dtype, device=device)
        down = torch.zeros(X, C, Fd, dtype=dtype, device=device)
        for e in range(X):
            g, u, d = self._names(e)
            gate[e, :F, :C] = tensors.pop(g)
            up[e, :F, :C] = tensors.pop(u)
            down[e, :, :F] = tensors.pop(d)
        self.gate, self.up, self.down = ops.moe_blocked(gate), ops.moe_blocked(up), ops.moe_blocked(down)
        if self.shared is not None:
            self.shared.bind(tensors, dtype, device)

    def weight_tensors(self):
        return [self.router]          # (a step reads only the matrices of the experts its tokens chose)

    def expert_bytes(self):
        """Bytes of one expert's three matrices on the device."""
        return sum(t[0].numel() * t.element_size() for t in (self.gate, self.up, self.down))

    def forward(self, ctx, h, x, accumulate=True):
        if not accumulate:
            raise ValueError("routed experts add into the stream")
        n = h.shape[0]
        if self.shared is not None:
            self.shared.forward(ctx, h, x)
        ids = ctx.scratch("moe.ids", (n, self.top), torch.int32)
        weights = ctx.scratch("moe.weights", (n, self.top), torch.float32)
        ops.moe_route(h, self.router, self.top, ids, weights)

        def scratch(tag, shape, dtype):
            # sized for the largest step: `capacity` rows for max_tokens rows of the stream
            most = ops.moe_capacity(ctx.max_tokens * self.top, self.experts)
            rows = {"moe.pos": ctx.max_tokens * self.top, "moe.tiles": most // 16}.get(tag, most)
            return ctx.workspace.get(f"{tag}.{self.top}.{self.experts}", shape, dtype, capacity=rows)
        ops.moe_experts(h, ids, weights, self.gate, self.up, self.down, self.limit, x, scratch)
        return None
