"""A feed-forward of routed experts, optionally beside a shared expert that every token runs.

    z = W_router h (float32),  s = sigmoid(z);  a token runs the `top` experts with the largest scores
    x += sum over its experts e of expert_e(s_e * h)  (+ shared(h))       the score multiplies the expert's INPUT and
                                                                           is not renormalised
    expert(y) = down( g' * sigmoid(1.702 g') * (u' + 1) ),  g' = min(gate y, L),  u' = clamp(up y, -L, L)

A second kind (`kind="gelu"`, `weighting="softmax_chosen"`, `router_bias`): experts without a gate, expert(y) =
down(gelu(up y)) with the exact gelu; the router's logits take a bias; a token's weights are the softmax over its chosen
logits alone and multiply the experts' OUTPUTS:  x += sum_e p_e expert_e(h)  (+ shared(h)).

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
    def __init__(self, prefix, hidden, experts, top, intermediate, limit=None, shared=None, router_name="router",
                 expert_names=None, kind="swish_limited", weighting="sigmoid", router_bias=None):
        """shared: a `FeedForward` part that every token runs as well (or None). expert_names: the checkpoint's
        names, behind the prefix, of expert number {}'s matrices (gate, up, down; up, down for kind "gelu").
        kind: "swish_limited" (gated, needs `limit`, weights on the experts' inputs) or "gelu" (no gate, weights on the
        outputs); weighting: "sigmoid" of each chosen logit or "softmax_chosen"; router_bias: the checkpoint's name,
        behind the prefix, of a bias on the router's logits (or None)."""
        self.prefix, self.hidden, self.experts, self.top = prefix, int(hidden), int(experts), int(top)
        self.intermediate, self.shared = int(intermediate), shared
        if kind not in ops.MOE_KINDS or weighting not in ops.MOE_WEIGHTS:
            raise ValueError("experts are 'swish_limited' or 'gelu', their weights 'sigmoid' or 'softmax_chosen'")
        self.kind, self.weighting = kind, weighting
        self.gated = kind == "swish_limited"
        self.limit = float(limit) if limit is not None else 0.0
        if not 0 < self.top <= self.experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"1 to {ops.MOE_MAX_EXPERTS} experts, of which `top` are chosen")
        if self.gated and not self.limit > 0:
            raise ValueError("the experts' limit must be positive")
        if expert_names is None:
            expert_names = ("e{}.gate", "e{}.up", "e{}.down") if self.gated else ("e{}.up", "e{}.down")
        self.router_name, self.expert_names = router_name, tuple(expert_names)
        self.router_bias_name = prefix + router_bias if router_bias else None
        self.router = self.router_bias = self.gate = self.up = self.down = None

    def parts(self):
        return [self.shared] if self.shared is not None else []

    def _names(self, e):
        return [self.prefix + n.format(e) for n in self.expert_names]

    def tensor_specs(self):
        C, F = self.hidden, self.intermediate
        specs = [TensorSpec(self.prefix + self.router_name, (self.experts, C), VECTOR, NORMAL)]
        if self.router_bias_name:
            specs.append(TensorSpec(self.router_bias_name, (self.experts,), VECTOR, NORMAL))
        for e in range(self.experts):
            *ins, down = self._names(e)
            specs += [TensorSpec(name, (F, C), MATRIX, NORMAL) for name in ins] + [TensorSpec(down, (C, F), MATRIX, NORMAL)]
        return specs + (self.shared.tensor_specs() if self.shared is not None else [])

    def bind(self, tensors, dtype, device):
        C, F, X = self.hidden, self.intermediate, self.experts
        Cd, Fd = ops.moe_pad(C), ops.moe_pad(F)
        self.router = tensors.pop(self.prefix + self.router_name).contiguous()        # float32: the router's precision
        if self.router_bias_name:
            self.router_bias = tensors.pop(self.router_bias_name).contiguous()
        gate = torch.zeros(X, Fd, Cd, dtype=dtype, device=device) if self.gated else None
        up = torch.zeros(X, Fd, Cd, dtype=dtype, device=device)
        down = torch.zeros(X, C, Fd, dtype=dtype, device=device)
        for e in range(X):
            *ins, d = self._names(e)
            if self.gated:
                gate[e, :F, :C] = tensors.pop(ins[0])
            up[e, :F, :C] = tensors.pop(ins[-1])
            down[e, :, :F] = tensors.pop(d)
        self.gate = ops.moe_blocked(gate) if self.gated else None
        self.up, self.down = ops.moe_blocked(up), ops.moe_blocked(down)
        if self.shared is not None:
            self.shared.bind(tensors, dtype, device)

    def weight_tensors(self):
        return [t for t in (self.router, self.router_bias) if t is not None]          # (a step reads only the matrices of the experts its tokens chose)

    def expert_bytes(self):
        """Bytes of one expert's three matrices on the device."""
        return sum(t[0].numel() * t.element_size() for t in (self.gate, self.up, self.down) if t is not None)

    def forward(self, ctx, h, x, accumulate=True):
        n = h.shape[0]
        # (with accumulate=False the shared expert writes x and the routed ones add to it, or it leaves the split-K sums of
        # its last product pending and the kernel that adds up a token's experts adds those too)
        pending = self.shared.forward(ctx, h, x, accumulate=accumulate) if self.shared is not None else None
        wrote = self.shared is not None and pending is None
        ids = ctx.scratch("moe.ids", (n, self.top), torch.int32)
        weights = ctx.scratch("moe.weights", (n, self.top), torch.float32)
        ops.moe_route(h, self.router, self.top, ids, weights, bias=self.router_bias, weighting=self.weighting)

        def scratch(tag, shape, dtype):
            # sized for the largest step: `capacity` rows for max_tokens rows of the stream
            most = ops.moe_capacity(ctx.max_tokens * self.top, self.experts)
            rows = {"moe.pos": ctx.max_tokens * self.top, "moe.tiles": most // 16}.get(tag, most)
            return ctx.workspace.get(f"{tag}.{self.top}.{self.experts}", shape, dtype, capacity=rows)
        ops.moe_experts(h, ids, weights, self.gate, self.up, self.down, self.limit, x, scratch, kind=self.kind,
                        accumulate=accumulate or wrote, more=pending)
        return None
