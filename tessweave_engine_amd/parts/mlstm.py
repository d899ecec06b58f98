"""The mLSTM: a recurrent mixer with a matrix memory per head, exponential gates and a running maximum that keeps them
in range (Beck et al., "xLSTM: Extended Long Short-Term Memory").

    q = W_q h * dim^-1/2, k = W_k h [heads x dim], v = W_v h [heads x value_dim]              (no biases)
    i = cap * tanh((W_i h + b_i) / cap),   f = logsigmoid(cap * tanh((W_f h + b_f) / cap))      (one of each per head)
    m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n <- the same with k alone
    o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
    out = W_o ( [ .. o_h / rms(o_h) .. ] * norm_weight * sigmoid(W_g h) )

S, n and m (all zero when a request opens, m too) are the mixer's whole memory: float32 states in its cache slot. The
packed product leaves float32 rows; gates, exponentials, the state and all products with it are float32 in both
precisions. One-token (and few-token) sequences are walked token by token, longer portions run in chunks of 16 on the
matrix unit: the same sums in another order.
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, FixedState
from ..kernels import ops
from ..weights.spec import NORMAL, ONE_PLUS_NORMAL, VECTOR, TensorSpec
from .base import Mixer
from .linear import Linear


def _round_up(v, m):
    return (int(v) + m - 1) // m * m


class MatrixLSTM(Mixer):
    STATE, NORMALISER, MAXIMUM = "mlstm.s", "mlstm.n", "mlstm.m"

    def __init__(self, prefix, hidden, heads, dim, value_dim, gate_cap, eps, names=("q", "k", "v", "g", "i", "f", "o"),
                 bias_suffix=".b", norm_name="norm", suffix=""):
        """gate_cap: the cap of the two gates' raw values; eps: of the per-head unit norm of the output; names: the
        checkpoint's names (behind the prefix) of the seven matrices; the gates' biases are `<name><bias_suffix>`."""
        if not 1 <= int(dim) <= 256:
            raise ValueError("the mLSTM kernels take key sizes up to 256")
        if not float(gate_cap) > 0:
            raise ValueError("the gates' cap must be positive")
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.heads, self.dim, self.value_dim = int(hidden), int(heads), int(dim), int(value_dim)
        self.gate_cap, self.eps = float(gate_cap), float(eps)
        H, D, E = self.heads, self.dim, self.value_dim
        # columns of the packed product
        self.columns = {"q": 0, "k": H * D, "v": 2 * H * D, "g": 2 * H * D + H * E, "i": 2 * H * D + 2 * H * E,
                        "f": 2 * H * D + 2 * H * E + H}
        self.width = 2 * H * D + 2 * H * E + 2 * H
        q, k, v, g, i, f, o = (prefix + n for n in self.names)
        self.proj = Linear([q, k, v, g, i, f], hidden, [H * D, H * D, H * E, H * E, H, H], suffixes=(suffix, ".bias"))
        self.bias_names = (i + bias_suffix, f + bias_suffix)
        self.norm_name = prefix + norm_name
        self.o = Linear([o], H * E, [hidden], suffixes=(suffix, ".bias"))
        self.i_bias = self.f_bias = self.norm_weight = None

    def parts(self):
        return [self.proj, self.o]

    def tensor_specs(self):
        # (the gates' biases are added inside the recurrence's kernel, in float32, not by the packed product)
        specs = self.proj.tensor_specs()
        specs += [TensorSpec(name, (self.heads,), VECTOR, NORMAL) for name in self.bias_names]
        return specs + self.o.tensor_specs() + [TensorSpec(self.norm_name, (self.heads * self.value_dim,), VECTOR, ONE_PLUS_NORMAL)]

    def bind(self, tensors, dtype, device):
        self.i_bias = tensors.pop(self.bias_names[0]).contiguous()
        self.f_bias = tensors.pop(self.bias_names[1]).contiguous()
        self.proj.bind(tensors, dtype, device)
        self.o.bind(tensors, dtype, device)
        self.norm_weight = tensors.pop(self.norm_name).contiguous()

    def weight_tensors(self):
        return [self.i_bias, self.f_bias, self.norm_weight]

    def cache_need(self):
        H, Dp, Ep = self.heads, _round_up(self.dim, 16), _round_up(self.value_dim, 16)
        return CacheNeed(states=((self.STATE, FixedState((H, Ep, Dp), "float32")),
                                 (self.NORMALISER, FixedState((2, H, Dp), "float32")),
                                 (self.MAXIMUM, FixedState((2, H), "float32"))))

    def forward(self, ctx, run, h, x, accumulate=True):
        n, H, D, E = ctx.n_tokens, self.heads, self.dim, self.value_dim
        col = self.columns
        proj = ctx.scratch("mlstm.proj", (n, self.width), torch.float32)
        self.proj.forward(ctx, h, proj)
        result = ctx.scratch("mlstm.o", (n, H * E), torch.float32)
        states = ctx.cache.states[run.cache_slot]
        common = (proj, col["q"], col["k"], col["v"], col["i"], col["f"], self.i_bias, self.f_bias, states[self.STATE],
                  states[self.NORMALISER], states[self.MAXIMUM], ctx.q_start, ctx.state_slots, ctx.state_phase)
        tail = (result, H, D, E, D ** -0.5, self.gate_cap)
        portions = ctx.n_seqs - ctx.n_decode
        if portions and ctx.max_q_len <= ops.MLSTM_WALK_TOKENS:
            ops.mlstm(*common, 0, ctx.n_seqs, *tail, walk=True)              # every sequence of the step is short
        else:
            if ctx.n_decode:
                ops.mlstm(*common, 0, ctx.n_decode, *tail, walk=True)
            if portions:
                # (one-token sequences own the first rows of a step: the portions' rows are the rest)
                ops.mlstm(*common, ctx.n_decode, portions, *tail, walk=False, first_row=ctx.n_decode)
        act = ctx.scratch("mlstm.act", (n, H * E))
        ops.head_norm_gate(result, proj[:, col["g"]:col["g"] + H * E], self.norm_weight, act, H, E, self.eps,
                           gate_activation="sigmoid")
        if ctx.defer_sums and self.o.deferrable(n):
            return self.o.forward_partials(ctx, act, "o")          # whoever norms next adds them up
        self.o.forward(ctx, act, x, residual=x if accumulate else None)
        return None
