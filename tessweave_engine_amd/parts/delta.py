"""The gated delta rule: a recurrent mixer whose state is corrected towards each new value before it is read.

    q, k [key_heads x dim], v [heads x value_dim] from one packed product (no biases), each through a short causal
    convolution over time per channel and SiLU; q and k made unit vectors per head, q times dim^-1/2
    beta = sigmoid(W_b h), decay = exp(-exp(A_log) * softplus(W_a h + dt_bias))           (one of each per head)
    S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                        (S float32 [dim, value_dim])
    out = W_o [ .. o_h / rms(o_h) * norm_weight * silu(g_h) .. ]                            (g from the same product)

Value head h reads key head h // (heads / key_heads). The state S and the convolutions' last inputs are the mixer's
whole memory: fixed-size float32 states in its cache slot, zero when a request opens. The packed product leaves float32
rows; the convolutions, unit norms, gates, the state and all products with it are float32 in both precisions.
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, FixedState
from ..kernels import ops
from ..weights.spec import NORMAL, ONE_PLUS_NORMAL, VECTOR, TensorSpec
from .base import Mixer
from .convolution import CausalConv
from .linear import Linear


class StackedTaps(CausalConv):
    """One causal convolution over several groups of channels side by side, each group's taps a checkpoint tensor of
    its own ([channels_i, taps]); on the device they are one [sum of channels, taps] tensor and one launch."""

    def __init__(self, names, channels, taps, state_name):
        super().__init__("|".join(names), sum(int(c) for c in channels), taps, state_name)
        self.tap_names, self.tap_channels = list(names), [int(c) for c in channels]

    def tensor_specs(self):
        return [TensorSpec(name, (c, self.taps), VECTOR, NORMAL) for name, c in zip(self.tap_names, self.tap_channels)]

    def bind(self, tensors, dtype, device):
        self.weight = torch.cat([tensors.pop(name) for name in self.tap_names], 0).contiguous()


class GatedDeltaRule(Mixer):
    STATE = "delta.s"
    CONV_STATE = "delta.conv"

    def __init__(self, prefix, hidden, heads, key_heads, dim, value_dim, taps, eps,
                 names=("q", "k", "v", "g", "b", "a", "o"), extras=("A_log", "dt_bias", "norm"), conv_suffix=".conv",
                 suffix=""):
        """taps: of the three convolutions; eps: of the per-head norm of the output; names: the checkpoint's names
        (behind the prefix) of the seven matrices, extras: of the per-head A_log and dt_bias and of the norm weight."""
        if heads % key_heads:
            raise ValueError("heads must be a multiple of key_heads")
        if not 1 <= int(dim) <= 256:
            raise ValueError("the delta rule's kernels take key sizes up to 256")
        self.prefix, self.names, self.extras = prefix, tuple(names), tuple(extras)
        self.hidden, self.heads, self.key_heads = int(hidden), int(heads), int(key_heads)
        self.dim, self.value_dim, self.eps = int(dim), int(value_dim), float(eps)
        H, G, D, E = self.heads, self.key_heads, self.dim, self.value_dim
        self.columns = {"q": 0, "k": G * D, "v": 2 * G * D, "g": 2 * G * D + H * E, "b": 2 * G * D + 2 * H * E,
                        "a": 2 * G * D + 2 * H * E + H}
        self.width = 2 * G * D + 2 * H * E + 2 * H
        self.proj = Linear([prefix + n for n in self.names[:6]], hidden, [G * D, G * D, H * E, H * E, H, H],
                           suffixes=(suffix, ".bias"))
        self.conv = StackedTaps([prefix + n + conv_suffix for n in self.names[:3]], [G * D, G * D, H * E], taps,
                                self.CONV_STATE)
        self.o = Linear([prefix + self.names[6]], H * E, [hidden], suffixes=(suffix, ".bias"))
        self.A_log = self.dt_bias = self.norm_weight = None

    def parts(self):
        return [self.proj, self.conv, self.o]

    def tensor_specs(self):
        p, (a_log, dt_bias, norm) = self.prefix, self.extras
        return (self.proj.tensor_specs() + self.conv.tensor_specs() + self.o.tensor_specs() +
                [TensorSpec(p + a_log, (self.heads,), VECTOR, NORMAL), TensorSpec(p + dt_bias, (self.heads,), VECTOR, NORMAL),
                 TensorSpec(p + norm, (self.value_dim,), VECTOR, ONE_PLUS_NORMAL)])

    def bind(self, tensors, dtype, device):
        self.proj.bind(tensors, dtype, device)
        self.conv.bind(tensors, dtype, device)
        self.o.bind(tensors, dtype, device)
        p, (a_log, dt_bias, norm) = self.prefix, self.extras
        self.A_log = tensors.pop(p + a_log).contiguous()
        self.dt_bias = tensors.pop(p + dt_bias).contiguous()
        self.norm_weight = tensors.pop(p + norm).contiguous()

    def weight_tensors(self):
        return [self.A_log, self.dt_bias, self.norm_weight]

    def cache_need(self):
        state = FixedState((self.heads, self.value_dim, ops.delta_key_extent(self.dim)), "float32")
        return CacheNeed(states=((self.STATE, state), self.conv.state_need()))

    def forward(self, ctx, run, h, x, accumulate=True):
        n, H, G, D, E = ctx.n_tokens, self.heads, self.key_heads, self.dim, self.value_dim
        col = self.columns
        proj = ctx.scratch("delta.proj", (n, self.width), torch.float32)
        self.proj.forward(ctx, h, proj)
        channels = self.conv.channels
        qkv = ctx.scratch("delta.qkv", (n, channels), torch.float32)
        self.conv.forward(ctx, run, proj[:, :channels], out32=qkv, activation="silu")
        result = ctx.scratch("delta.o", (n, H * E), torch.float32)
        state = ctx.cache.states[run.cache_slot][self.STATE]
        ops.delta_rule(qkv, col["q"], col["k"], col["v"], proj, col["b"], col["a"], self.A_log, self.dt_bias, state,
                       ctx.q_start, ctx.state_slots, 0, ctx.n_seqs, result, G, D, D ** -0.5, max_q_len=ctx.max_q_len)
        act = ctx.scratch("delta.act", (n, H * E))
        ops.head_norm_gate(result, proj[:, col["g"]:col["g"] + H * E], self.norm_weight, act, H, E, self.eps)
        self.o.forward(ctx, act, x, residual=x if accumulate else None)
        return None
