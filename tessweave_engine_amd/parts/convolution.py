"""A short causal convolution over time, per channel, with the request's last inputs as state.

out_t = identity * v_t + sum_j w[:, j] * v_(t - K + 1 + j) (+ bias): the last column of w meets the current
token, rows before the sequence's start are zeros. v is the input itself, or its RMS norm (`norm=`), in
which case norm, convolution and the rounding to the compute type are one kernel. The last K - 1 values v
of a request are part of its state, kept in float32 and held twice (`FixedState` of shape [2, K - 1, C]):
a step reads the copy `ctx.state_phase` names and writes the other, so a prompt portion's first tokens
never read what its last tokens write.
"""
from __future__ import annotations

import torch

from ..cache.spec import FixedState
from ..kernels import ops
from ..weights.spec import NORMAL, VECTOR, TensorSpec
from .base import Part


class CausalConv(Part):
    def __init__(self, name, channels, taps, state_name, bias_name=None, identity=0.0, norm=None):
        """name: the checkpoint's [channels, taps] tensor; bias_name: its [channels] bias or None;
        state_name: under which name the block's cache need lists this part's state;
        norm: an `RMSNorm` over the same channels that the input passes first (fused)."""
        if not 1 <= int(taps) <= ops.CONV_MAX_TAPS:
            raise ValueError(f"a causal convolution has 1 to {ops.CONV_MAX_TAPS} taps")
        self.name, self.channels, self.taps = name, int(channels), int(taps)
        self.bias_name, self.identity, self.norm, self.state_name = bias_name, float(identity), norm, state_name
        self.weight = self.bias = None

    def parts(self):
        return [self.norm] if self.norm is not None else []

    def tensor_specs(self):
        specs = [TensorSpec(self.name, (self.channels, self.taps), VECTOR, NORMAL)]
        if self.bias_name:
            specs.append(TensorSpec(self.bias_name, (self.channels,), VECTOR, NORMAL))
        return specs + (self.norm.tensor_specs() if self.norm is not None else [])

    def bind(self, tensors, dtype, device):
        self.weight = tensors.pop(self.name).contiguous()
        self.bias = tensors.pop(self.bias_name).contiguous() if self.bias_name else None
        if self.norm is not None:
            self.norm.bind(tensors, dtype, device)

    def weight_tensors(self):
        return [self.weight] + ([self.bias] if self.bias is not None else [])

    def state_need(self):
        return (self.state_name, FixedState((2, max(self.taps - 1, 1), self.channels), "float32"))

    def forward(self, ctx, run, src, out=None, out32=None, activation=None):
        """src: float32 rows (with a norm: the residual stream) or rows of the compute type.
        activation "silu": the result passes SiLU before it is written."""
        state = ctx.cache.states[run.cache_slot][self.state_name]
        scratch = ctx.scratch("conv.rows", (src.shape[0],), torch.float32) if self.norm is not None else None
        ops.causal_conv(src, self.weight, state, ctx.q_start, ctx.kv_len, ctx.state_slots, ctx.state_phase, ctx.n_seqs,
                        out=out, out32=out32, norm_weight=self.norm.weight if self.norm is not None else None,
                        eps=self.norm.eps if self.norm is not None else 0.0, bias=self.bias, identity=self.identity,
                        row_scratch=scratch, activation=activation)
        return out if out is not None else out32
