"""Token embedding and the output head (flow_engine/model.py:100,108-112,176,204).

The embedding is a row gather without scaling, into the float32 residual
stream. The head multiplies the normalised rows that were asked for by its
matrix and returns float32 logits; a tied head uses the embedding's matrix and
its own checkpoint key is accepted but never required.
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, FixedState
from ..kernels import ops
from ..weights.spec import MATRIX, NORMAL, TensorSpec
from .base import ROUNDED_STREAM, Part


class TokenEmbedding(Part):
    def __init__(self, name, vocab, hidden, suffix=".weight"):
        self.name, self.vocab, self.hidden = name, int(vocab), int(hidden)
        self.suffix = suffix
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name + self.suffix, (self.vocab, self.hidden), MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        self.weight = tensors.pop(self.name + self.suffix).contiguous()

    def forward(self, ctx):
        x = ctx.scratch("residual", (ctx.n_tokens, self.hidden), torch.float32)
        return ops.embed_gather(ctx.token_ids, self.weight, x, feed=ctx.token_feed)


class PositionedEmbedding(TokenEmbedding):
    """Token embedding plus a learned vector per position (not scaled): x = table[token] + positions[p].

    `keep` = (workspace tag, leading size): the sum is also written to the first rows of entry 0 of the float32
    scratch buffer [leading, largest step's rows, hidden] of that tag, for models whose later layers read the
    embedding output again."""

    def __init__(self, name, vocab, hidden, position_name, max_positions, suffix=".weight", keep=None):
        super().__init__(name, vocab, hidden, suffix)
        self.position_name, self.max_positions, self.keep = position_name, int(max_positions), keep
        self.positions = None

    def tensor_specs(self):
        return super().tensor_specs() + [TensorSpec(self.position_name + self.suffix, (self.max_positions, self.hidden),
                                                    MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        super().bind(tensors, dtype, device)
        self.positions = tensors.pop(self.position_name + self.suffix).contiguous()

    def forward(self, ctx):
        x = super().forward(ctx)
        copy = None
        if self.keep is not None:
            tag, leading = self.keep
            copy = ctx.workspace.get(tag, (leading, ctx.max_tokens, self.hidden), torch.float32)[0, :ctx.n_tokens]
        return ops.add_table_rows(x, self.positions, ctx.positions[0], copy=copy)


class HashedPairEmbedding(TokenEmbedding):
    """Token embedding times a scale, plus a row of a table indexed by a hash of (previous token, token), then a norm:

        x = norm( scale * table[token] + pairs[(previous * mul_prev + token * mul_cur) mod buckets] )

    A sequence's first token has no previous one and takes the pair table's last row (number `buckets`). The
    last token of a request is part of its state (`cache_need`: an int32 state in a cache slot of the part's
    own, which the model assigns), so a prompt cut into portions and a decoded token find their predecessor
    there. The state is held twice, as every state that one block of a launch reads and another writes. norm: an
    `RMSNorm` part (its weight and eps are used; embedding, sum and norm are one kernel). The normed row is left in
    the float32 residual stream and, rounded to the compute type, under `ctx.shared[ROUNDED_STREAM]`."""

    STATE = "last_token"

    def __init__(self, name, vocab, hidden, pair_name, buckets, mul_prev, mul_cur, norm, scale=1.0, suffix=".weight"):
        super().__init__(name, vocab, hidden, suffix)
        self.pair_name, self.buckets = pair_name, int(buckets)
        self.mul_prev, self.mul_cur, self.scale, self.norm = int(mul_prev), int(mul_cur), float(scale), norm
        if self.buckets <= 0 or self.mul_prev < 0 or self.mul_cur < 0:
            raise ValueError("buckets must be positive and the multipliers not negative")
        self.pairs = None
        self.cache_slot = None            # set by the model when it lays its cache out

    def parts(self):
        return [self.norm]

    def tensor_specs(self):
        return (super().tensor_specs() + [TensorSpec(self.pair_name + self.suffix, (self.buckets + 1, self.hidden), MATRIX, NORMAL)]
                + self.norm.tensor_specs())

    def bind(self, tensors, dtype, device):
        super().bind(tensors, dtype, device)
        self.pairs = tensors.pop(self.pair_name + self.suffix).contiguous()
        self.norm.bind(tensors, dtype, device)

    def cache_need(self):
        return CacheNeed(states=((self.STATE, FixedState((2,), "int32")),))

    def forward(self, ctx):
        if self.cache_slot is None:
            raise RuntimeError("the model has not given this embedding a cache slot (its cache layout was never asked for)")
        n = ctx.n_tokens
        x = ctx.scratch("residual", (n, self.hidden), torch.float32)
        rounded = ctx.scratch("stream.rounded", (n, self.hidden)) if ctx.dtype != torch.float32 else None
        state = ctx.cache.states[self.cache_slot][self.STATE]
        ops.embed_hashed(ctx.token_ids, self.weight, self.pairs, self.norm.weight, ctx.q_start, ctx.kv_len, ctx.state_slots,
                         ctx.state_phase, state, ctx.n_seqs, self.buckets, self.mul_prev, self.mul_cur, self.scale,
                         self.norm.eps, x, out=rounded, feed=ctx.token_feed)
        ctx.shared[ROUNDED_STREAM] = rounded if rounded is not None else x
        return x


class OutputHead(Part):
    def __init__(self, name, vocab, hidden, tied_to=None, suffix=".weight", scale=1.0, softcap=None):
        """scale: a factor on the logits, applied to the float32 product; softcap: the logits then pass
        softcap * tanh(logit / softcap)."""
        self.softcap = float(softcap) if softcap else 0.0
        self.name, self.vocab, self.hidden = name, int(vocab), int(hidden)
        self.suffix = suffix
        self.tied_to = tied_to
        self.scale = float(scale)
        self.weight = None

    def tensor_specs(self):
        if self.tied_to is not None:
            return [TensorSpec(self.name + self.suffix, (self.vocab, self.hidden), MATRIX, NORMAL,
                               optional_alias_of=self.tied_to.name + self.tied_to.suffix)]
        return [TensorSpec(self.name + self.suffix, (self.vocab, self.hidden), MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        # The head's matrix is kept in the matrix kernels' shuffled layout; a tied head makes its own
        # shuffled copy of the embedding (the gather reads rows, the head streams MFMA blocks).
        source = self.tied_to.weight if self.tied_to is not None else tensors.pop(self.name + self.suffix).contiguous()
        if torch.device(device).type == "cuda" and ops.can_shuffle(source):
            self.weight = ops.shuffle_weight(source)
        else:
            self.weight = source

    def matrix(self):
        return self.weight

    def weight_tensors(self):
        return [self.weight]          # (the embedding's table is not listed by its part: a step gathers a few rows of it)

    def forward(self, ctx, h):
        # The logits live in a shared scratch buffer: they are valid until the next step.
        logits = ctx.workspace.get("logits", (h.shape[0], self.vocab), torch.float32)
        ops.linear(h, self.matrix(), logits)
        if self.scale != 1.0:
            ops.scale_values(logits, self.scale)
        if self.softcap:
            ops.softcap_values(logits, self.softcap)
        return logits
