"""Attention whose queries and keys pass short causal convolutions and whole-row norms, and whose values are its keys.

    q = conv_q(W_q h), k = conv_k(W_k h)         a causal convolution over time per channel, its last inputs are state
    v = k                                         as it leaves the convolution: no value matrix
    q <- rotate(w_q * unit(q)), k <- rotate(w_k * unit(k))     unit(.) over ALL heads of the row at once, then the rotation
    position i sees j <= i with i - j < window, and the sequence's first `keep_first` positions whatever the distance
    p_j = exp(s_j) / (exp(sink) + sum_j' exp(s_j')),   s = scale * q . k      (sink: one fixed score without a value)
    out = W_o ( [heads' sums of p v] * sigmoid(W_g h) )

Query head a reads key head a // (heads / kv_heads). Keys and values are paged like every attention layer's (a windowed
cache group that never gives back the pages of the kept first tokens); the convolutions' last inputs are a float32
state of the cache slot. Convolutions, norms, angles, scores and the softmax are float32 in both precisions.

Two attention kernels serve it, both on the same pages. One-token sequences run the kernel that knows kept first keys
(`ops.attn_mixed`). Prompt portions run the engine's prompt kernel (`ops.attn_prefill`) over the window, with the sink;
in steps in which some query's window may have passed a kept token the prompt kernel leaves each row's softmax statistics
instead, and a small kernel (`ops.attn_kept_keys`) adds the kept keys in front of the row's window, and the sink.
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, PagedKV
from ..kernels import ops
from ..weights.spec import ONE_PLUS_NORMAL, VECTOR, TensorSpec
from .base import Mixer
from .delta import StackedTaps
from .linear import Linear


def _round_up(v, m):
    return (int(v) + m - 1) // m * m


def mixed_attention(ctx, q, keys, values, group, out, q_heads, kv_heads, value_dev, scale, window=0, keep_first=0, sink=None,
                    tag="attn.window", portions=True):
    """The step's one-token sequences and (unless portions=False) its prompt portions through the attention kernel that
    takes a window, kept first keys and a sink. keys [pages, kv_heads, page, key_dev], values [pages, kv_heads,
    value_dev, page]."""
    common = dict(window=window, keep_first=keep_first, sink=sink)
    span = window + _round_up(keep_first, 16) if window else 0        # most keys a query walks
    if ctx.n_decode:
        # A captured step is replayed for other lengths: its split count follows the step's length class.
        longest = ctx.kv_bound if ctx.capturing else ctx.max_kv_len
        most = ctx.kv_capacity
        if window:
            longest, most = min(longest, span), min(most, span)
        splits = ops.attn_mixed_splits(ctx.n_decode, longest)
        ws = None
        if splits > 1:
            # sized for the most splits any length class can ask for, so that it never grows under a capture
            floats = ops.attn_mixed_workspace_floats(ctx.n_decode, 1, q_heads, value_dev,
                                                     max(splits, ops.attn_mixed_splits(ctx.n_decode, most)))
            ws = ctx.workspace.get(tag + ".split", (floats,), torch.float32)
        ops.attn_mixed(q, keys, values, group.block_table, ctx.q_start, ctx.kv_len, 0, ctx.n_decode, 1, out, q_heads,
                       kv_heads, scale, splits=splits, workspace=ws, **common)
    if portions and ctx.n_seqs > ctx.n_decode:
        n_seqs = ctx.n_seqs - ctx.n_decode
        longest = min(ctx.max_kv_len, span + ctx.max_q_len) if window else ctx.max_kv_len
        splits = ops.attn_mixed_prefill_splits(ctx.n_tokens - ctx.n_decode, n_seqs, longest)
        ws = None
        if splits > 1:
            floats = ops.attn_mixed_workspace_floats(n_seqs, ctx.max_q_len, q_heads, value_dev, splits)
            ws = ctx.workspace.get(tag + ".split.rows", (floats,), torch.float32)
        ops.attn_mixed(q, keys, values, group.block_table, ctx.q_start, ctx.kv_len, ctx.n_decode, n_seqs, ctx.max_q_len,
                       out, q_heads, kv_heads, scale, splits=splits, workspace=ws, **common)
    return out


class ConvolvedWindowAttention(Mixer):
    CONV_STATE = "attention.conv"
    MAX_HEADS = 32                  # what the attention kernel's workgroup holds

    def __init__(self, prefix, hidden, q_heads, kv_heads, dim, position, taps, eps, window=None, keep_first=0, scale=None,
                 sink=0.0, names=("q", "k", "g", "o"), conv_suffix=".conv", norm_suffix=".norm", suffix=""):
        """position: a rotary encoding over at most `dim` elements (either pairing) or a `NoPositionEncoding`;
        taps: of the two convolutions; eps: of the two whole-row norms; window None: every earlier position is seen;
        sink: the fixed score in the softmax's denominator (0.0 adds one to it), None for none."""
        if q_heads % kv_heads:
            raise ValueError("q_heads must be a multiple of kv_heads")
        if not 1 <= int(dim) <= 256 or not 1 <= int(q_heads) <= self.MAX_HEADS:
            raise ValueError(f"the attention kernel takes head sizes up to 256 and up to {self.MAX_HEADS} heads")
        if position.rotary_dim > dim:
            raise ValueError("the rotary encoding must cover at most dim elements")
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.q_heads, self.kv_heads, self.dim = int(hidden), int(q_heads), int(kv_heads), int(dim)
        self.dim_dev = _round_up(dim, 16)
        self.position, self.eps = position, float(eps)
        self.window = int(window) if window else None
        self.keep_first = int(keep_first) if self.window else 0
        self.scale = float(scale) if scale is not None else self.dim ** -0.5
        self.sink_value = None if sink is None else float(sink)
        H, G, D = self.q_heads, self.kv_heads, self.dim
        q, k, g, o = (prefix + n for n in self.names)
        # one packed product with float32 rows: [q | k | gate], the gate's heads laid out like the attention's output
        self.proj = Linear([q, k, g], hidden, [H * D, G * D, H * D], pad_out=[None, None, (D, self.dim_dev)],
                           suffixes=(suffix, ".bias"))
        self.gate_col = (H + G) * D
        self.width = self.gate_col + H * self.dim_dev
        self.conv = StackedTaps([q + conv_suffix, k + conv_suffix], [H * D, G * D], taps, self.CONV_STATE)
        self.norm_names = (q + norm_suffix, k + norm_suffix)
        self.o = Linear([o], H * D, [hidden], pad_in=(D, self.dim_dev), suffixes=(suffix, ".bias"))
        self.q_weight = self.k_weight = self.sink = None

    def parts(self):
        return [self.proj, self.conv, self.o, self.position]

    def tensor_specs(self):
        H, G, D = self.q_heads, self.kv_heads, self.dim
        return (self.proj.tensor_specs() + self.conv.tensor_specs() + self.o.tensor_specs() +
                [TensorSpec(self.norm_names[0], (H * D,), VECTOR, ONE_PLUS_NORMAL),
                 TensorSpec(self.norm_names[1], (G * D,), VECTOR, ONE_PLUS_NORMAL)])

    def bind(self, tensors, dtype, device):
        self.proj.bind(tensors, dtype, device)
        self.conv.bind(tensors, dtype, device)
        self.o.bind(tensors, dtype, device)
        self.position.bind(tensors, dtype, device)
        self.q_weight = tensors.pop(self.norm_names[0]).contiguous()
        self.k_weight = tensors.pop(self.norm_names[1]).contiguous()
        if self.sink_value is not None:          # a constant of the design, one a head for the kernel
            self.sink = torch.full((self.q_heads,), self.sink_value, dtype=torch.float32, device=device)

    def weight_tensors(self):
        return [self.q_weight, self.k_weight]

    def cache_need(self):
        paged = PagedKV(self.kv_heads, self.dim_dev, self.window, None, self.keep_first)
        return CacheNeed(paged=paged, states=(self.conv.state_need(),))

    def forward(self, ctx, run, h, x, accumulate=True):
        n, H, G, D, Dp = ctx.n_tokens, self.q_heads, self.kv_heads, self.dim, self.dim_dev
        proj = ctx.scratch("window.proj", (n, self.width), torch.float32)
        self.proj.forward(ctx, h, proj)
        channels = self.conv.channels
        qk = ctx.scratch("window.qk", (n, channels), torch.float32)
        self.conv.forward(ctx, run, proj[:, :channels], out32=qk)
        cos, sin = self.position.tables(ctx)
        keys, values, g = ctx.cache.keys_values(run.cache_slot)
        pages = values
        values = values.view(values.shape[0], G, Dp, ctx.cache.page_size)
        group = ctx.groups[g]
        q = ctx.scratch("window.q", (n, H * Dp))
        ops.qk_finish(qk, 0, H * D, self.q_weight, self.k_weight, cos, sin, q, keys, values, group.slot_mapping, H, G, D,
                      self.position.rotary_dim, self.eps, adjacent=self.position.pairing == "adjacent")
        out = ctx.scratch("window.out", (n, H * Dp))
        window, portions = self.window or 0, ctx.n_seqs - ctx.n_decode
        mixed_attention(ctx, q, keys, values, group, out, H, G, Dp, self.scale, window=window, keep_first=self.keep_first,
                        sink=self.sink, portions=False)
        if portions:
            all_seen = not window or ctx.max_kv_len <= window      # no query of the step has a key behind its window
            seen = 0 if all_seen else window
            kept = bool(seen and self.keep_first)                  # some window may have passed a kept token
            longest = min(ctx.max_kv_len, seen + ctx.max_q_len) if seen else ctx.max_kv_len
            split = ops.attn_prefill_split(portions, H, G, ctx.max_q_len, longest)
            ws = None
            if split[0] > 1:
                ws = ctx.workspace.get("attn.prefill_split", (ops.attn_prefill_workspace_floats(n, H, Dp, split[0]),), torch.float32)
            stats = ctx.scratch("window.stats", (n, H, 2), torch.float32) if kept else None
            ops.attn_prefill(q, keys, pages, group.block_table, ctx.q_start, ctx.kv_len, ctx.n_decode, portions, ctx.max_q_len,
                             out, H, G, Dp, self.scale, window=seen, split=split, workspace=ws,
                             sink=None if kept else self.sink, stats=stats)
            if kept:       # the kept keys in front of the rows' windows, and the sink
                first_row = ctx.h_q_start[ctx.n_decode]
                ops.attn_kept_keys(q, keys, pages, group.block_table, ctx.q_start, ctx.kv_len, ctx.n_decode, portions, first_row,
                                   n - first_row, out, stats, H, G, Dp, self.scale, window, self.keep_first, sink=self.sink)
        ops.sigmoid_gate(out, proj[:, self.gate_col:])
        if ctx.defer_sums and self.o.deferrable(n):
            return self.o.forward_partials(ctx, out, "o")          # whoever norms next adds them up
        self.o.forward(ctx, out, x, residual=x if accumulate else None)
        return None
