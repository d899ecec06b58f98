"""Attention over a cached latent.

Every token leaves ONE normed vector c (L elements) and one rotated key part kr (R elements) that all heads share;
head a's key is [W_uk,a c | kr], its value W_uv,a c, its query [D unrotated | R rotated] elements:

    score_a(i, j) = scale * (q_plain,a(i) . W_uk,a c_j + q_turned,a(i) . kr_j),   causal softmax,   out = W_o [.. W_uv,a sum_j p c_j ..]

Only c and kr are cached; the engine's paged cache holds them like any other group (one key/value head whose key row
is [c | kr] and whose value is c). One-token sequences run the attention over that one head directly, for all query
heads at once: the products with W_uk and W_uv are moved to the query side and the output side (one small matrix per
head each, `ops.head_linear`), so a step reads every cached token once, at the latent's size. Prompt portions, with
many query rows against the same keys, go the other way round: the cached latents of their sequences are expanded
once a step (one product with [W_uk; W_uv] over the gathered key rows) into keys and values per head in scratch pages
of their own, and the engine's ordinary prompt attention runs on those. A layer may read the cache slot of another
layer (`LayerRun(writes_cache=False)`): it then has no down-projection of its own (`own_latent=False`) and uses that
layer's c and kr with its own queries and its own W_uk, W_uv.

Options: a learned sink per head (`sink_name`: exp(sink_a) more in head a's denominator, with no key and no value, not
scaled), an output gate (`gate_name`: the heads'
results times sigmoid(W_g h) before the output product), and a rotary encoding that pairs neighbouring elements: the
rotated rows of W_q and of the down-projection are then reordered once, when the weights are bound, into the order
that pairs element j with j + rot/2 (both sides of every score alike, so no score changes).
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, PagedKV
from ..kernels import ops
from ..weights.spec import MATRIX, NORMAL, ONE_PLUS_NORMAL, VECTOR, TensorSpec
from .base import Mixer
from .linear import Linear, pad_groups


def _round_up(v, m):
    return (int(v) + m - 1) // m * m


class LatentAttention(Mixer):
    def __init__(self, prefix, hidden, heads, dim, rot_dim, value_dim, latent, scale, position, eps, own_latent=True,
                 names=("q", "dkv", "dkv.norm", "uk", "uv", "o"), sink_name=None, gate_name=None):
        """position: a rotary encoding over `rot_dim` elements (its `rotary_dim` may be smaller: the rest of the
        rotated part passes unchanged). scale multiplies the scores as given."""
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.heads = int(hidden), int(heads)
        self.dim, self.rot_dim, self.value_dim, self.latent = int(dim), int(rot_dim), int(value_dim), int(latent)
        if min(self.heads, self.dim, self.rot_dim, self.value_dim, self.latent) <= 0:
            raise ValueError("heads and sizes must be positive")
        if position.rotary_dim <= 0 or position.rotary_dim > self.rot_dim:
            raise ValueError("the rotated part needs a rotary encoding of at most rot_dim elements")
        self.sink_name = prefix + sink_name if sink_name else None
        self.gate_name = prefix + gate_name if gate_name else None
        self.sink = None
        # sizes on the device: tails of zeros, which add nothing to a product
        self.dim_dev = _round_up(dim, 8)
        self.latent_dev, self.rot_dev = _round_up(latent, 16), _round_up(rot_dim, 16)
        self.key_dev = self.latent_dev + self.rot_dev
        # the size of an expanded head (prompt portions): keys [unrotated | rotated] and values side by side in one size
        self.value_dev = self.head_dev = _round_up(max(self.dim + self.rot_dim, self.value_dim), 16)
        if self.head_dev > 256:
            raise ValueError("the attention kernels take expanded heads (dim + rot_dim, value_dim) up to 256")
        # The one-head kernel of one-token sequences holds a key row's products in registers: latent + rotated part up
        # to 256 elements. A larger latent sends one-token sequences the prompt portions' way (expanded per step: right,
        # and slow; its scratch pages grow with the sequences, so such a model's steps are not replayed from graphs).
        self.one_head = self.key_dev <= 256
        if not self.one_head:
            self.graph_safe = False
        self.scale, self.eps, self.position, self.own_latent = float(scale), float(eps), position, bool(own_latent)
        self.proj = self.up = self.absorb = self.expand = self.latent_norm = None
        self.o = Linear([prefix + self.names[5]], heads * value_dim, [hidden], pad_in=(self.value_dim, self.value_dev),
                        suffixes=("", ".bias"))

    def _name(self, i):
        return self.prefix + self.names[i]

    def parts(self):
        # (`up`, the matrix of the prompt path, is a second arrangement of W_uk and W_uv, which `weight_tensors` already
        # names: a step reads one arrangement or the other, so it is not listed again)
        return [p for p in (self.proj, self.o, self.position) if p is not None]

    def tensor_specs(self):
        H, D, R, E, L, C = self.heads, self.dim, self.rot_dim, self.value_dim, self.latent, self.hidden
        specs = [TensorSpec(self._name(0), (H * (D + R), C), MATRIX, NORMAL)]
        if self.own_latent:
            specs += [TensorSpec(self._name(1), (L + R, C), MATRIX, NORMAL),
                      TensorSpec(self._name(2), (L,), VECTOR, ONE_PLUS_NORMAL)]
        specs += [TensorSpec(self._name(3), (H * D, L), MATRIX, NORMAL), TensorSpec(self._name(4), (H * E, L), MATRIX, NORMAL)]
        if self.sink_name:
            specs.append(TensorSpec(self.sink_name, (H,), VECTOR, NORMAL))
        if self.gate_name:
            specs.append(TensorSpec(self.gate_name, (H * E, C), MATRIX, NORMAL))
        return specs + self.o.tensor_specs()

    def bind(self, tensors, dtype, device):
        H, D, R, E, L = self.heads, self.dim, self.rot_dim, self.value_dim, self.latent
        Dp, Rp, Ep, Lp = self.dim_dev, self.rot_dev, self.value_dev, self.latent_dev
        q = tensors.pop(self._name(0)).view(H, D + R, self.hidden)
        # An encoding that pairs neighbours (2j with 2j + 1): the rotated rows are put into the order that pairs j with
        # j + rot/2, on the query side and the key side alike.
        order = list(range(R))
        if self.position.pairing == "adjacent":
            rot = self.position.rotary_dim
            order = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, R))
        turned = q[:, D:][:, order]
        # one packed product: [all heads' unrotated query parts | all heads' rotated parts | latent | shared key part | gate]
        rows = [pad_groups(q[:, :D].reshape(H * D, -1), 0, D, Dp), pad_groups(turned.reshape(H * R, -1), 0, R, Rp)]
        if self.own_latent:
            down = tensors.pop(self._name(1))
            rows += [pad_groups(down[:L], 0, L, Lp), pad_groups(down[L:][order], 0, R, Rp)]
            self.latent_norm = tensors.pop(self._name(2)).contiguous()
        self.q_col, self.c_col, self.kr_col = H * Dp, H * (Dp + Rp), H * (Dp + Rp) + Lp
        self.g_col = sum(r.shape[0] for r in rows)
        if self.gate_name:           # laid out like the heads' results
            rows.append(pad_groups(tensors.pop(self.gate_name), 0, E, Ep))
        if self.sink_name:
            self.sink = tensors.pop(self.sink_name).contiguous()
        packed = torch.cat(rows, 0).contiguous()
        self.proj_width = packed.shape[0]
        name = self.prefix + "packed"
        self.proj = Linear([name], self.hidden, [self.proj_width])
        self.proj.bind({name + ".weight": packed}, dtype, device)
        del q, rows, packed
        # query side: q_latent,a = W_uk,a^T q_plain,a ([Lp, Dp] per head); output side: W_uv,a ([Ep, Lp] per head)
        uk = tensors.pop(self._name(3)).view(H, D, L)
        self.absorb = uk.new_zeros(H, Lp, Dp)
        self.absorb[:, :L, :D] = uk.transpose(1, 2)
        uv = tensors.pop(self._name(4)).view(H, E, L)
        self.expand = uv.new_zeros(H, Ep, Lp)
        self.expand[:, :E, :L] = uv
        # prompt portions: [W_uk; W_uv] over the latent as one matrix (the heads' key parts, then their value parts)
        both = uk.new_zeros(H * (D + E), Lp)
        both[:H * D, :L] = uk.reshape(H * D, L)
        both[H * D:, :L] = uv.reshape(H * E, L)
        name = self.prefix + "expand"
        self.up = Linear([name], Lp, [H * (D + E)])
        self.up.bind({name + ".weight": both}, dtype, device)
        del both
        self.o.bind(tensors, dtype, device)
        self.position.bind(tensors, dtype, device)

    def weight_tensors(self):
        return [t for t in (self.absorb, self.expand, self.latent_norm, self.sink) if t is not None]

    def cache_need(self):
        return CacheNeed(paged=PagedKV(1, self.key_dev, None, self.latent_dev))

    def forward(self, ctx, run, h, x, accumulate=True):
        if run.writes_cache != self.own_latent:
            raise RuntimeError("a layer with a latent of its own writes its cache slot; one without reads another layer's")
        n, H = ctx.n_tokens, self.heads
        nd = ctx.n_decode if self.one_head else 0          # sequences that take the one-head kernel
        Lp, Rp, K, hd = self.latent_dev, self.rot_dev, self.key_dev, self.head_dev
        portions = ctx.n_seqs - nd
        longest_portion = max(ctx.max_q_len, 1)
        proj = ctx.scratch("latent.proj", (n, self.proj_width))
        self.proj.forward(ctx, h, proj)
        cos, sin = self.position.tables(ctx)
        keys, values, g = ctx.cache.keys_values(run.cache_slot)
        page = ctx.cache.page_size
        values = values.view(values.shape[0], 1, Lp, page)
        group = ctx.groups[g]
        q = ctx.scratch("latent.q", (n, H * K))
        q_full = ctx.scratch("latent.q_full", (n, H * hd)) if portions else None
        store = dict(keys=keys, values=values, slots=group.slot_mapping) if self.own_latent else {}
        ops.latent_finish(proj, self.q_col, self.c_col, self.kr_col, cos, sin, self.latent_norm, q, H, self.latent, Lp, Rp,
                          self.eps, q_full=q_full, dim=self.dim, dim_dev=self.dim_dev, full_from=nd, **store)
        out = ctx.scratch("latent.out", (n, H * hd))
        if nd:
            # one-token sequences: all heads over the one cached head, W_uk on the query side, W_uv on the output side
            ops.head_linear(proj[:nd], self.dim_dev, self.absorb, q[:nd], K)
            mixed = ctx.scratch("latent.mixed", (n, H * Lp))[:nd]
            longest = ctx.kv_bound if ctx.capturing else ctx.max_kv_len
            splits = ops.latent_decode_splits(nd, H, longest)
            ws = None
            if splits > 1:
                # sized for the most splits any length class can ask for, so that it never grows under a capture
                floats = ops.latent_decode_workspace_floats(nd, H, Lp, max(splits, ops.latent_decode_splits(nd, H, ctx.kv_capacity)))
                ws = ctx.workspace.get("latent.split", (floats,), torch.float32)
            ops.latent_decode(q[:nd], keys, values, group.block_table, ctx.q_start, ctx.kv_len, nd, mixed, H, self.scale,
                              splits=splits, workspace=ws, sink=self.sink)
            ops.head_linear(mixed, Lp, self.expand, out[:nd], hd)
        if portions:
            # prompt portions: their sequences' cached latents expanded per head into pages of this step's own
            own_pages = ctx.h_kv_page_start[ctx.n_seqs] - ctx.h_kv_page_start[nd]
            rows = ctx.workspace.get("latent.rows", (own_pages * page, K), ctx.dtype)
            own_table = ctx.workspace.get("latent.table", (ctx.n_seqs, group.block_table.shape[1]), torch.int32)
            ops.latent_gather(keys, group.block_table, ctx.kv_len, ctx.kv_page_start, nd, portions, own_pages, rows, own_table)
            up = ctx.workspace.get("latent.up", (own_pages * page, H * (self.dim + self.value_dim)), ctx.dtype)
            self.up.forward(ctx, rows[:, :Lp], up)
            own_keys = ctx.workspace.get("latent.keys", (own_pages, H, page, hd), ctx.dtype)
            own_values = ctx.workspace.get("latent.values", (own_pages, H, hd, page), ctx.dtype)
            ops.latent_expand_store(up, rows, Lp, own_keys, own_values, H, self.dim, self.rot_dim, self.value_dim)
            split = ops.attn_prefill_split(portions, H, H, longest_portion, ctx.max_kv_len)
            ws = None
            if split[0] > 1:
                ws = ctx.workspace.get("attn.prefill_split", (ops.attn_prefill_workspace_floats(n, H, hd, split[0]),), torch.float32)
            ops.attn_prefill(q_full, own_keys, own_values, own_table, ctx.q_start, ctx.kv_len, nd,
                             portions, longest_portion, out, H, H, hd, self.scale, split=split, workspace=ws, sink=self.sink)
        if self.gate_name:
            ops.sigmoid_gate(out, proj[:, self.g_col:self.g_col + H * hd])
        if ctx.defer_sums and self.o.deferrable(n):
            return self.o.forward_partials(ctx, out, "o")          # whoever norms next adds them up
        self.o.forward(ctx, out, x, residual=x if accumulate else None)
        return None
