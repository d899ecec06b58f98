"""A plain, slow implementation of the Rufusun decoder, one function per mechanism.

Written from the design's equations with ordinary tensor operations on whole sequences; it shares no
code with the package and keeps no cache: a sequence is always computed from its first token. The
tests compare the engine with it (prefill, decoding, portions and batches all have to give what this
gives for the whole sequence).

Notation: T tokens, C the model's width, H query (or value) heads, G key heads, D the query/key size of
a head, E its value size, V the vocabulary, F a feed-forward's inner size.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_half(x, positions, dims, base):
    """x [T, heads, >= dims]: the first `dims` elements of a head turn, element i with i + dims / 2, by
    the angle position * base^(-2i / dims); the rest pass."""
    half = dims // 2
    f = float(base) ** (-2.0 * torch.arange(half, dtype=torch.float64) / dims)
    angle = (positions.to(torch.float64).view(-1, 1, 1) * f.view(1, 1, -1))
    cos, sin = torch.cos(angle).to(x.dtype), torch.sin(angle).to(x.dtype)
    u, v, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], -1)


def capped_attention(h, w, m):
    """Causal softmax attention with biased projections, partial rotation, a given scale and a soft cap of
    the scores. w: the layer's mixer tensors by their short names ('q', 'q.b', ...), m: its sizes."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).view(T, H, D)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, D)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, E)
    pos = torch.arange(T)
    q = rotate_half(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_half(k, pos, m["rot"]["dims"], m["rot"]["base"])
    out = torch.zeros(T, H, E, dtype=h.dtype)
    visible = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        cap = m.get("softcap")
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~visible, float("-inf"))
        out[:, a] = torch.softmax(s, -1) @ v[:, g]
    return out.reshape(T, H * E) @ w["o"].T + w["o.b"]


def short_conv(x, taps):
    """x [T, channels], taps [channels, K]: causal convolution over time per channel; the last column of
    `taps` meets the current token, zeros stand before the start."""
    T, K = x.shape[0], taps.shape[1]
    padded = torch.cat([x.new_zeros(K - 1, x.shape[1]), x], 0)
    out = torch.zeros_like(x)
    for j in range(K):
        out = out + padded[j:j + T] * taps[:, j]
    return out


def delta_rule(q, k, v, beta, decay):
    """The gated delta rule of one head, token by token. q, k [T, D], v [T, E], beta, decay [T].
    S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, D = q.shape
    S = q.new_zeros(D, v.shape[1])
    out = []
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def delta_mixer(h, w, m, eps):
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = F.silu(short_conv(h @ w["q"].T, w["q.conv"])).view(T, G, D)
    k = F.silu(short_conv(h @ w["k"].T, w["k.conv"])).view(T, G, D)
    v = F.silu(short_conv(h @ w["v"].T, w["v.conv"])).view(T, H, E)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)                                                   # [T, H]
    decay = torch.exp(-torch.exp(w["A_log"]) * F.softplus(h @ w["a"].T + w["dt_bias"]))  # [T, H]
    gate = F.silu(h @ w["g"].T).view(T, H, E)
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        o = delta_rule(q[:, g], k[:, g], v[:, a], beta[:, a], decay[:, a])
        out[:, a] = rms_unit(o, eps) * w["norm"] * gate[:, a]
    return out.reshape(T, H * E) @ w["o"].T


def dense_ffn(h, w):
    return (F.silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def limited_expert(h, gate, up, down, limit):
    g = (h @ gate.T).clamp(max=limit)
    u = (h @ up.T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def routed_ffn(h, w, mlp):
    """Experts chosen by the largest sigmoid scores; a score multiplies its expert's INPUT; not renormalised;
    a shared expert is added for every token."""
    n, top = mlp["router"]["experts"], mlp["router"]["top"]
    scores = torch.sigmoid(h @ w["router"].T)
    chosen = torch.topk(scores, top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += limited_expert(scores[t, e] * h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"],
                                     mlp["expert"]["limit"])
    if mlp.get("shared"):
        out = out + limited_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"], mlp["shared"]["limit"])
    return out


def router_margin(h, w, mlp):
    """Per token: how far the last chosen expert's router logit lies above the best one not chosen (inf if all run)."""
    top = mlp["router"]["top"]
    z = torch.sort(h @ w["router"].T, -1, descending=True).values
    if top >= z.shape[1]:
        return torch.full((h.shape[0],), float("inf"), dtype=h.dtype)
    return z[:, top - 1] - z[:, top]


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer_order(config):
    """Indices of the layers in the order they run: layers start .. stop - 1 `times` times in a row."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(config, tensors, tokens, keep_layers=False, margins=None):
    """Logits [T, V] of a whole sequence (and, with keep_layers, the stream after every layer run). margins: a list
    that receives, per run of a layer with routed experts, every token's `router_margin`."""
    eps = config["norm"]["eps"]
    x = tensors["embed"][torch.tensor([int(t) for t in tokens], dtype=torch.long)]
    kept = []
    for i in layer_order(config):
        layer, p = config["layers"][i], f"l{i}."
        h1 = offset_norm(x, tensors[p + "norm1"], eps)
        mix = sub(tensors, p + "mix.")
        if layer["type"] == "attention":
            y = capped_attention(h1, mix, layer["mixer"])
        elif layer["type"] == "delta":
            y = delta_mixer(h1, mix, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp:
            h2 = offset_norm(x, tensors[p + "norm2"], eps)        # of the same x as the mixer's norm
            w = sub(tensors, p + "mlp.")
            y = y + (dense_ffn(h2, w) if mlp["kind"] == "dense" else routed_ffn(h2, w, mlp))
            if margins is not None and mlp["kind"] != "dense":
                margins.append(router_margin(h2, w, mlp))
        x = x + y
        kept.append(x)
    logits = (offset_norm(x, tensors["final.norm"], eps) @ tensors["head"].T) * config["logit_scale"]
    return (logits, torch.stack(kept)) if keep_layers else logits
