"""A plain, slow implementation of the Tadalorn decoder, one function per mechanism.

Written from the design's equations with ordinary tensor operations on whole sequences; it shares no
code with the package and keeps no cache: a sequence is always computed from its first token. The
tests compare the engine with it (prefill, decoding, portions and batches all have to give what this
gives for the whole sequence).

Notation: T tokens, C the model's width, H query heads, G key heads, D the query/key size of a head,
E its value size, R a rotated part, L a latent, V the vocabulary, F a feed-forward's inner size.
"""
from __future__ import annotations

import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_pairs(x, positions, dims, base):
    """x [T, heads, >= dims]: of the first `dims` elements of a head, element 2i turns with element 2i + 1 by the
    angle position * base^(-2i / dims); the rest pass. (A float32 run rounds the frequencies and the angles to
    float32: a thousand tokens in, an angle of hundreds of radians is then off by some 1e-5.)"""
    half = dims // 2
    f = (float(base) ** (-2.0 * torch.arange(half, dtype=torch.float64) / dims)).to(x.dtype)
    angle = positions.to(x.dtype).view(-1, 1, 1) * f.view(1, 1, -1)          # in the working precision, as everything
    cos, sin = torch.cos(angle), torch.sin(angle)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], -1).flatten(-2)
    return torch.cat([turned, x[..., dims:]], -1)


def causal_taps(u, w):
    """u [T, channels], w [channels, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    padded = torch.cat([u.new_zeros(taps - 1, u.shape[1]), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j]
    return y


def softmax_with_sink(scores, visible, sink):
    """Rows of `scores` [T, T] over the visible keys, with one more term exp(sink) in the denominator that has no
    value."""
    s = scores.masked_fill(~visible, -math.inf)
    top = torch.maximum(s.max(-1, keepdim=True).values, torch.as_tensor(sink, dtype=s.dtype))
    e = torch.exp(s - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))


def window_mask(T, size, keep_first):
    i, j = torch.arange(T).view(-1, 1), torch.arange(T).view(1, -1)
    return (j <= i) & ((i - j < size) | (j < keep_first))


def windowed_attention(h, w, m, eps):
    """Convolved q and k, values that are the convolved keys, norms over whole projections, rotation of pairs, a
    window that keeps the first tokens, a softmax with one added to its denominator, an output gate."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = causal_taps(h @ w["q"].T, w["q.conv"])
    k = causal_taps(h @ w["k"].T, w["k.conv"])
    v = k.view(T, G, D)
    q = rms_norm(q, w["q.norm"], eps).view(T, H, D)
    k = rms_norm(k, w["k.norm"], eps).view(T, G, D)
    pos = torch.arange(T)
    q = rotate_pairs(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_pairs(k, pos, m["rot"]["dims"], m["rot"]["base"])
    visible = window_mask(T, m["mask"]["size"], m["mask"]["keep_first"])
    out = torch.zeros(T, H, D, dtype=h.dtype)
    zero = torch.zeros((), dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        p = softmax_with_sink((q[:, a] @ k[:, g].T) * m["scale"], visible, zero)
        out[:, a] = p @ v[:, g]
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(T, -1) * gate) @ w["o"].T


def latent_attention(h, w, m, eps):
    """Causal attention whose keys and values are products of one normed latent per token, with one rotated key
    part for all heads, a learned sink per head and an output gate."""
    T = h.shape[0]
    H, D, R, E, L = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w["q"].T).view(T, H, D + R)
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :L], w["dkv.norm"], eps)
    pos = torch.arange(T)
    kr = rotate_pairs(down[:, L:].view(T, 1, R), pos, m["rot"]["dims"], m["rot"]["base"])[:, 0]
    qr = rotate_pairs(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    keys = (c @ w["uk"].T).view(T, H, D)
    values = (c @ w["uv"].T).view(T, H, E)
    visible = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for a in range(H):
        s = (q[:, a, :D] @ keys[:, a].T + qr[:, a] @ kr.T) * m["scale"]
        out[:, a] = softmax_with_sink(s, visible, w["sink"][a]) @ values[:, a]
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(T, -1) * gate) @ w["o"].T


def mlstm_steps(q, k, v, i_log, f_log):
    """The matrix memory token by token for one head. q, k [T, D], v [T, E], i_log, f_log [T].
    S [D, E], n [D] and the running maximum m all start at zero."""
    T, D = q.shape
    S, n, m = q.new_zeros(D, v.shape[1]), q.new_zeros(D), q.new_zeros(())
    out = []
    for t in range(T):
        m_new = torch.maximum(f_log[t] + m, i_log[t])
        keep, take = torch.exp(f_log[t] + m - m_new), torch.exp(i_log[t] - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        out.append((S.T @ q[t]) / (torch.maximum((n @ q[t]).abs(), torch.exp(-m)) + 1e-6))
    return torch.stack(out)


def mlstm(h, w, m, eps):
    T = h.shape[0]
    H, D, E, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, E)
    i_log = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)
    f_log = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    o = torch.stack([mlstm_steps(q[:, a], k[:, a], v[:, a], i_log[:, a], f_log[:, a]) for a in range(H)], 1)
    o = rms_unit(o, eps).reshape(T, H * E) * w["norm"]
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def dense_ff(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def plain_expert(h, up, down):
    return gelu_erf(h @ up.T) @ down.T


def router_margin(z, top):
    """Per token, how far the last chosen logit lies above the best one left out (infinite if all are chosen)."""
    if top >= z.shape[-1]:
        return torch.full(z.shape[:-1], math.inf, dtype=z.dtype)
    best = torch.topk(z, top + 1, dim=-1).values
    return best[..., top - 1] - best[..., top]


def routed_ff(h, w, mlp, margins=None):
    """Every token runs the `top` experts with the largest router logits, weighted by the softmax over those logits
    alone, and the shared expert if there is one."""
    T = h.shape[0]
    top = mlp["router"]["top"]
    z = h @ w["router"].T + w["router.b"]
    if margins is not None:
        margins.append(router_margin(z, top))
    best, ids = torch.topk(z, top, dim=-1)
    p = torch.softmax(best, -1)
    out = torch.zeros_like(h)
    for e in range(z.shape[-1]):
        share = (p * (ids == e)).sum(-1)                  # a token's weight for expert e, zero if it did not choose it
        rows = torch.nonzero((ids == e).any(-1)).flatten()
        if len(rows):
            out[rows] = out[rows] + share[rows, None] * plain_expert(h[rows], w[f"e{e}.up"], w[f"e{e}.down"])
    if mlp.get("shared") is not None:
        out = out + plain_expert(h, w["shared.up"], w["shared.down"])
    return out


MIXERS = {"attention": windowed_attention, "latent_attention": latent_attention, "mlstm": mlstm}


def sub(weights, prefix):
    """The tensors whose names start with `prefix`, by the rest of their names."""
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config, weights, tokens, dtype=torch.float64, layers_out=None, margins=None):
    """Logits [T, V] of a whole sequence. weights: name -> tensor (any float type). layers_out: a list that gets the
    stream after every layer; margins: a list that gets every routed layer's `router_margin` per token."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, mult = config["norm"]["eps"], config["residual_mult"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(config["layers"]):
        src = layer.get("weights_of", i)
        p = f"l{src}."
        y = MIXERS[layer["type"]](x, sub(w, p + "mix."), layer["mixer"], eps)
        x = x + mult * rms_norm(y, w[p + "norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            y = dense_ff(x, sub(w, p + "mlp.")) if mlp["kind"] == "dense" else routed_ff(x, sub(w, p + "mlp."), mlp, margins)
            x = x + mult * rms_norm(y, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_norm(x, w["final.norm"], eps)
    logits = x @ w["head"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
