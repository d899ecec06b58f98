"""Small Tadalorn configurations and weights made for testing.

The configurations differ from each other in every size, in the order of their layers and in what the design allows
to be absent, equal or one (a layer without a feed-forward, experts without a shared one, all experts chosen, one
head, one key head for all heads and one for each, a rotation over part of a head, a window shorter than a page, kept
first tokens that fill more than a page or none at all, a convolution of one tap, layers that run with another layer's
weights, sizes that are no multiples of 16, 8 or 4). Weights are drawn so that every path matters: norm weights away
from one, forget gates close to one (a lost state shows hundreds of tokens later), router rows and biases that spread
the tokens over the experts, sinks of both signs.
"""
from __future__ import annotations

import math

import torch

from kanavik_util import Driver, row_error, write_folder  # noqa: F401  (the same driver of the package's step function)


def attention(heads, kv_heads, dim, rot_dims, scale, conv, size, keep_first, base=10000.0, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "conv": conv,
         "mask": {"size": size, "keep_first": keep_first}, "rot": {"base": base, "dims": rot_dims}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, rot_dims=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dims or rot_dim}}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def mlstm(heads, dim, vdim, gate_cap, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, "mlp": mlp}


def same_as(layer, source):
    d = dict(layer)
    d["weights_of"] = source
    return d


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    d = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def config(layers, width, vocab, mult=1.0, softcap=None, eps=1e-5):
    c = {"architecture": "Tadalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}
    if softcap:
        c["logit_softcap"] = softcap
    return c


# head sizes that are no multiples of 16; a window shorter than a page with three kept tokens; the first attention layer
# runs a second time with its weights and a cache of its own; two of five experts and three of three; a latent layer
# without a feed-forward; one mLSTM head of odd sizes
_A = attention(6, 3, 24, 16, 0.3, 4, 9, 3, base=100.0, mlp=dense(136))
CONFIG_ODD = config([_A,
                     mlstm(3, 20, 24, 8.0, mlp=moe(5, 2, 40, shared=56)),
                     latent(3, 24, 8, 40, 48, 0.2, base=500.0, mlp=moe(3, 3, 24)),
                     same_as(_A, 0),
                     latent(2, 16, 16, 8, 20, 0.35),
                     mlstm(1, 13, 10, 3.0, mlp=dense(50))],
                    width=88, vocab=211, mult=0.7, softcap=9.0)
# latent first; many experts; one key head per head; a convolution of one tap; more kept tokens than a page holds and
# than the window is long; no kept tokens; a rotation over half of the rotated part; a key size of 128; no soft cap
_L = latent(8, 32, 32, 32, 96, 0.2, base=1e6, rot_dims=16, mlp=moe(16, 4, 64, shared=32))
CONFIG_WIDE = config([_L,
                      attention(8, 8, 32, 32, 0.2, 1, 64, 0, base=1e6, mlp=dense(192)),
                      mlstm(2, 128, 64, 15.0, mlp=moe(4, 1, 32)),
                      same_as(_L, 0),
                      attention(4, 1, 64, 32, 0.11, 3, 5, 20, base=1e4, mlp=dense(200)),
                      mlstm(4, 32, 80, 6.0)],
                     width=128, vocab=300, mult=1.0, eps=1e-6)
# one mLSTM layer and nothing else; sizes that are no multiples of 4
CONFIG_ONE = config([mlstm(2, 13, 10, 5.0)], width=48, vocab=97, mult=0.4, softcap=30.0)

CONFIGS = {"odd": CONFIG_ODD, "wide": CONFIG_WIDE, "one": CONFIG_ONE}


def tensor_shapes(c):
    """Names and shapes of a checkpoint, written from the design's naming and not from the package's parts."""
    C = c["width"]
    shapes = {"embed": (c["vocab"], C), "head": (c["vocab"], C), "final.norm": (C,)}
    for i, lay in enumerate(c["layers"]):
        if lay.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", lay["mixer"]
        H, D, E = m["heads"], m["dim"], m["vdim"]
        shapes[p + "norm1"] = (C,)
        q = p + "mix."
        if lay["type"] == "attention":
            G, K = m["kv_heads"], m["conv"]
            shapes.update({q + "q": (H * D, C), q + "k": (G * D, C), q + "q.conv": (H * D, K), q + "k.conv": (G * D, K),
                           q + "q.norm": (H * D,), q + "k.norm": (G * D,), q + "g": (H * E, C), q + "o": (C, H * E)})
        elif lay["type"] == "latent_attention":
            R, L = m["rot_dim"], m["kv_rank"]
            shapes.update({q + "q": (H * (D + R), C), q + "dkv": (L + R, C), q + "dkv.norm": (L,), q + "uk": (H * D, L),
                           q + "uv": (H * E, L), q + "sink": (H,), q + "g": (H * E, C), q + "o": (C, H * E)})
        else:
            shapes.update({q + "q": (H * D, C), q + "k": (H * D, C), q + "v": (H * E, C), q + "g": (H * E, C), q + "o": (C, H * E),
                           q + "norm": (H * E,), q + "i": (H, C), q + "i.b": (H,), q + "f": (H, C), q + "f.b": (H,)})
        mlp = lay["mlp"]
        if mlp:
            shapes[p + "norm2"] = (C,)
            q = p + "mlp."
            if mlp["kind"] == "dense":
                F = mlp["ff"]
                shapes.update({q + "gate": (F, C), q + "up": (F, C), q + "down": (C, F)})
            else:
                F = mlp["expert"]["ff"]
                shapes[q + "router"] = (mlp["router"]["experts"], C)
                shapes[q + "router.b"] = (mlp["router"]["experts"],)
                for e in range(mlp["router"]["experts"]):
                    shapes.update({q + f"e{e}.up": (F, C), q + f"e{e}.down": (C, F)})
                if mlp.get("shared"):
                    F = mlp["shared"]["ff"]
                    shapes.update({q + "shared.up": (F, C), q + "shared.down": (C, F)})
    return shapes


def make_weights(c, seed, sharp=1.0):
    """{name: bfloat16 tensor}: what a checkpoint of configuration C holds. SHARP multiplies what scales an attention
    layer's scores (the whole-row query norm's weight; a latent layer's query matrix): above one, a softmax
    concentrates on its best key, wherever that lies."""
    g = torch.Generator().manual_seed(seed)
    kinds = {f"l{i}.": lay["type"] for i, lay in enumerate(c["layers"])}
    out = {}
    for name, shape in tensor_shapes(c).items():
        parts = name.split(".")
        leaf = parts[-1]
        kind = kinds.get(parts[0] + ".", "")
        normal = torch.randn(shape, generator=g)
        if name == "embed":
            t = normal
        elif leaf in ("norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.3 * normal
        elif leaf == "norm":
            t = 1.0 + 0.3 * normal
            if kind == "attention" and parts[-2] == "q":
                t = t * sharp
        elif leaf == "conv":
            t = 0.6 * normal
        elif leaf == "sink":
            t = 1.5 * normal
        elif leaf == "router":
            t = 3.0 * normal / math.sqrt(shape[-1])
        elif leaf == "b" and parts[-2] == "router":
            t = 0.5 * normal
        elif leaf == "b" and parts[-2] == "f":
            t = 4.0 + normal                                   # forget gates of 0.95 to 0.999: the state remembers
        elif leaf == "b":
            t = 0.5 * normal
        else:                                                  # linear maps [out, in]
            t = normal / math.sqrt(shape[-1])
            if kind == "latent_attention" and leaf == "q":
                t = t * sharp
            if leaf in ("i", "f") and kind == "mlstm":
                t = t * 2.0                                    # the gates move, and meet their cap now and then
        out[name] = t.to(torch.bfloat16)
    return out
