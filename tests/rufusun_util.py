"""Small Rufusun configurations and weights made for testing.

The configurations differ from each other in every size, in the order of their layers and in what the design allows
to be absent or equal (a layer without a feed-forward, experts without a shared one, all experts chosen, a rotation
that covers part of a head, no soft cap, values larger and smaller than keys, one key head for all heads and one for
each, a convolution of one tap, a loop over both kinds of layer, no loop, sizes that are no multiples of 16, 8 or 4).
Weights are drawn so that every path matters: norm weights far from zero, decays close to one (a lost state shows
hundreds of tokens later), router rows that spread the tokens over the experts, gate and up values beyond the limits.
"""
from __future__ import annotations

import math

import torch

from kanavik_util import Driver, row_error, write_folder  # noqa: F401  (the same driver of the package's step function)


def attention(heads, kv_heads, dim, vdim, rot_dims, scale, softcap=None, base=10000.0, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
         "rot": {"base": base, "dims": rot_dims}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def delta(heads, kv_heads, dim, vdim, conv, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit, shared=None):
    d = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        d["shared"] = {"ff": shared[0], "limit": shared[1]}
    return d


def config(layers, width, vocab, logit_scale, loop=None, eps=1e-5):
    c = {"architecture": "Rufusun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
         "layers": layers}
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


# attention first; head sizes that are no multiples of 16, values larger than keys and smaller; a rotation over part of
# a head; two of five experts and three of three; a delta layer with two blocks of value columns and no feed-forward;
# the loop repeats a delta layer and an attention layer (pages and state of their own per pass)
CONFIG_ODD = config([attention(6, 3, 24, 40, 16, 0.3, softcap=5.0, base=100.0, mlp=dense(136)),
                     delta(4, 2, 20, 24, 4, mlp=moe(5, 2, 40, 1.2, shared=(56, 0.8))),
                     delta(3, 3, 40, 72, 2),
                     attention(2, 1, 16, 8, 8, 0.45, base=500.0, mlp=moe(3, 3, 24, 2.5))],
                    width=88, vocab=211, logit_scale=0.7, loop=(2, 4, 2))
# delta first; many experts; one key head per head in attention; a convolution of one tap; a key size of 128; no loop
CONFIG_WIDE = config([delta(8, 2, 64, 32, 4, mlp=dense(192)),
                      attention(8, 8, 32, 32, 32, 0.2, softcap=50.0, base=1e6, mlp=moe(16, 4, 64, 7.0, shared=(32, 3.0))),
                      delta(1, 1, 128, 128, 1),
                      attention(4, 2, 64, 16, 32, 0.11, base=1e4, mlp=dense(200))],
                     width=128, vocab=300, logit_scale=1.0, eps=1e-6)
# one delta layer run three times and nothing else; sizes that are no multiples of 4
CONFIG_ONE = config([delta(2, 1, 13, 10, 3)], width=48, vocab=97, logit_scale=2.5, loop=(0, 1, 3))

CONFIGS = {"odd": CONFIG_ODD, "wide": CONFIG_WIDE, "one": CONFIG_ONE}


def tensor_shapes(c):
    """Names and shapes of a checkpoint, written from the design's naming and not from the package's parts."""
    C = c["width"]
    shapes = {"embed": (c["vocab"], C), "head": (c["vocab"], C), "final.norm": (C,)}
    for i, lay in enumerate(c["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        shapes[p + "norm1"] = (C,)
        if lay["type"] == "attention":
            shapes.update({p + "mix.q": (H * D, C), p + "mix.q.b": (H * D,), p + "mix.k": (G * D, C), p + "mix.k.b": (G * D,),
                           p + "mix.v": (G * E, C), p + "mix.v.b": (G * E,), p + "mix.o": (C, H * E), p + "mix.o.b": (C,)})
        else:
            K = m["conv"]
            shapes.update({p + "mix.q": (G * D, C), p + "mix.q.conv": (G * D, K), p + "mix.k": (G * D, C),
                           p + "mix.k.conv": (G * D, K), p + "mix.v": (H * E, C), p + "mix.v.conv": (H * E, K),
                           p + "mix.b": (H, C), p + "mix.a": (H, C), p + "mix.A_log": (H,), p + "mix.dt_bias": (H,),
                           p + "mix.norm": (E,), p + "mix.g": (H * E, C), p + "mix.o": (C, H * E)})
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
                for e in range(mlp["router"]["experts"]):
                    shapes.update({q + f"e{e}.gate": (F, C), q + f"e{e}.up": (F, C), q + f"e{e}.down": (C, F)})
                if mlp.get("shared"):
                    F = mlp["shared"]["ff"]
                    shapes.update({q + "shared.gate": (F, C), q + "shared.up": (F, C), q + "shared.down": (C, F)})
    return shapes


def make_weights(c, seed, sharp=1.0):
    """{name: bfloat16 tensor}: what a checkpoint of configuration C holds. SHARP multiplies every attention layer's
    query matrix and bias: above one, a softmax concentrates on its best key, wherever that lies."""
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
            t = 0.3 * normal                                   # stored around zero
        elif leaf == "norm":
            t = 1.0 + 0.3 * normal
        elif leaf == "conv":
            t = 0.5 * normal
        elif leaf == "A_log":
            t = -1.0 + 0.7 * normal
        elif leaf == "dt_bias":
            t = -3.0 + normal                                  # decays of 0.9 to 0.999: the state remembers
        elif leaf == "router":
            t = 3.0 * normal / math.sqrt(shape[-1])
        elif len(shape) == 1:                                  # biases
            t = 0.3 * normal
            if kind == "attention" and parts[-2] == "q":
                t = t * sharp
        else:                                                  # linear maps [out, in]
            t = normal / math.sqrt(shape[-1])
            if kind == "attention" and leaf == "q":
                t = t * sharp
            if leaf in ("gate", "up") and "mlp" in parts:
                t = t * 2.0                                    # experts' limits are met
        out[name] = t.to(torch.bfloat16)
    return out
