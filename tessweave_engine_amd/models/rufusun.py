"""The Rufusun decoder: its typed configuration and its model assembled from parts.

config.json gives every size and every constant that differs between models of the design:

    architecture "Rufusun", vocab, width, norm.eps, logit_scale, loop: {start, stop, times} (optional),
    layers: [{type: "attention", mixer: {heads, kv_heads, dim, vdim, scale, softcap, rot: {base, dims}}, mlp: ...},
             {type: "delta", mixer: {heads, kv_heads, dim, vdim, conv}, mlp: ...}, ...]
    mlp: null, {kind: "dense", ff} or {kind: "moe", router: {experts, top}, expert: {ff, limit}, shared: {ff, limit}}

A layer (`parts.ParallelBlock`) runs its mixer and its feed-forward side by side, each behind an RMS norm of its own
whose weight is stored around zero, both of the same stream: x <- x + mixer(norm1(x)) + ff(norm2(x)). Mixers: causal
softmax attention with grouped key/value heads, biased projections, rotary positions on the first `rot.dims` elements of
a head, a scale from the configuration and a soft cap of the scores, values of a size of their own
(`parts.GroupedQueryAttention`); or the gated delta rule behind short convolutions (`parts.GatedDeltaRule`).
Feed-forwards: SiLU-gated (`parts.GatedFeedForward`), or routed experts with a limited swish beside a shared expert
(`parts.RoutedExperts`), or none. `loop` runs layers start .. stop - 1 `times` times in a row with the same weights;
every pass has a cache slot (pages, state) of its own: the schedule names a block several times. Output: the same
kind of norm, the head, and a scale on the logits. Tensor names are the checkpoint's own: `embed`, `l<i>.norm1`,
`l<i>.mix.q`, `l<i>.mix.q.b`, `l<i>.mix.q.conv`, `l<i>.mlp.e<j>.gate`, `l<i>.mlp.shared.up`, `final.norm`, `head`.

Constants the design fixes (not in config.json) live in the parts: the norms' offset of one, the unit norms' 1e-6 and
the queries' dim^-1/2 of the delta rule, the experts' 1.702 and their `up + 1`.
"""
from __future__ import annotations

from dataclasses import dataclass
import json

from ..config.model_config import ConfigError, eos_tuple
from ..config.registry import register_architecture
from ..parts import (DecoderModel, GatedDeltaRule, GatedFeedForward, GroupedQueryAttention, LayerRun, OutputHead,
                     ParallelBlock, RMSNorm, RotaryEmbedding, RoutedExperts, TokenEmbedding)
from ..kernels.ops import CONV_MAX_TAPS, MOE_MAX_EXPERTS

MIXERS = ("attention", "delta")
NO_POSITION_LIMIT = 1 << 30      # the design has no learned positions: nothing bounds a request's length but the cache


def _need(d, key, where):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json lacks {where}{key!r}")
    return d[key]


def _positive(value, what):
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"{what} must be a positive integer, found {value!r}")
    return value


def _positive_float(value, what):
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not float(value) > 0:
        raise ConfigError(f"{what} must be a positive number, found {value!r}")
    return float(value)


def _check_mlp(mlp, i):
    where = f"layers[{i}].mlp."
    kind = _need(mlp, "kind", where)
    if kind == "dense":
        _positive(_need(mlp, "ff", where), f"layer {i}: ff")
    elif kind == "moe":
        router, expert = _need(mlp, "router", where), _need(mlp, "expert", where)
        experts = _positive(_need(router, "experts", where + "router."), f"layer {i}: experts")
        top = _positive(_need(router, "top", where + "router."), f"layer {i}: top")
        if top > experts or experts > MOE_MAX_EXPERTS:
            raise ConfigError(f"layer {i}: top must not exceed experts, and experts not {MOE_MAX_EXPERTS}")
        for part, name in ((expert, "expert"), (mlp.get("shared"), "shared")):
            if part is not None:
                _positive(_need(part, "ff", where + name + "."), f"layer {i}: {name}.ff")
                _positive_float(_need(part, "limit", where + name + "."), f"layer {i}: {name}.limit")
    else:
        raise ConfigError(f"layer {i}: feed-forward kind {kind!r} is not built (known: 'dense', 'moe')")


@dataclass(frozen=True)
class RufusunConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    logit_scale: float
    loop: tuple                   # (start, stop, times); (0, 0, 1) when nothing repeats
    layers: tuple                 # the layer entries of config.json, as immutable JSON text each
    max_position_embeddings: int = NO_POSITION_LIMIT
    eos_token_ids: tuple = ()

    ARCHITECTURE = "Rufusun"
    MODEL_TYPE = "rufusun"

    @classmethod
    def from_dict(cls, d):
        if d.get("architecture", d.get("model_type")) not in (cls.ARCHITECTURE, cls.MODEL_TYPE):
            raise ConfigError(f"architecture {d.get('architecture')!r} is not {cls.ARCHITECTURE!r}")
        layers = _need(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("'layers' must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            kind = _need(layer, "type", where)
            if kind not in MIXERS:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is not built (known: {', '.join(MIXERS)})")
            m = _need(layer, "mixer", where)
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _positive(_need(m, key, where + "mixer."), f"layer {i}: {key}")
            if m["heads"] % m["kv_heads"]:
                raise ConfigError(f"layer {i}: heads must be a multiple of kv_heads")
            if kind == "attention":
                if m["dim"] % 2 or max(m["dim"], m["vdim"]) > 256:
                    raise ConfigError(f"layer {i}: the attention kernels take even key sizes, and key and value sizes up to 256")
                _positive_float(_need(m, "scale", where + "mixer."), f"layer {i}: scale")
                cap = m.get("softcap")
                if cap is not None and cap != 0:
                    _positive_float(cap, f"layer {i}: softcap")
                rot = _need(m, "rot", where + "mixer.")
                dims = _positive(_need(rot, "dims", where + "mixer.rot."), f"layer {i}: rot.dims")
                if dims % 2 or dims > m["dim"]:
                    raise ConfigError(f"layer {i}: rot.dims must be even and at most dim")
                if not float(_need(rot, "base", where + "mixer.rot.")) > 1:
                    raise ConfigError(f"layer {i}: rot.base must be greater than 1")
            else:
                if m["dim"] > 256:
                    raise ConfigError(f"layer {i}: the delta rule's kernels take key sizes up to 256")
                taps = _positive(_need(m, "conv", where + "mixer."), f"layer {i}: conv")
                if taps > CONV_MAX_TAPS:
                    raise ConfigError(f"layer {i}: a convolution has at most {CONV_MAX_TAPS} taps")
            if layer.get("mlp") is not None:
                _check_mlp(layer["mlp"], i)
        loop = d.get("loop")
        start, stop, times = 0, 0, 1
        if loop is not None:
            start, stop, times = (_need(loop, key, "loop.") for key in ("start", "stop", "times"))
            for v in (start, stop, times):
                if isinstance(v, bool) or not isinstance(v, int):
                    raise ConfigError("loop.start, loop.stop and loop.times must be integers")
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError("loop must name layers start .. stop - 1 of the model and run them at least once")
        eps = _positive_float(_need(_need(d, "norm", ""), "eps", "norm."), "norm.eps")
        scale = d.get("logit_scale", 1.0)
        if isinstance(scale, bool) or not isinstance(scale, (int, float)):
            raise ConfigError("logit_scale must be a number")
        return cls(architecture=cls.ARCHITECTURE, vocab_size=_positive(_need(d, "vocab", ""), "vocab"),
                   hidden_size=_positive(_need(d, "width", ""), "width"), norm_eps=eps, logit_scale=float(scale),
                   loop=(start, stop, times), layers=tuple(json.dumps(layer, sort_keys=True) for layer in layers),
                   eos_token_ids=eos_tuple(d.get("eos_token_id")))

    def layer_dicts(self):
        return [json.loads(text) for text in self.layers]

    def layer_order(self):
        """Indices of the layers in the order they run."""
        start, stop, times = self.loop
        n = len(self.layers)
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))

    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
             "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale, "layers": self.layer_dicts()}
        if self.loop != (0, 0, 1):
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d

    def describe(self):
        return self.to_dict()


def _feed_forward(prefix, C, mlp):
    names = lambda p: [p + "gate", p + "up", p + "down"]       # noqa: E731
    if mlp["kind"] == "dense":
        return GatedFeedForward(names(prefix), C, mlp["ff"], activation="silu", suffix="")
    shared = mlp.get("shared")
    if shared is not None:
        shared = GatedFeedForward(names(prefix + "shared."), C, shared["ff"], activation="swish_limited",
                                  limit=shared["limit"], suffix="")
    return RoutedExperts(prefix, C, mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"],
                         mlp["expert"]["limit"], shared=shared)


def build_rufusun(config: RufusunConfig, packed=True):
    c = config
    C, layers = c.hidden_size, c.layer_dicts()
    encodings = {}

    def rotary(rot, size):
        """One part per distinct encoding: its tables are formed once a step for all layers that share it."""
        key = (float(rot["base"]), int(rot["dims"]))
        if key not in encodings:
            encodings[key] = RotaryEmbedding(max(size, rot["dims"]), rot["base"], rot["dims"])
        return encodings[key]

    def norm(name):
        return RMSNorm(name, C, c.norm_eps, suffix="", offset=1.0)

    blocks = []
    for i, layer in enumerate(layers):
        p, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "attention":
            mixer = GroupedQueryAttention(p + "mix.", C, m["heads"], m["kv_heads"], m["dim"], rotary(m["rot"], m["dim"]),
                                          qkv_bias=True, o_bias=True, scale=m["scale"], softcap=m.get("softcap") or None,
                                          value_dim=m["vdim"], names=("q", "k", "v", "o"), suffixes=("", ".b"))
        else:
            mixer = GatedDeltaRule(p + "mix.", C, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], c.norm_eps)
        mlp = layer.get("mlp")
        ffn = _feed_forward(p + "mlp.", C, mlp) if mlp is not None else None
        blocks.append(ParallelBlock(C, norm(p + "norm1"), mixer, norm(p + "norm2") if ffn is not None else None, ffn))
    # every run of a layer has a cache slot of its own: a repeated layer shares its weights, not its pages or state
    schedule = [LayerRun(block, slot) for slot, block in enumerate(c.layer_order())]
    embedding = TokenEmbedding("embed", c.vocab_size, C, suffix="")
    head = OutputHead("head", c.vocab_size, C, suffix="", scale=c.logit_scale)
    return DecoderModel(c, embedding, blocks, norm("final.norm"), head, schedule=schedule, defer_sums=False)


register_architecture(RufusunConfig.ARCHITECTURE, RufusunConfig.MODEL_TYPE, RufusunConfig, build_rufusun, replace=True)
