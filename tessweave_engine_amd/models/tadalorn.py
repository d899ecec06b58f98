"""The Tadalorn decoder: its typed configuration and its model assembled from parts.

config.json gives every size and every constant that differs between models of the design:

    architecture "Tadalorn", vocab, width, norm.eps, residual_mult, logit_softcap,
    layers: [{type: "attention", mixer: {heads, kv_heads, dim, vdim, scale, conv, mask: {size, keep_first}, rot: {base, dims}}, mlp: ...},
             {type: "latent_attention", mixer: {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {base, dims}}, mlp: ...},
             {type: "mlstm", mixer: {heads, dim, vdim, gate_cap}, mlp: ...},
             {..., weights_of: j}, ...]
    mlp: null, {kind: "dense", ff} or {kind: "moe", router: {experts, top}, expert: {ff}, shared: {ff} or absent}

A layer (`parts.ResultNormBlock`) norms each sublayer's RESULT and scales it into the stream, and its sublayers read the
stream itself: x <- x + m norm1(mixer(x)); x <- x + m norm2(ff(x)), m = residual_mult. Mixers: windowed attention behind
short convolutions whose values are its keys, with whole-row norms, kept first tokens, one added to the softmax's
denominator and an output gate (`parts.ConvolvedWindowAttention`); attention over a cached latent with a learned sink
per head and an output gate (`parts.LatentAttention`); the mLSTM's matrix memory (`parts.MatrixLSTM`). Both attentions
rotate neighbouring pairs of elements. Feed-forwards: SiLU-gated (`parts.GatedFeedForward`), or routed experts without a
gate behind the exact gelu, weighted by the softmax over the chosen logits, beside a shared expert of the same form
(`parts.RoutedExperts`, `parts.PlainFeedForward`), or none. A layer with `weights_of: j` runs layer j's block (mixer,
feed-forward and norms) with a cache slot of its own: the schedule names that block once more. Output: an RMS norm, the
head, a soft cap on the logits. Tensor names are the checkpoint's own: `embed`, `l<i>.norm1`, `l<i>.mix.q`,
`l<i>.mix.q.conv`, `l<i>.mix.q.norm`, `l<i>.mix.dkv.norm`, `l<i>.mix.sink`, `l<i>.mix.i.b`, `l<i>.mlp.e<j>.up`,
`l<i>.mlp.router.b`, `l<i>.mlp.shared.up`, `final.norm`, `head`.

Constants the design fixes (not in config.json) live in the parts: the one in the windowed softmax's denominator (a
sink of score 0), the mLSTM's dim^-1/2 on its queries, its 1e-6 and its maximum that starts at zero.
"""
from __future__ import annotations

from dataclasses import dataclass
import json

from ..config.model_config import ConfigError, eos_tuple
from ..config.registry import register_architecture
from ..parts import (ConvolvedWindowAttention, DecoderModel, GatedFeedForward, LatentAttention, LayerRun, MatrixLSTM,
                     OutputHead, PlainFeedForward, ResultNormBlock, RMSNorm, RotaryEmbedding, RoutedExperts,
                     TokenEmbedding)
from ..kernels.ops import CONV_MAX_TAPS, MOE_MAX_EXPERTS

MIXERS = ("attention", "latent_attention", "mlstm")
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


def _check_rot(m, i, limit):
    rot = _need(m, "rot", f"layers[{i}].mixer.")
    dims = _positive(_need(rot, "dims", f"layers[{i}].mixer.rot."), f"layer {i}: rot.dims")
    if dims % 2 or dims > limit:
        raise ConfigError(f"layer {i}: rot.dims must be even and at most the rotated size {limit}")
    if not float(_need(rot, "base", f"layers[{i}].mixer.rot.")) > 1:
        raise ConfigError(f"layer {i}: rot.base must be greater than 1")


def _check_mixer(kind, m, i):
    where = f"layers[{i}].mixer."
    for key in ("heads", "dim", "vdim"):
        _positive(_need(m, key, where), f"layer {i}: {key}")
    if kind == "attention":
        _positive(_need(m, "kv_heads", where), f"layer {i}: kv_heads")
        if m["heads"] % m["kv_heads"]:
            raise ConfigError(f"layer {i}: heads must be a multiple of kv_heads")
        if m["vdim"] != m["dim"]:
            raise ConfigError(f"layer {i}: this attention's values are its keys, so vdim must equal dim")
        if m["dim"] > 256 or m["heads"] > ConvolvedWindowAttention.MAX_HEADS:
            raise ConfigError(f"layer {i}: the attention kernel takes head sizes up to 256 and up to "
                              f"{ConvolvedWindowAttention.MAX_HEADS} heads")
        _positive_float(_need(m, "scale", where), f"layer {i}: scale")
        taps = _positive(_need(m, "conv", where), f"layer {i}: conv")
        if taps > CONV_MAX_TAPS:
            raise ConfigError(f"layer {i}: a convolution has at most {CONV_MAX_TAPS} taps")
        mask = _need(m, "mask", where)
        _positive(_need(mask, "size", where + "mask."), f"layer {i}: mask.size")
        keep = _need(mask, "keep_first", where + "mask.")
        if isinstance(keep, bool) or not isinstance(keep, int) or keep < 0:
            raise ConfigError(f"layer {i}: mask.keep_first must be an integer, zero or more")
        _check_rot(m, i, m["dim"])
    elif kind == "latent_attention":
        for key in ("rot_dim", "kv_rank"):
            _positive(_need(m, key, where), f"layer {i}: {key}")
        _positive_float(_need(m, "scale", where), f"layer {i}: scale")
        if max(m["dim"] + m["rot_dim"], m["vdim"]) > 256:
            raise ConfigError(f"layer {i}: the attention kernels take heads (dim + rot_dim, vdim) up to 256")
        _check_rot(m, i, m["rot_dim"])
    else:
        if m["dim"] > 256:
            raise ConfigError(f"layer {i}: the mLSTM's kernels take key sizes up to 256")
        _positive_float(_need(m, "gate_cap", where), f"layer {i}: gate_cap")


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
        _positive(_need(expert, "ff", where + "expert."), f"layer {i}: expert.ff")
        if mlp.get("shared") is not None:
            _positive(_need(mlp["shared"], "ff", where + "shared."), f"layer {i}: shared.ff")
    else:
        raise ConfigError(f"layer {i}: feed-forward kind {kind!r} is not built (known: 'dense', 'moe')")


@dataclass(frozen=True)
class TadalornConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    residual_mult: float
    logit_softcap: float          # 0.0: none
    layers: tuple                 # the layer entries of config.json, as immutable JSON text each
    max_position_embeddings: int = NO_POSITION_LIMIT
    eos_token_ids: tuple = ()

    ARCHITECTURE = "Tadalorn"
    MODEL_TYPE = "tadalorn"

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
            _check_mixer(kind, _need(layer, "mixer", where), i)
            if layer.get("mlp") is not None:
                _check_mlp(layer["mlp"], i)
            source = layer.get("weights_of")
            if source is not None:
                if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < len(layers) or source == i:
                    raise ConfigError(f"layer {i}: weights_of must name another layer of the model")
                if layers[source].get("weights_of") is not None:
                    raise ConfigError(f"layer {i}: weights_of names layer {source}, which has no weights of its own")
                for key in ("type", "mixer", "mlp"):
                    if json.dumps(layer.get(key), sort_keys=True) != json.dumps(layers[source].get(key), sort_keys=True):
                        raise ConfigError(f"layer {i}: a layer that uses layer {source}'s weights must equal it in its {key}")
        eps = _positive_float(_need(_need(d, "norm", ""), "eps", "norm."), "norm.eps")
        mult = d.get("residual_mult", 1.0)
        if isinstance(mult, bool) or not isinstance(mult, (int, float)):
            raise ConfigError("residual_mult must be a number")
        cap = d.get("logit_softcap")
        if cap is not None and cap != 0:
            _positive_float(cap, "logit_softcap")
        return cls(architecture=cls.ARCHITECTURE, vocab_size=_positive(_need(d, "vocab", ""), "vocab"),
                   hidden_size=_positive(_need(d, "width", ""), "width"), norm_eps=eps, residual_mult=float(mult),
                   logit_softcap=float(cap or 0.0), layers=tuple(json.dumps(layer, sort_keys=True) for layer in layers),
                   eos_token_ids=eos_tuple(d.get("eos_token_id")))

    def layer_dicts(self):
        return [json.loads(text) for text in self.layers]

    def weight_sources(self):
        """Per layer, the layer whose tensors it runs with (itself unless `weights_of` names another)."""
        return [layer.get("weights_of", i) if layer.get("weights_of") is not None else i
                for i, layer in enumerate(self.layer_dicts())]

    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
             "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "layers": self.layer_dicts()}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d

    def describe(self):
        return self.to_dict()


def _feed_forward(prefix, C, mlp):
    if mlp["kind"] == "dense":
        return GatedFeedForward([prefix + "gate", prefix + "up", prefix + "down"], C, mlp["ff"], activation="silu", suffix="")
    shared = mlp.get("shared")
    if shared is not None:
        # (where its last product splits K, the sums are added up by the kernel that adds up a token's experts)
        shared = PlainFeedForward([prefix + "shared.up", prefix + "shared.down"], C, shared["ff"], suffix="",
                                  activation="gelu")
    return RoutedExperts(prefix, C, mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"], shared=shared,
                         kind="gelu", weighting="softmax_chosen", router_bias="router.b")


def build_tadalorn(config: TadalornConfig, packed=True):
    c = config
    C, layers = c.hidden_size, c.layer_dicts()
    encodings = {}

    def rotary(rot, size):
        """One part per distinct encoding: its tables are formed once a step for all layers that share it."""
        key = (float(rot["base"]), int(rot["dims"]))
        if key not in encodings:
            encodings[key] = RotaryEmbedding(max(size, rot["dims"]), rot["base"], rot["dims"], pairing="adjacent")
        return encodings[key]

    def norm(name):
        return RMSNorm(name, C, c.norm_eps, suffix="")

    sources = c.weight_sources()
    blocks, block_of = [], {}
    for i, layer in enumerate(layers):
        if sources[i] != i:
            continue
        p, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "attention":
            mixer = ConvolvedWindowAttention(p + "mix.", C, m["heads"], m["kv_heads"], m["dim"], rotary(m["rot"], m["dim"]),
                                             m["conv"], c.norm_eps, window=m["mask"]["size"],
                                             keep_first=m["mask"]["keep_first"], scale=m["scale"], sink=0.0)
        elif layer["type"] == "latent_attention":
            mixer = LatentAttention(p + "mix.", C, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"],
                                    rotary(m["rot"], m["rot_dim"]), c.norm_eps, sink_name="sink", gate_name="g")
        else:
            mixer = MatrixLSTM(p + "mix.", C, m["heads"], m["dim"], m["vdim"], m["gate_cap"], c.norm_eps)
        mlp = layer.get("mlp")
        ffn = _feed_forward(p + "mlp.", C, mlp) if mlp is not None else None
        block_of[i] = len(blocks)
        blocks.append(ResultNormBlock(C, mixer, norm(p + "norm1"), ffn, norm(p + "norm2") if ffn is not None else None,
                                      mult=c.residual_mult, unused_names=() if ffn is not None else (p + "norm2",)))
    # every layer has a cache slot of its own: a layer that runs another's block shares its weights, not its pages or state
    schedule = [LayerRun(block_of[sources[i]], i) for i in range(len(layers))]
    embedding = TokenEmbedding("embed", c.vocab_size, C, suffix="")
    head = OutputHead("head", c.vocab_size, C, suffix="", softcap=c.logit_softcap or None)
    return DecoderModel(c, embedding, blocks, norm("final.norm"), head, schedule=schedule)


register_architecture(TadalornConfig.ARCHITECTURE, TadalornConfig.MODEL_TYPE, TadalornConfig, build_tadalorn, replace=True)
