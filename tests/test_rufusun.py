"""The Rufusun design without a GPU: configuration, registry, tensor names, cache needs and schedule, and the plain
implementation's mechanisms against closed forms (so that the oracle the GPU tests use is itself pinned)."""
import json
import math

import pytest
import torch

import plain_rufusun as plain
from rufusun_util import CONFIGS, make_weights, tensor_shapes, write_folder


@pytest.mark.parametrize("name", list(CONFIGS))
def test_config_registry_and_tensor_names(name, tmp_path):
    from tessweave_engine_amd.config import build_model, config_from_dict, read_model_config
    c = CONFIGS[name]
    config = config_from_dict(c)
    assert config.architecture == "Rufusun" and config.vocab_size == c["vocab"]
    assert config_from_dict(config.to_dict()) == config
    model = build_model(config)
    specs = {s.name: s.shape for s in model.tensor_specs() if s.optional_alias_of is None}
    assert specs == tensor_shapes(c)
    folder = write_folder(tmp_path, c, make_weights(c, 0))
    assert read_model_config(folder) == config
    assert config.layer_order() == plain.layer_order(c)


def test_config_rejections():
    from tessweave_engine_amd.config import ConfigError, config_from_dict
    base = json.loads(json.dumps(CONFIGS["odd"]))
    for change in (lambda c: c["layers"][0].__setitem__("type", "other"),
                   lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 4),
                   lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7),
                   lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 26),
                   lambda c: c["layers"][0]["mixer"].pop("scale"),
                   lambda c: c["layers"][0]["mlp"].__setitem__("kind", "experts"),
                   lambda c: c["layers"][1]["mixer"].__setitem__("conv", 0),
                   lambda c: c["layers"][1]["mixer"].__setitem__("conv", 9),
                   lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 6),
                   lambda c: c["layers"][1]["mlp"]["expert"].__setitem__("limit", 0),
                   lambda c: c["layers"][2]["mixer"].__setitem__("dim", 300),
                   lambda c: c["loop"].__setitem__("stop", 5),
                   lambda c: c["loop"].__setitem__("times", 0),
                   lambda c: c.pop("width"),
                   lambda c: c["norm"].__setitem__("eps", 0)):
        c = json.loads(json.dumps(base))
        change(c)
        with pytest.raises(ConfigError):
            config_from_dict(c)


def test_cache_layout_and_schedule():
    """Every run of a layer has a cache slot of its own (a repeated layer shares weights, not pages or state);
    attention layers page keys and values laid out with the larger of the two sizes rounded up to 16; delta layers
    hold a float32 state [heads, value size, key size rounded up to 4] and the convolutions' last inputs, twice."""
    from tessweave_engine_amd.config import build_model, config_from_dict
    model = build_model(config_from_dict(CONFIGS["odd"]))
    layout = model.cache_layout()
    assert [(r.block, r.cache_slot, r.writes_cache) for r in model.schedule] == \
        [(0, 0, True), (1, 1, True), (2, 2, True), (3, 3, True), (2, 4, True), (3, 5, True)]
    assert layout.needs[0].paged.kv_heads == 3 and layout.needs[0].paged.head_dim == 48
    assert layout.needs[3].paged == layout.needs[5].paged and layout.needs[3].paged.head_dim == 16
    assert len(layout.groups) == 2 and layout.groups[1].slots == (3, 5)
    states = dict(layout.needs[2].states)
    assert states["delta.s"].shape == (3, 72, 40) and states["delta.conv"].shape == (2, 1, 40 * 3 * 2 + 3 * 72)
    assert dict(layout.needs[1].states)["delta.conv"].shape == (2, 3, 2 * 2 * 20 + 4 * 24)
    assert dict(layout.needs[4].states) == states
    assert not layout.shares_prefixes and not model.defers_sums
    one = build_model(config_from_dict(CONFIGS["one"]))
    assert dict(one.cache_layout().needs[2].states)["delta.s"].shape == (2, 10, 16)
    assert [r.block for r in one.schedule] == [0, 0, 0]


def test_random_weights_and_inspect_on_the_command_line(tmp_path, capsys):
    from tessweave_engine_amd.cli import main
    from tessweave_engine_amd.config import read_model_config
    source = tmp_path / "config.json"
    source.write_text(json.dumps(CONFIGS["wide"]))
    folder = tmp_path / "model"
    assert main(["random-weights", str(source), str(folder), "--seed", "3"]) == 0
    assert read_model_config(folder).to_dict()["layers"] == CONFIGS["wide"]["layers"]
    from safetensors import safe_open
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        assert {k: tuple(f.get_slice(k).get_shape()) for k in f.keys()} == tensor_shapes(CONFIGS["wide"])
        assert f.get_tensor("l0.norm1").float().abs().max() < 0.2          # stored around zero
    capsys.readouterr()
    assert main(["inspect", str(folder), "--kv-blocks", "10", "--block-size", "16"]) == 0
    assert "Rufusun" in capsys.readouterr().out


# ---- the plain implementation's mechanisms against closed forms --------------------------------------------

def test_offset_norm():
    x = torch.randn(5, 12, dtype=torch.float64) * 3
    y = plain.offset_norm(x, torch.zeros(12, dtype=torch.float64), 1e-9)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64))
    assert torch.allclose(plain.offset_norm(x, torch.full((12,), -1.0, dtype=torch.float64), 1e-5), torch.zeros_like(x))


def test_short_convolution_meets_the_current_token_with_its_last_tap():
    x = torch.zeros(6, 2, dtype=torch.float64)
    x[2] = torch.tensor([1.0, 10.0])
    taps = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], dtype=torch.float64)
    y = plain.short_conv(x, taps)
    assert y[:, 0].tolist() == [0, 0, 3, 2, 1, 0] and y[:, 1].tolist() == [0, 0, 60, 50, 40, 0]


def test_delta_rule_closed_forms():
    """One token: S = beta k v^T, o = beta (k . q) v. Orthonormal keys written with beta 1 and no decay are read back
    exactly; writing a key again replaces its value (the correction, not a sum); with beta 0 nothing is written;
    the decay multiplies what was there before the token's own write."""
    D, E = 4, 3
    eye = torch.eye(D, dtype=torch.float64)
    v = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0], [7.0, 8.0, 9.0]], dtype=torch.float64)
    ones = torch.ones(3, dtype=torch.float64)
    o = plain.delta_rule(0.5 * eye[:1], eye[:1], v[:1], 0.25 * ones[:1], ones[:1])
    assert torch.allclose(o, 0.25 * 0.5 * v[:1])
    k = torch.stack([eye[0], eye[1], eye[0]])
    q = torch.stack([eye[0], eye[0] + eye[1], eye[0]])
    o = plain.delta_rule(q, k, v, ones, ones)
    assert torch.allclose(o, torch.stack([v[0], v[0] + v[1], v[2]]))
    o = plain.delta_rule(q, k, v, torch.tensor([1.0, 0.0, 0.0], dtype=torch.float64), ones)
    assert torch.allclose(o, torch.stack([v[0], v[0], v[0]]))
    g = torch.tensor([1.0, 0.5, 0.5], dtype=torch.float64)
    o = plain.delta_rule(q, k, v, torch.tensor([1.0, 1.0, 0.0], dtype=torch.float64), g)
    assert torch.allclose(o, torch.stack([v[0], 0.5 * v[0] + v[1], 0.25 * v[0]]))


def test_attention_closed_forms():
    """Zero queries average the values seen so far plus the bias path (causal, v not rotated, key/value head of a query
    head); a huge score is capped: with cap c two keys whose raw scores are far above c weigh the same."""
    T, C = 5, 6
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 1.0, "softcap": None, "rot": {"base": 10.0, "dims": 2}}
    g = torch.Generator().manual_seed(0)
    h = torch.randn(T, C, generator=g, dtype=torch.float64)
    w = {"q": torch.zeros(8, C, dtype=torch.float64), "q.b": torch.zeros(8, dtype=torch.float64),
         "k": torch.randn(4, C, generator=g, dtype=torch.float64), "k.b": torch.zeros(4, dtype=torch.float64),
         "v": torch.randn(3, C, generator=g, dtype=torch.float64), "v.b": torch.tensor([1.0, 2.0, 3.0], dtype=torch.float64),
         "o": torch.cat([torch.eye(3, dtype=torch.float64), torch.eye(3, dtype=torch.float64)], 1)[:, :6].repeat(2, 1)[:C],
         "o.b": torch.full((C,), 0.5, dtype=torch.float64)}
    v = h @ w["v"].T + w["v.b"]
    mean = torch.cumsum(v, 0) / torch.arange(1, T + 1, dtype=torch.float64).view(-1, 1)
    want = torch.cat([mean, mean], 1) @ w["o"].T + 0.5
    assert torch.allclose(plain.capped_attention(h, w, m), want)
    # the cap: queries and keys from biases only, unrotated part, scores 400 and 900 -> both about the cap
    m2 = dict(m, softcap=2.0, rot={"base": 10.0, "dims": 2})
    w2 = dict(w, **{"q.b": torch.tensor([0, 0, 20.0, 0] * 2, dtype=torch.float64), "k": torch.zeros(4, C, dtype=torch.float64)})
    w2["k"][2] = torch.tensor([1.0, 0, 0, 0, 0, 0], dtype=torch.float64)
    h2 = torch.zeros(2, C, dtype=torch.float64)
    h2[0, 0], h2[1, 0] = 20.0, 45.0
    out = plain.capped_attention(h2, w2, m2)
    v2 = h2 @ w2["v"].T + w2["v.b"]
    both = torch.cat([(v2[0] + v2[1]) / 2] * 2) @ w2["o"].T + 0.5
    assert torch.allclose(out[1], both, atol=1e-9)


def test_experts_closed_forms():
    """The limited swish at and beyond its limits; the score multiplies the expert's input (not its output), is not
    renormalised, and the shared expert is added for every token."""
    one = torch.ones(1, 1, dtype=torch.float64)
    y = plain.limited_expert(torch.tensor([[10.0]], dtype=torch.float64), one, -one, one, 2.0)
    assert torch.allclose(y, torch.tensor([[2.0 / (1 + math.exp(-1.702 * 2.0)) * (-2.0 + 1.0)]], dtype=torch.float64))
    y = plain.limited_expert(torch.tensor([[-10.0]], dtype=torch.float64), one, one, one, 2.0)
    assert torch.allclose(y, torch.tensor([[-10.0 / (1 + math.exp(17.02)) * (-2.0 + 1.0)]], dtype=torch.float64))
    C = 4
    g = torch.Generator().manual_seed(1)
    w = {"router": torch.tensor([[5.0, 0, 0, 0], [0, 5.0, 0, 0], [0, 0, 0.1, 0]], dtype=torch.float64)}
    for e in range(3):
        w[f"e{e}.gate"], w[f"e{e}.up"] = (torch.randn(5, C, generator=g, dtype=torch.float64) for _ in range(2))
        w[f"e{e}.down"] = torch.randn(C, 5, generator=g, dtype=torch.float64)
    mlp = {"router": {"experts": 3, "top": 1}, "expert": {"ff": 5, "limit": 1.5}}
    h = torch.tensor([[1.0, 0.2, 0, 0.3], [0.1, 2.0, 0, 0]], dtype=torch.float64)
    out = plain.routed_ffn(h, w, mlp)
    for t, e in ((0, 0), (1, 1)):
        s = 1 / (1 + math.exp(-5.0 * h[t, e].item()))
        assert torch.allclose(out[t], plain.limited_expert(s * h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], 1.5)[0])
    mlp2 = dict(mlp, router={"experts": 3, "top": 2}, shared={"ff": 5, "limit": 0.5})
    w.update({"shared.gate": w["e2.gate"], "shared.up": w["e2.up"], "shared.down": w["e2.down"]})
    out2 = plain.routed_ffn(h[:1], w, mlp2)
    s0, s1 = 1 / (1 + math.exp(-5.0)), 1 / (1 + math.exp(-1.0))
    want = (plain.limited_expert(s0 * h[:1], w["e0.gate"], w["e0.up"], w["e0.down"], 1.5) +
            plain.limited_expert(s1 * h[:1], w["e1.gate"], w["e1.up"], w["e1.down"], 1.5) +
            plain.limited_expert(h[:1], w["e2.gate"], w["e2.up"], w["e2.down"], 0.5))
    assert torch.allclose(out2, want)


def test_parallel_layer_and_loop():
    """Both norms read the same stream (the feed-forward does not see the mixer's result), and a looped layer runs
    with the same weights again on its own result."""
    c = CONFIGS["one"]
    weights = {k: v.double() for k, v in make_weights(c, 2).items()}
    toks = [3, 50, 7, 7, 90, 1]
    logits, layers = plain.forward(c, weights, toks, keep_layers=True)
    assert layers.shape[0] == 3
    x = weights["embed"][torch.tensor(toks)]
    for run in range(3):
        h = plain.offset_norm(x, weights["l0.norm1"], c["norm"]["eps"])
        x = x + plain.delta_mixer(h, plain.sub(weights, "l0.mix."), c["layers"][0]["mixer"], c["norm"]["eps"])
        assert torch.allclose(layers[run], x)
    assert torch.allclose(logits, plain.offset_norm(x, weights["final.norm"], 1e-5) @ weights["head"].T * 2.5)
    c2 = CONFIGS["wide"]
    w2 = {k: v.double() for k, v in make_weights(c2, 3).items()}
    _, layers2 = plain.forward(c2, w2, toks, keep_layers=True)
    x = w2["embed"][torch.tensor(toks)]
    h1, h2 = (plain.offset_norm(x, w2[f"l0.norm{i}"], 1e-6) for i in (1, 2))
    want = x + plain.delta_mixer(h1, plain.sub(w2, "l0.mix."), c2["layers"][0]["mixer"], 1e-6) + plain.dense_ffn(h2, plain.sub(w2, "l0.mlp."))
    assert torch.allclose(layers2[0], want)
