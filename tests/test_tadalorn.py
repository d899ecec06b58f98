"""The Tadalorn design without a GPU: configuration, registry, tensor names, cache needs and schedule, the cache
manager's kept first pages, and the plain implementation's mechanisms against closed forms (so that the oracle the GPU
tests use is itself pinned)."""
import json
import math

import pytest
import torch

import plain_tadalorn as plain
from tadalorn_util import CONFIGS, make_weights, tensor_shapes, write_folder


@pytest.mark.parametrize("name", list(CONFIGS))
def test_config_registry_and_tensor_names(name, tmp_path):
    from tessweave_engine_amd.config import build_model, config_from_dict, read_model_config
    c = CONFIGS[name]
    config = config_from_dict(c)
    assert config.architecture == "Tadalorn" and config.vocab_size == c["vocab"]
    assert config_from_dict(config.to_dict()) == config
    model = build_model(config)
    specs = {s.name: s.shape for s in model.tensor_specs() if s.optional_alias_of is None}
    assert specs == tensor_shapes(c)
    folder = write_folder(tmp_path, c, make_weights(c, 0))
    assert read_model_config(folder) == config


def test_config_rejections():
    from tessweave_engine_amd.config import ConfigError, config_from_dict
    base = json.loads(json.dumps(CONFIGS["odd"]))
    for change in (lambda c: c["layers"][0].__setitem__("type", "other"),
                   lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 4),
                   lambda c: c["layers"][0]["mixer"].__setitem__("vdim", 32),
                   lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7),
                   lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 26),
                   lambda c: c["layers"][0]["mixer"].pop("scale"),
                   lambda c: c["layers"][0]["mixer"].__setitem__("conv", 0),
                   lambda c: c["layers"][0]["mixer"].__setitem__("conv", 9),
                   lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0),
                   lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("keep_first", -1),
                   lambda c: c["layers"][0]["mlp"].__setitem__("kind", "experts"),
                   lambda c: c["layers"][1]["mixer"].__setitem__("gate_cap", 0),
                   lambda c: c["layers"][1]["mixer"].__setitem__("dim", 300),
                   lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 6),
                   lambda c: c["layers"][2]["mixer"]["rot"].__setitem__("dims", 10),
                   lambda c: c["layers"][2]["mixer"].pop("kv_rank"),
                   lambda c: c["layers"][3].__setitem__("weights_of", 3),
                   lambda c: c["layers"][3].__setitem__("weights_of", 9),
                   lambda c: c["layers"][3].__setitem__("weights_of", 1),
                   lambda c: c["layers"][4].__setitem__("weights_of", 3),
                   lambda c: c.pop("width"),
                   lambda c: c.__setitem__("logit_softcap", -1.0),
                   lambda c: c["norm"].__setitem__("eps", 0)):
        c = json.loads(json.dumps(base))
        change(c)
        with pytest.raises(ConfigError):
            config_from_dict(c)


def test_cache_layout_and_schedule():
    """Every layer has a cache slot of its own (a layer that runs with another's weights shares its block, not its pages
    or state); windowed layers page keys and values in a group that keeps the first tokens; latent layers page one head
    of latent + rotated part; mLSTM layers hold S [heads, values, keys] (rounded up to 16), and n and m twice."""
    from tessweave_engine_amd.config import build_model, config_from_dict
    model = build_model(config_from_dict(CONFIGS["odd"]))
    layout = model.cache_layout()
    assert [(r.block, r.cache_slot, r.writes_cache) for r in model.schedule] == \
        [(0, 0, True), (1, 1, True), (2, 2, True), (0, 3, True), (3, 4, True), (4, 5, True)]
    assert len(model.blocks) == 5
    a = layout.needs[0].paged
    assert (a.kv_heads, a.head_dim, a.window, a.keep_first) == (3, 32, 9, 3) and layout.needs[3].paged == a
    assert dict(layout.needs[0].states)["attention.conv"].shape == (2, 3, 6 * 24 + 3 * 24)
    lat = layout.needs[2].paged
    assert (lat.kv_heads, lat.head_dim, lat.value_dim, lat.window) == (1, 48 + 16, 48, None)
    states = dict(layout.needs[1].states)
    assert states["mlstm.s"].shape == (3, 32, 32) and states["mlstm.n"].shape == (2, 3, 32) and states["mlstm.m"].shape == (2, 3)
    assert dict(layout.needs[5].states)["mlstm.s"].shape == (1, 16, 16)
    assert not layout.shares_prefixes
    wide = build_model(config_from_dict(CONFIGS["wide"]))
    assert [r.block for r in wide.schedule] == [0, 1, 2, 0, 3, 4]
    assert wide.cache_layout().needs[4].paged.keep_first == 20


def test_kept_first_pages_stay_when_the_window_has_passed_them():
    """A windowed group with kept first tokens: the pages of the first `keep_first` tokens are never given back, the
    others return as the window passes them, and a closed request returns everything."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.cache.spec import CacheLayout, CacheNeed, PagedKV
    layout = CacheLayout([CacheNeed(paged=PagedKV(2, 16, window=6, keep_first=5)), CacheNeed(paged=PagedKV(2, 16, window=6))])
    cache = CacheManager(layout, 4, 40, 2, device=None)
    seq = cache.open("a")
    for upto in (3, 11, 12, 30, 31, 50):
        cache.ensure(seq, upto)
        cache.advance(seq, upto)
        cache.check()
    kept, plain_window = seq.tables
    assert kept[0] >= 0 and kept[1] >= 0                     # tokens 0 .. 4 lie in blocks 0 and 1
    assert all(p < 0 for p in kept[2:(50 - 6 + 1) // 4]) and all(p >= 0 for p in kept[(50 - 6 + 1) // 4:])
    assert all(p < 0 for p in plain_window[:(50 - 6 + 1) // 4])
    assert cache.pages_needed(0, 1000, 16) == cache.pages_needed(1, 1000, 16) + 2
    cache.close(seq)
    assert all(len(pool.free) == 40 for pool in cache.pools)


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
    capsys.readouterr()
    assert main(["inspect", str(folder), "--kv-blocks", "10", "--block-size", "16"]) == 0
    assert "Tadalorn" in capsys.readouterr().out


# ---- the plain implementation's mechanisms against closed forms --------------------------------------------

F64 = torch.float64


def test_rotation_of_pairs_and_short_convolution():
    x = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 5.0, 6.0]]], dtype=F64).repeat(3, 1, 1)
    y = plain.rotate_pairs(x, torch.arange(3), 4, 100.0)
    for p in range(3):
        a0, a1 = p * 1.0, p * 100.0 ** -0.5
        want = [math.cos(a0), math.sin(a0), -2.0 * math.sin(a1), 2.0 * math.cos(a1), 5.0, 6.0]
        assert torch.allclose(y[p, 0], torch.tensor(want, dtype=F64))
    u = torch.zeros(6, 2, dtype=F64)
    u[2] = torch.tensor([1.0, 10.0])
    taps = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], dtype=F64)
    y = plain.causal_taps(u, taps)
    assert y[:, 0].tolist() == [0, 0, 3, 2, 1, 0] and y[:, 1].tolist() == [0, 0, 60, 50, 40, 0]


def test_window_mask_and_sink():
    m = plain.window_mask(9, 3, 2)
    assert m[8].tolist() == [True, True, False, False, False, False, True, True, True]
    assert m[3].tolist() == [True, True, True, True, False, False, False, False, False]
    assert m[4].tolist() == [True, True, True, True, True, False, False, False, False]
    assert plain.window_mask(5, 2, 0)[4].tolist() == [False, False, False, True, True]
    s = torch.zeros(3, 3, dtype=F64)
    p = plain.softmax_with_sink(s, torch.tril(torch.ones(3, 3, dtype=torch.bool)), torch.zeros((), dtype=F64))
    assert torch.allclose(p.sum(-1), torch.tensor([1 / 2, 2 / 3, 3 / 4], dtype=F64))           # one added to the denominator
    p = plain.softmax_with_sink(s, torch.tril(torch.ones(3, 3, dtype=torch.bool)), torch.tensor(math.log(3.0), dtype=F64))
    assert torch.allclose(p.sum(-1), torch.tensor([1 / 4, 2 / 5, 3 / 6], dtype=F64))


def test_windowed_attention_closed_form():
    """Zero query weights: every visible key weighs the same and the sink as much as one key, so a head's result is the
    sum of the visible convolved keys over (their number + 1), times the gate; the values are the keys BEFORE norm and
    rotation; query head a reads key head a // (heads / kv_heads)."""
    T, C = 7, 5
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 1.0, "conv": 2, "mask": {"size": 3, "keep_first": 1},
         "rot": {"base": 10.0, "dims": 2}}
    g = torch.Generator().manual_seed(0)
    h = torch.randn(T, C, generator=g, dtype=F64)
    w = {"q": torch.zeros(8, C, dtype=F64), "k": torch.randn(4, C, generator=g, dtype=F64),
         "q.conv": torch.randn(8, 2, generator=g, dtype=F64), "k.conv": torch.tensor([[0.5, 2.0]] * 4, dtype=F64),
         "q.norm": torch.ones(8, dtype=F64), "k.norm": torch.ones(4, dtype=F64), "g": torch.zeros(8, C, dtype=F64),
         "o": torch.cat([torch.eye(4, dtype=F64), torch.eye(4, dtype=F64)], 1)[:C - 1].repeat(2, 1)[:C]}
    k = h @ w["k"].T
    v = 2.0 * k + 0.5 * torch.cat([torch.zeros(1, 4, dtype=F64), k[:-1]])
    mask = plain.window_mask(T, 3, 1).to(F64)
    mean = (mask @ v) / (mask.sum(-1, keepdim=True) + 1.0)
    want = (torch.cat([mean, mean], 1) * 0.5) @ w["o"].T
    assert torch.allclose(plain.windowed_attention(h, w, m, 1e-5), want)


def test_latent_attention_closed_form():
    """Zero query weights and a sink of log 2: uniform weights over the causal keys with two more in the denominator; the
    values are W_uv times the NORMED latent; the rotated key part is not normed."""
    T, C = 4, 6
    m = {"heads": 1, "dim": 2, "rot_dim": 2, "vdim": 3, "kv_rank": 4, "scale": 0.7, "rot": {"base": 10.0, "dims": 2}}
    g = torch.Generator().manual_seed(1)
    h = torch.randn(T, C, generator=g, dtype=F64)
    w = {"q": torch.zeros(4, C, dtype=F64), "dkv": torch.randn(6, C, generator=g, dtype=F64),
         "dkv.norm": torch.tensor([1.0, 2.0, 0.5, 1.5], dtype=F64), "uk": torch.randn(2, 4, generator=g, dtype=F64),
         "uv": torch.randn(3, 4, generator=g, dtype=F64), "sink": torch.tensor([math.log(2.0)], dtype=F64),
         "g": torch.zeros(3, C, dtype=F64), "o": torch.randn(C, 3, generator=g, dtype=F64)}
    c = plain.rms_norm((h @ w["dkv"].T)[:, :4], w["dkv.norm"], 1e-5)
    v = c @ w["uv"].T
    mean = torch.cumsum(v, 0) / (torch.arange(1, T + 1, dtype=F64).view(-1, 1) + 2.0)
    assert torch.allclose(plain.latent_attention(h, w, m, 1e-5), (mean * 0.5) @ w["o"].T)
    # the rotated parts matter: a query that only has a rotated part prefers the key whose rotated part it meets
    w2 = dict(w, q=torch.randn(4, C, generator=g, dtype=F64))
    assert not torch.allclose(plain.latent_attention(h, w2, m, 1e-5), plain.latent_attention(h, w, m, 1e-5))


def test_mlstm_closed_forms():
    """One token with input gate i and forget gate f (logarithms): m = max(f, i) since m starts at ZERO, S = exp(i - m) k v^T,
    o = exp(i - m) (k . q) v / (max(exp(i - m) |k . q|, exp(-m)) + 1e-6). With f = 0 and i = 0 throughout, the state is
    the plain sum of k v^T and the denominator max(|n . q|, 1)."""
    q = torch.tensor([[1.0, 2.0]], dtype=F64)
    k = torch.tensor([[0.5, -1.0]], dtype=F64)
    v = torch.tensor([[3.0, 4.0, 5.0]], dtype=F64)
    for i_log, f_log in ((-2.0, -0.1), (1.5, -3.0), (-5.0, -4.0)):
        o = plain.mlstm_steps(q, k, v, torch.tensor([i_log], dtype=F64), torch.tensor([f_log], dtype=F64))
        m = max(f_log + 0.0, i_log)
        kq = float(k[0] @ q[0])
        want = math.exp(i_log - m) * kq * v[0] / (max(abs(math.exp(i_log - m) * kq), math.exp(-m)) + 1e-6)
        assert torch.allclose(o[0], want)
    g = torch.Generator().manual_seed(2)
    T = 6
    q, k, v = (torch.randn(T, n, generator=g, dtype=F64) for n in (3, 3, 2))
    zero = torch.zeros(T, dtype=F64)
    o = plain.mlstm_steps(q, k, v, zero, zero)
    for t in range(T):
        S = k[:t + 1].T @ v[:t + 1]
        n = k[:t + 1].sum(0)
        assert torch.allclose(o[t], (S.T @ q[t]) / (max(abs(float(n @ q[t])), 1.0) + 1e-6))
    # the gates' caps: a huge raw value is capped
    m = {"heads": 1, "dim": 3, "vdim": 2, "gate_cap": 2.0}
    C = 4
    h = torch.randn(T, C, generator=g, dtype=F64)
    w = {n: torch.randn(r, C, generator=g, dtype=F64) for n, r in (("q", 3), ("k", 3), ("v", 2), ("g", 2))}
    w.update({"i": torch.zeros(1, C, dtype=F64), "f": torch.zeros(1, C, dtype=F64), "i.b": torch.tensor([50.0], dtype=F64),
              "f.b": torch.tensor([-50.0], dtype=F64), "norm": torch.ones(2, dtype=F64), "o": torch.randn(C, 2, generator=g, dtype=F64)})
    capped = plain.mlstm(h, w, m, 1e-5)
    w2 = dict(w, **{"i.b": torch.tensor([60.0], dtype=F64)})
    assert torch.allclose(capped, plain.mlstm(h, w2, m, 1e-5))


def test_experts_closed_forms():
    """The exact gelu; the weights are the softmax over the CHOSEN logits alone and multiply the experts' outputs; the
    bias takes part in the choice; the shared expert is added for every token."""
    z = torch.tensor([-1.0, 0.0, 2.0], dtype=F64)
    assert torch.allclose(plain.gelu_erf(z), z * 0.5 * (1 + torch.erf(z / math.sqrt(2.0))))
    C = 4
    g = torch.Generator().manual_seed(1)
    w = {"router": torch.tensor([[5.0, 0, 0, 0], [0, 5.0, 0, 0], [0, 0, 0.1, 0]], dtype=F64), "router.b": torch.tensor([0.0, 0.0, 3.0], dtype=F64)}
    for e in range(3):
        w[f"e{e}.up"] = torch.randn(5, C, generator=g, dtype=F64)
        w[f"e{e}.down"] = torch.randn(C, 5, generator=g, dtype=F64)
    mlp = {"router": {"experts": 3, "top": 2}, "expert": {"ff": 5}}
    h = torch.tensor([[1.0, 0.2, 0, 0.3], [0.1, 2.0, 0, 0]], dtype=F64)
    out = plain.routed_ff(h, w, mlp)
    for t, (a, b) in enumerate(((0, 2), (1, 2))):
        za, zb = 5.0 * h[t, a].item(), 3.0
        pa = math.exp(za) / (math.exp(za) + math.exp(zb))
        want = pa * plain.plain_expert(h[t:t + 1], w[f"e{a}.up"], w[f"e{a}.down"]) + \
            (1 - pa) * plain.plain_expert(h[t:t + 1], w[f"e{b}.up"], w[f"e{b}.down"])
        assert torch.allclose(out[t], want[0])
    w.update({"shared.up": w["e1.up"], "shared.down": w["e1.down"]})
    out2 = plain.routed_ff(h, w, dict(mlp, shared={"ff": 5}))
    assert torch.allclose(out2, out + plain.plain_expert(h, w["e1.up"], w["e1.down"]))
    assert plain.router_margin(torch.tensor([[3.0, 1.0, 2.5]], dtype=F64), 1).item() == 0.5


def test_layer_arrangement_shared_weights_and_soft_cap():
    """The norm is on the sublayer's RESULT, scaled by the multiplier, and the sublayers read the stream itself; a layer
    with another's weights runs the same block on its own input; the logits pass the soft cap."""
    c = CONFIGS["odd"]
    weights = {k: v.double() for k, v in make_weights(c, 2).items()}
    toks = [3, 50, 7, 7, 90, 1, 200, 4]
    layers = []
    logits = plain.forward(c, weights, toks, layers_out=layers)
    assert len(layers) == 6
    eps, mult = c["norm"]["eps"], c["residual_mult"]
    x = weights["embed"][torch.tensor(toks)]
    y = plain.windowed_attention(x, plain.sub(weights, "l0.mix."), c["layers"][0]["mixer"], eps)
    x = x + mult * plain.rms_norm(y, weights["l0.norm1"], eps)
    x = x + mult * plain.rms_norm(plain.dense_ff(x, plain.sub(weights, "l0.mlp.")), weights["l0.norm2"], eps)
    assert torch.allclose(layers[0], x)
    x = layers[2]
    y = plain.windowed_attention(x, plain.sub(weights, "l0.mix."), c["layers"][0]["mixer"], eps)
    x = x + mult * plain.rms_norm(y, weights["l0.norm1"], eps)
    x = x + mult * plain.rms_norm(plain.dense_ff(x, plain.sub(weights, "l0.mlp.")), weights["l0.norm2"], eps)
    assert torch.allclose(layers[3], x)
    x = layers[3]
    y = plain.latent_attention(x, plain.sub(weights, "l4.mix."), c["layers"][4]["mixer"], eps)
    assert torch.allclose(layers[4], x + mult * plain.rms_norm(y, weights["l4.norm1"], eps))           # no feed-forward
    raw = plain.rms_norm(layers[5], weights["final.norm"], eps) @ weights["head"].T
    assert torch.allclose(logits, 9.0 * torch.tanh(raw / 9.0)) and logits.abs().max() < 9.0
