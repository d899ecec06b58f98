"""The Rufusun design on the GPU against the plain implementation (`plain_rufusun.py`).

Mechanisms alone (each kernel against the plain function of the same mechanism: the paired norm, the convolution with
its activation and carried inputs, the gated delta rule over differently cut sequences in reused slots, the per-head
norm with its gate, the router with ties, the grouped experts with few and many rows, the limited swish in the gated
product's epilogue and in its own kernel), then whole models through the package's loader, cache manager and step
function: prefill against token-by-token decoding, portions down to two tokens, unequal batches against each request
alone, few pages and slots that are freed and used again, attention made sharp so that single keys far back carry
the result, a state that must survive hundreds of tokens, long decoding from HIP graphs, sizes drawn at random, and
greedy generation through the scheduler.

Bars: float32 rows must agree with the float64 plain implementation to 2e-5 of the logits' spread (the kernels sum
in other orders); bfloat16 to 3 % of it (bfloat16 rounds to 0.4 %, a few dozen roundings deep). A router may send a
token whose two best experts nearly tie the other way in bfloat16, and a unit norm behind sums that nearly cancel
magnifies its inputs' rounding: one bfloat16 row in fifty may lie up to twice as far. A token whose router logits
nearly tie between the last expert chosen and the next (`plain.router_margin` under CLOSE) may go the other way in
bfloat16, whose rounding of the router's input moves a logit by a few hundredths: in bfloat16 the rows of a sequence
before its first such token are held to the bar (one in twenty up to three times as far: the narrow models here round
coarsely), and of all rows the typical one must stay within the bar and at most one in ten (or five) may lie beyond three times
it, since a token that ran another expert is far off and leaves its mark on what follows. The float32 runs hold
every row to the strict bar, and every kernel that runs in bfloat16 is the same template.
"""
import math
import random

import numpy as np
import pytest
import torch

import plain_rufusun as plain
from rufusun_util import CONFIGS, Driver, attention, config, delta, dense, make_weights, moe, row_error, write_folder

pytestmark = pytest.mark.gpu

BAR = {"float32": 2e-5, "bfloat16": 3e-2}
CLOSE = 0.1


def reference(c, weights, toks):
    """(logits [T, V], per token the smallest router margin over all runs of routed layers) of the plain implementation."""
    margins = []
    logits = plain.forward(c, double(weights), toks, margins=margins).numpy()
    least = torch.stack(margins).min(0).values.numpy() if margins else np.full(len(toks), np.inf)
    return logits, least


def tdtype(name):
    return getattr(torch, name)


def ints(values, device):
    return torch.tensor(values, dtype=torch.int32, device=device)


def double(weights):
    return {k: v.double() for k, v in weights.items()}


# ---------------------------------------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,C", [(5, 88), (70, 1000), (3, 4097), (4, 4096), (2, 90), (2, 6000)])
def test_paired_norm(device, dtype, n, C):
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(n)
    x = (torch.randn(n, C, generator=g) * 3).to(device)
    w1, w2 = (0.3 * torch.randn(C, generator=g) for _ in range(2))
    out1, out2 = (torch.empty(n, C, dtype=tdtype(dtype), device=device) for _ in range(2))
    ops.rmsnorm_pair(x, (1 + w1).to(device), 1e-5, out1, (1 + w2).to(device), out2)
    tol = 1e-5 if dtype == "float32" else 1e-2
    for out, w in ((out1, w1), (out2, w2)):
        want = plain.offset_norm(x.double().cpu(), w.double(), 1e-5)
        assert ((out.double().cpu() - want).abs() <= tol * (1 + want.abs())).all()
    alone = torch.empty_like(out1)
    ops.rmsnorm_pair(x, (1 + w1).to(device), 1e-5, alone)
    assert torch.equal(alone, out1)


@pytest.mark.parametrize("taps,C", [(4, 44), (3, 46), (1, 20), (2, 600)])
def test_convolution_with_silu_carries_its_inputs(device, taps, C):
    """Three sequences in differently cut portions over three steps, in state slots with stale contents; the rows are
    columns of a wider float32 tensor, as a packed projection leaves them."""
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(taps)
    lens = {"a": 9, "b": 4, "c": 6}
    xs = {k: torch.randn(n, C, generator=g) for k, n in lens.items()}
    w = 0.5 * torch.randn(C, taps, generator=g)
    want = {k: torch.nn.functional.silu(plain.short_conv(v.double(), w.double())) for k, v in xs.items()}
    state = torch.full((3, 2, max(taps - 1, 1), C), 7.0, device=device)
    slot = {"a": 2, "b": 0, "c": 1}
    for s in slot.values():
        state[s] = 0                                                    # what opening a request does
    state[slot["b"], 1] = 9.0                                           # the copy a first step does not read may hold anything
    at, steps_of = {k: 0 for k in lens}, {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for parts in ([("c", 1), ("a", 5), ("b", 2)], [("c", 1), ("a", 1)], [("a", 3), ("b", 2), ("c", 4)]):
        rows = torch.cat([xs[k][at[k]:at[k] + n] for k, n in parts])
        wide = torch.zeros(rows.shape[0], C + 12, device=device)
        wide[:, :C] = rows.to(device)
        starts = np.cumsum([0] + [n for _, n in parts]).tolist()
        out = torch.empty(rows.shape[0], C, device=device)
        ops.causal_conv(wide[:, :C], w.to(device), state, ints(starts, device), ints([at[k] + n for k, n in parts], device),
                        ints([slot[k] for k, _ in parts], device), ints([steps_of[k] & 1 for k, _ in parts], device), len(parts),
                        out32=out, activation="silu")
        for i, (k, n) in enumerate(parts):
            got[k].append(out[starts[i]:starts[i] + n].cpu())
            at[k] += n
            steps_of[k] += 1
    for k in lens:
        assert torch.allclose(torch.cat(got[k]).double(), want[k], atol=1e-5), k


def plain_delta_heads(q, k, v, b, a, A_log, dt_bias, H, G, D, E):
    """float64 [T, H * E]: the recurrence of every head from raw q, k (unit norms inside), b and a."""
    T = q.shape[0]
    q = q.view(T, G, D)
    k = k.view(T, G, D)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(b)
    decay = torch.exp(-torch.exp(A_log) * torch.nn.functional.softplus(a + dt_bias))
    out = [plain.delta_rule(q[:, h // (H // G)], k[:, h // (H // G)], v.view(T, H, E)[:, h], beta[:, h], decay[:, h]) for h in range(H)]
    return torch.stack(out, 1).reshape(T, H * E)


@pytest.mark.parametrize("most", [1, 64], ids=["walked", "chunks_solved"])
@pytest.mark.parametrize("H,G,D,E", [(4, 2, 20, 24), (3, 3, 40, 72), (2, 1, 13, 10), (1, 1, 128, 128), (2, 2, 256, 16), (8, 1, 64, 64)])
def test_delta_rule_over_cut_sequences_in_reused_slots(device, H, G, D, E, most):
    """Three sequences cut differently over four steps (portions of 37 and 21 tokens across chunks of the kernel, two
    tokens, single tokens), the state carried in slots that held another request before. Decays near one: what the
    first tokens wrote still weighs at the end. Once with every token walked in turn, once with every step (its single
    tokens too) through the kernel that solves 16 tokens at once."""
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(H * 100 + D)
    lens = {"a": 60, "b": 25, "c": 9}
    W = 2 * G * D + H * E
    rows = {k: torch.randn(n, W, generator=g) for k, n in lens.items()}
    ab = {k: torch.randn(n, 2 * H + 3, generator=g) for k, n in lens.items()}          # b at 1.., a at 1 + H..
    A_log, dt_bias = -1.0 + 0.5 * torch.randn(H, generator=g), -3.0 + torch.randn(H, generator=g)
    want = {k: plain_delta_heads(rows[k][:, :G * D].double(), rows[k][:, G * D:2 * G * D].double(), rows[k][:, 2 * G * D:].double(),
                                 ab[k][:, 1:1 + H].double(), ab[k][:, 1 + H:1 + 2 * H].double(), A_log.double(), dt_bias.double(),
                                 H, G, D, E) for k in lens}
    state = torch.randn(4, H, E, ops.delta_key_extent(D), generator=g).to(device)       # stale contents everywhere
    slot = {"a": 3, "b": 1, "c": 0}
    for s in slot.values():
        state[s] = 0
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for parts in ([("c", 1), ("a", 37), ("b", 2)], [("c", 1), ("b", 1), ("a", 1)], [("b", 1), ("a", 21), ("c", 7)], [("a", 1), ("b", 21)]):
        parts = [(k, n) for k, n in parts if n]
        qkv = torch.cat([rows[k][at[k]:at[k] + n] for k, n in parts]).to(device)
        gates = torch.cat([ab[k][at[k]:at[k] + n] for k, n in parts]).to(device)
        starts = np.cumsum([0] + [n for _, n in parts]).tolist()
        out = torch.full((qkv.shape[0], H * E), float("nan"), device=device)
        ops.delta_rule(qkv, 0, G * D, 2 * G * D, gates, 1, 1 + H, A_log.to(device), dt_bias.to(device), state,
                       ints(starts, device), ints([slot[k] for k, _ in parts], device), 0, len(parts), out, G, D, D ** -0.5,
                       max_q_len=most)
        for i, (k, n) in enumerate(parts):
            got[k].append(out[starts[i]:starts[i] + n].cpu())
            at[k] += n
    for k in lens:
        res = torch.cat(got[k]).double()
        assert torch.isfinite(res).all()
        assert (res - want[k]).abs().max() < 2e-5 * max(1.0, want[k].abs().max().item()), (k, (res - want[k]).abs().max())
    # a second request in a's slot starts from zero once the slot is cleared, whatever a left there
    state[slot["a"]] = 0
    out = torch.empty(lens["c"], H * E, device=device)
    ops.delta_rule(rows["c"].to(device), 0, G * D, 2 * G * D, ab["c"].to(device), 1, 1 + H, A_log.to(device), dt_bias.to(device), state,
                   ints([0, lens["c"]], device), ints([slot["a"]], device), 0, 1, out, G, D, D ** -0.5, max_q_len=most)
    assert (out.cpu().double() - want["c"]).abs().max() < 2e-5 * max(1.0, want["c"].abs().max().item())


@pytest.mark.parametrize("H,G,D,E", [(2, 1, 64, 48), (1, 1, 128, 20), (2, 2, 200, 16)])
def test_delta_rule_long_portions_solved_in_chunks(device, H, G, D, E):
    """500 tokens in portions of 333 and 167 (neither a multiple of a chunk's 16 tokens) beside a second sequence of one
    token a step: thirty chunks whose states follow from each other, slow decays, value columns in one to three blocks."""
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(D + E)
    n = 500
    W = 2 * G * D + H * E
    rows, ab = torch.randn(n, W, generator=g), torch.randn(n, 2 * H, generator=g)
    other, other_ab = torch.randn(2, W, generator=g), torch.randn(2, 2 * H, generator=g)
    A_log, dt_bias = -2.0 + 0.5 * torch.randn(H, generator=g), -3.0 + torch.randn(H, generator=g)

    def plain_of(r, gates):
        return plain_delta_heads(r[:, :G * D].double(), r[:, G * D:2 * G * D].double(), r[:, 2 * G * D:].double(),
                                 gates[:, :H].double(), gates[:, H:].double(), A_log.double(), dt_bias.double(), H, G, D, E)
    want, want_other = plain_of(rows, ab), plain_of(other, other_ab)
    state = torch.zeros(3, H, E, ops.delta_key_extent(D), device=device)
    got, got_other, at = [], [], 0
    for step, take in enumerate((333, 167)):
        qkv = torch.cat([other[step:step + 1], rows[at:at + take]]).to(device)
        gates = torch.cat([other_ab[step:step + 1], ab[at:at + take]]).to(device)
        out = torch.full((take + 1, H * E), float("nan"), device=device)
        ops.delta_rule(qkv, 0, G * D, 2 * G * D, gates, 0, H, A_log.to(device), dt_bias.to(device), state,
                       ints([0, 1, take + 1], device), ints([2, 0], device), 0, 2, out, G, D, D ** -0.5, max_q_len=take)
        got_other.append(out[:1].cpu())
        got.append(out[1:].cpu())
        at += take
    for res, ref in ((torch.cat(got).double(), want), (torch.cat(got_other).double(), want_other)):
        assert torch.isfinite(res).all()
        assert (res - ref).abs().max() < 1e-4 * max(1.0, ref.abs().max().item()), (res - ref).abs().max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_norm_with_gate(device, dtype):
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    n, H, E = 7, 3, 72
    o, gate = torch.randn(n, H * E, generator=g) * 4, torch.randn(n, H * E + 5, generator=g)
    w = 1 + 0.3 * torch.randn(E, generator=g)
    out = torch.empty(n, H * E, dtype=tdtype(dtype), device=device)
    ops.head_norm_gate(o.to(device), gate.to(device)[:, 5:], w.to(device), out, H, E, 1e-5)
    want = (plain.rms_unit(o.double().view(n, H, E), 1e-5) * w.double() * torch.nn.functional.silu(gate[:, 5:].double()).view(n, H, E)).view(n, -1)
    tol = 1e-5 if dtype == "float32" else 1e-2
    assert ((out.double().cpu() - want).abs() <= tol * (1 + want.abs())).all()


@pytest.mark.parametrize("C,X,top", [(72, 70, 4), (90, 7, 3), (64, 1, 1), (2048, 16, 2)])
def test_router_picks_the_largest_and_the_lowest_index_on_ties(device, C, X, top):
    """Widths with and without 16-byte rows, an odd number of experts, one expert."""
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    n = 40
    h = torch.randn(n, C, generator=g)
    router = torch.randn(X, C, generator=g) / math.sqrt(C)
    if X > 60:
        router[5] = router[60]                                          # experts 5 and 60 always tie
        router[9] = router[60] + 0.0
    ids = torch.empty(n, top, dtype=torch.int32, device=device)
    weights = torch.empty(n, top, device=device)
    ops.moe_route(h.to(device), router.to(device), top, ids, weights)
    z = h.double() @ router.double().T
    for t in range(n):
        order = sorted(range(X), key=lambda e: (-round(z[t, e].item(), 9), e))
        chosen = ids[t].tolist()
        for e in chosen:
            if X > 60 and e in (9, 60):
                assert 5 in chosen and chosen.index(5) < chosen.index(e)
        clear = [e for i, e in enumerate(order[:top]) if top == X or z[t, order[top]] < z[t, e] - 1e-4]
        assert set(clear) <= set(chosen)
        assert torch.allclose(weights[t].cpu().double(), torch.sigmoid(z[t, chosen]), atol=1e-5)
    # bfloat16 rows: the products are float32 of the rows as they are
    hb = h.to(torch.bfloat16)
    ops.moe_route(hb.to(device), router.to(device), top, ids, weights)
    zb = hb.double() @ router.double().T
    assert torch.allclose(weights.cpu().double(), torch.sigmoid(torch.gather(zb, 1, ids.cpu().long())), atol=1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,C,X,top,F", [(1, 88, 5, 2, 40), (9, 128, 16, 4, 64), (300, 96, 3, 3, 24), (130, 72, 64, 1, 100), (17, 64, 2, 1, 32),
                                         (40, 64, 2, 1, 32), (7, 90, 6, 2, 40), (700, 256, 16, 2, 96)])
def test_grouped_experts(device, dtype, n, C, X, top, F):
    """Against the plain expert, row by row, for given choices and scores (few rows, many rows an expert, experts
    nobody chose, sizes that are no multiples of 32); the result is added to what x held."""
    from tessweave_engine_amd.kernels import ops
    from tessweave_engine_amd.parts.base import Workspace
    dt = tdtype(dtype)
    g = torch.Generator().manual_seed(n + X)
    h = torch.randn(n, C, generator=g).to(dt)
    gate, up = (2 * torch.randn(X, F, C, generator=g) / math.sqrt(C) for _ in range(2))
    down = torch.randn(X, C, F, generator=g) / math.sqrt(F)
    gate, up, down = gate.to(dt), up.to(dt), down.to(dt)
    ids = torch.stack([torch.randperm(X, generator=g)[:top] for _ in range(n)]).to(torch.int32)
    if X > 4 and top == 1:
        ids[ids == 1] = 0                                                # nobody runs expert 1
    weights = torch.rand(n, top, generator=g)
    limit = 1.3
    Cd, Fd = ops.moe_pad(C), ops.moe_pad(F)
    gd, ud, dd = torch.zeros(X, Fd, Cd, dtype=dt), torch.zeros(X, Fd, Cd, dtype=dt), torch.zeros(X, C, Fd, dtype=dt)
    gd[:, :F, :C], ud[:, :F, :C], dd[:, :, :F] = gate, up, down
    x0 = torch.randn(n, C, generator=g)
    x = x0.clone().to(device)
    ws = Workspace(device)
    ops.moe_experts(h.to(device), ids.to(device), weights.to(device), ops.moe_blocked(gd.to(device)),
                    ops.moe_blocked(ud.to(device)), ops.moe_blocked(dd.to(device)), limit, x,
                    lambda tag, shape, dtype: ws.get(tag, shape, dtype))
    want = x0.double().clone()
    for t in range(n):
        for r in range(top):
            e = int(ids[t, r])
            y = (weights[t, r] * h[t].float()).to(dt).double()           # the scaled input is rounded to the compute type
            want[t] += plain.limited_expert(y[None], gate[e].double(), up[e].double(), down[e].double(), limit)[0]
    err = (x.cpu().double() - want).abs().max().item()
    assert err < (2e-5 if dtype == "float32" else 3e-2) * max(1.0, want.abs().max().item()), err


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("m,F,C", [(3, 48, 88), (200, 96, 128), (70, 56, 64)])
def test_limited_swish_in_the_gated_product_and_alone(device, dtype, m, F, C):
    from tessweave_engine_amd.kernels import ops
    dt = tdtype(dtype)
    g = torch.Generator().manual_seed(m)
    x = torch.randn(m, C, generator=g).to(dt)
    gate, up = (2 * torch.randn(F, C, generator=g) / math.sqrt(C) for _ in range(2))
    gate, up = gate.to(dt), up.to(dt)
    limit = 0.9
    gv, uv = (x.double() @ gate.double().T).clamp(max=limit), (x.double() @ up.double().T).clamp(-limit, limit)
    want = gv * torch.sigmoid(1.702 * gv) * (uv + 1)
    tol = 1e-5 if dtype == "float32" else 2e-2
    if F % 16 == 0:
        w = ops.shuffle_weight(ops.interleave_glu_rows(gate, up).to(device))
        out = torch.empty(m, F, dtype=dt, device=device)
        ops.linear_glu(x.to(device), w, out, activation="swish_limited", factor=limit)
        assert ((out.double().cpu() - want).abs() <= tol * (1 + want.abs())).all()
    gu = torch.cat([x.double() @ gate.double().T, x.double() @ up.double().T], 1).to(dt)
    out = torch.empty(m, F, dtype=dt, device=device)
    ops.swish_limited_mul(gu.to(device), out, limit)
    gv, uv = gu[:, :F].double().clamp(max=limit), gu[:, F:].double().clamp(-limit, limit)
    want = gv * torch.sigmoid(1.702 * gv) * (uv + 1)
    assert ((out.double().cpu() - want).abs() <= tol * (1 + want.abs())).all()


# ---------------------------------------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------------------------------------

LENGTHS = {"odd": [61, 3, 40, 1, 29, 75], "wide": [50, 37, 2, 66], "one": [44, 9, 30]}


@pytest.fixture(scope="module", params=list(CONFIGS))
def model(request, tmp_path_factory, device):
    name = request.param
    c = CONFIGS[name]
    weights = make_weights(c, seed=len(name))
    folder = write_folder(tmp_path_factory.mktemp("rufusun_" + name), c, weights)
    g = torch.Generator().manual_seed(50 + len(name))
    tokens = {f"r{i}": torch.randint(0, c["vocab"], (n,), generator=g).tolist() for i, n in enumerate(LENGTHS[name])}
    both = {rid: reference(c, weights, toks) for rid, toks in tokens.items()}
    return dict(name=name, config=c, weights=weights, folder=folder, tokens=tokens, want={k: v[0] for k, v in both.items()},
                margin={k: v[1] for k, v in both.items()})


def check_rows(err, dtype, what="", margin=None):
    """ERR: one relative error per row of ONE sequence (or of several, without margins)."""
    err = np.asarray(err)
    if dtype == "bfloat16":
        margin = np.full(len(err), np.inf) if margin is None else np.asarray(margin)
        close = margin < CLOSE
        behind = np.cumsum(close) > 0                              # rows that may have read what a close call left
        sure = err[~behind]
        if len(sure):
            assert sure.max() < 3 * BAR[dtype], (what, int(sure.argmax()), float(sure.max()))
            assert (sure > BAR[dtype]).sum() <= max(1, len(sure) // 20), (what, np.nonzero(sure > BAR[dtype])[0].tolist())
        assert np.median(err) < BAR[dtype], (what, float(np.median(err)))
        assert (err > 3 * BAR[dtype]).sum() <= max(5, len(err) // 10), (what, np.nonzero(err > 3 * BAR[dtype])[0].tolist())
    else:
        assert err.max() < BAR[dtype], (what, int(err.argmax()), float(err.max()))


def check_all(model, got, dtype, only=None):
    for rid, want in model["want"].items():
        if only is not None and rid not in only:
            continue
        assert np.isfinite(got[rid]).all()
        check_rows(row_error(got[rid], want), dtype, rid, model["margin"][rid])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts(model, dtype):
    d = Driver(model["folder"], dtype, pages=24, page_size=8)
    got = d.run([[(rid, len(toks))] for rid, toks in model["tokens"].items()], model["tokens"])
    check_all(model, got, dtype)
    d.close()


def test_stream_after_every_layer(model):
    """float32: the residual stream after each layer run (a looped layer counts each time) against the plain one's."""
    from tessweave_engine_amd.engine.step import StepEntry
    rid = "r0"
    toks = model["tokens"][rid]
    _, want = plain.forward(model["config"], double(model["weights"]), toks, keep_layers=True)
    d = Driver(model["folder"], "float32", pages=24, page_size=8, graphs=False)
    seq = d.cache.open(rid)
    ctx, ordered, _ = d.stepper.prepare([StepEntry(seq, list(toks), [len(toks) - 1])])
    seen = []
    ctx.segment_end = lambda i: seen.append(ctx.scratch("residual", (ctx.n_tokens, model["config"]["width"]), torch.float32).clone())
    with torch.cuda.stream(d.stepper.stream):
        d.stepper.upload(ctx)
        d.model.forward(ctx)
    d.stepper.synchronize()
    d.stepper.finish(ordered)
    assert len(seen) == len(want)
    for i, (got, ref) in enumerate(zip(seen, want)):
        assert torch.allclose(got.cpu().double(), ref, atol=2e-5 * max(1.0, ref.abs().max().item())), i
    d.close()


@pytest.mark.parametrize("dtype,graphs", [("float32", True), ("float32", False), ("bfloat16", True)])
def test_token_by_token(model, dtype, graphs):
    """Every token decoded alone from the first on (the first tokens of a sequence included)."""
    rid = "r0"
    d = Driver(model["folder"], dtype, pages=24, page_size=4, graphs=graphs)
    got = d.run([[(rid, 1)] for _ in model["tokens"][rid]], model["tokens"])
    check_all(model, got, dtype, only=[rid])
    if graphs:
        assert d.model.graph_safe_model and d.stepper.graph_replays > 0
    d.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [[2], [3, 1, 2], [16, 5, 2, 2, 9], [7, 8, 1]])
def test_portions(model, dtype, sizes):
    rid = max(model["tokens"], key=lambda r: len(model["tokens"][r]))
    total, schedule, i = len(model["tokens"][rid]), [], 0
    while total:
        n = min(sizes[i % len(sizes)], total)
        schedule.append([(rid, n)])
        total -= n
        i += 1
    d = Driver(model["folder"], dtype, pages=40, page_size=4)
    got = d.run(schedule, model["tokens"])
    check_all(model, got, dtype, only=[rid])
    d.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [0, 1])
def test_unequal_batches_few_pages_two_slots(model, dtype, seed):
    """Portions of some requests beside single tokens of others; at most two requests live, so that every state slot
    is used again (delta states, convolution inputs), and a page pool that only just holds them."""
    rng = random.Random(seed)
    tokens = model["tokens"]
    pending, live, schedule = list(tokens), {}, []
    while pending or live:
        while pending and len(live) < 2:
            rid = pending.pop(0)
            live[rid] = dict(left=len(tokens[rid]), prompt=rng.randrange(1, len(tokens[rid]) + 1))
        parts = []
        for rid, r in list(live.items()):
            if len(live) > 1 and rng.random() < 0.25:
                continue
            n = min(r["left"], rng.choice([2, 3, 5, 11, 16]) if r["prompt"] > 0 else 1)
            r["prompt"] -= n
            r["left"] -= n
            parts.append((rid, n))
            if r["left"] == 0:
                del live[rid]
        if parts:
            schedule.append(parts)
    page = 8
    longest = sorted(len(t) for t in tokens.values())[-2:]
    pages = sum((n + page - 1) // page for n in longest)
    d = Driver(model["folder"], dtype, pages=pages, page_size=page, max_requests=2)
    got = d.run(schedule, tokens)
    check_all(model, got, dtype)
    d.close()


def test_ways_of_cutting_agree(model):
    """float32: whole, token by token and in portions beside another request differ by rounding only."""
    tokens = model["tokens"]
    rid, other = "r0", "r2"
    runs = []
    for schedule in ([[(rid, len(tokens[rid]))]],
                     [[(rid, 1)] for _ in tokens[rid]],
                     [[(other, 1), (rid, 5)]] + [[(rid, 2), (other, 1)] for _ in range(500)]):
        d = Driver(model["folder"], "float32", pages=40, page_size=4)
        fixed, used = [], {}
        for parts in schedule:
            parts = [(r, min(n, len(tokens[r]) - used.get(r, 0))) for r, n in parts]
            parts = [(r, n) for r, n in parts if n > 0]
            for r, n in parts:
                used[r] = used.get(r, 0) + n
            if parts:
                fixed.append(parts)
        runs.append(d.run(fixed, tokens)[rid])
        d.close()
    for other_run in runs[1:]:
        assert row_error(other_run, runs[0]).max() < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "wide"])
def test_sharp_attention_over_a_long_prompt(device, tmp_path, dtype, name):
    """Queries eight times as large: every softmax sits on one or two keys, wherever they lie among hundreds (far back,
    at a page's edge, the first token), as far as the soft cap lets it. 600 tokens: 330 in one step, then portions of
    64, 15, 2 and single tokens, on pages of four tokens handed out in an order of their own. float32 rows must agree
    to 1e-3, where a key that is lost or seen wrongly moves a row by a tenth and more; in bfloat16 the typical row must
    stay within the bar."""
    c = CONFIGS[name]
    weights = make_weights(c, seed=13, sharp=8.0 if dtype == "float32" else 3.0)
    folder = write_folder(tmp_path, c, weights)
    toks = torch.randint(0, c["vocab"], (600,), generator=torch.Generator().manual_seed(4)).tolist()
    want = plain.forward(c, double(weights), toks).numpy()
    d = Driver(folder, dtype, pages=180, page_size=4, max_step_tokens=64)
    warm = {"w0": toks[:37], "w1": toks[:90]}
    d.step([("w0", 37), ("w1", 90)], warm)
    d.end("w0")
    schedule = [[("a", 330)], [("a", 64)], [("a", 15)], [("a", 2)]] + [[("a", 1)]] * 9 + [[("a", 90)], [("a", 90)]]
    got = d.run(schedule, {"a": toks})["a"]
    d.end("w1")
    err = row_error(got, want)
    if dtype == "float32":
        assert err.max() < 1e-3, (int(err.argmax()), float(err.max()))
    else:
        assert np.median(err) < BAR[dtype], float(np.median(err))
    d.close()


def test_a_state_that_remembers_its_first_tokens(device, tmp_path):
    """One delta layer whose decay is one and whose writes are strong (A_log very negative, b large): the logits at
    the end depend on the first tokens. Two prompts that differ in their first three tokens only must differ at token
    200 and later, and each must match the plain implementation whether it ran whole, or in portions and single tokens."""
    c = config([delta(2, 1, 64, 48, 2, mlp=dense(64))], width=64, vocab=50, logit_scale=1.0)
    weights = make_weights(c, seed=4)
    weights["l0.mix.A_log"] = torch.full((2,), -12.0).to(torch.bfloat16)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(9)
    base = torch.randint(0, 50, (260,), generator=g).tolist()
    other = [(t + 7) % 50 for t in base[:3]] + base[3:]
    tokens = {"a": base, "b": other}
    want = {k: plain.forward(c, double(weights), v).numpy() for k, v in tokens.items()}
    assert row_error(want["a"][200:], want["b"][200:]).min() > 1e-3
    d = Driver(folder, "float32", pages=40, page_size=16, max_requests=2)
    got = d.run([[("a", 260)], [("b", 100)], [("b", 2)]] + [[("b", 1)]] * 17 + [[("b", 141)]], tokens)
    for k in tokens:
        assert row_error(got[k], want[k]).max() < BAR["float32"], k
    d.close()


def random_config(seed):
    """A configuration nobody chose: one to five layers of both kinds in any order, any feed-forward, sizes of every
    parity, a loop or none."""
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["dense", "moe", "moe", None])
        if kind == "dense":
            mlp = dense(rng.choice([24, 40, 100, 136]))
        elif kind == "moe":
            experts = rng.choice([1, 2, 6, 9, 33])
            shared = (rng.choice([8, 24, 50]), rng.uniform(0.5, 4.0)) if rng.random() < 0.6 else None
            mlp = moe(experts, rng.randint(1, min(experts, 4)), rng.choice([8, 20, 48, 70]), rng.uniform(0.5, 8.0), shared)
        else:
            mlp = None
        G = rng.choice([1, 2, 3])
        H = G * rng.choice([1, 2, 4])
        if rng.random() < 0.5:
            D = rng.choice([8, 12, 34, 64, 80])
            layers.append(attention(H, G, D, rng.choice([4, 8, 20, 64, 96]), rng.choice([d for d in (2, 4, 8, 12, 34, 64, 80) if d <= D]),
                                    rng.uniform(0.05, 0.5), rng.choice([None, 3.0, 30.0]), rng.choice([50.0, 1e4, 1e6]), mlp))
        else:
            layers.append(delta(H, G, rng.choice([4, 9, 16, 50, 96, 130]), rng.choice([3, 8, 20, 64, 100]), rng.randint(1, 5), mlp))
    loop = None
    if rng.random() < 0.6:
        a = rng.randrange(len(layers))
        loop = (a, rng.randint(a + 1, len(layers)), rng.randint(1, 3))
    return config(layers, width=rng.choice([40, 56, 100, 136, 192]), vocab=rng.randint(30, 400), logit_scale=rng.choice([1.0, 0.3, 4.0]),
                  loop=loop, eps=rng.choice([1e-6, 1e-5, 1e-3]))


@pytest.mark.parametrize("seed", list(range(10)))
def test_configurations_drawn_at_random(device, tmp_path, seed):
    """Whole prompts in one batch, then a prompt in portions with its last tokens one by one beside another request, in
    both precisions, for sizes nobody chose."""
    c = random_config(seed)
    weights = make_weights(c, seed=100 + seed)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(seed)
    tokens = {"a": torch.randint(0, c["vocab"], (83,), generator=g).tolist(), "b": torch.randint(0, c["vocab"], (21,), generator=g).tolist()}
    want = {k: reference(c, weights, v) for k, v in tokens.items()}
    for dtype in ("float32", "bfloat16"):
        d = Driver(folder, dtype, pages=40, page_size=4, max_requests=2)
        whole = d.run([[("a", 83), ("b", 21)]], tokens)
        cut = d.run([[("a", 30)], [("a", 17), ("b", 2)], [("a", 2), ("b", 1)], [("a", 24), ("b", 9)]] + [[("a", 1), ("b", 1)]] * 10, tokens)
        for got in (whole, cut):
            for k in tokens:
                check_rows(row_error(got[k], want[k][0]), dtype, (seed, c["width"], k), want[k][1])
        d.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompt_in_one_step(device, tmp_path, dtype):
    """1,700 tokens: 1,500 in one step (the delta rule over many chunks, prompt attention over many tiles, experts
    with hundreds of rows each), then a portion of 150 behind them and single tokens, beside a second, short request."""
    c = CONFIGS["odd"]
    weights = make_weights(c, seed=17)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(6)
    tokens = {"a": torch.randint(0, c["vocab"], (1700,), generator=g).tolist(), "b": torch.randint(0, c["vocab"], (40,), generator=g).tolist()}
    want = {k: reference(c, weights, v) for k, v in tokens.items()}
    d = Driver(folder, dtype, pages=120, page_size=16, max_requests=2)
    got = d.run([[("a", 1500), ("b", 3)], [("a", 150), ("b", 1)]] + [[("a", 1), ("b", 1)]] * 36 + [[("a", 14)]], tokens)
    for k in tokens:
        check_rows(row_error(got[k], want[k][0]), dtype, k, want[k][1])
    d.close()


def test_long_decoding_from_graphs(device, tmp_path):
    """400 tokens decoded one by one from graphs after a short prompt, two requests side by side."""
    c = CONFIGS["odd"]
    weights = make_weights(c, seed=11)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(3)
    tokens = {"a": torch.randint(0, c["vocab"], (420,), generator=g).tolist(),
              "b": torch.randint(0, c["vocab"], (409,), generator=g).tolist()}
    want = {k: plain.forward(c, double(weights), v).numpy() for k, v in tokens.items()}
    d = Driver(folder, "float32", pages=70, page_size=16)
    got = d.run([[("a", 20), ("b", 9)]] + [[("a", 1), ("b", 1)] for _ in range(400)], tokens)
    for k in tokens:
        err = row_error(got[k], want[k])
        assert err.max() < BAR["float32"], (k, int(err.argmax()), float(err.max()))
    assert d.stepper.graph_replays > 300
    d.close()


@pytest.mark.parametrize("name", ["odd", "wide"])
def test_greedy_generation_through_the_scheduler(device, tmp_path, name):
    """`engine_for(...).generate`: the package's entry point, scheduler, sampler and lookahead. Every generated
    token must be the plain implementation's best token for the text so far (checked where its lead is clear)."""
    from tessweave_engine_amd.cli import engine_for
    c = CONFIGS[name]
    weights = make_weights(c, seed=21)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(8)
    prompts = [torch.randint(0, c["vocab"], (n,), generator=g).tolist() for n in (5, 23, 1, 40, 12, 30)]
    engine = engine_for(folder, dtype="float32", max_context=128, kv_blocks=60, block_size=8, max_active=3,
                        prefill_chunk=16, no_prefix_cache=False)
    try:
        outputs = engine.generate(prompts, max_tokens=24, temperature=0.0)
    finally:
        engine.close()
    clear = 0
    for prompt, out in zip(prompts, outputs):
        assert len(out) == 24
        logits = plain.forward(c, double(weights), prompt + out)[len(prompt) - 1:-1]
        top = logits.topk(2, -1)
        for t, token in enumerate(out):
            if top.values[t, 0] - top.values[t, 1] > 1e-3:
                assert token == int(top.indices[t, 0]), (t, token)
                clear += 1
    assert clear > 100
