"""Every mechanism of the Famepel design alone: the kernel (its torch twin on the CPU, the HIP kernel on the GPU in
float32 and bfloat16) against the plain implementation's function for it, at sizes of all kinds."""

import math

import pytest
import torch

import plain_famepel as plain
from simple_inference_amd.parts import FEED_FORWARDS, MIXERS, POSITION_ENCODINGS, BuildEnv
from simple_inference_amd.parts.context import LayerCache
from test_feduzen_mechanisms import step_context
from test_mogisun_mechanisms import BACKENDS, close, context, lowered, rnd, setup


def f32(t, dev):
    return t.float().to(dev).contiguous()


def done(y):
    """A mixer's result, its last product computed if the kernels left it pending."""
    return y.compute() if hasattr(y, "compute") else y


def rounded(t):
    """The float64 values of a tensor that the engine keeps in float32."""
    return t.float().double()


def portions(lengths, cuts):
    """Steps over sequences of the given lengths: every step a list of (sequence, first token, tokens); the sequences
    advance by the sizes of ``cuts`` in turn, each from another place of the list, and some steps leave one out."""
    done, steps, i = [0] * len(lengths), [], 0
    while any(d < n for d, n in zip(done, lengths)):
        step = []
        for s, n in enumerate(lengths):
            if done[s] >= n or (i + s) % 4 == 3 and len(step) > 0:
                continue
            take = min(cuts[(i + 2 * s) % len(cuts)], n - done[s])
            step.append((s, done[s], take))
            done[s] += take
        step.sort(key=lambda e: e[2] != 1)      # single tokens first, as the step function lays them out
        steps.append(step)
        i += 1
    return steps


def rows_of(step, offsets):
    return torch.cat([torch.arange(offsets[s] + a, offsets[s] + a + n) for s, a, n in step])


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width", [96, 50, 176, 1024, 2056])
def test_dynamic_tanh_of_the_sum_and_of_what_is_added(backend, width):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(width)
    n = 7
    res = rnd(g, n, width, std=2.0)
    delta, delta64 = lowered(rnd(g, n, width, std=1.5), dtype, dev)
    T = {}
    for name in ("post", "pre"):
        T[name], T[name + ".b"] = 1 + rnd(g, width, std=0.3), rnd(g, width, std=0.4)
        T[name + ".alpha"] = torch.tensor([0.3 + float(torch.rand(1, generator=g))], dtype=torch.float64)
    ls = rnd(g, width, std=0.7)
    terms = lambda name, scale: (f32(T[name], dev), f32(T[name + ".b"], dev), f32(T[name + ".alpha"], dev), scale)
    T64 = {name: rounded(t) for name, t in T.items()}
    want_sum = rounded(res) + plain.dynamic_tanh(delta64, T64, "post") * rounded(ls)
    want = plain.dynamic_tanh(want_sum, T64, "pre")
    # all rows: the residual is left updated
    r = f32(res, dev)
    out = k.dyt_norm(r, delta, terms("post", f32(ls, dev)), terms("pre", None), dtype)
    close(r, want_sum, 3e-6)
    close(out, want, tol)
    # chosen rows: the residual stays
    r = f32(res, dev)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=dev)
    out = k.dyt_norm(r, delta, terms("post", f32(ls, dev)), terms("pre", None), dtype, rows)
    close(r, rounded(res), 0)
    close(out, want[[5, 0, 5]], tol)
    # the sum alone; a delta that is added as it is; no delta at all
    r = f32(res, dev)
    assert k.dyt_norm(r, delta, terms("post", f32(ls, dev)), None, dtype) is None
    close(r, want_sum, 3e-6)
    r = f32(res, dev)
    out = k.dyt_norm(r, delta, None, terms("pre", None), dtype)
    close(out, plain.dynamic_tanh(rounded(res) + delta64, T64, "pre"), tol)
    r = f32(res, dev)
    out = k.dyt_norm(r, None, None, terms("pre", f32(ls, dev)), dtype)
    close(out, plain.dynamic_tanh(rounded(res), T64, "pre") * rounded(ls), tol)
    close(r, rounded(res), 0)


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("channels,taps,first_col", [(40, 4, 16), (7, 2, 0), (130, 5, 3), (64, 1, 8), (256, 3, 0)])
def test_short_convolution_reads_its_last_inputs_from_the_state(backend, channels, taps, first_col):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(channels + taps)
    lengths, slots, offset = [23, 1, 41, 6], [5, 0, 3, 1], 11
    w, b = rnd(g, channels, taps, std=0.5), rnd(g, channels, std=0.3)
    width = first_col + channels + 5
    rows, rows64 = lowered(rnd(g, sum(lengths), width), dtype, dev)
    offsets = [sum(lengths[:s]) for s in range(len(lengths))]
    want = torch.cat([plain.silu(plain.causal_conv(rows64[o:o + n, first_col:first_col + channels], rounded(w), rounded(b)))
                      for o, n in zip(offsets, lengths)])
    state = torch.zeros(7, offset + channels * (taps - 1) + 3, device=dev)
    state[:, :offset] = 7.0                      # what lies in front of the kept inputs is not the convolution's
    got = torch.zeros(sum(lengths), channels, dtype=torch.float64)
    for step in portions(lengths, [2, 1, 9, 1, 3, 17]):
        ctx = context(dev, [n for _, _, n in step], [slots[s] for s, _, _ in step])
        idx = rows_of(step, offsets)
        out = k.causal_conv(rows[idx.to(dev)].contiguous(), first_col, f32(w, dev), f32(b, dev), "silu", ctx, state, offset)
        got[idx] = out.double().cpu()
    close(got, want, tol)
    assert float((state[:, :offset] - 7.0).abs().max()) == 0 and float(state[:, offset + channels * (taps - 1):].abs().max()) == 0
    for s, (o, n) in enumerate(zip(offsets, lengths) if taps > 1 else []):     # the row holds the last inputs, oldest first
        kept = state[slots[s], offset:offset + channels * (taps - 1)].view(taps - 1, channels).double().cpu()
        seq = torch.cat([torch.zeros(taps - 1, channels, dtype=torch.float64), rows64[o:o + n, first_col:first_col + channels]])
        close(kept, seq[seq.shape[0] - (taps - 1):], 1e-6)
    # without the activation
    ctx = context(dev, [lengths[0]], [6])
    out = k.causal_conv(rows[:lengths[0]].contiguous(), first_col, f32(w, dev), f32(b, dev), None, ctx, state, offset)
    close(out, plain.causal_conv(rows64[:lengths[0], first_col:first_col + channels], rounded(w), rounded(b)), tol)


# ---------------------------------------------------------------------------------------------------------------
def mamba_tensors(g, H, P, N, G, taps):
    inner, ch = H * P, H * P + 2 * G * N
    return {"conv": rnd(g, ch, taps, std=0.5), "conv.b": rnd(g, ch, std=0.2), "dt_bias": rnd(g, H, std=0.5),
            "A_log": rnd(g, H, std=0.7), "D": rnd(g, H), "norm": 1 + rnd(g, inner, std=0.2)}


def run_mamba(k, dev, dtype, rows, T, m, eps, lengths, slots, cuts, state=None):
    """The convolution and the recurrence over projected rows, step by step; returns all outputs and the state."""
    H, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner, ch = H * P, H * P + 2 * G * N
    if state is None:
        state = torch.zeros(8, H * N * P + ch * (taps - 1), device=dev)
    offsets = [sum(lengths[:s]) for s in range(len(lengths))]
    got = torch.zeros(sum(lengths), inner, dtype=torch.float64)
    w = {name: f32(t, dev) for name, t in T.items()}
    for step in portions(lengths, cuts):
        ctx = context(dev, [n for _, _, n in step], [slots[s] for s, _, _ in step])
        idx = rows_of(step, offsets)
        proj = rows[idx.to(dev)].contiguous()
        xbc = k.causal_conv(proj, inner, w["conv"], w["conv.b"], "silu", ctx, state, H * N * P)
        y = k.ssd_scan(proj, xbc, w["dt_bias"], w["A_log"], w["D"], w["norm"], H, P, N, G, m["norm_groups"], eps, ctx, state)
        got[idx] = y.double().cpu()
    return got, state


def plain_mamba(rows64, T, m, eps, dtype=torch.float32):
    """The plain mixer with the unit matrix before and behind: its input is the projected row.  The convolved rows are
    rounded where the engine hands them on in bfloat16 (the recurrence adds up hundreds of them, and what it sums of
    their rounding is no fault of its own)."""
    width, inner = rows64.shape[1], m["heads"] * m["vdim"]
    T64 = {"p." + name: rounded(t) for name, t in T.items()}
    T64["p.in"], T64["p.o"] = torch.eye(width, dtype=torch.float64), torch.eye(inner, dtype=torch.float64)
    if dtype == torch.float32:
        return plain.mamba2(rows64, T64, "p", m, eps)
    z, xbc, dt = plain.mamba2_inputs(rows64, T64, "p", m)
    return plain.state_space(z, xbc.to(dtype).double(), dt, T64, "p", m, eps)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,P,N,G,parts,taps", [(4, 16, 24, 2, 2, 4), (1, 48, 16, 1, 1, 2), (6, 32, 64, 3, 2, 4), (5, 12, 10, 1, 5, 3),
                                               (3, 24, 8, 3, 1, 1), (4, 64, 128, 1, 4, 4), (2, 128, 64, 2, 1, 5)])
def test_state_space_recurrence_carries_its_state_through_any_cut(backend, H, P, N, G, parts, taps):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(H * P + N)
    m = {"heads": H, "vdim": P, "state": N, "groups": G, "norm_groups": parts, "conv": taps}
    T = mamba_tensors(g, H, P, N, G, taps)
    lengths, slots = [37, 1, 70, 5], [2, 7, 0, 4]
    rows, rows64 = lowered(rnd(g, sum(lengths), 2 * H * P + 2 * G * N + H), dtype, dev)
    offsets = [sum(lengths[:s]) for s in range(len(lengths))]
    want = torch.cat([plain_mamba(rows64[o:o + n], T, m, 1e-5, dtype) for o, n in zip(offsets, lengths)])
    got, state = run_mamba(k, dev, dtype, rows, T, m, 1e-5, lengths, slots, [2, 1, 33, 1, 3, 64, 1, 1])
    close(got, want, tol)
    whole, state2 = run_mamba(k, dev, dtype, rows, T, m, 1e-5, lengths, slots, [100])
    close(whole, want, tol)
    close(state, state2, 2e-5 if dtype == torch.float32 else tol)      # however it was cut, the same state is left
    assert float(state[[1, 3, 5, 6]].abs().max()) == 0                 # and nobody else's row was touched


@pytest.mark.parametrize("backend", BACKENDS)
def test_state_space_recurrence_remembers_one_token_over_a_long_decode(backend):
    """The first token writes with a large step; every later token's step is next to nothing and the decay next to
    none, so all that the outputs 300 tokens later can show is what the first token left in the state."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(11)
    H, P, N, G = 3, 16, 24, 1
    m = {"heads": H, "vdim": P, "state": N, "groups": G, "norm_groups": 1, "conv": 1}
    T = mamba_tensors(g, H, P, N, G, 1)
    T["A_log"].fill_(-18.0)
    T["dt_bias"].zero_()
    T["D"].zero_()
    n = 330
    raw = rnd(g, n, 2 * H * P + 2 * N + H)
    raw[:, -H:] = -30.0
    raw[0, -H:] = 3.0
    rows, rows64 = lowered(raw, dtype, dev)
    want = plain_mamba(rows64, T, m, 1e-6, dtype)
    assert float(want[-1].abs().min()) > 1e-3
    other = rows64.clone()
    other[0, H * P:2 * H * P] += 1.0
    assert float((plain_mamba(other, T, m, 1e-6)[-1] - want[-1]).abs().max()) > 0.1    # the first token is what they show
    got, _ = run_mamba(k, dev, dtype, rows, T, m, 1e-6, [n], [3], [1])
    close(got[[1, 2, 100, 299, 329]], want[[1, 2, 100, 299, 329]], tol)


# ---------------------------------------------------------------------------------------------------------------
def run_hgrn(k, dev, rows, T, H, D, Dv, eps, lengths, slots, cuts):
    state = torch.zeros(8, H, D, Dv, device=dev)
    offsets = [sum(lengths[:s]) for s in range(len(lengths))]
    got = torch.zeros(sum(lengths), H * Dv, dtype=torch.float64)
    for step in portions(lengths, cuts):
        ctx = context(dev, [n for _, _, n in step], [slots[s] for s, _, _ in step])
        idx = rows_of(step, offsets)
        y = k.hgrn2_scan(rows[idx.to(dev)].contiguous(), f32(T["f.b"], dev), f32(T["lower"], dev), f32(T["norm"], dev),
                         H, D, Dv, eps, ctx, state)
        got[idx] = y.double().cpu()
    return got, state


def plain_hgrn(rows64, T, H, D, Dv, eps):
    """The plain mixer with matrices that pick the row's three parts, and the unit matrix behind."""
    eye = torch.eye(rows64.shape[1], dtype=torch.float64)
    T64 = {"p.q": eye[:H * D], "p.f": eye[H * D:2 * H * D], "p.v": eye[2 * H * D:], "p.o": torch.eye(H * Dv, dtype=torch.float64)}
    T64.update({"p." + name: rounded(t) for name, t in T.items()})
    return plain.hgrn2(rows64, T64, "p", {"heads": H, "dim": D, "vdim": Dv}, eps)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,D,Dv", [(3, 20, 12), (1, 32, 32), (4, 32, 64), (2, 8, 24), (3, 12, 20), (2, 128, 128), (5, 64, 16)])
def test_forget_gate_recurrence_carries_its_state_through_any_cut(backend, H, D, Dv):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(H * D + Dv)
    T = {"f.b": rnd(g, H * D, std=0.5), "lower": torch.rand(H * D, generator=g, dtype=torch.float64) * 0.9,
         "norm": 1 + rnd(g, Dv, std=0.2)}
    lengths, slots = [37, 1, 70, 5], [2, 7, 0, 4]
    rows, rows64 = lowered(rnd(g, sum(lengths), 2 * H * D + H * Dv), dtype, dev)
    offsets = [sum(lengths[:s]) for s in range(len(lengths))]
    want = torch.cat([plain_hgrn(rows64[o:o + n], T, H, D, Dv, 1e-5) for o, n in zip(offsets, lengths)])
    got, state = run_hgrn(k, dev, rows, T, H, D, Dv, 1e-5, lengths, slots, [2, 1, 33, 1, 3, 64, 1, 1])
    close(got, want, tol)
    whole, state2 = run_hgrn(k, dev, rows, T, H, D, Dv, 1e-5, lengths, slots, [100])
    close(whole, want, tol)
    close(state, state2, 2e-5 if dtype == torch.float32 else tol)
    assert float(state[[1, 3, 5, 6]].abs().max()) == 0


@pytest.mark.parametrize("backend", BACKENDS)
def test_forget_gate_recurrence_remembers_one_token_over_a_long_decode(backend):
    """The first token's gates are at their lower bound 0 (all of it is written), every later token's at 1 (nothing
    forgotten, nothing written): the outputs 300 tokens later are the first token's values seen through the query."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(12)
    H, D, Dv, n = 2, 16, 24, 330
    T = {"f.b": torch.zeros(H * D, dtype=torch.float64), "lower": torch.zeros(H * D, dtype=torch.float64),
         "norm": 1 + rnd(g, Dv, std=0.2)}
    raw = rnd(g, n, 2 * H * D + H * Dv)
    raw[:, H * D:2 * H * D] = 60.0
    raw[0, H * D:2 * H * D] = -60.0
    rows, rows64 = lowered(raw, dtype, dev)
    want = plain_hgrn(rows64, T, H, D, Dv, 1e-6)
    v0 = rows64[0, 2 * H * D:].view(H, Dv)
    unit = v0 / torch.sqrt((v0 * v0).mean(-1, keepdim=True) + 1e-6) * rounded(T["norm"])
    q = plain.silu(rows64[-1, :H * D]).view(H, D).sum(-1, keepdim=True)
    close(want[-1].view(H, Dv), unit * torch.sign(q), 1e-3)           # the state is v0 in every row
    got, state = run_hgrn(k, dev, rows, T, H, D, Dv, 1e-6, [n], [3], [1])
    close(got[[0, 1, 100, 299, 329]], want[[0, 1, 100, 299, 329]], tol)
    close(state[3, :, 5], v0, tol)


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,groups,width", [(6, 2, (3, 1), 96), (8, 2, (4, 2), 128), (12, 4, (3, 2), 50), (5, 2, None, 64),
                                                      (4, 2, (4, 2), 64), (9, 3, (3, 3), 100), (16, 1, (2, 1), 256), (7, 7, None, 48),
                                                      (64, 6, (8, 3), 128), (10, 5, (2, 1), 72)])
def test_the_router_keeps_the_best_groups_and_weighs_by_the_scores(backend, experts, top, groups, width):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(experts * top + width)
    n = 33
    h, h64 = lowered(rnd(g, n, width), dtype, dev)
    router = rnd(g, experts, width, std=0.3)
    r = {"experts": experts, "top": top, "scale": 1.7}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    want_ids, want_w = plain.route(h64, {"p.router": rounded(router)}, "p", r)
    ids, weights = k.moe_route(h, f32(router, dev), top, score="sigmoid", groups=groups, scale=1.7)
    ids, weights = ids.cpu().long(), weights.double().cpu()
    for t in range(n):
        assert sorted(ids[t].tolist()) == sorted(want_ids[t].tolist()), t
        order = {e: i for i, e in enumerate(want_ids[t].tolist())}
        place = [order[e] for e in ids[t].tolist()]
        close(weights[t], want_w[t][place], 1e-5)
    close(weights.sum(-1), torch.full((n,), 1.7, dtype=torch.float64), 1e-5)


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_group_is_judged_by_its_two_best_scores_not_by_its_best(backend):
    k, dev, dtype, tol = setup(backend)
    # six experts in two groups; the router is the unit matrix, so a row of the input is the row of logits
    logits = torch.tensor([[3.0, -5.0, -5.0, 1.0, 1.0, 0.5],        # the best expert's group loses: .95 + .01 < .73 + .73
                           [3.0, 0.5, -5.0, 1.0, 1.0, 0.5],         # .95 + .62 > 1.46: now it wins
                           [0.0, 0.0, 0.0, 0.0, 0.0, 0.0],          # all alike: the lower group, the lower experts
                           [-2.0, -2.0, 4.0, 4.0, -9.0, -9.0]],     # .12 + .98 > .98 + 0
                          dtype=torch.float64)
    h, _ = lowered(logits, dtype, dev)
    eye = torch.eye(6, device=dev)
    ids, weights = k.moe_route(h, eye, 2, score="sigmoid", groups=(2, 1), scale=2.0)
    assert ids.cpu().tolist() == [[3, 4], [0, 1], [0, 1], [2, 0]]
    s = torch.sigmoid(logits)
    close(weights[0], torch.tensor([1.0, 1.0]), 1e-6)
    close(weights[1], 2 * s[1, :2] / s[1, :2].sum(), 1e-5)
    close(weights[3], 2 * s[3, [2, 0]] / s[3, [2, 0]].sum(), 1e-5)
    # both groups kept: the best experts wherever they are; three groups of two, of which two are kept
    ids, _ = k.moe_route(h, eye, 2, score="sigmoid", groups=(2, 2), scale=1.0)
    assert ids.cpu().tolist() == [[0, 3], [0, 3], [0, 1], [2, 3]]
    ids, _ = k.moe_route(h, eye, 3, score="sigmoid", groups=(3, 2), scale=1.0)
    assert ids.cpu().tolist() == [[0, 4, 5], [0, 4, 1], [0, 1, 2], [2, 3, 0]]
    # a group of one expert counts its one score
    ids, _ = k.moe_route(h, eye, 2, score="sigmoid", groups=(6, 2), scale=1.0)
    assert ids.cpu().tolist() == [[0, 3], [0, 3], [0, 1], [2, 3]]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,groups,width,ff,n", [(6, 2, (3, 1), 96, 40, 9), (5, 3, None, 50, 24, 4), (8, 2, (4, 2), 128, 64, 130)])
def test_experts_chosen_by_sigmoid_scores_weighted_and_summed(backend, experts, top, groups, width, ff, n):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(experts + width)
    env = BuildEnv(k, torch.device(dev), dtype, 64)
    params = {"hidden_size": width, "experts": experts, "top": top, "expert_size": ff, "score": "sigmoid",
              "groups": groups, "route_scale": 2.5}
    part = FEED_FORWARDS.get("moe")(params, env)
    T64, bound = {}, {}
    bound["router"], T64["p.router"] = lowered(rnd(g, experts, width, std=0.3), torch.float32, dev)
    for e in range(experts):
        for name, shape in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff))):
            bound[f"{name}{e}"], T64[f"p.e{e}.{name}"] = lowered(rnd(g, *shape, std=0.15), dtype, dev)
    part.bind(bound)
    h, h64 = lowered(rnd(g, n, width), dtype, dev)
    mlp = {"router": {"experts": experts, "top": top, "scale": 2.5}}
    if groups:
        mlp["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    out = part.forward(h, context(dev, [n], [0]))
    close(out, plain.experts(h64, T64, "p", mlp), tol)


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dims,base,scaling", [
    (32, 10000.0, (4.0, 64, 16.0, 2.0)), (8, 10000.0, (4.0, 64, 16.0, 2.0)), (64, 500000.0, (32.0, 4096, 32.0, 1.0)),
    (16, 100.0, (2.0, 8, 4.0, 1.0)),             # the ramp begins before pair 0 and ends behind the last one
    (6, 777.0, (16.0, 100000, 2.0, 1.5)),        # every pair turns too fast to be stretched
    (12, 50.0, (3.0, 4, 1000.0, 900.0)),         # every pair is stretched
    (24, 10000.0, (8.0, 512, 9.0, 8.9)),         # the ramp's ends fall on one pair: a step
    (20, 1000.0, None)])
def test_frequencies_stretched_along_a_ramp_and_tables_raised(dims, base, scaling):
    rot = {"dims": dims, "base": base}
    sc = None
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
        sc = dict(rot["scaling"], rope_type="yarn")
    env = BuildEnv(None, torch.device("cpu"), torch.float32, 700)
    part = POSITION_ENCODINGS.get("rope")({"rotary_dim": dims, "theta": base, "scaling": sc, "pairing": "interleaved",
                                            "angles": "float64"}, env)
    cos, sin = part.tables()
    want_cos, want_sin = plain.rotary_tables(700, rot)
    assert cos.dtype == torch.float32 and tuple(cos.shape) == (700, dims // 2)
    close(cos, want_cos, 1e-6)
    close(sin, want_sin, 1e-6)
    if scaling:
        close(cos[0], torch.full((dims // 2,), 0.1 * math.log(scaling[0]) + 1, dtype=torch.float64), 1e-7)


# ---------------------------------------------------------------------------------------------------------------
def latent_part(k, dev, dtype, g, m, width, eps, max_positions=1024, kv_from=None):
    """A latent-attention mixer of the package with random weights, and the same numbers under the plain names."""
    env = BuildEnv(k, torch.device(dev), dtype, max_positions)
    sc = dict(m["rot"]["scaling"], rope_type="yarn") if m["rot"].get("scaling") else None
    params = {"hidden_size": width, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
              "value_head_dim": m["vdim"], "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": m["scale"],
              "norm_eps": eps, "sink": True, "kv_from_layer": kv_from,
              "position": {"kind": "rope", "params": {"rotary_dim": m["rot"]["dims"], "theta": m["rot"]["base"],
                                                      "scaling": sc, "pairing": "interleaved", "angles": "float64"}}}
    part = MIXERS.get("latent_attention")(params, env)
    H, qk = m["heads"], m["dim"] + m["rot_dim"]
    shapes = {"dq": (m["q_rank"], width), "uq": (H * qk, m["q_rank"]), "uk": (H * m["dim"], m["kv_rank"]),
              "uv": (H * m["vdim"], m["kv_rank"]), "o": (width, H * m["vdim"])}
    if kv_from is None:
        shapes["dkv"] = (m["kv_rank"] + m["rot_dim"], width)
    bound, T64 = {}, {}
    for name, shape in shapes.items():
        bound[name], T64["p." + name] = lowered(rnd(g, *shape, std=shape[1] ** -0.5), dtype, dev)
    vectors = {"dq_norm": ("dq.norm", 1 + rnd(g, m["q_rank"], std=0.2)), "sink": ("sink", rnd(g, H, std=1.5))}
    if kv_from is None:
        vectors["dkv_norm"] = ("dkv.norm", 1 + rnd(g, m["kv_rank"], std=0.2))
    for name, (plain_name, t) in vectors.items():
        bound[name], T64["p." + plain_name] = f32(t, dev), rounded(t)
    return part, bound, T64


def pages_for(part, dev, dtype, n_pages, page, table):
    need = part.cache_need()
    vdim = need.value_dim if getattr(need, "value_dim", None) else need.head_dim
    return LayerCache(k_pages=torch.zeros(n_pages, 1, page, need.head_dim, dtype=dtype, device=dev),
                      v_pages=torch.zeros(n_pages, 1, vdim, page, dtype=dtype, device=dev), block_table=table, page_size=page)


def prefix_context(dev, runs, table, k):
    """The step that brings the tokens in front of ``runs``' portions (for the sequences that have any)."""
    import types
    rows = [s for s, (first, _) in enumerate(runs) if first > 0]
    firsts = [runs[s][0] for s in rows]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    cu = [0]
    for n in firsts:
        cu.append(cu[-1] + n)
    ctx = types.SimpleNamespace(
        n_tokens=cu[-1], n_seqs=len(rows), positions=i32([p for n in firsts for p in range(n)]),
        seq_of_token=i32([s for s, n in enumerate(firsts) for _ in range(n)]), cu_q=i32(cu), kv_len=i32(firsts),
        max_kv_len=max(firsts), max_q_len=max(firsts), n_decode_seqs=0, q_lens=firsts, kv_bound=0, max_run_kv_len=max(firsts),
        kernels=k, extra={})
    return ctx, table[rows].contiguous(), rows


LATENTS = [
    dict(heads=3, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=40, scale=0.2, rot={"base": 10000.0, "dims": 8, "scaling": dict(
        factor=4.0, original=64, fast=16.0, slow=2.0)}),
    dict(heads=1, dim=24, rot_dim=16, vdim=40, q_rank=16, kv_rank=24, scale=0.3, rot={"base": 1000.0, "dims": 8}),
    dict(heads=4, dim=64, rot_dim=32, vdim=64, q_rank=48, kv_rank=96, scale=0.11, rot={"base": 50000.0, "dims": 32, "scaling": dict(
        factor=16.0, original=128, fast=32.0, slow=1.0)}),
    dict(heads=5, dim=12, rot_dim=6, vdim=20, q_rank=14, kv_rank=22, scale=0.4, rot={"base": 777.0, "dims": 4}),
    dict(heads=2, dim=128, rot_dim=64, vdim=128, q_rank=96, kv_rank=192, scale=0.07, rot={"base": 10000.0, "dims": 64}),
    # more heads on the one cached row than a decode workgroup takes: dealt out as two groups of 12, as 17 of one
    dict(heads=24, dim=16, rot_dim=16, vdim=16, q_rank=32, kv_rank=48, scale=0.15, rot={"base": 10000.0, "dims": 16}),
    dict(heads=17, dim=8, rot_dim=8, vdim=24, q_rank=24, kv_rank=24, scale=0.2, rot={"base": 500.0, "dims": 8}),
    # a cached row wider than any head the matrix-core attention is built for
    dict(heads=2, dim=32, rot_dim=32, vdim=40, q_rank=24, kv_rank=288, scale=0.1, rot={"base": 10000.0, "dims": 32}),
]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("m,page", list(zip(LATENTS, [8, 16, 16, 4, 16, 16, 8, 16])))
def test_latent_attention_in_prompts_portions_and_decoding_and_from_another_layers_pages(backend, m, page):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(m["kv_rank"])
    width, eps = 72, 1e-5
    part, bound, T64 = latent_part(k, dev, dtype, g, m, width, eps)
    part.bind(bound)
    reader, bound2, T64b = latent_part(k, dev, dtype, g, m, width, eps, kv_from=0)
    reader.bind(bound2)
    # a whole prompt, a portion that begins in the middle of a page, single tokens at a page's first and last place, the
    # very first token of a sequence
    runs = [(0, 150), (page + 3, 61), (3 * page, 1), (5 * page - 1, 1), (0, 1), (77, 2)]
    ctx, table, n_pages, runs = step_context(dev, runs, page, k)
    cache = pages_for(part, dev, dtype, n_pages, page, table)
    inputs = [lowered(rnd(g, first + n, width), dtype, dev) for first, n in runs]
    inputs2 = [lowered(rnd(g, first + n, width), dtype, dev) for first, n in runs]
    before, before_table, rows = prefix_context(dev, runs, table, k)
    cache.block_table = before_table
    done(part.forward(torch.cat([inputs[s][0][:runs[s][0]] for s in rows]), before, cache))
    cache.block_table = table
    got = done(part.forward(torch.cat([x[first:] for (x, _), (first, n) in zip(inputs, runs)]), ctx, cache))
    got2 = done(reader.forward(torch.cat([x[first:] for (x, _), (first, n) in zip(inputs2, runs)]), ctx, cache))
    want, want2 = [], []
    for (_, x64), (_, y64), (first, n) in zip(inputs, inputs2, runs):
        kv = plain.latent_kv(x64, T64, "p", m, eps)
        if dtype == torch.bfloat16:        # what the pages hold is rounded
            kv = tuple(t.to(dtype).double() for t in kv)
        want.append(plain.latent_attention(x64, T64, "p", m, eps, kv)[first:])
        want2.append(plain.latent_attention(y64, T64b, "p", m, eps, kv)[first:])
    close(got, torch.cat(want), tol)
    close(got2, torch.cat(want2), tol)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("decoding", [False, True])
def test_one_far_latent_is_found_among_hundreds_and_one_ahead_is_not(backend, decoding):
    """One position's latent is made to stand out for the last query: its input row is a large multiple of one unit
    vector that the latent's first channel reads, the first unrotated key channel of every head reads that channel,
    and the last token's query is large there.  The result is then that position's value, wherever it lies: at
    position 0, at a page's first and last place, hundreds of positions back; the plain implementation says the
    same.  Planted one position ahead of the query, inside the same portion, it is not seen."""
    k, dev, dtype, tol = setup(backend)
    m = dict(heads=2, dim=16, rot_dim=8, vdim=16, q_rank=12, kv_rank=32, scale=0.5, rot={"base": 10000.0, "dims": 8})
    width, eps, page, L = 40, 1e-6, 16, 500
    for place in (0, 16, 31, 250, 463, 498, 499):
        g = torch.Generator().manual_seed(3)
        part, bound, T64 = latent_part(k, dev, dtype, g, m, width, eps)
        for t in (bound, T64):
            for name in ("dkv", "p.dkv", "uk", "p.uk", "dq", "p.dq", "uq", "p.uq"):
                if name in t:
                    t[name].mul_(0.1)
        for t, pre in ((bound, ""), (T64, "p.")):
            t[pre + "dkv"][0].zero_()
            t[pre + "dkv"][0, 0] = 1.0                                   # latent channel 0 reads input element 0
            t[pre + "uk"].view(2, 16, 32)[:, 0].zero_()
            t[pre + "uk"].view(2, 16, 32)[:, 0, 0] = 1.0                 # key channel 0 of both heads reads latent channel 0
            t[pre + "dq"][0].zero_()
            t[pre + "dq"][0, 1] = 1.0                                    # the query's latent channel 0 reads input element 1
            t[pre + "uq"].view(2, 24, 12)[:, 0].zero_()
            t[pre + "uq"].view(2, 24, 12)[:, 0, 0] = 4.0
            t[pre + "sink"].fill_(-3.0)
            for name in ("dkv_norm", "dq_norm") if pre == "" else ("dkv.norm", "dq.norm"):
                t[pre + name].fill_(1.0)
        part.bind(bound)
        raw = rnd(g, L, width, std=0.3)
        raw[:, :2] = 0.0
        raw[place] = 0.0
        raw[place, 0] = 50.0                                             # its latent is sqrt(32) times the unit vector
        query = L - 2                                                    # the last token but one asks; place 499 lies ahead
        raw[query, 1] = 50.0
        x, x64 = lowered(raw, dtype, dev)
        first = L - 1 if decoding else L - 45
        ask = L - 1 if decoding else query
        if decoding:
            raw[L - 1, 1], raw[query, 1] = 50.0, 0.0
            x, x64 = lowered(raw, dtype, dev)
        ctx, table, n_pages, runs = step_context(dev, [(first, L - first)], page, k)
        cache = pages_for(part, dev, dtype, n_pages, page, table)
        before, before_table, _ = prefix_context(dev, runs, table, k)
        done(part.forward(x[:first].contiguous(), before, cache))
        got = done(part.forward(x[first:].contiguous(), ctx, cache)).double().cpu()[ask - first]
        kv = plain.latent_kv(x64, T64, "p", m, eps)
        if dtype == torch.bfloat16:
            kv = tuple(t.to(dtype).double() for t in kv)
        want = plain.latent_attention(x64, T64, "p", m, eps, kv)[ask]
        close(got, want, tol)
        # what the result would be if the planted position were all that is seen
        v = (kv[0][place] @ T64["p.uv"].T) @ T64["p.o"].T
        seen = place <= ask
        assert (float((got - v).abs().max()) < 0.05 * float(v.abs().max())) == seen, (place, decoding)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,in_dim,out_dim,tail,rotary,spare", [(3, 16, 40, 8, 8, 0), (24, 128, 192, 64, 64, 0), (5, 12, 22, 6, 4, 4),
                                                                    (2, 192, 128, 0, 0, 64), (1, 24, 24, 16, 8, 8), (4, 40, 100, 0, 0, 0)])
@pytest.mark.parametrize("n", [1, 7, 16, 45, 300])
def test_a_product_per_head_with_the_turned_tail_behind_it(backend, heads, in_dim, out_dim, tail, rotary, spare, n):
    """Few rows, many rows, sizes the wide loads take and sizes they do not: the same numbers."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(heads * in_dim + n)
    in_stride, out_stride = in_dim + tail + spare, out_dim + tail + 3
    x, x64 = lowered(rnd(g, n, heads * in_stride), dtype, dev)
    w, w64 = lowered(rnd(g, heads, out_dim, in_dim, std=in_dim ** -0.5), dtype, dev)
    positions = torch.randint(0, 500, (n,), generator=g)
    cos64, sin64 = plain.rotary_tables(500, {"dims": max(rotary, 2), "base": 1000.0})
    rotation = (rotary, f32(cos64, dev), f32(sin64, dev), positions.to(torch.int32).to(dev)) if rotary else None
    got = k.headwise_linear(x, w, in_stride, out_stride, tail=tail, rotation=rotation).double().cpu().view(n, heads, out_stride)
    xs = x64.view(n, heads, in_stride)
    close(got[:, :, :out_dim], torch.einsum("nhi,hoi->nho", xs[:, :, :in_dim], w64), tol)
    if tail:
        behind = xs[:, :, in_dim:in_dim + tail]
        if rotary:
            behind = plain.rotate_pairs(behind, rounded(cos64)[positions], rounded(sin64)[positions])
        close(got[:, :, out_dim:out_dim + tail], behind, tol)
    assert float(got[:, :, out_dim + tail:].abs().max()) == 0
