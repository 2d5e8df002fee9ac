"""Every mechanism of the Tadinex design alone: the kernel (its torch twin on the CPU, the HIP kernel on the GPU in
float32 and bfloat16) against the plain implementation's function for it, at sizes of all kinds."""

import math

import pytest
import torch

import plain_tadinex as plain
from simple_inference_amd.parts import MIXERS, BuildEnv
from simple_inference_amd.parts.context import LayerCache
from test_famepel_mechanisms import done, f32, portions, rounded, rows_of
from test_feduzen_mechanisms import empty_cache, step_context
from test_mogisun_mechanisms import BACKENDS, close, context, lowered, rnd, setup


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width", [96, 50, 176, 1024, 2056, 8200])
def test_scaled_terms_go_into_the_residual_inside_the_norm(backend, width):
    """``x += f1 d1 + f2 d2`` and the norm of the sum with a gain stored as its distance from one: all rows (the
    residual keeps the sum), chosen rows (it does not), one term, and the sum alone."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(width)
    n, eps = 7, 1e-5
    res = rnd(g, n, width, std=2.0)
    d1, d1_64 = lowered(rnd(g, n, width, std=1.5), dtype, dev)
    d2, d2_64 = lowered(rnd(g, n, width, std=1.5), dtype, dev)
    T = {"w": rnd(g, width, std=0.3).float().double()}
    gain = (T["w"].float() + 1.0).to(dev)
    want_sum = rounded(res) + 0.42 * d1_64 - 1.3 * d2_64
    want = plain.offset_norm(want_sum, T, "w", eps)
    r = f32(res, dev)
    out = k.add_rmsnorm(r, None, gain, eps, dtype, terms=[(d1, 0.42), (d2, -1.3)])
    close(r, want_sum, 3e-6)
    close(out, want, tol)
    r = f32(res, dev)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=dev)
    out = k.add_rmsnorm(r, None, gain, eps, dtype, rows, terms=[(d1, 0.42), (d2, -1.3)])
    close(r, rounded(res), 0)
    close(out, want[[5, 0, 5]], tol)
    r = f32(res, dev)
    out = k.add_rmsnorm(r, None, gain, eps, dtype, terms=[(d2, 0.7)])
    close(out, plain.offset_norm(rounded(res) + 0.7 * d2_64, T, "w", eps), tol)
    r = f32(res, dev)
    assert k.add_rmsnorm(r, None, None, 0.0, dtype, terms=[(d1, 0.42), (d2, -1.3)]) is None
    close(r, want_sum, 3e-6)
    close(k.scaled_sum([(d1, 0.42), (d2, -1.3)]), 0.42 * d1_64 - 1.3 * d2_64, tol)


@pytest.mark.parametrize("backend", BACKENDS)
def test_exact_gelu_and_the_clamped_gate(backend):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(3)
    for n, width, inter in ((5, 64, 40), (33, 128, 72), (19, 64, 27)):
        x, x64 = lowered(rnd(g, n, width), dtype, dev)
        w, w64 = lowered(rnd(g, 2 * inter, width, std=0.4), dtype, dev)
        close(k.activated_linear(x, w, "gelu"), plain.gelu_erf(x64 @ w64.T), tol)
        for limit in (0.6, 2.5):
            z = x64 @ w64.T
            gate, up = z[:, :inter].clamp(max=limit), z[:, inter:].clamp(-limit, limit)
            want = gate * torch.sigmoid(1.702 * gate) * (up + 1.0)
            assert float((z[:, :inter] > limit).sum()) > 0 and float((z[:, inter:] < -limit).sum()) > 0
            close(k.gated_linear(x, w, activation=("clamped", limit)), want, tol)


# ---------------------------------------------------------------------------------------------------------------
DELTA_SHAPES = [(4, 2, 12, 20), (1, 1, 8, 8), (2, 2, 64, 64), (4, 1, 128, 128), (6, 3, 56, 24), (1, 1, 40, 200),
                (2, 1, 264, 96)]


def delta_reference(qkv64, proj64, cols, T, H, G, D, Dv, eps):
    """The plain functions on convolved rows: unit vectors, write strengths, decays, the recurrence, norm and gate."""
    n = qkv64.shape[0]
    q = plain.unit(qkv64[:, :G * D].reshape(n, G, D)) * D ** -0.5
    kk = plain.unit(qkv64[:, G * D:2 * G * D].reshape(n, G, D))
    v = qkv64[:, 2 * G * D:].reshape(n, H, Dv)
    beta = torch.sigmoid(proj64[:, cols[1]:cols[1] + H])
    step = torch.nn.functional.softplus(proj64[:, cols[2]:cols[2] + H] + T["dt_bias"], threshold=1e9)
    decay = torch.exp(-torch.exp(T["A_log"]) * step)
    o = plain.rms(plain.delta_rule(q, kk, v, beta, decay), eps) * T["norm"]
    return o.reshape(n, H * Dv) * plain.silu(proj64[:, cols[0]:cols[0] + H * Dv])


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,Dv", DELTA_SHAPES)
def test_the_delta_rule_carries_its_state_through_any_cut(backend, H, G, D, Dv):
    """Three sequences of unequal length in scattered slots, fed in portions of unequal sizes down to one token, the
    batch's order changing: every output is the plain recurrence's over the whole sequence, and nobody else's slot is
    touched.  The matrices lie at the front of a longer state row."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(H * 1000 + D)
    lengths, slots = [38, 6, 22], [4, 0, 2]
    cols = (3, 3 + H * Dv + 2, 3 + H * Dv + 2 + H)
    qkvs = [lowered(rnd(g, n, 2 * G * D + H * Dv), dtype, dev) for n in lengths]
    projs = [lowered(rnd(g, n, cols[2] + H + 1, std=1.5), dtype, dev) for n in lengths]
    T = {"A_log": rounded(rnd(g, H, std=0.7)), "dt_bias": rounded(rnd(g, H, std=0.7)), "norm": rounded(1 + rnd(g, Dv, std=0.3))}
    tail = 5
    state = torch.zeros(6, H * D * Dv + tail, dtype=torch.float32, device=dev)
    state[:, H * D * Dv:] = 3.0
    eps = 1e-5
    offsets = [sum(lengths[:s]) for s in range(len(lengths))]
    got = torch.zeros(sum(lengths), H * Dv, dtype=torch.float64)
    for step in portions(lengths, [2, 1, 9, 1, 3, 17]):
        ctx = context(dev, [n for _, _, n in step], [slots[s] for s, _, _ in step])
        pick = lambda rows: torch.cat([rows[s][0][a:a + n] for s, a, n in step]).contiguous()
        out = k.delta_rule(pick(qkvs), pick(projs), cols, f32(T["A_log"], dev), f32(T["dt_bias"], dev), f32(T["norm"], dev),
                           H, G, D, Dv, eps, ctx, state)
        got[rows_of(step, offsets)] = out.double().cpu()
    want = torch.cat([delta_reference(qkvs[s][1], projs[s][1], cols, T, H, G, D, Dv, eps) for s in range(len(lengths))])
    close(got, want, tol * 2)
    assert float(state[[1, 3, 5], :H * D * Dv].abs().max()) == 0.0
    assert float((state[:, H * D * Dv:] - 3.0).abs().max()) == 0.0      # what lies behind the matrices is not theirs


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_delta_rule_replaces_what_a_key_holds(backend):
    """Built inputs: one key direction is written with value a, then, 300 tokens of other directions later, written
    again with value b at full strength: a query along it then reads b and nothing of a (a plain sum of writes would
    read a + b); without the second write it still reads a, faded by the decays on the way."""
    k, dev, dtype, tol = setup(backend)
    H = G = 1
    D, Dv, n = 16, 8, 330
    g = torch.Generator().manual_seed(1)
    cols = (0, Dv, Dv + 1)
    qkv = torch.zeros(n, 2 * D + Dv, dtype=torch.float64)
    proj = torch.zeros(n, Dv + 2, dtype=torch.float64)
    proj[:, :Dv] = 2.0                            # an open output gate
    proj[:, Dv] = 30.0                            # write at full strength
    proj[:, Dv + 1] = -4.0                        # small steps: slow decay
    e = torch.eye(D, dtype=torch.float64)
    for t in range(n):
        qkv[t, D:2 * D] = e[1 + t % (D - 1)]      # keys along the other axes
        qkv[t, :D] = e[0]                         # everybody asks along the first
        qkv[t, 2 * D:] = rnd(g, Dv)
    a, b = torch.arange(Dv, dtype=torch.float64) - 3.5, torch.linspace(2, -1, Dv, dtype=torch.float64)
    qkv[5, D:2 * D], qkv[5, 2 * D:] = e[0], a
    again = qkv.clone()
    again[310, D:2 * D], again[310, 2 * D:] = e[0], b
    T = {"A_log": torch.zeros(1, dtype=torch.float64), "dt_bias": torch.zeros(1, dtype=torch.float64),
         "norm": torch.ones(Dv, dtype=torch.float64)}
    outs = {}
    for name, rows in (("once", qkv), ("again", again)):
        state = torch.zeros(2, D * Dv, dtype=torch.float32, device=dev)
        x, x64 = lowered(rows, dtype, dev)
        p, p64 = lowered(proj, dtype, dev)
        got = []
        for lo, hi in [(0, 7), (7, 9)] + [(t, t + 1) for t in range(9, n)]:      # a portion, two tokens, then decoding
            ctx = context(dev, [hi - lo], [1])
            got.append(k.delta_rule(x[lo:hi].contiguous(), p[lo:hi].contiguous(), cols, f32(T["A_log"], dev),
                                    f32(T["dt_bias"], dev), f32(T["norm"], dev), H, G, D, Dv, 1e-6, ctx, state))
        outs[name] = torch.cat(got).double().cpu()
        close(outs[name], delta_reference(x64, p64, cols, T, H, G, D, Dv, 1e-6), tol * 2)
    cos = lambda u, v: float((u * v).sum() / u.norm() / v.norm())
    assert cos(outs["once"][n - 1], a) > 0.99 and cos(outs["again"][n - 1], b) > 0.99
    assert cos(outs["again"][309], a) > 0.99      # until the second write the first is what is read


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,D,Dv", [(3, 24, 40), (1, 8, 8), (2, 64, 64), (2, 128, 128), (5, 56, 24), (1, 40, 200)])
def test_decaying_attention_carries_its_state_through_any_cut(backend, H, D, Dv):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(H * 1000 + D)
    lengths, slots = [38, 6, 22], [4, 0, 2]
    width = 2 * H * D + 2 * H * Dv
    projs = [lowered(rnd(g, n, width), dtype, dev) for n in lengths]
    decays = [0.5 + 0.499 * i / max(H - 1, 1) for i in range(H)]
    norm = rounded(1 + rnd(g, H * Dv, std=0.3))
    state = torch.zeros(6, H, D, Dv, dtype=torch.float32, device=dev)
    eps = 1e-5
    offsets = [sum(lengths[:s]) for s in range(len(lengths))]
    got = torch.zeros(sum(lengths), H * Dv, dtype=torch.float64)
    for step in portions(lengths, [2, 1, 9, 1, 3, 17]):
        ctx = context(dev, [n for _, _, n in step], [slots[s] for s, _, _ in step])
        rows = torch.cat([projs[s][0][a:a + n] for s, a, n in step]).contiguous()
        out = k.decay_attention(rows, torch.tensor(decays, dtype=torch.float32, device=dev), f32(norm, dev), H, D, Dv,
                                eps, ctx, state)
        got[rows_of(step, offsets)] = out.double().cpu()
    for s, n in enumerate(lengths):
        p = projs[s][1]
        act = plain.silu(p[:, :2 * H * D + H * Dv]).to(dtype).double()      # the activations are rounded once
        q, kk = act[:, :H * D].reshape(n, H, D), act[:, H * D:2 * H * D].reshape(n, H, D)
        v = act[:, 2 * H * D:].reshape(n, H, Dv)
        o = torch.zeros(n, H, Dv, dtype=torch.float64)
        for h in range(H):
            S = torch.zeros(D, Dv, dtype=torch.float64)
            for t in range(n):
                S = decays[h] * S + torch.outer(kk[t, h], v[t, h])
                o[t, h] = S.T @ q[t, h]
        want = plain.rms(o.reshape(n, H * Dv), eps) * norm * torch.sigmoid(p[:, 2 * H * D + H * Dv:])
        close(got[offsets[s]:offsets[s] + n], want, tol * 2)
    assert float(state[[1, 3, 5]].abs().max()) == 0.0


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_mixer_of_the_plain_implementation_is_the_decaying_attention_part(backend):
    """The part as the plan builds it (stacked projections, its own tensor names) against the plain function."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(11)
    hidden, H, D, Dv, n = 64, 2, 16, 24, 29
    mx = {"heads": H, "dim": D, "vdim": Dv, "decay": [0.8, 0.97]}
    env = BuildEnv(kernels=k, device=torch.device(dev), dtype=dtype, max_positions=64)
    part = MIXERS.get("decay_attention")({"hidden_size": hidden, "num_heads": H, "key_dim": D, "value_dim": Dv,
                                          "decay": mx["decay"], "norm_eps": 1e-5}, env)
    T, bound = {}, {}
    for name, spec in part.weight_specs().items():
        t = rnd(g, *spec.shape, std=0.3) + (1.0 if spec.role == "vector" else 0.0)
        bound[name], T["m." + name] = lowered(t, torch.float32 if spec.role == "vector" else dtype, dev)
    part.bind(bound)
    h, h64 = lowered(rnd(g, n, hidden), dtype, dev)
    state = torch.zeros(2, H, D, Dv, dtype=torch.float32, device=dev)
    outs = []
    for lo, hi in ((0, 17), (17, 19), (19, 20), (20, n)):
        outs.append(done(part.forward(h[lo:hi].contiguous(), context(dev, [hi - lo], [1]), LayerCache(state=state))))
    close(torch.cat(outs), plain.decaying_attention(h64, T, "m", mx, 1e-5), tol * 3)


# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,width", [(5, 1, 96), (8, 3, 128), (11, 2, 50), (7, 7, 64), (70, 6, 128)])
def test_the_router_scores_all_outputs_chooses_with_the_correction_and_weighs_without(backend, experts, top, width):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(experts)
    h, h64 = lowered(rnd(g, 9, width), dtype, dev)
    router = rnd(g, experts, width, std=0.3).float()
    correction = rnd(g, experts, std=0.2).float()
    correction[0] = 5.0                                      # always chosen, whatever its score
    ids, weights = k.moe_route(h, router.to(dev), top, score="softmax_all", correction=correction.to(dev))
    T = {"m.router": router.double(), "m.correction": correction.double()}
    want_ids, want_w = plain.route(h64, T, "m", {"router": {"top": top}})
    s = torch.softmax(h64 @ router.double().T, -1)
    ranked = s + correction.double()
    for t in range(9):
        got = ids[t].tolist()
        assert len(set(got)) == top and 0 in got
        rest = [float(ranked[t][e]) for e in range(experts) if e not in got]
        assert not rest or float(ranked[t][got].min()) >= max(rest) - 1e-6
        close(weights[t], s[t][got] / s[t][got].sum(), 1e-5)
        close(weights[t].sort().values, want_w[t].sort().values, 1e-4)
    # without a correction the scores alone decide
    ids, weights = k.moe_route(h, router.to(dev), top, score="softmax_all")
    for t in range(9):
        rest = [float(s[t][e]) for e in range(experts) if e not in ids[t].tolist()]
        assert not rest or float(s[t][ids[t].long().cpu()].min()) >= max(rest) - 1e-6


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,identity,top,width,ff,shared,n", [
    (5, 1, 2, 96, 40, False, 11), (8, 2, 3, 128, 24, True, 11), (4, 3, 2, 50, 17, True, 11), (3, 0, 3, 64, 128, False, 11),
    # steps of many slots, which the GPU sorts by expert and multiplies in tiles; slots of experts without tensors
    # take no place in a tile
    (8, 2, 2, 160, 96, True, 203), (6, 10, 1, 64, 32, False, 70), (3, 1, 4, 128, 288, True, 64)])
def test_clamped_experts_and_experts_that_return_their_input(backend, experts, identity, top, width, ff, shared, n):
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(ff + identity)
    limit = 0.9
    h, h64 = lowered(rnd(g, n, width), dtype, dev)
    w1, w1_64 = lowered(rnd(g, experts, 2 * ff, width, std=0.15), dtype, dev)
    w2, w2_64 = lowered(rnd(g, experts, width, ff, std=0.1), dtype, dev)
    ids = torch.stack([torch.randperm(experts + identity, generator=g)[:top] for _ in range(n)]).to(torch.int32)
    weights = torch.softmax(rnd(g, n, top), -1).float()
    sh = sh64 = None
    if shared:
        sh, sh64 = lowered(rnd(g, n, width), dtype, dev)
    got = k.moe_experts(h, w1, w2, ids.to(dev), weights.to(dev), sh, None, activation=("clamped", limit),
                        identity=identity)
    want = torch.zeros(n, width, dtype=torch.float64)
    for t in range(n):
        for e, p in zip(ids[t].tolist(), weights[t].double()):
            if e >= experts:
                want[t] += p * h64[t]
                continue
            T = {"e.gate": w1_64[e][:ff], "e.up": w1_64[e][ff:], "e.down": w2_64[e]}
            want[t] += p * plain.clamped_expert(h64[t:t + 1], T, "e", limit)[0]
    if shared:
        want = want + sh64
    assert identity == 0 or int((ids >= experts).sum()) > 0
    close(got, want, tol * 2)


# ---------------------------------------------------------------------------------------------------------------
def window_part(k, dev, dtype, g, hidden, H, G, D, window, dims, scaling, scale=0.2, base=10000.0):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    mx = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "mask": {"size": window}, "rot": rot, "scale": scale}
    env = BuildEnv(kernels=k, device=torch.device(dev), dtype=dtype, max_positions=512)
    sc = dict(rot["scaling"], rope_type="yarn") if scaling else None
    part = MIXERS.get("attention")({
        "hidden_size": hidden, "num_heads": H, "num_kv_heads": G, "head_dim": D, "window": window, "scale": scale,
        "qk_norm": {"eps": 1e-5}, "sink": True, "value_from_key": True,
        "position": {"kind": "rope", "params": {"rotary_dim": dims, "theta": base, "scaling": sc, "angles": "float64"}}}, env)
    names = {"q": "m.q", "k": "m.k", "o": "m.o", "q_norm": "m.q.norm", "k_norm": "m.k.norm", "sink": "m.sink"}
    T, bound = {}, {}
    for name, spec in part.weight_specs().items():
        t = rnd(g, *spec.shape, std=0.3) + (1.0 if name.endswith("_norm") else 0.0)
        bound[name], T[names[name]] = lowered(t, torch.float32 if spec.role == "vector" else dtype, dev)
    part.bind(bound)
    return part, mx, T


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,window,dims,scaling,page", [
    (4, 2, 16, 11, 8, (4.0, 64, 16.0, 2.0), 8), (2, 2, 24, 40, 24, None, 16), (4, 1, 64, 24, 32, (16.0, 128, 32.0, 1.0), 16),
    (5, 5, 12, 7, 4, (2.0, 40, 8.0, 1.0), 16), (1, 1, 32, 1, 16, None, 16), (6, 2, 80, 33, 40, (3.0, 256, 24.0, 1.0), 16)])
def test_window_attention_whose_values_are_its_keys_as_projected(backend, H, G, D, window, dims, scaling, page):
    """A prompt in portions and decoded tokens (positions that pass the window and pages' borders) against the plain
    function over the whole sequence: values that are the keys before norm and rotation, the sink, the window."""
    k, dev, dtype, tol = setup(backend)
    g = torch.Generator().manual_seed(H * 100 + D)
    hidden, n = 64, 93
    part, mx, T = window_part(k, dev, dtype, g, hidden, H, G, D, window, dims, scaling)
    h, h64 = lowered(rnd(g, n, hidden), dtype, dev)
    want = plain.window_attention(h64, T, "m", mx, 1e-5)
    need = part.cache_need()
    pages = -(-n // page) + 1
    table = torch.arange(pages - 1, -1, -1, dtype=torch.int32, device=dev).view(1, pages).contiguous()
    cache = empty_cache(dev, dtype, pages, G, page, need.head_dim, need.value_dim, table)
    outs, at = [], 0
    for take in [17, 2, 30, 1, 1, 9] + [1] * 33:
        ctx, _, _, _ = step_context(dev, [(at, take)], page, k)
        cache.block_table = table
        outs.append(done(part.forward(h[at:at + take].contiguous(), ctx, cache)))
        at += take
    assert at == n
    close(torch.cat(outs), want, tol * 3)


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_key_at_the_windows_edge_is_seen_and_the_next_one_is_not(backend):
    """One position's input is replaced by a far larger one (its value, the key as projected, then dwarfs all others):
    a query ``window - 1`` places later reads it, a query ``window`` places later gives what it gave before, in a
    prompt and in decoding, with the changed position at a page's last and first place and in the middle of one."""
    k, dev, dtype, tol = setup(backend)
    if dtype == torch.bfloat16:
        pytest.skip("a question of which keys are visible: float32 decides it")
    H = G = 1
    D, window, page, hidden = 16, 21, 8, 32
    g = torch.Generator().manual_seed(2)
    part, mx, T = window_part(k, dev, dtype, g, hidden, H, G, D, window, 8, None, scale=1.0)
    n = 70
    for planted in (15, 16, 40):
        base = rnd(g, n, hidden, std=0.3)
        other = base.clone()
        other[planted] = 8.0 * rnd(g, hidden)
        inside, outside = planted + window - 1, planted + window
        for prefix in (n, 12):                                   # all as one prompt; or a short prompt and decoding
            rows = []
            for inputs in (base, other):
                h, h64 = lowered(inputs, dtype, dev)
                pages = -(-n // page)
                table = torch.randperm(pages, generator=torch.Generator().manual_seed(planted)).to(torch.int32)
                table = table.view(1, pages).to(dev).contiguous()
                cache = empty_cache(dev, dtype, pages, G, page, D, D, table)
                outs, at = [], 0
                for take in [prefix] + [1] * (n - prefix):
                    ctx, _, _, _ = step_context(dev, [(at, take)], page, k)
                    cache.block_table = table
                    outs.append(done(part.forward(h[at:at + take].contiguous(), ctx, cache)))
                    at += take
                rows.append(torch.cat(outs).double().cpu())
                close(rows[-1], plain.window_attention(h64, T, "m", mx, 1e-5), 3e-5)
            size = float(rows[0].abs().max())
            assert float((rows[0][inside] - rows[1][inside]).abs().max()) > 1e-3 * size
            assert float((rows[0][outside:] - rows[1][outside:]).abs().max()) <= 1e-6 * size
            assert float((rows[0][:planted] - rows[1][:planted]).abs().max()) == 0.0
