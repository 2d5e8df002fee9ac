"""A plain, slow implementation of the Famepel design: whole sequences, no cache, float64, one function per mechanism.

It shares no code with the package.  ``cfg`` is the design's config.json as a dictionary and ``T`` maps checkpoint
names to tensors.  Notation: ``x`` the residual stream ``[n, width]``, ``h`` a sublayer's input.

* norm (dynamic tanh): ``tanh(a x) w + b`` with a scalar ``a``; no statistic.
* layer: ``x += ls1 * N1b(mixer(N1(x)))``, then ``x += ls2 * N2b(ff(N2(x)))`` if it has a feed-forward.
* ``rms(y) = y / sqrt(mean(y^2) + eps)``.
"""

import math

import torch

F64 = torch.float64


def _t(T, name):
    return T[name].to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def dynamic_tanh(x, T, name):
    return torch.tanh(_t(T, name + ".alpha") * x) * _t(T, name) + _t(T, name + ".b")


# ---------------------------------------------------------------------------------------------------------
def causal_conv(u, w, b):
    """``out[t, c] = b[c] + sum_j w[c, j] u[t - (taps - 1) + j, c]``: the last tap meets the current token, zeros
    stand before the sequence."""
    n, _ = u.shape
    taps = w.shape[1]
    out = torch.zeros_like(u) + b
    for j in range(taps):
        shift = taps - 1 - j
        if shift < n:
            out[shift:] += u[: n - shift] * w[:, j]
    return out


def mamba2_inputs(h, T, p, m):
    """The mixer's projection and convolution: ``z [n, inner]``, the convolved ``[x | B | C]`` rows and the raw step
    sizes ``[n, heads]``."""
    heads, vdim, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * vdim
    proj = h @ _t(T, p + ".in").T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    return z, silu(causal_conv(xbc, _t(T, p + ".conv"), _t(T, p + ".conv.b"))), dt


def state_space(z, xbc, dt, T, p, m, eps):
    """The recurrence over convolved rows, the gate and the norm in parts: ``[n, inner]``."""
    heads, vdim, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, n = heads * vdim, z.shape[0]
    x = xbc[:, :inner].reshape(n, heads, vdim)
    B = xbc[:, inner:inner + G * N].reshape(n, G, N)
    C = xbc[:, inner + G * N:].reshape(n, G, N)
    dt = torch.nn.functional.softplus(dt + _t(T, p + ".dt_bias"), threshold=1e9)
    a = torch.exp(_t(T, p + ".A_log"))
    D = _t(T, p + ".D")
    y = torch.zeros(n, heads, vdim, dtype=F64)
    for hd in range(heads):
        g = hd // (heads // G)
        S = torch.zeros(N, vdim, dtype=F64)
        for t in range(n):
            S = torch.exp(-a[hd] * dt[t, hd]) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + D[hd] * x[t, hd]
    y = y.reshape(n, inner) * silu(z)
    parts = m["norm_groups"]
    return rms(y.reshape(n, parts, inner // parts), eps).reshape(n, inner) * _t(T, p + ".norm")


def mamba2(h, T, p, m, eps):
    z, xbc, dt = mamba2_inputs(h, T, p, m)
    return state_space(z, xbc, dt, T, p, m, eps) @ _t(T, p + ".o").T


# ---------------------------------------------------------------------------------------------------------
def hgrn2(h, T, p, m, eps):
    heads, dim, vdim, n = m["heads"], m["dim"], m["vdim"], h.shape[0]
    q = silu(h @ _t(T, p + ".q").T).reshape(n, heads, dim)
    v = (h @ _t(T, p + ".v").T).reshape(n, heads, vdim)
    low = _t(T, p + ".lower")
    f = (low + (1 - low) * torch.sigmoid(h @ _t(T, p + ".f").T + _t(T, p + ".f.b"))).reshape(n, heads, dim)
    o = torch.zeros(n, heads, vdim, dtype=F64)
    for hd in range(heads):
        S = torch.zeros(dim, vdim, dtype=F64)
        for t in range(n):
            S = f[t, hd][:, None] * S + torch.outer(1 - f[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = rms(o, eps) * _t(T, p + ".norm")
    return o.reshape(n, heads * vdim) @ _t(T, p + ".o").T


# ---------------------------------------------------------------------------------------------------------
def rotary_tables(n, rot):
    """cos and sin ``[n, dims / 2]`` with the frequencies stretched by wavelength and the amplitude raised."""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2 * i / dims)
    amp = 1.0
    sc = rot.get("scaling")
    if sc:
        def at(turns):
            return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(at(sc["fast"])), 0)
        hi = min(math.ceil(at(sc["slow"])), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        amp = 0.1 * math.log(sc["factor"]) + 1
    ang = torch.arange(n, dtype=F64)[:, None] * f
    return ang.cos() * amp, ang.sin() * amp


def rotate_pairs(u, cos, sin):
    """``u [n, ..., r]``: the first ``2 * cos.shape[1]`` elements in neighbouring pairs, the rest unchanged."""
    d = 2 * cos.shape[1]
    shape = [u.shape[0]] + [1] * (u.dim() - 2) + [d // 2]
    c, s = cos.reshape(shape), sin.reshape(shape)
    a, b = u[..., 0:d:2], u[..., 1:d:2]
    out = u.clone()
    out[..., 0:d:2] = a * c - b * s
    out[..., 1:d:2] = b * c + a * s
    return out


def latent_kv(h, T, p, m, eps):
    """The cached part of latent attention: the normed latent ``[n, kv_rank]`` and the rotated shared key part."""
    n = h.shape[0]
    d = h @ _t(T, p + ".dkv").T
    c = rms(d[:, :m["kv_rank"]], eps) * _t(T, p + ".dkv.norm")
    cos, sin = rotary_tables(n, m["rot"])
    return c, rotate_pairs(d[:, m["kv_rank"]:], cos, sin)


def latent_attention(h, T, p, m, eps, kv):
    H, dim, rd, vdim, n = m["heads"], m["dim"], m["rot_dim"], m["vdim"], h.shape[0]
    c, k_rot = kv
    cq = rms(h @ _t(T, p + ".dq").T, eps) * _t(T, p + ".dq.norm")
    q = (cq @ _t(T, p + ".uq").T).reshape(n, H, dim + rd)
    cos, sin = rotary_tables(n, m["rot"])
    q_plain, q_rot = q[..., :dim], rotate_pairs(q[..., dim:], cos, sin)
    k_plain = (c @ _t(T, p + ".uk").T).reshape(n, H, dim)
    v = (c @ _t(T, p + ".uv").T).reshape(n, H, vdim)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    scores = scores.masked_fill(~mask, -math.inf)
    sink = _t(T, p + ".sink")
    top = torch.maximum(scores.max(-1).values, sink[:, None])
    e = torch.exp(scores - top[..., None])
    w = e / (e.sum(-1) + torch.exp(sink[:, None] - top))[..., None]
    out = torch.einsum("hij,jhd->ihd", w, v).reshape(n, H * vdim)
    return out @ _t(T, p + ".o").T


# ---------------------------------------------------------------------------------------------------------
def route(h, T, p, r):
    """ids ``[n, top]`` and weights ``[n, top]`` of the chosen experts."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ _t(T, p + ".router").T)
    allowed = torch.ones_like(s, dtype=torch.bool)
    g = r.get("groups")
    if g:
        per = E // g["count"]
        grouped = s.reshape(-1, g["count"], per)
        score = grouped.topk(min(2, per), dim=-1).values.sum(-1)
        best = score.topk(g["keep"], dim=-1).indices
        keep = torch.zeros_like(score, dtype=torch.bool).scatter_(1, best, True)
        allowed = keep[:, :, None].expand(-1, -1, per).reshape(-1, E)
    ids = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    chosen = s.gather(1, ids)
    return ids, chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * r.get("scale", 1.0)


def experts(h, T, p, mlp):
    ids, w = route(h, T, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t].tolist(), w[t]):
            q = f"{p}.e{e}"
            out[t] += wt * ((silu(h[t] @ _t(T, q + ".gate").T) * (h[t] @ _t(T, q + ".up").T)) @ _t(T, q + ".down").T)
    return out


# ---------------------------------------------------------------------------------------------------------
def forward(cfg, T, tokens, return_layers=False):
    """Logits ``[n, vocab]`` of a whole sequence (and the residual stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = _t(T, "embed")[torch.as_tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    kept, after = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        h = dynamic_tanh(x, T, p + ".norm1")
        if layer["type"] == "mamba2":
            y = mamba2(h, T, p + ".mix", m, eps)
        elif layer["type"] == "hgrn2":
            y = hgrn2(h, T, p + ".mix", m, eps)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = latent_kv(h, T, p + ".mix", m, eps)
            y = latent_attention(h, T, p + ".mix", m, eps, kept[i if src is None else src])
        else:
            raise ValueError(layer["type"])
        x = x + dynamic_tanh(y, T, p + ".norm1b") * _t(T, p + ".ls1")
        if layer.get("mlp") is not None:
            y = experts(dynamic_tanh(x, T, p + ".norm2"), T, p + ".mlp", layer["mlp"])
            x = x + dynamic_tanh(y, T, p + ".norm2b") * _t(T, p + ".ls2")
        after.append(x.clone())
    logits = dynamic_tanh(x, T, "final.norm") @ _t(T, "head").T
    return (logits, torch.stack(after)) if return_layers else logits
