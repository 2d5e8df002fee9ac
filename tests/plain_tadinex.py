"""A plain, slow implementation of the Tadinex design: whole sequences, no cache, float64, one function per mechanism.

It shares no code with the package.  ``cfg`` is the design's config.json as a dictionary and ``T`` maps checkpoint
names to tensors.  Notation: ``x`` the residual stream ``[n, width]``, ``h`` a sublayer's input, ``m`` the layer
multiplier.

* norm: ``N(x) = x / sqrt(mean(x^2) + eps) * (1 + w)``: the gain is stored as its distance from one.
* layer: ``x += m * mixer(N1(x))``, then ``x += m * ff(N2(x))`` if the layer has a feed-forward.
* mixers: the gated delta rule behind short convolutions (``delta``), and softmax attention over a window beside a
  linear attention with a constant decay, both reading the same input (``parallel``).
* feed-forwards: ``W_down gelu(W_up h)``, or routed experts with a clamped gated activation, identity experts and a
  shared expert.
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


def offset_norm(x, T, name, eps):
    return rms(x, eps) * (1.0 + _t(T, name))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


# ---------------------------------------------------------------------------------------------------------
# the delta-rule mixer
def causal_conv(u, w):
    """``out[t, c] = sum_j w[c, j] u[t - (taps - 1) + j, c]``: the last tap meets the current token, zeros stand
    before the sequence."""
    n = u.shape[0]
    taps = w.shape[1]
    out = torch.zeros_like(u)
    for j in range(taps):
        shift = taps - 1 - j
        if shift < n:
            out[shift:] += u[: n - shift] * w[:, j]
    return out


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_inputs(h, T, p, mx):
    """q, k ``[n, kv_heads, dim]`` (unit vectors, q scaled), v ``[n, heads, vdim]``, the write strengths and the
    decays ``[n, heads]``."""
    n = h.shape[0]
    H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = silu(causal_conv(h @ _t(T, p + ".q").T, _t(T, p + ".q.conv"))).reshape(n, G, D)
    k = silu(causal_conv(h @ _t(T, p + ".k").T, _t(T, p + ".k.conv"))).reshape(n, G, D)
    v = silu(causal_conv(h @ _t(T, p + ".v").T, _t(T, p + ".v.conv"))).reshape(n, H, Dv)
    q, k = unit(q) * D ** -0.5, unit(k)
    beta = torch.sigmoid(h @ _t(T, p + ".b").T)
    step = torch.nn.functional.softplus(h @ _t(T, p + ".a").T + _t(T, p + ".dt_bias"), threshold=1e9)
    decay = torch.exp(-torch.exp(_t(T, p + ".A_log")) * step)
    return q, k, v, beta, decay


def delta_rule(q, k, v, beta, decay):
    """Per head: the state fades, the value the key would read out now is replaced, in part, by the new one, and the
    query reads the state that already holds this token."""
    n, H, Dv = v.shape
    G, D = q.shape[1], q.shape[2]
    o = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(n):
            S = decay[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    return o


def delta_mixer(h, T, p, mx, eps):
    n = h.shape[0]
    H, Dv = mx["heads"], mx["vdim"]
    o = delta_rule(*delta_inputs(h, T, p, mx))
    o = rms(o, eps) * _t(T, p + ".norm")
    o = o.reshape(n, H * Dv) * silu(h @ _t(T, p + ".g").T)
    return o @ _t(T, p + ".o").T


# ---------------------------------------------------------------------------------------------------------
# the two mixers side by side
def ramp_frequencies(rot):
    """Turning speed of every pair of the rotated elements and the factor on both tables."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def pair_of(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(pair_of(sc["fast"])), 0)
    hi = min(math.ceil(pair_of(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / sc["factor"] * ramp + f * (1 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half(x, rot):
    """``x [n, heads, dim]``: element ``i`` of the first ``dims`` turns with element ``i + dims / 2``."""
    dims = rot["dims"]
    f, amp = ramp_frequencies(rot)
    a = torch.arange(x.shape[0], dtype=F64)[:, None] * f[None, :]
    c, s = (torch.cos(a) * amp)[:, None, :], (torch.sin(a) * amp)[:, None, :]
    u, w = x[..., : dims // 2], x[..., dims // 2: dims]
    out = x.clone()
    out[..., : dims // 2] = u * c - w * s
    out[..., dims // 2: dims] = w * c + u * s
    return out


def window_attention(h, T, p, mx, eps):
    n = h.shape[0]
    H, G, D = mx["heads"], mx["kv_heads"], mx["dim"]
    q = (h @ _t(T, p + ".q").T).reshape(n, H, D)
    k = (h @ _t(T, p + ".k").T).reshape(n, G, D)
    v = k                                    # the values are the keys as projected
    q = rotate_half(rms(q, eps) * _t(T, p + ".q.norm"), mx["rot"])
    kr = rotate_half(rms(k, eps) * _t(T, p + ".k.norm"), mx["rot"])
    pos = torch.arange(n)
    dist = pos[:, None] - pos[None, :]
    seen = (dist >= 0) & (dist < mx["mask"]["size"])
    sink = _t(T, p + ".sink")
    out = torch.zeros(n, H, D, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        sc = (q[:, hd] @ kr[:, g].T) * mx["scale"]
        sc = sc.masked_fill(~seen, float("-inf"))
        top = torch.maximum(sc.max(-1).values, sink[hd])
        e = torch.exp(sc - top[:, None])
        out[:, hd] = (e / (e.sum(-1, keepdim=True) + torch.exp(sink[hd] - top)[:, None])) @ v[:, g]
    return out.reshape(n, H * D) @ _t(T, p + ".o").T


def decaying_attention(h, T, p, mx, eps):
    n = h.shape[0]
    H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
    q = silu(h @ _t(T, p + ".q").T).reshape(n, H, D)
    k = silu(h @ _t(T, p + ".k").T).reshape(n, H, D)
    v = silu(h @ _t(T, p + ".v").T).reshape(n, H, Dv)
    o = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(n):
            S = mx["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = rms(o.reshape(n, H * Dv), eps) * _t(T, p + ".norm")
    return (o * torch.sigmoid(h @ _t(T, p + ".g").T)) @ _t(T, p + ".o").T


def parallel_mixer(h, T, p, mx, eps):
    if mx["left"].get("vdim", mx["left"]["dim"]) != mx["left"]["dim"]:
        raise ValueError("values that are the keys have the keys' width")
    return (mx["left_scale"] * window_attention(h, T, p + ".left", mx["left"], eps)
            + mx["right_scale"] * decaying_attention(h, T, p + ".right", mx["right"], eps))


# ---------------------------------------------------------------------------------------------------------
# feed-forwards
def dense(h, T, p):
    return gelu_erf(h @ _t(T, p + ".up").T) @ _t(T, p + ".down").T


def clamped_expert(h, T, p, limit):
    g = torch.clamp(h @ _t(T, p + ".gate").T, max=limit)
    u = torch.clamp(h @ _t(T, p + ".up").T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ _t(T, p + ".down").T


def route(h, T, p, mlp):
    """(ids [n, top], weights [n, top]): chosen by score plus correction, weighted by the scores alone."""
    s = torch.softmax(h @ _t(T, p + ".router").T, -1)
    order = torch.sort(s + _t(T, p + ".correction"), dim=-1, descending=True, stable=True).indices[:, : mlp["router"]["top"]]
    w = torch.gather(s, 1, order)
    return order, w / (w.sum(-1, keepdim=True) + 1e-20)


def experts(h, T, p, mlp):
    real = mlp["router"]["experts"]       # the router's further outputs stand for experts that return their input
    ids, w = route(h, T, p, mlp)
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(ids.shape[1]):
            e = int(ids[t, k])
            y[t] += w[t, k] * (clamped_expert(h[t:t + 1], T, f"{p}.e{e}", mlp["expert"]["limit"])[0] if e < real else h[t])
    if mlp.get("shared"):
        y = y + clamped_expert(h, T, p + ".shared", mlp["shared"]["limit"])
    return y


# ---------------------------------------------------------------------------------------------------------
def layer_streams(cfg, T, tokens):
    """The residual stream after every layer, ``[layers, n, width]``, and the last one normed."""
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = _t(T, "embed")[torch.as_tensor(tokens, dtype=torch.long)] * cfg.get("embedding", {}).get("scale", 1.0)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        h = offset_norm(x, T, p + ".norm1", eps)
        if layer["type"] == "delta":
            x = x + m * delta_mixer(h, T, p + ".mix", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            x = x + m * parallel_mixer(h, T, p + ".mix", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = offset_norm(x, T, p + ".norm2", eps)
            x = x + m * (dense(h, T, p + ".mlp") if mlp["kind"] == "dense" else experts(h, T, p + ".mlp", mlp))
        after.append(x.clone())
    return torch.stack(after), offset_norm(x, T, "final.norm", eps)


def forward(cfg, T, tokens):
    """Logits ``[n, vocab]`` of a whole sequence."""
    return layer_streams(cfg, T, tokens)[1] @ _t(T, "head").T
