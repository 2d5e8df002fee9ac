"""Plain torch twins of the device kernels, one per kernel, with the kernels' signatures.

Two uses, both in tests only:

* on the GPU, each HIP kernel is compared alone with its twin;
* on the CPU, where the HIP kernels cannot run, a ``TwinKernels`` object is handed to
  the engine in place of the kernel library, so that the cache manager, the step
  function, the scheduler and trace replay can be tested without a GPU.

The engine itself has no such path: without its compiled kernels it refuses to start.
"""

from __future__ import annotations

import torch


class TwinKernels:
    name = "torch-twins"

    # -- embedding ---------------------------------------------------------
    def place_tokens(self, token_ids, dst_rows, src_tokens, src_rows):
        token_ids[dst_rows.long()] = src_tokens[src_rows.long()]

    def embed(self, token_ids, table, scale=1.0):
        return table[token_ids.long()].float() * scale

    def cast(self, x, dtype):
        return x.to(dtype)

    # -- residual += rms norm of a sublayer's output ---------------------------
    def norm_add(self, residual, y, weight, eps, out_dtype):
        yf = y.float()
        residual.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * weight.float())
        return residual if out_dtype == torch.float32 else residual.to(out_dtype)

    # -- residual add + rms norm ---------------------------------------------
    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype, rows=None, gate=None, gate_bias=None,
                    delta_bias=None, terms=None):
        if terms is not None:      # the delta as several results with a constant factor each
            delta = None
            for y, f in terms:
                delta = y.float() * f if delta is None else delta + y.float() * f
        elif delta is not None:
            delta = self._gated(delta, gate, gate_bias, delta_bias)
        if rows is None:
            if delta is not None:
                residual.add_(delta)
            x = residual
        else:
            x = residual[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()]
        if weight is None:
            return None
        var = x.pow(2).mean(-1, keepdim=True)
        return (x * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)

    def scaled_sum(self, terms):
        total = None
        for y, f in terms:
            total = y.float() * f if total is None else total + y.float() * f
        return total.to(terms[0][0].dtype)

    @staticmethod
    def _gated(delta, gate, gate_bias, delta_bias):
        d = delta.float()
        if delta_bias is not None:
            d = d + delta_bias.float()
        if gate is not None:
            z = gate.float()
            if gate_bias is not None:
                z = z + gate_bias.float()
            d = d * torch.sigmoid(z)
        return d

    def gated_add(self, residual, delta, gate=None, gate_bias=None, delta_bias=None):
        residual.add_(self._gated(delta, gate, gate_bias, delta_bias))

    def add_bias(self, y, bias):
        y.copy_((y.float() + bias.float()).to(y.dtype))
        return y

    def head_gate(self, out, logits, n_heads):
        n = out.shape[0]
        gated = out.float().view(n, n_heads, -1) * torch.sigmoid(logits.float())[:, :, None]
        out.copy_(gated.view(n, -1).to(out.dtype))
        return out

    def side_by_side(self, a, b, dtype):
        return torch.cat([a, b], dim=-1).to(dtype)

    def scale_softcap(self, logits, scale=1.0, cap=None):
        logits.mul_(scale)
        if cap is not None:
            logits.copy_(cap * torch.tanh(logits / cap))
        return logits

    # -- linear attention with a state ------------------------------------------
    def gla_recurrent(self, proj, columns, a2, a2_bias, norm_weight, n_heads, key_dim, value_dim, tau, q_scale, eps,
                      ctx, cache):
        N = proj.shape[0]
        H, D, Dv, rank = n_heads, key_dim, value_dim, a2.shape[1]
        cq, ck, cv, cg, ca = columns
        p = proj.float()
        q = p[:, cq:cq + H * D].view(N, H, D) * q_scale
        k = p[:, ck:ck + H * D].view(N, H, D)
        v = p[:, cv:cv + H * Dv].view(N, H, Dv)
        g = p[:, cg:cg + H * Dv]
        z = p[:, ca:ca + rank] @ a2.float().T
        if a2_bias is not None:
            z = z + a2_bias.float()
        alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(N, H, D)
        out = torch.zeros(N, H, Dv)
        cu, slots = ctx.cu_q.tolist(), ctx.state_slots.tolist()
        for s in range(ctx.n_seqs):
            S = cache.state[slots[s]]            # [H, D, Dv] float, updated in place
            for t in range(cu[s], cu[s + 1]):
                S.mul_(alpha[t][:, :, None]).add_(k[t][:, :, None] * v[t][:, None, :])
                out[t] = torch.einsum("hd,hdv->hv", q[t], S)
        out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_weight.float()
        return (out.view(N, H * Dv) * torch.nn.functional.silu(g)).to(proj.dtype)

    # -- norm without a statistic ------------------------------------------------------
    @staticmethod
    def _dyt(x, terms):
        w, b, alpha, scale = terms
        y = torch.tanh(alpha.float() * x.float()) * w.float() + b.float()
        return y * scale.float() if scale is not None else y

    def dyt_norm(self, residual, delta, post, pre, out_dtype, rows=None):
        add = None
        if delta is not None:
            add = self._dyt(delta, post) if post is not None else delta.float()
        if rows is None:
            if add is not None:
                residual.add_(add)
            x = residual
        else:
            x = residual[rows.long()]
            if add is not None:
                x = x + add[rows.long()]
        return self._dyt(x, pre).to(out_dtype) if pre is not None else None

    # -- short convolution and recurrences with a state -------------------------------------
    def causal_conv(self, proj, first_col, weight, bias, activation, ctx, state, state_offset):
        channels, taps = weight.shape
        u = proj[:, first_col:first_col + channels].float()
        out = torch.zeros_like(u)
        cu, slots = ctx.cu_q.tolist(), ctx.state_slots.tolist()
        w = weight.float()
        for s in range(ctx.n_seqs):
            past = state[slots[s], state_offset:state_offset + channels * (taps - 1)].view(taps - 1, channels)
            seq = torch.cat([past, u[cu[s]:cu[s + 1]]], dim=0)
            n = cu[s + 1] - cu[s]
            acc = bias.float().expand(n, channels).clone() if bias is not None else torch.zeros(n, channels)
            for j in range(taps):
                acc += seq[j:j + n] * w[:, j]
            out[cu[s]:cu[s + 1]] = acc
            if taps > 1:
                past.copy_(seq[n:])
        if activation == "silu":
            out = torch.nn.functional.silu(out)
        return out.to(proj.dtype)

    def ssd_scan(self, proj, xbc, dt_bias, a_log, d_skip, norm_weight, n_heads, head_dim, state_size, groups,
                 norm_groups, eps, ctx, state):
        n, H, P, N, G = proj.shape[0], n_heads, head_dim, state_size, groups
        inner = H * P
        z = proj[:, :inner].float()
        dt = torch.nn.functional.softplus(proj[:, proj.shape[1] - H:].float() + dt_bias.float(), threshold=1e9)
        decay = torch.exp(-torch.exp(a_log.float()) * dt)
        x = xbc[:, :inner].float().view(n, H, P)
        B = xbc[:, inner:inner + G * N].float().view(n, G, N).repeat_interleave(H // G, dim=1)
        C = xbc[:, inner + G * N:].float().view(n, G, N).repeat_interleave(H // G, dim=1)
        y = torch.zeros(n, H, P)
        cu, slots = ctx.cu_q.tolist(), ctx.state_slots.tolist()
        for s in range(ctx.n_seqs):
            S = state[slots[s], :H * N * P].view(H, N, P)
            for t in range(cu[s], cu[s + 1]):
                S.mul_(decay[t][:, None, None]).add_((dt[t][:, None] * B[t])[:, :, None] * x[t][:, None, :])
                y[t] = torch.einsum("hn,hnp->hp", C[t], S)
        y = (y + d_skip.float()[None, :, None] * x).view(n, inner) * torch.nn.functional.silu(z)
        parts = y.view(n, norm_groups, inner // norm_groups)
        y = (parts * torch.rsqrt(parts.pow(2).mean(-1, keepdim=True) + eps)).view(n, inner) * norm_weight.float()
        return y.to(proj.dtype)

    def delta_rule(self, qkv, proj, columns, a_log, dt_bias, norm_weight, n_heads, n_kv_heads, key_dim, value_dim, eps,
                   ctx, state):
        n, H, G, D, Dv = qkv.shape[0], n_heads, n_kv_heads, key_dim, value_dim
        cg, cb, ca = columns
        x, p = qkv.float(), proj.float()
        q = x[:, :G * D].view(n, G, D)
        k = x[:, G * D:2 * G * D].view(n, G, D)
        v = x[:, 2 * G * D:].view(n, H, Dv)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
        beta = torch.sigmoid(p[:, cb:cb + H])
        step = torch.nn.functional.softplus(p[:, ca:ca + H] + dt_bias.float(), threshold=1e9)
        decay = torch.exp(-torch.exp(a_log.float()) * step)
        out = torch.zeros(n, H, Dv)
        cu, slots = ctx.cu_q.tolist(), ctx.state_slots.tolist()
        for s in range(ctx.n_seqs):
            S = state[slots[s], :H * D * Dv].view(H, D, Dv)
            for t in range(cu[s], cu[s + 1]):
                S.mul_(decay[t][:, None, None])
                u = beta[t][:, None] * (v[t] - torch.einsum("hd,hdv->hv", k[t], S))
                S.add_(k[t][:, :, None] * u[:, None, :])
                out[t] = torch.einsum("hd,hdv->hv", q[t], S)
        out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_weight.float()
        return (out.view(n, H * Dv) * torch.nn.functional.silu(p[:, cg:cg + H * Dv])).to(qkv.dtype)

    def decay_attention(self, proj, decays, norm_weight, n_heads, key_dim, value_dim, eps, ctx, state):
        n, H, D, Dv = proj.shape[0], n_heads, key_dim, value_dim
        act = torch.nn.functional.silu(proj[:, :2 * H * D + H * Dv].float()).to(proj.dtype).float()
        q = act[:, :H * D].view(n, H, D)
        k = act[:, H * D:2 * H * D].view(n, H, D)
        v = act[:, 2 * H * D:].view(n, H, Dv)
        g = proj[:, 2 * H * D + H * Dv:].float()
        out = torch.zeros(n, H, Dv)
        cu, slots = ctx.cu_q.tolist(), ctx.state_slots.tolist()
        for s in range(ctx.n_seqs):
            S = state[slots[s]]
            for t in range(cu[s], cu[s + 1]):
                S.mul_(decays.float()[:, None, None]).add_(k[t][:, :, None] * v[t][:, None, :])
                out[t] = torch.einsum("hd,hdv->hv", q[t], S)
        out = out.view(n, H * Dv)
        out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_weight.float()
        return (out * torch.sigmoid(g)).to(proj.dtype)

    def hgrn2_scan(self, proj, f_bias, lower, norm_weight, n_heads, key_dim, value_dim, eps, ctx, state):
        n, H, D, Dv = proj.shape[0], n_heads, key_dim, value_dim
        p = proj.float()
        q = torch.nn.functional.silu(p[:, :H * D]).to(proj.dtype).float().view(n, H, D)
        low = lower.float()
        f = (low + (1 - low) * torch.sigmoid(p[:, H * D:2 * H * D] + f_bias.float())).view(n, H, D)
        v = p[:, 2 * H * D:].view(n, H, Dv)
        out = torch.zeros(n, H, Dv)
        cu, slots = ctx.cu_q.tolist(), ctx.state_slots.tolist()
        for s in range(ctx.n_seqs):
            S = state[slots[s]]
            for t in range(cu[s], cu[s + 1]):
                S.mul_(f[t][:, :, None]).add_((1 - f[t])[:, :, None] * v[t][:, None, :])
                out[t] = torch.einsum("hd,hdv->hv", q[t], S)
        out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_weight.float()
        return out.view(n, H * Dv).to(proj.dtype)

    # -- latent attention ------------------------------------------------------------------
    @staticmethod
    def _rotate_pairs(x, rotary_dim, cos, sin, pos):
        """``x [n, ..., r]`` float: neighbouring pairs of the first ``rotary_dim`` elements turned by the tables' rows."""
        if rotary_dim == 0:
            return x
        shape = [x.shape[0]] + [1] * (x.dim() - 2) + [rotary_dim // 2]
        c, s = cos[pos.long()].view(shape), sin[pos.long()].view(shape)
        a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        out = x.clone()
        out[..., 0:rotary_dim:2] = a * c - b * s
        out[..., 1:rotary_dim:2] = b * c + a * s
        return out

    def latent_prepare(self, proj, q_rank, q_gain, kv_rank, kv_gain, rot_dim, rotary_dim, cos, sin, eps, ctx, cache,
                       page_dim=None):
        p = proj.float()
        cq = p[:, :q_rank]
        cq = (cq * torch.rsqrt(cq.pow(2).mean(-1, keepdim=True) + eps) * q_gain.float()).to(proj.dtype)
        if kv_rank:
            a = p[:, q_rank:q_rank + kv_rank]
            c = (a * torch.rsqrt(a.pow(2).mean(-1, keepdim=True) + eps) * kv_gain.float()).to(proj.dtype)
            b = self._rotate_pairs(p[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim], rotary_dim, cos, sin,
                                   ctx.positions).to(proj.dtype)
            pos = ctx.positions.long()
            ps = cache.page_size
            page = cache.block_table.long()[ctx.seq_of_token.long(), pos // ps]
            off = pos % ps
            cache.k_pages[page, 0, off, :kv_rank] = c
            cache.k_pages[page, 0, off, kv_rank:kv_rank + rot_dim] = b
            cache.v_pages[page, 0, :kv_rank, off] = c
        return cq

    def headwise_linear(self, x, w, in_stride, out_stride, tail=0, rotation=None):
        n = x.shape[0]
        H, out_dim, in_dim = w.shape
        xs = x.float().view(n, H, in_stride)
        y = torch.zeros(n, H, out_stride)
        y[:, :, :out_dim] = torch.einsum("nhi,hoi->nho", xs[:, :, :in_dim], w.float())
        if tail:
            t = xs[:, :, in_dim:in_dim + tail]
            if rotation is not None:
                rotary_dim, cos, sin, positions = rotation
                t = self._rotate_pairs(t, rotary_dim, cos, sin, positions)
            y[:, :, out_dim:out_dim + tail] = t
        return y.view(n, H * out_stride).to(x.dtype)

    # -- mixture of experts ---------------------------------------------------------
    def moe_route(self, h, router, top, score="softmax", groups=None, scale=1.0, correction=None):
        logits = h.float() @ router.float().T
        if score == "softmax_all":
            sc = torch.softmax(logits, -1)
            ranked = sc + correction.float() if correction is not None else sc
            order = torch.sort(ranked, dim=-1, descending=True, stable=True).indices[:, :top]
            chosen = torch.gather(sc, 1, order)
            return order.to(torch.int32), chosen / (chosen.sum(-1, keepdim=True) + 1e-20)
        if score == "sigmoid":
            sc = torch.sigmoid(logits)
            ranked = sc
            if groups is not None:
                count, keep = groups
                per = sc.shape[1] // count
                g = sc.view(-1, count, per)
                gscore = torch.sort(g, dim=-1, descending=True).values[:, :, :2].sum(-1)
                best = torch.sort(gscore, dim=-1, descending=True, stable=True).indices[:, :keep]
                allowed = torch.zeros_like(gscore, dtype=torch.bool).scatter_(1, best, True)
                ranked = sc.masked_fill(~allowed[:, :, None].expand(-1, -1, per).reshape(sc.shape), -1.0)
            order = torch.sort(ranked, dim=-1, descending=True, stable=True).indices[:, :top]
            chosen = torch.gather(sc, 1, order)
            return order.to(torch.int32), chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * scale
        order = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :top]
        best = torch.gather(logits, 1, order)
        return order.to(torch.int32), torch.softmax(best, -1)

    @staticmethod
    def _glu(g, u, activation):
        if activation is None:
            return torch.nn.functional.silu(g) * u
        kind, limit = activation
        assert kind == "clamped"
        g, u = g.clamp(max=limit), u.clamp(-limit, limit)
        return g * torch.sigmoid(1.702 * g) * (u + 1.0)

    def moe_experts(self, h, w_gate_up, w_down, ids, weights, shared=None, shared_gate=None, activation=None,
                    identity=0):
        n, top = ids.shape
        ff = w_gate_up.shape[1] // 2
        real = w_gate_up.shape[0]
        x = h.float()
        y = torch.zeros(n, w_down.shape[1])
        for t in range(n):
            for k in range(top):
                e = int(ids[t, k])
                if e >= real:       # an expert without tensors: its input comes back
                    assert e < real + identity
                    y[t] += weights[t, k] * x[t]
                    continue
                gu = w_gate_up[e].float() @ x[t]
                a = self._glu(gu[:ff], gu[ff:], activation).to(h.dtype).float()
                y[t] += weights[t, k] * (w_down[e].float() @ a)
        if shared is not None:
            s = shared.float()
            if shared_gate is not None:
                s = s * torch.sigmoid(shared_gate.float())
            y = y + s
        return y.to(h.dtype)

    # -- matrix product ------------------------------------------------------
    def linear(self, x, w, out_float32=False):
        y = x.float() @ w.float().T
        return y if out_float32 else y.to(x.dtype)

    pending_linear = linear   # computed at once: the twin's norm always has a kernel of its own

    def gated_linear(self, x, w_gate_up, activation=None):
        if activation is not None:
            gu = self.linear(x, w_gate_up).float()
            inter = gu.shape[-1] // 2
            return self._glu(gu[:, :inter], gu[:, inter:], activation).to(x.dtype)
        return self.swiglu(self.linear(x, w_gate_up))

    # -- feed-forward activation --------------------------------------------
    def swiglu(self, gu):
        inter = gu.shape[-1] // 2
        g, u = gu[:, :inter].float(), gu[:, inter:].float()
        return (g * torch.sigmoid(g) * u).to(gu.dtype)

    def activated_linear(self, x, w, activation):
        z = self.linear(x, w).float()
        if activation == "relu2":
            a = torch.relu(z) ** 2
        elif activation == "gelu_tanh":
            a = 0.5 * z * (1 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        elif activation == "gelu":
            a = 0.5 * z * (1 + torch.erf(z * 0.7071067811865476))
        else:
            raise ValueError(activation)
        return a.to(x.dtype)

    def qkv_to_cache(self, x, w_qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache,
                     value_dim=None, bias=None, qk_norm=None, q_temp=None, extra_columns=0, values_are_keys=False):
        qkv = self.linear(x, w_qkv)
        self.rope_kv_write(qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache,
                           value_dim=value_dim, bias=bias, qk_norm=qk_norm, q_temp=q_temp,
                           values_are_keys=values_are_keys)
        if extra_columns:
            return qkv, qkv[:, qkv.shape[1] - extra_columns:]
        return qkv

    # -- rotation + cache write ----------------------------------------------
    def rope_kv_write(self, qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache,
                      value_dim=None, bias=None, qk_norm=None, q_temp=None, values_are_keys=False):
        N = qkv.shape[0]
        pos = ctx.positions.long()
        value_dim = value_dim or head_dim
        if bias is not None:
            own = bias.numel()
            qkv[:, :own] = (qkv[:, :own].float() + bias.float()).to(qkv.dtype)
        q = qkv[:, :n_heads * head_dim].view(N, n_heads, head_dim)

        def normed(x, gain):
            if qk_norm is None:
                return x
            xf = x.float()
            return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + qk_norm[2]) * gain.float()).to(x.dtype)

        def rotate(x):
            if rotary_dim == 0:
                return x
            half = rotary_dim // 2
            c = cos[pos][:, None, :]
            s = sin[pos][:, None, :]
            xf = x.float()
            a, b = xf[..., :half], xf[..., half:rotary_dim]
            out = xf.clone()
            out[..., :half] = a * c - b * s
            out[..., half:rotary_dim] = b * c + a * s
            return out.to(x.dtype)

        qn = normed(q, qk_norm[0] if qk_norm else None)
        if q_temp is not None:
            temp = 1.0 + q_temp[0] * torch.log((torch.div(pos + 1, q_temp[1], rounding_mode="floor") + 1).float())
            qn = (qn.float() * temp[:, None, None]).to(q.dtype)
        q.copy_(rotate(qn))
        if n_kv_written == 0:
            return
        kv0 = n_heads * head_dim
        k = qkv[:, kv0:kv0 + n_kv_written * head_dim].view(N, n_kv_written, head_dim)
        v0 = kv0 if values_are_keys else kv0 + n_kv_written * head_dim      # the keys as projected serve as values
        v = qkv[:, v0:v0 + n_kv_written * value_dim].view(N, n_kv_written, value_dim)
        k = rotate(normed(k, qk_norm[1] if qk_norm else None))
        ps = cache.page_size
        seq = ctx.seq_of_token.long()
        page = cache.block_table.long()[seq, pos // ps]
        off = pos % ps
        cache.k_pages[page, :, off, :] = k
        cache.v_pages[page, :, :, off] = v

    # -- attention over the pages --------------------------------------------
    def paged_attention(self, qkv, n_heads, n_kv_heads, head_dim, scale, window, ctx, cache, value_dim=None,
                        chunk=None, sinks=None):
        N = qkv.shape[0]
        value_dim = value_dim or head_dim
        q = qkv[:, :n_heads * head_dim].view(N, n_heads, head_dim).float()
        out = torch.zeros(N, n_heads, value_dim, dtype=torch.float32, device=qkv.device)
        ps = cache.page_size
        group = n_heads // n_kv_heads
        cu = ctx.cu_q.tolist()
        kv_len = ctx.kv_len.tolist()
        table = cache.block_table.long()
        for s in range(ctx.n_seqs):
            L = kv_len[s]
            lo = 0
            first = kv_len[s] - (cu[s + 1] - cu[s])
            if window is not None:
                lo = max(0, first - window + 1)
            if chunk is not None:
                lo = max(lo, first - first % chunk)
            idx = torch.arange(lo, L, device=qkv.device)
            pages = table[s, idx // ps]
            k = cache.k_pages[pages, :, idx % ps, :].float()          # [T, Hkv, D]
            v = cache.v_pages[pages, :, :, idx % ps].float()          # [T, Hkv, D]
            qs = q[cu[s]:cu[s + 1]]
            qpos = torch.arange(first, L, device=qkv.device)
            visible = idx[None, :] <= qpos[:, None]
            if window is not None:
                visible &= idx[None, :] > qpos[:, None] - window
            if chunk is not None:
                visible &= idx[None, :] // chunk == qpos[:, None] // chunk
            for h in range(n_heads):
                sc = (qs[:, h] @ k[:, h // group].T) * scale
                sc = sc.masked_fill(~visible, float("-inf"))
                if sinks is not None:    # one more term in the denominator: a column whose value is nothing
                    sc = torch.cat([sc, sinks[h].float().expand(sc.shape[0], 1)], dim=-1)
                    out[cu[s]:cu[s + 1], h] = torch.softmax(sc, -1)[:, :-1] @ v[:, h // group]
                else:
                    out[cu[s]:cu[s + 1], h] = torch.softmax(sc, -1) @ v[:, h // group]
        return out.view(N, n_heads * value_dim).to(qkv.dtype)

    # -- sampling --------------------------------------------------------------
    def sample(self, logits, temperature, top_k, top_p, uniform, all_greedy=False, filters=None):
        if all_greedy:
            return torch.argmax(logits.double(), dim=-1).to(torch.int32)
        out = []
        for r in range(logits.shape[0]):
            row = logits[r].double()
            t = float(temperature[r])
            if t == 0.0:
                out.append(int(torch.argmax(row)))
                continue
            row = row / t
            k = int(top_k[r])
            V = row.shape[0]
            if 0 < k < V:
                kth = torch.sort(row, descending=True).values[k - 1]
                row = torch.where(row < kth, torch.full_like(row, float("-inf")), row)
            p = float(top_p[r])
            if p < 1.0:
                srt, idx = torch.sort(row, descending=True)
                cum = torch.softmax(srt, -1).cumsum(-1)
                rem = torch.zeros_like(cum, dtype=torch.bool)
                if p > 0.0:
                    rem[1:] = cum[:-1] > p
                else:
                    rem[1:] = True
                row = row.masked_fill(torch.zeros_like(rem).scatter(0, idx, rem), float("-inf"))
            cdf = torch.softmax(row, -1).cumsum(-1)
            out.append(min(int((cdf <= float(uniform[r]) * cdf[-1]).sum()), V - 1))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
