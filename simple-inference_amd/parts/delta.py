"""The gated delta rule: a mixer whose memory is a matrix state per head that is corrected, not only added to.

For a token with input ``h`` (``H`` value heads of width ``Dv``, ``G`` query/key heads of width ``D``, value head ``i``
reading query/key head ``i // (H / G)``):

    q, k, v = silu(conv(Wq h)), silu(conv(Wk h)), silu(conv(Wv h))     a short causal convolution per channel
    q <- q / sqrt(sum(q^2) + 1e-6) * D^(-1/2),  k <- k / sqrt(sum(k^2) + 1e-6)          per head
    beta = sigmoid(Wb h),  g = exp(-exp(A_log) * softplus(Wa h + dt_bias))              per value head
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                        S [D, Dv], in this order
    y = Wo (concat_i(o_i / rms(o_i) * w) * silu(Wg h))                                  w [Dv], shared by the heads

A request's row of state holds, in float32, the ``H`` matrices and behind them the last ``taps - 1`` inputs of the
convolution (zeros before the first token); the cache manager hands it in as ``cache.state``.  All input projections
are one stacked matrix ``[q | k | v | g | b | a]``; the convolution reads its first columns.  Unit norms, write
strengths, decays, the state and the output norm are float32 in both modes.
"""

from __future__ import annotations

import torch

from .plan import StateNeed, TensorSpec
from .registry import register_mixer


@register_mixer("gated_delta")
class GatedDeltaRule:
    """params: hidden_size, num_heads, num_kv_heads, key_dim, value_dim, conv_taps, norm_eps."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.key_dim = int(params["key_dim"])
        self.value_dim = int(params["value_dim"])
        self.taps = int(params["conv_taps"])
        self.eps = float(params["norm_eps"])
        if self.num_heads % self.num_kv_heads or self.taps < 1:
            raise ValueError(f"{self.num_heads} heads do not share {self.num_kv_heads} query/key heads evenly (or the "
                             f"convolution has no tap)")
        self.qk = self.num_kv_heads * self.key_dim
        self.inner = self.num_heads * self.value_dim
        self.channels = 2 * self.qk + self.inner
        check = getattr(env.kernels, "check_recurrent_geometry", None)
        if check is not None:
            check(self.key_dim, self.value_dim)
        self.env = env
        self.w_in = self.w_o = self.conv_w = self.a_log = self.dt_bias = self.norm = None
        self.columns = None

    takes_scaled_rows = False

    def weight_specs(self):
        H = self.num_heads
        return {
            "q": TensorSpec((self.qk, self.hidden)), "k": TensorSpec((self.qk, self.hidden)),
            "v": TensorSpec((self.inner, self.hidden)), "g": TensorSpec((self.inner, self.hidden)),
            "b": TensorSpec((H, self.hidden)), "a": TensorSpec((H, self.hidden)),
            "q_conv": TensorSpec((self.qk, self.taps), "vector"), "k_conv": TensorSpec((self.qk, self.taps), "vector"),
            "v_conv": TensorSpec((self.inner, self.taps), "vector"),
            "a_log": TensorSpec((H,), "vector"), "dt_bias": TensorSpec((H,), "vector"),
            "norm": TensorSpec((self.value_dim,), "vector"), "o": TensorSpec((self.hidden, self.inner)),
        }

    def bind(self, tensors):
        H = self.num_heads
        stacked = [tensors[n] for n in ("q", "k", "v", "g", "b", "a")]
        pad = -(-2 * H // 8) * 8 - 2 * H          # zero rows, so that a projected row keeps its alignment
        if pad:
            stacked.append(tensors["a"].new_zeros((pad, self.hidden)))
        self.w_in = torch.cat(stacked, dim=0).contiguous()
        g_col = self.channels
        self.columns = (g_col, g_col + self.inner, g_col + self.inner + H)      # gate, write strength, step size
        self.conv_w = torch.cat([tensors["q_conv"], tensors["k_conv"], tensors["v_conv"]], dim=0).float().contiguous()
        self.a_log, self.dt_bias = tensors["a_log"].contiguous(), tensors["dt_bias"].contiguous()
        self.norm = tensors["norm"].contiguous()
        self.w_o = tensors["o"].contiguous()
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:
            prepare(self.w_o)

    def cache_need(self):
        return None

    @property
    def matrix_floats(self) -> int:
        return self.num_heads * self.key_dim * self.value_dim

    def state_need(self):
        return StateNeed((self.matrix_floats + self.channels * (self.taps - 1),), "float32", 0.0)

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        proj = k.linear(h, self.w_in)
        qkv = k.causal_conv(proj, 0, self.conv_w, None, "silu", ctx, cache.state, self.matrix_floats)
        out = k.delta_rule(qkv, proj, self.columns, self.a_log, self.dt_bias, self.norm, self.num_heads,
                           self.num_kv_heads, self.key_dim, self.value_dim, self.eps, ctx, cache.state)
        return k.pending_linear(out, self.w_o)
