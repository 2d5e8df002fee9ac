"""State-space mixer with a scalar decay per head (the Mamba-2 form) behind a short causal convolution.

For a token with input ``h`` (``H`` heads of width ``P``, state size ``N``, ``G`` groups of heads that share their
``B`` and ``C``; ``inner = H P``):

    [z | x | B | C | dt] = W_in h                  z, x [inner]; B, C [G N]; dt [H]
    [x | B | C] <- silu(conv(x | B | C))           per channel, over the token and the ``taps - 1`` before it
    dt_h  = softplus(dt_h + dt_bias_h)
    S_h  <- exp(-exp(A_log_h) dt_h) S_h + dt_h B_g x_h^T        S_h [N, P], g = h // (H / G)
    y_h   = S_h^T C_g + D_h x_h
    y     = W_o (rms_groups(y * silu(z)) * w)      the root mean square over each of ``norm_groups`` equal parts

A request's row of state holds, in float32, the ``H`` matrices ``S_h`` and behind them the last ``taps - 1`` inputs of
the convolution (zeros before the first token); the cache manager hands it in as ``cache.state``.  The step sizes,
decays, the state and the norm are float32 in both modes.
"""

from __future__ import annotations

from .plan import StateNeed, TensorSpec
from .registry import register_mixer


@register_mixer("mamba2")
class Mamba2Mixer:
    """params: hidden_size, num_heads, head_dim, state_size, groups, conv_taps, norm_groups, norm_eps."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.head_dim = int(params["head_dim"])
        self.state_size = int(params["state_size"])
        self.groups = int(params["groups"])
        self.taps = int(params["conv_taps"])
        self.norm_groups = int(params["norm_groups"])
        self.eps = float(params["norm_eps"])
        self.inner = self.num_heads * self.head_dim
        if self.num_heads % self.groups or self.inner % self.norm_groups or self.taps < 1:
            raise ValueError(f"{self.num_heads} heads of {self.head_dim} do not split into {self.groups} groups and "
                             f"{self.norm_groups} norm parts (or the convolution has no tap)")
        self.channels = self.inner + 2 * self.groups * self.state_size
        check = getattr(env.kernels, "check_recurrent_geometry", None)
        if check is not None:
            check(self.state_size, self.head_dim)
        self.env = env
        self.w_in = self.w_o = self.conv_w = self.conv_b = self.dt_bias = self.a_log = self.d = self.norm = None

    takes_scaled_rows = False

    def weight_specs(self):
        return {
            "in": TensorSpec((2 * self.inner + 2 * self.groups * self.state_size + self.num_heads, self.hidden)),
            "conv": TensorSpec((self.channels, self.taps), "vector"), "conv_bias": TensorSpec((self.channels,), "vector"),
            "dt_bias": TensorSpec((self.num_heads,), "vector"), "a_log": TensorSpec((self.num_heads,), "vector"),
            "d": TensorSpec((self.num_heads,), "vector"), "norm": TensorSpec((self.inner,), "vector"),
            "o": TensorSpec((self.hidden, self.inner)),
        }

    def bind(self, tensors):
        self.w_in, self.w_o = tensors["in"].contiguous(), tensors["o"].contiguous()
        self.conv_w, self.conv_b = tensors["conv"].contiguous(), tensors["conv_bias"].contiguous()
        self.dt_bias, self.a_log, self.d = (tensors[n].contiguous() for n in ("dt_bias", "a_log", "d"))
        self.norm = tensors["norm"].contiguous()
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:
            prepare(self.w_o)

    def cache_need(self):
        return None

    @property
    def matrix_floats(self) -> int:
        return self.num_heads * self.state_size * self.head_dim

    def state_need(self):
        return StateNeed((self.matrix_floats + self.channels * (self.taps - 1),), "float32", 0.0)

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        proj = k.linear(h, self.w_in)
        xbc = k.causal_conv(proj, self.inner, self.conv_w, self.conv_b, "silu", ctx, cache.state, self.matrix_floats)
        y = k.ssd_scan(proj, xbc, self.dt_bias, self.a_log, self.d, self.norm, self.num_heads, self.head_dim,
                       self.state_size, self.groups, self.norm_groups, self.eps, ctx, cache.state)
        return k.pending_linear(y, self.w_o)
