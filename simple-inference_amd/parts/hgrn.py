"""Gated linear recurrence whose forget gate also decides what is written (the HGRN-2 form).

For a token with input ``h`` (``H`` heads, gate width ``D``, value width ``Dv``):

    q = silu(W_q h)                                   [H, D]
    v = W_v h                                         [H, Dv]
    f = l + (1 - l) * sigmoid(W_f h + b)              [H, D]   a forget gate per channel, never below ``l``
    S_h <- diag(f_h) S_h + (1 - f_h) v_h^T            S_h [D, Dv]; what is forgotten makes room for what is written
    o_h = S_h^T q_h
    y   = W_o concat_h(o_h / rms(o_h) * w)            w [Dv], shared by the heads

A request's state is all zeros before its first token, float32 in both modes, and kept in the request's state slot.
The three input projections are one stacked matrix ``[q | f | v]``; gates, the state and the norm are float32.
"""

from __future__ import annotations

import torch

from .plan import StateNeed, TensorSpec
from .registry import register_mixer


@register_mixer("hgrn2")
class Hgrn2Mixer:
    """params: hidden_size, num_heads, key_dim, value_dim, norm_eps."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.key_dim = int(params["key_dim"])
        self.value_dim = int(params["value_dim"])
        self.eps = float(params["norm_eps"])
        check = getattr(env.kernels, "check_recurrent_geometry", None)
        if check is not None:
            check(self.key_dim, self.value_dim)
        self.env = env
        self.w_in = self.w_o = self.f_bias = self.lower = self.norm = None

    takes_scaled_rows = False

    def weight_specs(self):
        qk, v = self.num_heads * self.key_dim, self.num_heads * self.value_dim
        return {"q": TensorSpec((qk, self.hidden)), "f": TensorSpec((qk, self.hidden)), "v": TensorSpec((v, self.hidden)),
                "f_bias": TensorSpec((qk,), "vector"), "lower": TensorSpec((qk,), "vector"),
                "norm": TensorSpec((self.value_dim,), "vector"), "o": TensorSpec((self.hidden, v))}

    def bind(self, tensors):
        self.w_in = torch.cat([tensors["q"], tensors["f"], tensors["v"]], dim=0).contiguous()
        self.w_o = tensors["o"].contiguous()
        self.f_bias, self.lower, self.norm = (tensors[n].contiguous() for n in ("f_bias", "lower", "norm"))
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:
            prepare(self.w_o)

    def cache_need(self):
        return None

    def state_need(self):
        return StateNeed((self.num_heads, self.key_dim, self.value_dim), "float32", 0.0)

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        proj = k.linear(h, self.w_in)
        y = k.hgrn2_scan(proj, self.f_bias, self.lower, self.norm, self.num_heads, self.key_dim, self.value_dim,
                         self.eps, ctx, cache.state)
        return k.pending_linear(y, self.w_o)
