"""Linear attention with a constant decay per head: a mixer whose memory is a matrix state per head.

For a token with input ``h`` (``H`` heads, key width ``D``, value width ``Dv``):

    q, k, v = silu(Wq h), silu(Wk h), silu(Wv h)
    S <- decay_i S + k v^T;  o = S^T q                      per head i, S [D, Dv]; the state already holds this token
    y = Wo (rms(concat_i(o_i)) * w * sigmoid(Wg h))         the root mean square over all heads together, w [H Dv]

A request's state is all zeros before its first token, float32 in both modes, and kept in the request's state slot;
the cache manager hands it in as ``cache.state``.  The four input projections are one stacked matrix.
"""

from __future__ import annotations

import torch

from .plan import StateNeed, TensorSpec
from .registry import register_mixer


@register_mixer("decay_attention")
class DecayAttention:
    """params: hidden_size, num_heads, key_dim, value_dim, decay (one number a head), norm_eps."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.key_dim = int(params["key_dim"])
        self.value_dim = int(params["value_dim"])
        self.decay = [float(x) for x in params["decay"]]
        if len(self.decay) != self.num_heads:
            raise ValueError(f"{len(self.decay)} decays for {self.num_heads} heads")
        self.eps = float(params["norm_eps"])
        check = getattr(env.kernels, "check_recurrent_geometry", None)
        if check is not None:
            check(self.key_dim, self.value_dim)
        self.env = env
        self.w_in = self.w_o = self.norm = self.decays = None

    takes_scaled_rows = False

    def weight_specs(self):
        qk, v = self.num_heads * self.key_dim, self.num_heads * self.value_dim
        return {"q": TensorSpec((qk, self.hidden)), "k": TensorSpec((qk, self.hidden)), "v": TensorSpec((v, self.hidden)),
                "g": TensorSpec((v, self.hidden)), "norm": TensorSpec((v,), "vector"), "o": TensorSpec((self.hidden, v))}

    def bind(self, tensors):
        self.w_in = torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0).contiguous()
        self.norm = tensors["norm"].contiguous()
        self.w_o = tensors["o"].contiguous()
        self.decays = torch.tensor(self.decay, dtype=torch.float32, device=self.w_o.device)
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
        out = k.decay_attention(proj, self.decays, self.norm, self.num_heads, self.key_dim, self.value_dim, self.eps,
                                ctx, cache.state)
        return k.pending_linear(out, self.w_o)
