"""Mixture of experts: every token runs ``top`` of ``experts`` small gated feed-forwards.

    z = R h                                   router logits, float32 (``h`` as the compute dtype holds it)
    chosen: the ``top`` largest logits (ties: the lower index); weights: softmax over the chosen logits alone
    y = sum_k weight_k * W2_e (silu(Wg_e h) * (Wu_e h))        e = the k-th chosen expert; experts have no biases
    y += sigmoid(s . h) * Ws2 (silu(Wsg h) * (Wsu h))          a shared expert every token runs, if the layer has one,
                                                              scaled by a scalar of the token's own

Another way to choose and weigh, by parameters (``score: "sigmoid"``): the scores are ``s = sigmoid(z)``; with
``groups: (count, keep)`` the experts form ``count`` equal groups of neighbours, a group's score is the sum of its two
largest ``s``, and only experts of the ``keep`` best groups can be chosen; the ``top`` largest ``s`` among those are
chosen and weighted by ``s / (sum of the chosen s + 1e-20) * route_scale``.

Further forms, each a parameter: ``score: "softmax_all"`` takes the softmax over all router outputs as the scores,
chooses by ``s + correction`` (``correction: True``: a vector of the checkpoint, added for the choice only) and weighs
the chosen by ``s / (sum of the chosen s + 1e-20)``; ``identity_experts: n`` gives the router ``n`` further outputs
behind the experts' own, experts without tensors that return their input; ``activation: "clamped"`` (with ``limit``,
and ``shared_limit`` for the shared expert) makes an expert ``W2 (g * sigmoid(1.702 g) * (u + 1))`` with ``g = min(Wg h,
limit)`` and ``u = clamp(Wu h, -limit, limit)``.

The experts' matrices are stacked at load (``[E, 2 ff, hidden]`` with the gate rows first, ``[E, hidden, ff]``); the
shared expert's gate and up rows and its scalar gate are one stacked matrix.  Routing happens on the device: no
count or index comes back to the host, so a step's launches do not depend on who was routed where.
"""

from __future__ import annotations

import torch

from .plan import TensorSpec
from .registry import register_feed_forward


@register_feed_forward("moe")
class MixtureOfExperts:
    """params: hidden_size, experts, top, expert_size, and optionally shared_size (a shared expert of that
    intermediate size), shared_gate (default True: the shared expert's output is scaled by a sigmoid), score
    ("softmax", the default, "sigmoid" or "softmax_all"), groups ((count, keep), with sigmoid scores), route_scale,
    correction, identity_experts, activation ("swiglu", the default, or "clamped"), limit and shared_limit."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.experts = int(params["experts"])
        self.top = int(params["top"])
        self.inter = int(params["expert_size"])
        if not 0 < self.top <= self.experts + int(params.get("identity_experts", 0)):
            raise ValueError(f"top {self.top} is not between 1 and the number of experts {self.experts}")
        self.score = str(params.get("score", "softmax"))
        if self.score not in ("softmax", "sigmoid", "softmax_all"):
            raise ValueError(f"score must be 'softmax', 'sigmoid' or 'softmax_all', got {self.score!r}")
        self.identity = int(params.get("identity_experts", 0))
        self.correction = bool(params.get("correction", False))
        if self.identity < 0 or (self.correction and self.score != "softmax_all"):
            raise ValueError("a correction of the choice comes with scores over all router outputs")
        self.activation = str(params.get("activation", "swiglu"))
        if self.activation not in ("swiglu", "clamped"):
            raise ValueError(f"activation must be 'swiglu' or 'clamped', got {self.activation!r}")
        self.glu = self.shared_glu = None
        if self.activation == "clamped":
            self.glu = ("clamped", float(params["limit"]))
            if params.get("shared_size"):
                self.shared_glu = ("clamped", float(params.get("shared_limit", params["limit"])))
        groups = params.get("groups")
        self.groups = (int(groups[0]), int(groups[1])) if groups else None
        self.route_scale = float(params.get("route_scale", 1.0))
        if self.score != "sigmoid" and (self.groups is not None or self.route_scale != 1.0):
            raise ValueError("expert groups and a scale on the weights come with sigmoid scores")
        if self.groups is not None:
            count, keep = self.groups
            if count <= 0 or self.experts % count or not 0 < keep <= count or self.top > self.experts // count * keep:
                raise ValueError(f"{self.experts} experts in {count} groups of which {keep} are kept cannot give {self.top}")
        shared = params.get("shared_size")
        self.shared_inter = int(shared) if shared else 0
        self.shared_gate = bool(params.get("shared_gate", True)) and self.shared_inter > 0
        self.env = env
        self.router = self.w_gate_up = self.w_down = self.w_shared_in = self.w_shared_down = None

    def weight_specs(self):
        specs = {"router": TensorSpec((self.experts + self.identity, self.hidden), "float_matrix")}
        if self.correction:
            specs["correction"] = TensorSpec((self.experts + self.identity,), "vector")
        for e in range(self.experts):
            specs[f"gate{e}"] = TensorSpec((self.inter, self.hidden))
            specs[f"up{e}"] = TensorSpec((self.inter, self.hidden))
            specs[f"down{e}"] = TensorSpec((self.hidden, self.inter))
        if self.shared_inter:
            specs["shared_gate"] = TensorSpec((self.shared_inter, self.hidden))
            specs["shared_up"] = TensorSpec((self.shared_inter, self.hidden))
            specs["shared_down"] = TensorSpec((self.hidden, self.shared_inter))
            if self.shared_gate:
                specs["shared_scale"] = TensorSpec((1, self.hidden))
        return specs

    def bind(self, tensors):
        E = range(self.experts)
        self.router = tensors["router"].contiguous()
        self.choice_bias = tensors["correction"].contiguous() if self.correction else None
        self.w_gate_up = torch.stack([torch.cat([tensors[f"gate{e}"], tensors[f"up{e}"]], dim=0) for e in E]).contiguous()
        self.w_down = torch.stack([tensors[f"down{e}"] for e in E]).contiguous()
        if self.shared_inter:
            self.w_shared_in = torch.cat([tensors["shared_gate"], tensors["shared_up"]], dim=0).contiguous()
            self.w_shared_down = tensors["shared_down"].contiguous()
            self.w_shared_scale = tensors["shared_scale"].contiguous() if self.shared_gate else None

    def forward(self, h, ctx):
        k = self.env.kernels
        if self.score == "softmax":
            ids, weights = k.moe_route(h, self.router, self.top)
        elif self.score == "softmax_all":
            ids, weights = k.moe_route(h, self.router, self.top, score=self.score, correction=self.choice_bias)
        else:
            ids, weights = k.moe_route(h, self.router, self.top, score=self.score, groups=self.groups,
                                       scale=self.route_scale)
        shared = scale = None
        if self.shared_inter:
            inner = k.gated_linear(h, self.w_shared_in) if self.shared_glu is None else \
                k.gated_linear(h, self.w_shared_in, activation=self.shared_glu)
            shared = k.linear(inner, self.w_shared_down)
            if self.shared_gate:
                scale = k.linear(h, self.w_shared_scale)
        if self.glu is None and not self.identity:
            return k.moe_experts(h, self.w_gate_up, self.w_down, ids, weights, shared, scale)
        return k.moe_experts(h, self.w_gate_up, self.w_down, ids, weights, shared, scale, activation=self.glu,
                             identity=self.identity)
