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
    ("softmax", the default, or "sigmoid"), groups ((count, keep), with sigmoid scores) and route_scale."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.experts = int(params["experts"])
        self.top = int(params["top"])
        self.inter = int(params["expert_size"])
        if not 0 < self.top <= self.experts:
            raise ValueError(f"top {self.top} is not between 1 and the number of experts {self.experts}")
        self.score = str(params.get("score", "softmax"))
        if self.score not in ("softmax", "sigmoid"):
            raise ValueError(f"score must be 'softmax' or 'sigmoid', got {self.score!r}")
        groups = params.get("groups")
        self.groups = (int(groups[0]), int(groups[1])) if groups else None
        self.route_scale = float(params.get("route_scale", 1.0))
        if self.score == "softmax" and (self.groups is not None or self.route_scale != 1.0):
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
        specs = {"router": TensorSpec((self.experts, self.hidden), "float_matrix")}
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
        else:
            ids, weights = k.moe_route(h, self.router, self.top, score=self.score, groups=self.groups,
                                       scale=self.route_scale)
        shared = scale = None
        if self.shared_inter:
            shared = k.linear(k.gated_linear(h, self.w_shared_in), self.w_shared_down)
            if self.shared_gate:
                scale = k.linear(h, self.w_shared_scale)
        return k.moe_experts(h, self.w_gate_up, self.w_down, ids, weights, shared, scale)
