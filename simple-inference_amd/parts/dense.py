"""Dense feed-forward without a gate: ``y = act(h Wu^T) Wd^T``.

``act`` is named by the ``activation`` parameter: ``relu2`` is the square of ``max(z, 0)``, ``gelu_tanh`` is
``0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))``, ``gelu`` is ``0.5 z (1 + erf(z / sqrt(2)))``.  The activation is computed in float32 on the product and
rounded once; for few rows it is part of the product's own kernel.
"""

from __future__ import annotations

from .plan import TensorSpec
from .registry import register_feed_forward

ACTIVATIONS = ("relu2", "gelu_tanh", "gelu")


@register_feed_forward("dense")
class DenseFeedForward:
    """params: hidden_size, intermediate_size, activation."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.activation = str(params["activation"])
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"activation {self.activation!r} is not one of {', '.join(ACTIVATIONS)}")
        self.env = env
        self.w_up = None
        self.w_down = None

    def weight_specs(self):
        return {"up": TensorSpec((self.inter, self.hidden)), "down": TensorSpec((self.hidden, self.inter))}

    def bind(self, tensors):
        self.w_up = tensors["up"].contiguous()
        self.w_down = tensors["down"].contiguous()
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:   # the kernels may keep a copy of their own of a weight for their few-row product
            prepare(self.w_down)

    def forward(self, h, ctx):
        k = self.env.kernels
        return k.linear(k.activated_linear(h, self.w_up, self.activation), self.w_down)
