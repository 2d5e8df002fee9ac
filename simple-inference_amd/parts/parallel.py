"""Several mixers side by side: each reads the same input, and the layer's result is their weighted sum.

    y = sum_b scale_b * mixer_b(h)

``branches`` names the mixers (``{name: {"kind", "params", "scale"}}``); a branch's tensors are this part's tensors
``<name>.<the branch's own name>``.  The run of the layer still owns one set of pages and one state row: at most one
branch may keep pages and at most one a state, and each finds its own in the ``LayerCache`` the layer is handed.  The
sum is not taken here: the terms go on with their factors (``ScaledSum``), and whoever adds the result into the
residual adds them one by one.
"""

from __future__ import annotations

from .context import ScaledSum
from .registry import MIXERS, register_mixer


@register_mixer("parallel")
class ParallelMixers:
    """params: branches ({name: {"kind": mixer kind, "params": its params, "scale": its factor (default 1)}})."""

    def __init__(self, params, env):
        branches = params["branches"]
        if not branches:
            raise ValueError("mixers side by side need at least one branch")
        self.branches = [(str(name), MIXERS.get(b["kind"])(b["params"], env), float(b.get("scale", 1.0)))
                         for name, b in branches.items()]
        if sum(m.cache_need() is not None for _, m, _ in self.branches) > 1:
            raise ValueError("at most one of the mixers side by side keeps pages")
        if sum(m.state_need() is not None for _, m, _ in self.branches) > 1:
            raise ValueError("at most one of the mixers side by side keeps a state")
        if any(getattr(m, "kv_from_layer", None) is not None for _, m, _ in self.branches):
            raise ValueError("a mixer beside another reads no other layer's pages")
        self.env = env

    takes_scaled_rows = False

    def weight_specs(self):
        return {f"{name}.{local}": spec for name, m, _ in self.branches for local, spec in m.weight_specs().items()}

    def bind(self, tensors):
        for name, m, _ in self.branches:
            m.bind({local: tensors[f"{name}.{local}"] for local in m.weight_specs()})

    def cache_need(self):
        return next((m.cache_need() for _, m, _ in self.branches if m.cache_need() is not None), None)

    def state_need(self):
        return next((m.state_need() for _, m, _ in self.branches if m.state_need() is not None), None)

    def forward(self, h, ctx, cache):
        return ScaledSum([(m.forward(h, ctx, cache), scale) for _, m, scale in self.branches], self.env.kernels)
