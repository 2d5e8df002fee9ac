"""Root-mean-square norm (reference: ``ops/rmsnorm.py:41-46``, ``kernels/rmsnorm_kernel.py:105-113``).

``y = x * rsqrt(mean(x^2) + eps) * w`` with the statistic, the normalisation and
the gain in float32 and one rounding to the compute dtype, as the reference's
fused kernel does.  The add of the pending residual delta is fused in front.

The same norm can sit behind a sublayer instead of in front of it (``add_normed``): the residual then grows by
the norm of what the sublayer returned, ``x += y * rsqrt(mean(y^2) + eps) * w``, statistic and sum in float32.
"""

from __future__ import annotations

from .context import BiasedDelta, ScaledSum
from .plan import TensorSpec
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm:
    """params: size, eps, and optionally unit_offset (default False): the stored vector is the gain's distance from
    one, ``y = x * rsqrt(mean(x^2) + eps) * (1 + w)``; the one is added once, in float32, when the vector is bound."""

    def __init__(self, params, env):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.unit_offset = bool(params.get("unit_offset", False))
        self.env = env
        self.weight = None

    def weight_specs(self):
        return {"weight": TensorSpec((self.size,), "vector")}

    def bind(self, tensors):
        self.weight = tensors["weight"]
        if self.unit_offset:
            self.weight = (self.weight.float() + 1.0).contiguous()

    gives_scaled_rows = True

    def plain_form(self):
        """What this norm is, as plain data, for kernels that can run a whole block in one call (None for a
        subclass with a forward of its own: it is no longer what this form describes)."""
        if type(self).forward is not RMSNorm.forward:
            return None
        # (a gain stored as its distance from one is an ordinary gain once it is bound)
        return {"kind": "rmsnorm", "weight": self.weight, "eps": self.eps, "size": self.size}

    def add_normed(self, stream, y):
        """``stream.residual += norm(y)``, in one kernel; returns the new residual in the compute dtype (the input
        of the next sublayer), which the stream also keeps as ``lowered``."""
        if hasattr(y, "compute"):     # a product left pending for a norm in front of the next sublayer: not this one
            y = y.compute()
        out = self.env.kernels.norm_add(stream.residual, y, self.weight, self.eps, self.env.dtype)
        stream.lowered = out
        return out

    def forward(self, stream, rows=None, scaled_ok=False):
        """Adds ``stream.delta`` into ``stream.residual`` and returns the normed rows.

        With ``rows`` (int32 indices) only those rows are computed and the residual
        is left as it was: that form ends a forward pass.

        ``scaled_ok``: the caller also takes the rows undivided by their root mean square (the kernels'
        ``ScaledRows``).  Then a delta that is a product not yet computed is computed into the residual by the
        product's own kernel, and the product after the norm divides: the norm has no kernel of its own.
        """
        k = self.env.kernels
        if stream.post is not None:     # the pending result passes a norm of its own first: that norm's kernel adds it
            stream.settle(k)
        if stream.gate is not None or isinstance(stream.raw_delta, BiasedDelta):
            return self._gated(stream, rows)
        if stream.scale is not None or isinstance(stream.raw_delta, ScaledSum):
            # the delta, or its several terms, with a constant factor each: all added inside the norm's kernel
            out = k.add_rmsnorm(stream.residual, None, self.weight, self.eps, self.env.dtype, rows,
                                terms=stream.scaled_terms())
            if rows is None:
                stream.delta = None
            return out
        if scaled_ok and rows is None and hasattr(stream.raw_delta, "compute") and hasattr(k, "linear_into_residual"):
            out = k.linear_into_residual(stream.raw_delta, stream.residual, self.weight, self.eps)
            stream.delta = None
            return out
        out = self.env.kernels.add_rmsnorm(
            stream.residual, stream.delta, self.weight, self.eps, self.env.dtype, rows)
        if rows is None:
            stream.delta = None
        return out

    def _gated(self, stream, rows):
        """The same with a delta that passes an elementwise sigmoid gate (``stream.gate``) and may still lack its
        bias: ``residual += (delta + bias) * sigmoid(gate logits + gate bias)``, all inside the norm's kernel."""
        raw, bias = stream.raw_delta, None
        if isinstance(raw, BiasedDelta):
            raw, bias = raw.value(), raw.bias
        elif hasattr(raw, "compute"):
            raw = raw.compute()
        logits, gate_bias = stream.gate if stream.gate is not None else (None, None)
        if logits is None:      # a bias alone: nothing to fuse it into
            raw, bias = self.env.kernels.add_bias(raw, bias), None
            out = self.env.kernels.add_rmsnorm(stream.residual, raw, self.weight, self.eps, self.env.dtype, rows)
        else:
            out = self.env.kernels.add_rmsnorm(stream.residual, raw, self.weight, self.eps, self.env.dtype, rows,
                                               gate=logits, gate_bias=gate_bias, delta_bias=bias)
        if rows is None:
            stream.delta = None
        return out


@register_norm("dyt")
class DynamicTanh:
    """A norm without a statistic: ``y = tanh(a * x) * w + b`` with a learned scalar ``a``, elementwise, in float32
    with one rounding.  With ``scaled`` it has a second vector ``s`` and gives ``(tanh(a * x) * w + b) * s`` (a layer
    scale on a sublayer's normed result).

    params: size, and optionally scaled (default False).

    In front of a sublayer (``forward``) it first adds what is pending into the float32 residual; a pending result
    that passes a norm of this kind on its way (``stream.post``) is normed and added in the same kernel.  Behind a
    sublayer (``add_normed``) it adds its own output into the residual.
    """

    def __init__(self, params, env):
        self.size = int(params["size"])
        self.scaled = bool(params.get("scaled", False))
        self.env = env
        self.weight = self.bias = self.alpha = self.scale = None

    def weight_specs(self):
        specs = {"weight": TensorSpec((self.size,), "vector"), "bias": TensorSpec((self.size,), "vector"),
                 "alpha": TensorSpec((), "vector")}
        if self.scaled:
            specs["scale"] = TensorSpec((self.size,), "vector")
        return specs

    def bind(self, tensors):
        self.weight, self.bias = tensors["weight"].contiguous(), tensors["bias"].contiguous()
        self.alpha = tensors["alpha"].reshape(1).contiguous()
        self.scale = tensors["scale"].contiguous() if self.scaled else None

    def terms(self):
        """(weight, bias, alpha, scale or None): what the kernels need of this norm."""
        return (self.weight, self.bias, self.alpha, self.scale)

    def add_normed(self, stream, y):
        """``stream.residual += norm(y)``; returns nothing (no sublayer reads the un-normed residual)."""
        if hasattr(y, "compute"):
            y = y.compute()
        self.env.kernels.dyt_norm(stream.residual, y, self.terms(), None, self.env.dtype)

    def forward(self, stream, rows=None, scaled_ok=False):
        """Adds what is pending into ``stream.residual`` and returns the normed rows; with ``rows`` (int32 indices)
        only those rows are computed and the residual is left as it was."""
        k = self.env.kernels
        post = stream.post
        if stream.gate is not None or isinstance(stream.raw_delta, BiasedDelta) or (
                post is not None and not isinstance(post, DynamicTanh)):
            stream.settle(k)
            post = None
        delta = stream.delta
        out = k.dyt_norm(stream.residual, delta, post.terms() if (post is not None and delta is not None) else None,
                         self.terms(), self.env.dtype, rows)
        if rows is None:
            stream.delta = None
        return out
