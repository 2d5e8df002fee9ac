"""The arrangement of parts in a layer.

Pre-norm (reference: ``model/block.py:135-147``):
``x += mixer(norm1(x))``; ``x += feed_forward(norm2(x))``.  Each add is carried
as the stream's pending delta and summed into the float32 residual by the norm
that follows (the next layer's, or the model's last norm).  With ``residual_scale`` (a parameter of the block, from
the layer's ``block_params``) every sublayer's result is multiplied by that constant on its way into the residual
(``stream.scale``); a pre-norm layer may have no feed-forward.

Output-norm: ``x += norm1(mixer(x))``; ``x += norm2(feed_forward(x))``.  Mixer and feed-forward take the
un-normed stream as input (rounded to the compute dtype), and each norm is applied to its sublayer's result; the kernel that adds the normed
output into the float32 residual also leaves the rounded residual for the next sublayer.  A layer of this kind
may have no feed-forward.

Gated pre-norm: ``h = norm1(x); x += sigmoid(G1 h + g1) * mixer(h)``, then the same with the feed-forward if the
layer has one.  Each sublayer's result passes an elementwise gate computed from the sublayer's own input; the gate's
logits travel with the pending delta (``stream.gate``) and the sigmoid, the product and the sum happen inside the
kernel of the norm that follows.
"""

from __future__ import annotations

from .registry import register_block


@register_block("prenorm")
class PreNormBlock:
    def __init__(self, mixer, feed_forward=None, mixer_norm=None, feed_forward_norm=None, residual_scale=None):
        if mixer_norm is None or (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a pre-norm block has a mixer with its norm, and a feed-forward with its norm or neither")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm
        self.residual_scale = None if residual_scale is None or float(residual_scale) == 1.0 else float(residual_scale)
        self.plain_forms = None   # kept by kernels that run the block in one call: what they made of the parts

    def plain_form(self):
        """What this block is, as plain data, for kernels that can make all of its launches in one call: its kind
        (the order in which the parts run is this file's affair: the docstring above) and what each part says it is
        (its own ``plain_form``; None for a part that has none, and such a block goes part by part)."""
        if type(self).forward is not PreNormBlock.forward or self.residual_scale is not None or self.feed_forward is None:
            return None
        form = lambda part: getattr(part, "plain_form", lambda: None)()
        return {"kind": "prenorm", "mixer_norm": form(self.mixer_norm), "mixer": form(self.mixer),
                "feed_forward_norm": form(self.feed_forward_norm), "feed_forward": form(self.feed_forward)}

    def forward(self, stream, ctx, cache):
        # Kernels that can make all of a block's launches in one call are shown the block (they look at what it and
        # its parts say they are, ``plain_form``, and take it or leave it); else part by part.
        whole = getattr(ctx.kernels, "prenorm_block", None)
        if whole is not None and whole(self, stream, ctx, cache):
            return
        h = _normed(self.mixer_norm, self.mixer, stream)
        stream.delta = self.mixer.forward(h, ctx, cache)
        stream.scale = self.residual_scale
        if self.feed_forward is None:
            return
        h = _normed(self.feed_forward_norm, self.feed_forward, stream)
        stream.delta = self.feed_forward.forward(h, ctx)
        stream.scale = self.residual_scale


def _normed(norm, consumer, stream):
    """The norm's rows for ``consumer``.  A norm that ``gives_scaled_rows`` may leave the division by the root mean
    square to a consumer that ``takes_scaled_rows`` (one that hands its input to the kernels' products only)."""
    if getattr(norm, "gives_scaled_rows", False) and getattr(consumer, "takes_scaled_rows", False):
        return norm.forward(stream, scaled_ok=True)
    return norm.forward(stream)


@register_block("output_norm")
class OutputNormBlock:
    def __init__(self, mixer, mixer_norm, feed_forward=None, feed_forward_norm=None):
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("an output-norm block has a feed-forward and its norm, or neither")
        self.mixer = mixer
        self.mixer_norm = mixer_norm
        self.feed_forward = feed_forward
        self.feed_forward_norm = feed_forward_norm

    def forward(self, stream, ctx, cache):
        if stream.raw_delta is not None:
            raise NotImplementedError("an output-norm block cannot follow a block that leaves its sum to the next norm")
        x = stream.lowered
        if x is None:    # the first block of a step, or the residual is already of the compute dtype
            x = stream.residual
            if x.dtype != self.mixer_norm.env.dtype:
                x = ctx.kernels.cast(x, self.mixer_norm.env.dtype)
        x = self.mixer_norm.add_normed(stream, self.mixer.forward(x, ctx, cache))
        if self.feed_forward is not None:
            self.feed_forward_norm.add_normed(stream, self.feed_forward.forward(x, ctx))


@register_block("gated_prenorm")
class GatedPreNormBlock:
    def __init__(self, mixer, mixer_norm, mixer_gate, feed_forward=None, feed_forward_norm=None, feed_forward_gate=None):
        if not ((feed_forward is None) == (feed_forward_norm is None) == (feed_forward_gate is None)):
            raise ValueError("a gated pre-norm block has a feed-forward with its norm and its gate, or none of them")
        self.mixer, self.mixer_norm, self.mixer_gate = mixer, mixer_norm, mixer_gate
        self.feed_forward, self.feed_forward_norm, self.feed_forward_gate = feed_forward, feed_forward_norm, feed_forward_gate

    def forward(self, stream, ctx, cache):
        h = self.mixer_norm.forward(stream)
        logits = self.mixer_gate.logits(h)     # before the mixer: its input is the same rows
        stream.delta = self.mixer.forward(h, ctx, cache)
        stream.gate = (logits, self.mixer_gate.bias)
        if self.feed_forward is not None:
            h = self.feed_forward_norm.forward(stream)
            logits = self.feed_forward_gate.logits(h)
            stream.delta = self.feed_forward.forward(h, ctx)
            stream.gate = (logits, self.feed_forward_gate.bias)


@register_block("sandwich")
class SandwichBlock:
    """``x += post1(mixer(norm1(x)))``, then ``x += post2(feed_forward(norm2(x)))`` if the layer has a feed-forward:
    a norm in front of each sublayer and another on its result.  The result travels as the stream's pending delta
    with its norm (``stream.post``); the norm in front of the next sublayer (or the model's last) norms it, adds it
    into the float32 residual and norms the sum for its own sublayer, in one kernel where both norms are of a kind
    whose kernel can (``dyt``)."""

    def __init__(self, mixer, mixer_norm, mixer_post_norm, feed_forward=None, feed_forward_norm=None,
                 feed_forward_post_norm=None):
        if not ((feed_forward is None) == (feed_forward_norm is None) == (feed_forward_post_norm is None)):
            raise ValueError("a sandwich block has a feed-forward with both of its norms, or none of them")
        self.mixer, self.mixer_norm, self.mixer_post_norm = mixer, mixer_norm, mixer_post_norm
        self.feed_forward, self.feed_forward_norm = feed_forward, feed_forward_norm
        self.feed_forward_post_norm = feed_forward_post_norm

    def forward(self, stream, ctx, cache):
        h = self.mixer_norm.forward(stream)
        stream.delta = self.mixer.forward(h, ctx, cache)
        stream.post = self.mixer_post_norm
        if self.feed_forward is not None:
            h = self.feed_forward_norm.forward(stream)
            stream.delta = self.feed_forward.forward(h, ctx)
            stream.post = self.feed_forward_post_norm
