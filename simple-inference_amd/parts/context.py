"""What parts are built with and what a step hands to them."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Optional

import torch


@dataclass
class BuildEnv:
    """Where and with what a model's parts are built."""

    kernels: Any            # the object that launches the device kernels
    device: torch.device
    dtype: torch.dtype      # compute dtype: torch.bfloat16 or torch.float32
    max_positions: int      # absolute positions the engine will ever use (sizes rotation tables)
    _shared: Dict[Any, Any] = field(default_factory=dict)  # parts shared between layers, by spec key


@dataclass
class StepContext:
    """One batch of tokens: runs of consecutive tokens of several requests.

    Token ``t`` of the flat batch belongs to sequence ``seq_of_token[t]`` and stands
    at absolute position ``positions[t]``.  Sequence ``s`` brings tokens
    ``cu_q[s] .. cu_q[s+1]`` and holds ``kv_len[s]`` tokens once the step is done,
    so its first new token stands at ``kv_len[s] - (cu_q[s+1] - cu_q[s])``.
    All tensors are int32 on the device.
    """

    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    seq_of_token: torch.Tensor
    cu_q: torch.Tensor
    kv_len: torch.Tensor
    state_slots: torch.Tensor
    logit_rows: Optional[torch.Tensor]
    n_logit_rows: int
    max_q_len: int          # host-side facts for choosing kernels and grids
    max_kv_len: int
    kernels: Any = None
    block_tables: list = field(default_factory=list)  # one [n_seqs, width] table per cache group
    n_decode_seqs: int = 0  # sequences 0 .. n_decode_seqs-1 bring exactly one token (they are sorted first)
    q_lens: list = field(default_factory=list)  # host copy: tokens each sequence brings
    kv_bound: int = 0  # replayed graphs: an upper bound of kv_len that fixes grids (0: use max_kv_len)
    max_run_kv_len: int = 0  # the longest kv_len among the sequences that bring more than one token (0: not known)
    extra: dict = field(default_factory=dict)  # name -> int32 [n_tokens]: what the step's entries brought beside tokens


@dataclass
class LayerCache:
    """What one run of one layer may touch of the caches in this step."""

    k_pages: Optional[torch.Tensor] = None      # [pages, kv_heads, page_size, head_dim]
    v_pages: Optional[torch.Tensor] = None      # [pages, kv_heads, head_dim, page_size]
    block_table: Optional[torch.Tensor] = None  # [n_seqs, max_pages] int32, -1 where no page
    page_size: int = 0
    state: Optional[torch.Tensor] = None        # [slots, *state_shape]; row = ctx.state_slots[s]


class ResidualStream:
    """The hidden state between parts: a 32-bit residual and a delta not yet added.

    Parts produce deltas in the compute dtype; the sum over the residual is kept
    in float32 in both modes.  The add is fused into the norm that follows it.

    A part may leave its last product uncomputed (an object with ``compute()``, as the kernels'
    ``pending_linear`` returns): ``raw_delta`` shows it to a norm that can have it computed
    straight into the residual; ``delta`` computes it for everybody else.

    ``lowered`` is the residual in the compute dtype, if the kernel that last changed the residual left it (a
    sublayer that reads the residual itself, not a norm of it, takes it from there); setting a delta forgets it.

    ``gate`` belongs to the pending delta: ``(logits, bias)`` of an elementwise sigmoid gate that the delta passes
    on its way into the residual (``residual += delta * sigmoid(logits + bias)``).  It is set after the delta and
    forgotten with it; whoever adds the delta (a norm, ``settle``) reads it.  A delta may also be a
    ``BiasedDelta``: a result whose bias is still to be added, which the gated add takes in passing.

    ``post`` belongs to the pending delta too: a norm part that the delta passes on its way into the residual
    (``residual += post(delta)``, for blocks that norm a sublayer's result as well as its input).  It is set after
    the delta and forgotten with it; a norm that can apply it inside its own kernel does so, everybody else has it
    applied by ``settle`` (the norm's ``add_normed``).

    ``scale`` belongs to the pending delta as well: a constant factor on its way into the residual (``residual +=
    scale * delta``), set after the delta and forgotten with it.  A delta may be a ``ScaledSum``, several results
    with a factor each that nobody has added up yet; a sum that can take the terms one by one does.
    """

    __slots__ = ("residual", "raw_delta", "lowered", "gate", "post", "scale")

    def __init__(self, residual: torch.Tensor, delta: Optional[torch.Tensor] = None):
        self.residual = residual
        self.raw_delta = delta
        self.lowered = None
        self.gate = None
        self.post = None
        self.scale = None

    @property
    def delta(self):
        if hasattr(self.raw_delta, "compute"):
            self.raw_delta = self.raw_delta.compute()
        return self.raw_delta

    @delta.setter
    def delta(self, value):
        self.raw_delta = value
        self.gate = None
        self.post = None
        self.scale = None
        if value is not None:
            self.lowered = None

    def scaled_terms(self):
        """The pending delta as ``[(tensor, factor)]`` with the stream's own factor multiplied in."""
        raw, own = self.raw_delta, 1.0 if self.scale is None else float(self.scale)
        if isinstance(raw, ScaledSum):
            return [(y, f * own) for y, f in raw.values()]
        return [(self.delta, own)]

    def settle(self, kernels) -> torch.Tensor:
        """Adds what is pending into the residual (no norm follows) and returns the residual."""
        raw = self.raw_delta
        if raw is None:
            return self.residual
        if self.scale is not None or isinstance(raw, ScaledSum):
            if self.post is not None or self.gate is not None:
                raise NotImplementedError("a scaled delta passes neither a gate nor a norm of its own")
            kernels.add_rmsnorm(self.residual, None, None, 0.0, self.residual.dtype, terms=self.scaled_terms())
            self.delta = None
            return self.residual
        if self.post is not None:
            post = self.post
            post.add_normed(self, raw)
            self.delta = None
            return self.residual
        bias = None
        if isinstance(raw, BiasedDelta):
            raw, bias = raw.value(), raw.bias
        elif hasattr(raw, "compute"):
            raw = raw.compute()
        gate, gate_bias = self.gate if self.gate is not None else (None, None)
        kernels.gated_add(self.residual, raw, gate, gate_bias, bias)
        self.delta = None
        return self.residual


class ScaledSum:
    """A sublayer's result that is a sum of several, each with a constant factor: ``sum_i factor_i * y_i``.  A sum
    into the residual that can take the terms one by one reads ``terms``; everybody else gets the tensor from
    ``compute()``."""

    __slots__ = ("terms", "kernels")

    def __init__(self, terms, kernels):
        self.terms, self.kernels = list(terms), kernels

    def values(self):
        """``[(tensor, factor)]``, products that were left pending computed."""
        self.terms = [(y.compute() if hasattr(y, "compute") else y, f) for y, f in self.terms]
        return self.terms

    def compute(self):
        return self.kernels.scaled_sum(self.values())


class BiasedDelta:
    """A sublayer's result whose bias is not added yet: ``y + bias``.  A sum that can take the bias in passing reads
    ``value()`` and ``bias``; everybody else gets the tensor from ``compute()``."""

    __slots__ = ("y", "bias", "kernels")

    def __init__(self, y, bias, kernels):
        self.y, self.bias, self.kernels = y, bias, kernels

    def value(self):
        if hasattr(self.y, "compute"):
            self.y = self.y.compute()
        return self.y

    def compute(self):
        return self.kernels.add_bias(self.value(), self.bias)
