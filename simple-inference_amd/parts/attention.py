"""Grouped-query attention over the paged cache (reference: ``ops/attention.py:70-228``,
serving form ``serving/paged_decoder.py:133-185``).

Order inside the mixer, as in the reference's serving path: project q, k, v (no
bias) -> rotate q and k by absolute position -> write k (rotated) and v into
the pages -> attend over the pages, the tokens just written included -> output
projection.  Query head ``h`` reads key/value head ``h // (Hq / Hkv)`` (reference:
``kernels/attention_kernel.py:108-251``).  Scores are ``(q . k) * scale`` with the
scale applied after the dot; key ``j`` is visible to a query at position ``p`` iff
``j <= p`` and, with a window ``w``, ``j > p - w``.

The three projections are stacked into one ``[(Hq + 2 Hkv) D, H]`` matrix at load.
A mixer whose ``kv_from_layer`` is set projects only q and reads the pages that
the named layer's latest run wrote.

Further forms, each switched on by a parameter of its own and free to combine:

* ``value_head_dim``: value heads of another width ``Dv`` than the keys'; the stacked matrix is then
  ``[Hq D + Hkv D + Hkv Dv, H]`` and the output projection takes ``Hq Dv`` columns.
* ``bias``: q, k and v have biases, added to the projections before anything else.
* ``qk_norm`` (``{"eps": e}``): every q and k head is divided by its root mean square over the head
  (``x / sqrt(mean(x^2) + e)``) and multiplied by a gain of size ``D`` that all heads share (one for q, one for k),
  after the bias and before the rotation.
* ``chunk``: the sequence's absolute positions are cut into blocks ``[b*chunk, (b+1)*chunk)``; a query attends
  causally inside its block and to nothing before the block's first position (how a prompt was fed in portions
  does not move the blocks).
* ``sink``: a learned logit per query head that competes in the softmax but carries no value: the weights of
  the real keys are ``exp(s_j) / (sum_i exp(s_i) + exp(sink_h))``, with ``sink_h`` taken as it is (``scale``
  applies to the dot products only).
* ``qk_norm`` with ``"gain": False``: the same division by the root mean square without learned gains.
* ``q_temp`` (``{"coef": c, "every": n}``): a query at position ``p`` is multiplied by
  ``1 + c * ln(floor((p + 1) / n) + 1)`` after its norm, so late queries score more sharply.
* ``out_gate``: head ``h``'s output is multiplied by ``sigmoid((G x)_h)``, a scalar for every token and head, ``G
  [Hq, H]`` reading the mixer's own input; its rows ride at the end of the stacked projection.
* ``value_from_key``: there is no value projection: a position's values are its keys as projected (with their bias,
  before norm and rotation); the stacked matrix is ``[(Hq + Hkv) D, H]``.
* ``o_bias``: the output projection has a bias; it is handed on with the result (``BiasedDelta``) so that the sum
  into the residual can take it in passing.
"""

from __future__ import annotations

import torch

from .context import BiasedDelta
from .plan import PagedKVNeed, TensorSpec
from .registry import POSITION_ENCODINGS, register_mixer


def _shared_position_encoding(spec, env):
    kind = spec["kind"] if isinstance(spec, dict) else spec.kind
    params = spec["params"] if isinstance(spec, dict) else spec.params
    key = ("position", kind, repr(sorted(params.items(), key=lambda kv: kv[0])))
    if key not in env._shared:
        env._shared[key] = POSITION_ENCODINGS.get(kind)(params, env)
    return env._shared[key]


@register_mixer("attention")
class Attention:
    """params: hidden_size, num_heads, num_kv_heads, head_dim, position
    (``{"kind", "params"}``), and optionally window, scale, kv_from_layer, value_head_dim, bias, qk_norm, chunk,
    sink, q_temp, out_gate, o_bias, value_from_key."""

    def __init__(self, params, env):
        self.hidden = int(params["hidden_size"])
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}")
        self.window = params.get("window")
        if self.window is not None:
            self.window = int(self.window)
            if self.window <= 0:
                raise ValueError(f"window must be positive, got {self.window}")
        scale = params.get("scale")
        self.scale = float(scale) if scale is not None else 1.0 / (self.head_dim ** 0.5)
        self.kv_from_layer = params.get("kv_from_layer")
        self.value_dim = int(params.get("value_head_dim") or self.head_dim)
        self.bias = bool(params.get("bias", False))
        qk_norm = params.get("qk_norm")
        self.qk_norm_eps = float(qk_norm["eps"]) if qk_norm else None
        self.qk_norm_gain = bool(qk_norm.get("gain", True)) if qk_norm else False
        q_temp = params.get("q_temp")
        self.q_temp = (float(q_temp["coef"]), int(q_temp["every"])) if q_temp else None
        if self.q_temp is not None and self.q_temp[1] <= 0:
            raise ValueError(f"q_temp.every must be positive, got {self.q_temp[1]}")
        self.out_gate = bool(params.get("out_gate", False))
        self.o_bias = bool(params.get("o_bias", False))
        self.value_from_key = bool(params.get("value_from_key", False))
        if self.value_from_key and (self.value_dim != self.head_dim or params.get("kv_from_layer") is not None):
            raise ValueError("values that are the keys have the keys' width, and the mixer projects its own keys")
        self.chunk = params.get("chunk")
        if self.chunk is not None:
            self.chunk = int(self.chunk)
            if self.chunk <= 0:
                raise ValueError(f"chunk must be positive, got {self.chunk}")
        self.sink = bool(params.get("sink", False))
        if self.kv_from_layer is not None and (self.bias or self.qk_norm_eps is not None or self.value_dim != self.head_dim
                                               or self.out_gate or self.q_temp is not None):
            raise ValueError("a mixer that reads another layer's keys and values has plain q heads of the keys' width")
        self.position = _shared_position_encoding(params.get("position", {"kind": "none", "params": {}}), env)
        if self.position.rotary_dim > self.head_dim:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head_dim {self.head_dim}")
        check = getattr(env.kernels, "check_attention_geometry", None)
        if check is not None:     # sizes the kernels refuse are refused here, when the model is built
            check(self.num_heads, self.num_kv_heads, max(self.head_dim, self.value_dim))
        # kernels that want keys and values of one width say at which width this mixer should keep its pages
        page_dim = getattr(env.kernels, "attention_page_dim", None)
        self.page_dim = page_dim(self.head_dim, self.value_dim, env.dtype) if page_dim is not None and self._options() else None
        self.env = env
        self.w_qkv = None
        self.w_o = None
        self.b_qkv = self.q_gain = self.k_gain = self.sinks = self.b_o = None
        self.gate_columns = 0

    takes_scaled_rows = True   # the input goes to ``qkv_to_cache`` only

    @property
    def writes_kv(self) -> bool:
        return self.kv_from_layer is None

    def weight_specs(self):
        q = self.num_heads * self.head_dim
        kv = self.num_kv_heads * self.head_dim
        v = self.num_kv_heads * self.value_dim
        specs = {"q": TensorSpec((q, self.hidden)), "o": TensorSpec((self.hidden, self.num_heads * self.value_dim))}
        if self.writes_kv:
            specs["k"] = TensorSpec((kv, self.hidden))
            if not self.value_from_key:
                specs["v"] = TensorSpec((v, self.hidden))
        if self.bias:
            specs.update({"q_bias": TensorSpec((q,), "vector"), "k_bias": TensorSpec((kv,), "vector")})
            if not self.value_from_key:
                specs["v_bias"] = TensorSpec((v,), "vector")
        if self.qk_norm_eps is not None and self.qk_norm_gain:
            specs.update({"q_norm": TensorSpec((self.head_dim,), "vector"), "k_norm": TensorSpec((self.head_dim,), "vector")})
        if self.sink:
            specs["sink"] = TensorSpec((self.num_heads,), "vector")
        if self.out_gate:
            specs["gate"] = TensorSpec((self.num_heads, self.hidden))
        if self.o_bias:
            specs["o_bias"] = TensorSpec((self.hidden,), "vector")
        return specs

    def bind(self, tensors):
        stacked = [tensors["q"]]
        if self.writes_kv:
            stacked += [tensors["k"]] if self.value_from_key else [tensors["k"], tensors["v"]]
        if self.out_gate:   # the gate's rows behind v, filled up with zero rows so that a projected row stays aligned
            self.gate_columns = -(-self.num_heads // 8) * 8
            g = tensors["gate"]
            stacked += [g, g.new_zeros((self.gate_columns - self.num_heads, self.hidden))]
        self.w_qkv = torch.cat(stacked, dim=0).contiguous()
        self.w_o = tensors["o"].contiguous()
        if self.page_dim is not None:   # the attention's rows come with page_dim elements a head: zero columns for the rest
            wide = self.w_o.new_zeros((self.hidden, self.num_heads, self.page_dim))
            wide[:, :, :self.value_dim] = self.w_o.view(self.hidden, self.num_heads, self.value_dim)
            self.w_o = wide.view(self.hidden, self.num_heads * self.page_dim)
        if self.bias:
            self.b_qkv = torch.cat([tensors[n] for n in ("q_bias", "k_bias", "v_bias") if n in tensors]).contiguous()
        if self.qk_norm_eps is not None and self.qk_norm_gain:
            self.q_gain, self.k_gain = tensors["q_norm"].contiguous(), tensors["k_norm"].contiguous()
        elif self.qk_norm_eps is not None:
            self.q_gain = self.k_gain = torch.ones(self.head_dim, dtype=torch.float32, device=self.w_qkv.device)
        if self.o_bias:
            self.b_o = tensors["o_bias"].contiguous()
        if self.sink:
            self.sinks = tensors["sink"].contiguous()
        prepare = getattr(self.env.kernels, "prepare_pending_weight", None)
        if prepare is not None:   # the kernels may keep a copy of their own of a weight whose product is left pending
            prepare(self.w_o)

    def plain_form(self):
        """What this mixer is, as plain data, for kernels that can run a whole block in one call; None for the forms
        that only ``forward`` covers (reading another layer's keys and values)."""
        if not self.writes_kv or type(self).forward is not Attention.forward or self._options():
            return None     # a subclass with a forward of its own is no longer what this form describes
        cos, sin = self.position.tables()
        return {"kind": "paged_attention", "w_qkv": self.w_qkv, "w_o": self.w_o, "hidden": self.hidden,
                "n_heads": self.num_heads, "n_kv_heads": self.num_kv_heads, "head_dim": self.head_dim,
                "rotary_dim": self.position.rotary_dim, "cos": cos, "sin": sin, "scale": self.scale,
                "window": self.window}

    def _options(self) -> bool:
        """Whether any of the further forms is switched on (the kernels then get them as keyword arguments)."""
        return (self.bias or self.qk_norm_eps is not None or self.sink or self.chunk is not None
                or self.value_dim != self.head_dim or self.q_temp is not None or self.out_gate or self.value_from_key)

    def cache_need(self):
        if self.page_dim is not None:
            return PagedKVNeed(self.num_kv_heads, self.page_dim, self.window, None, self.chunk)
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window,
                           self.value_dim if self.value_dim != self.head_dim else None, self.chunk)

    def state_need(self):
        return None

    def forward(self, h, ctx, cache):
        k = self.env.kernels
        cos, sin = self.position.tables()
        project, attend = {}, {}
        if self._options():   # only then: a kernels object that knows none of these forms serves the plain mixer
            if self.value_dim != self.head_dim:
                project["value_dim"] = self.value_dim
                if self.page_dim is None:
                    attend["value_dim"] = self.value_dim
            if self.page_dim is not None:
                project["page_dim"] = self.page_dim
            if self.bias:
                project["bias"] = self.b_qkv
            if self.qk_norm_eps is not None:
                project["qk_norm"] = (self.q_gain, self.k_gain, self.qk_norm_eps)
            if self.chunk is not None:
                attend["chunk"] = self.chunk
            if self.sink:
                attend["sinks"] = self.sinks
            if self.q_temp is not None:
                project["q_temp"] = self.q_temp
            if self.out_gate:
                project["extra_columns"] = self.gate_columns
            if self.value_from_key:
                project["values_are_keys"] = True
        qkv = k.qkv_to_cache(
            h, self.w_qkv, self.num_heads, self.num_kv_heads if self.writes_kv else 0, self.head_dim,
            self.position.rotary_dim, cos, sin, ctx, cache, **project)
        gate_logits = None
        if self.out_gate:
            qkv, further = qkv
            gate_logits = further[:, :self.num_heads]
        out = k.paged_attention(
            qkv, self.num_heads, self.num_kv_heads, self.page_dim or self.head_dim, self.scale, self.window, ctx, cache,
            **attend)
        if gate_logits is not None:
            out = k.head_gate(out, gate_logits, self.num_heads)
        y = k.pending_linear(out, self.w_o)   # the norm after it may have it added into the residual
        return BiasedDelta(y, self.b_o, k) if self.o_bias else y
