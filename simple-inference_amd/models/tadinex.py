"""``Tadinex``: a pre-norm decoder whose sublayers' results are scaled by one constant, whose mixers are a gated delta
rule or a windowed softmax attention beside a decaying linear attention, and whose feed-forwards are dense or routed.

All that is particular to the design is here: which parts a layer has and what the tensors are called.

* A layer is a pre-norm block with ``residual_scale``: ``x += m * mixer(N1(x))`` and, if it has a feed-forward,
  ``x += m * ff(N2(x))``; every ``N`` is an RMS norm whose gain is stored as its distance from one.
* ``delta``: the gated delta rule of ``parts/delta.py`` behind convolutions of ``conv`` taps.
* ``parallel``: ``parts/parallel.py`` over the ``attention`` part (window, a sink per head, q/k norm with gains,
  rotation of the first ``rot.dims`` elements with ramp-scaled frequencies, the values being the keys as projected)
  and ``parts/decay_attention.py``, with the two factors of the configuration.
* ``dense``: ``W_down gelu(W_up h)`` with the exact gelu.  ``moe``: scores over all router outputs, the choice
  corrected by a stored vector, identity experts behind the experts with tensors, clamped gated experts, a shared
  expert without a gate of its own.
* The embedding is multiplied by ``embedding.scale``; the last norm is of the same kind; the head is untied.

Checkpoint names: ``embed``, ``final.norm``, ``head``; layer ``i``: ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``
(under ``.left`` and ``.right`` for the two mixers side by side), ``l<i>.mlp.*``.
"""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.tadinex_config import ClampedExperts, DeltaMixer, DenseMlp, ParallelMixer, TadinexConfig
from ..parts.plan import LayerSpec, ModelPlan, PartSpec


def _mixer(cfg: TadinexConfig, m, p: str) -> PartSpec:
    if isinstance(m, DeltaMixer):
        return PartSpec("gated_delta", {
            "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
            "value_dim": m.vdim, "conv_taps": m.conv, "norm_eps": cfg.norm_eps,
        }, {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "g": f"{p}.g", "b": f"{p}.b", "a": f"{p}.a",
            "q_conv": f"{p}.q.conv", "k_conv": f"{p}.k.conv", "v_conv": f"{p}.v.conv", "a_log": f"{p}.A_log",
            "dt_bias": f"{p}.dt_bias", "norm": f"{p}.norm", "o": f"{p}.o"}, role="mixer")
    assert isinstance(m, ParallelMixer)
    left, right = m.left, m.right
    scaling = dict(left.rot.scaling.to_dict(), rope_type="yarn") if left.rot.scaling is not None else None
    branches = {
        "left": {"kind": "attention", "scale": m.left_scale, "params": {
            "hidden_size": cfg.width, "num_heads": left.heads, "num_kv_heads": left.kv_heads, "head_dim": left.dim,
            "window": left.window, "scale": left.scale, "qk_norm": {"eps": cfg.norm_eps}, "sink": True,
            "value_from_key": True,
            "position": {"kind": "rope", "params": {"rotary_dim": left.rot.dims, "theta": left.rot.base,
                                                    "scaling": scaling, "angles": "float64"}}}},
        "right": {"kind": "decay_attention", "scale": m.right_scale, "params": {
            "hidden_size": cfg.width, "num_heads": right.heads, "key_dim": right.dim, "value_dim": right.vdim,
            "decay": list(right.decay), "norm_eps": cfg.norm_eps}},
    }
    names = {"left.q": f"{p}.left.q", "left.k": f"{p}.left.k", "left.o": f"{p}.left.o",
             "left.q_norm": f"{p}.left.q.norm", "left.k_norm": f"{p}.left.k.norm", "left.sink": f"{p}.left.sink"}
    names.update({f"right.{n}": f"{p}.right.{n}" for n in ("q", "k", "v", "g", "norm", "o")})
    return PartSpec("parallel", {"branches": branches}, names, role="mixer")


def _feed_forward(cfg: TadinexConfig, mlp, p: str) -> PartSpec:
    if isinstance(mlp, DenseMlp):
        return PartSpec("dense", {"hidden_size": cfg.width, "intermediate_size": mlp.ff, "activation": "gelu"},
                        {"up": f"{p}.up", "down": f"{p}.down"}, role="feed_forward")
    assert isinstance(mlp, ClampedExperts)
    names = {"router": f"{p}.router", "correction": f"{p}.correction"}
    for e in range(mlp.experts):
        names.update({f"gate{e}": f"{p}.e{e}.gate", f"up{e}": f"{p}.e{e}.up", f"down{e}": f"{p}.e{e}.down"})
    params = {"hidden_size": cfg.width, "experts": mlp.experts, "top": mlp.top, "expert_size": mlp.ff,
              "score": "softmax_all", "correction": True, "identity_experts": mlp.identity, "activation": "clamped",
              "limit": mlp.limit}
    if mlp.shared_ff is not None:
        params.update({"shared_size": mlp.shared_ff, "shared_gate": False, "shared_limit": mlp.shared_limit})
        names.update({"shared_gate": f"{p}.shared.gate", "shared_up": f"{p}.shared.up", "shared_down": f"{p}.shared.down"})
    return PartSpec("moe", params, names, role="feed_forward")


def tadinex_plan(cfg: TadinexConfig) -> ModelPlan:
    def norm(name, role="norm"):
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "unit_offset": True}, {"weight": name}, role=role)

    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        parts = {"mixer_norm": norm(f"{p}.norm1"), "mixer": _mixer(cfg, layer.mixer, f"{p}.mix")}
        if layer.mlp is not None:
            parts.update({"feed_forward_norm": norm(f"{p}.norm2"),
                          "feed_forward": _feed_forward(cfg, layer.mlp, f"{p}.mlp")})
        layers.append(LayerSpec(block="prenorm", parts=parts, block_params={"residual_scale": cfg.residual_mult}))
    return ModelPlan(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                         "scale": cfg.embedding_scale}, {"weight": "embed"}),
        layers=layers,
        final_norm=norm("final.norm", role=""),
        head=PartSpec("head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False}, {"weight": "head"}),
    )


register_architecture("Tadinex", TadinexConfig.from_dict, tadinex_plan, replace=True)
