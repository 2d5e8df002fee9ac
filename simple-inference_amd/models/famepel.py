"""``Famepel``: a decoder whose layers norm every sublayer's input and result with a dynamic tanh, and whose mixers
are a state-space mixer, a gated linear recurrence or latent attention; feed-forwards are routed experts.

All that is particular to the design is here: which parts a layer has and what the tensors are called.

* A layer is a sandwich block: ``x += ls1 * N1b(mixer(N1(x)))`` and, if it has a feed-forward, ``x += ls2 *
  N2b(ff(N2(x)))``; every ``N`` is ``tanh(a x) w + b`` with its own scalar ``a``, and ``ls`` a vector per sublayer.
* ``mamba2``: the state-space mixer of ``parts/ssm.py``; ``hgrn2``: the gated linear recurrence of ``parts/hgrn.py``;
  ``latent_attention``: ``parts/latent_attention.py`` with a sink per head, interleaved rotation of the shared key
  part with ramp-scaled frequencies, and optionally another layer's cached latent (``kv_from``).
* ``moe``: experts chosen by sigmoid scores among the best groups of experts, weights normalised and scaled.
* The embedding is multiplied by ``embedding.scale``; the last norm is of the same kind; the head is untied.

Checkpoint names: ``embed``, ``final.norm`` (``.b``, ``.alpha``), ``head``; layer ``i``: ``l<i>.norm1``, ``.norm1b``,
``.norm2``, ``.norm2b`` (each with ``.b`` and ``.alpha``), ``l<i>.ls1``, ``l<i>.ls2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""

from __future__ import annotations

from ..config.famepel_config import FamepelConfig, Hgrn2, LatentAttention, Mamba2
from ..config.registry import register_architecture
from ..parts.plan import LayerSpec, ModelPlan, PartSpec


def _mixer(cfg: FamepelConfig, m, p: str) -> PartSpec:
    if isinstance(m, Mamba2):
        return PartSpec("mamba2", {
            "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.vdim, "state_size": m.state,
            "groups": m.groups, "conv_taps": m.conv, "norm_groups": m.norm_groups, "norm_eps": cfg.norm_eps,
        }, {"in": f"{p}.in", "conv": f"{p}.conv", "conv_bias": f"{p}.conv.b", "dt_bias": f"{p}.dt_bias",
            "a_log": f"{p}.A_log", "d": f"{p}.D", "norm": f"{p}.norm", "o": f"{p}.o"}, role="mixer")
    if isinstance(m, Hgrn2):
        return PartSpec("hgrn2", {
            "hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim,
            "norm_eps": cfg.norm_eps,
        }, {"q": f"{p}.q", "f": f"{p}.f", "v": f"{p}.v", "f_bias": f"{p}.f.b", "lower": f"{p}.lower",
            "norm": f"{p}.norm", "o": f"{p}.o"}, role="mixer")
    assert isinstance(m, LatentAttention)
    scaling = None
    if m.rot.scaling is not None:
        scaling = dict(m.rot.scaling.to_dict(), rope_type="yarn")
    names = {"dq": f"{p}.dq", "dq_norm": f"{p}.dq.norm", "uq": f"{p}.uq", "uk": f"{p}.uk", "uv": f"{p}.uv",
             "sink": f"{p}.sink", "o": f"{p}.o"}
    if m.kv_from is None:
        names.update({"dkv": f"{p}.dkv", "dkv_norm": f"{p}.dkv.norm"})
    return PartSpec("latent_attention", {
        "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
        "value_head_dim": m.vdim, "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale,
        "norm_eps": cfg.norm_eps, "sink": True, "kv_from_layer": m.kv_from,
        "position": {"kind": "rope", "params": {"rotary_dim": m.rot.dims, "theta": m.rot.base, "scaling": scaling,
                                                "pairing": "interleaved", "angles": "float64"}},
    }, names, role="mixer")


def _feed_forward(cfg: FamepelConfig, mlp, p: str) -> PartSpec:
    names = {"router": f"{p}.router"}
    for e in range(mlp.experts):
        names.update({f"gate{e}": f"{p}.e{e}.gate", f"up{e}": f"{p}.e{e}.up", f"down{e}": f"{p}.e{e}.down"})
    return PartSpec("moe", {"hidden_size": cfg.width, "experts": mlp.experts, "top": mlp.top, "expert_size": mlp.ff,
                            "score": "sigmoid", "groups": mlp.groups, "route_scale": mlp.scale},
                    names, role="feed_forward")


def famepel_plan(cfg: FamepelConfig) -> ModelPlan:
    def norm(name, scale=None):
        weights = {"weight": name, "bias": name + ".b", "alpha": name + ".alpha"}
        if scale is not None:
            weights["scale"] = scale
        return PartSpec("dyt", {"size": cfg.width, "scaled": scale is not None}, weights, role="norm")

    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        parts = {"mixer_norm": norm(f"{p}.norm1"), "mixer": _mixer(cfg, layer.mixer, f"{p}.mix"),
                 "mixer_post_norm": norm(f"{p}.norm1b", f"{p}.ls1")}
        if layer.mlp is not None:
            parts.update({"feed_forward_norm": norm(f"{p}.norm2"),
                          "feed_forward": _feed_forward(cfg, layer.mlp, f"{p}.mlp"),
                          "feed_forward_post_norm": norm(f"{p}.norm2b", f"{p}.ls2")})
        layers.append(LayerSpec(block="sandwich", parts=parts))
    final = norm("final.norm")
    final.role = ""
    return ModelPlan(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                         "scale": cfg.embedding_scale}, {"weight": "embed"}),
        layers=layers,
        final_norm=final,
        head=PartSpec("head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False}, {"weight": "head"}),
    )


register_architecture("Famepel", FamepelConfig.from_dict, famepel_plan, replace=True)
