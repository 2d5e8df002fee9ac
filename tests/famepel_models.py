"""Small Famepel configurations for the tests, their model folders, and runners over them.

The configurations differ from one another in every size and option: state-space mixers with one group and with
several, one norm part and several, convolutions of 1, 2, 4 and 5 taps; forget-gate recurrences with one head and
with several, key and value widths that differ; latent attention with one head and with several, latents narrower and
wider than the heads, a rotation of all of the shared key part and of a part of it, with and without frequency
scaling, layers that read another layer's latent; experts with and without groups, groups of one expert, all groups
kept, top 1 to 4; layers without a feed-forward; every order of the three mixers; an embedding scale of 1 and others.
"""

from __future__ import annotations

import copy
import json

import torch
from safetensors import safe_open

import plain_famepel as plain
from mogisun_models import TOLERANCE, err, make_runner, rel_err, rms_err  # noqa: F401  (the same runners and measures)


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups,
                                        "state": state, "vdim": vdim}}


def _hgrn(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": {"dim": dim, "heads": heads, "vdim": vdim}}


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, dims=None, scaling=None, kv_from=None):
    rot = {"base": base, "dims": dims or rot_dim}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    m = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot, "rot_dim": rot_dim,
         "scale": scale, "vdim": vdim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def _moe(experts, top, ff, scale=1.0, groups=None):
    router = {"experts": experts, "scale": scale, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


def _layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def _model(vocab, width, eps, scale, layers):
    return {"architecture": "Famepel", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "layers": layers}


_LAT_A = dict(heads=3, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=40, scale=0.2, base=10000.0,
              scaling=(4.0, 64, 16.0, 2.0))
_LAT_C = dict(heads=4, dim=64, rot_dim=32, vdim=64, q_rank=48, kv_rank=96, scale=0.11, base=50000.0,
              scaling=(16.0, 128, 32.0, 1.0))

CONFIGS = {
    # latent attention first, read again by the last layer; groups of experts of which one is kept
    "a": _model(211, 96, 1e-5, 4.0, [
        _layer(_latent(**_LAT_A), _moe(6, 2, 40, 2.0, (3, 1))),
        _layer(_ssm(4, 16, 24, 2, 4, 2), None),
        _layer(_hgrn(3, 20, 12), _moe(4, 1, 24)),
        _layer(_latent(**_LAT_A, kv_from=0), _moe(6, 3, 16, 0.5, (2, 2)))]),
    # one head everywhere; convolution of two taps; groups of one expert; a rotation of half the shared key part
    "b": _model(160, 64, 3e-6, 1.0, [
        _layer(_hgrn(1, 32, 32), _moe(4, 2, 32, 1.0, (4, 2))),
        _layer(_ssm(1, 48, 16, 1, 2, 1), _moe(3, 3, 20)),
        _layer(_latent(1, 24, 16, 40, 16, 24, 0.3, 1000.0, dims=8), None)]),
    # sizes at which the GPU takes its matrix-core attention and its few-row products
    "c": _model(300, 128, 1e-6, 8.0, [
        _layer(_ssm(6, 32, 64, 3, 4, 2), _moe(8, 2, 64, 2.5, (4, 2))),
        _layer(_latent(**_LAT_C), _moe(8, 2, 64, 2.5, (4, 2))),
        _layer(_hgrn(4, 32, 64), _moe(4, 2, 128)),
        _layer(_ssm(4, 64, 32, 4, 3, 4), None),
        _layer(_latent(**_LAT_C, kv_from=1), _moe(6, 4, 64, 1.0, (3, 2)))]),
    # no latent attention at all; a convolution of one tap (no inputs to keep) and of five
    "d": _model(97, 48, 1e-5, 2.0, [
        _layer(_ssm(2, 24, 8, 1, 1, 1), _moe(2, 1, 16, 3.0)),
        _layer(_hgrn(2, 8, 24), None),
        _layer(_ssm(3, 16, 12, 3, 5, 3), _moe(5, 2, 8, 1.0, (5, 3)))]),
    # sizes that are multiples of nothing the kernels like: every vector path has to step aside
    "e": _model(131, 100, 2e-6, 1.3, [
        _layer(_latent(5, 12, 6, 20, 14, 22, 0.4, 777.0, dims=4, scaling=(2.0, 40, 8.0, 1.0)), _moe(7, 2, 36, 1.2)),
        _layer(_hgrn(3, 12, 20), _moe(9, 3, 10, 0.7, (3, 2))),
        _layer(_ssm(5, 12, 10, 1, 4, 5), None)]),
}

PAGE_SIZE = {"a": 8, "b": 16, "c": 16, "d": 4, "e": 16}


def all_experts(cfg):
    """The configuration with every expert chosen for every token and every group kept: what remains of routing are
    the weights, which do not jump.  (With fewer, two scores that nearly tie pick another expert under bfloat16's
    rounding of the router's input, and the outputs then differ by an expert, not by rounding.)"""
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if layer["mlp"]:
            router = layer["mlp"]["router"]
            router["top"] = router["experts"]
            if "groups" in router:
                router["groups"]["keep"] = router["groups"]["count"]
    return cfg


def tame(tensors, seed=0):
    """Vectors that the random mode draws around 1 and that mean something else: biases around 0, lower bounds of the
    forget gates inside (0, 1), convolution weights and decays of a size that keeps the recurrences lively."""
    g = torch.Generator().manual_seed(1000 + seed)
    for name, t in tensors.items():
        draw = lambda std: torch.randn(t.shape, generator=g) * std
        if name.endswith((".b", ".dt_bias", ".sink", ".A_log")):
            t.copy_(draw(0.5))
        elif name.endswith(".lower"):
            t.copy_(torch.rand(t.shape, generator=g) * 0.9)
        elif name.endswith(".mix.conv"):
            t.copy_(draw(0.5))
        elif name.endswith(".alpha"):
            t.copy_(0.5 + torch.rand(t.shape, generator=g))


def write_model(folder, name_or_config, seed=0, std=0.08, spread=0.3, change=None):
    """config.json + model.safetensors with the package's random mode: matrices N(0, std), vectors 1 + N(0, spread),
    then ``tame``; ``change(tensors)`` may edit the tensors before they are written."""
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import build_model
    from simple_inference_amd.weights import random_tensors, write_model_folder

    cfg = copy.deepcopy(CONFIGS[name_or_config] if isinstance(name_or_config, str) else name_or_config)
    model, mcfg = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    tensors = random_tensors(model.expected_tensors(), seed, std, spread, "bfloat16")
    tame(tensors, seed)
    if change is not None:
        change(tensors)
    write_model_folder(folder, mcfg.to_dict(), tensors)
    return folder


def read_model(folder):
    with open(f"{folder}/config.json") as f:
        cfg = json.load(f)
    w = {}
    with safe_open(f"{folder}/model.safetensors", framework="pt") as f:
        for k in f.keys():
            w[k] = f.get_tensor(k).double()
    return cfg, w


def plain_logits(folder, tokens):
    cfg, w = read_model(folder)
    return plain.forward(cfg, w, tokens).float()
