"""Small Tadinex configurations for the tests, their model folders, and runners over them.

The configurations differ from one another in every size and option: delta-rule mixers with as many query/key heads
as value heads and with fewer, key and value widths that differ, convolutions of 1 to 5 taps; windowed attention with
one key/value head and with several, windows shorter and longer than a page, a rotation of all of a head and of a part
of it, with and without frequency scaling; decaying attention with one head and with several; dense feed-forwards,
experts with and without identity experts, with and without a shared expert, top 1 to 4; layers without a
feed-forward; every order of the two mixers; a layer multiplier of 1 and others.
"""

from __future__ import annotations

import copy
import json

import torch
from safetensors import safe_open

import plain_tadinex as plain
from mogisun_models import TOLERANCE, err, make_runner, rel_err, rms_err  # noqa: F401  (the same runners and measures)


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}}


def _parallel(heads, kv_heads, dim, window, scale, base, dims, scaling, r_heads, r_dim, r_vdim, decay, ls, rs):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "parallel", "mixer": {
        "left": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": window}, "rot": rot, "scale": scale,
                 "vdim": dim},
        "left_scale": ls,
        "right": {"decay": list(decay), "dim": r_dim, "heads": r_heads, "vdim": r_vdim},
        "right_scale": rs}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, identity, top, ff, limit, shared=None):
    mlp = {"kind": "moe", "router": {"experts": experts, "identity": identity, "top": top},
           "expert": {"ff": ff, "limit": limit}}
    if shared:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


def _layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def _model(vocab, width, eps, scale, mult, layers):
    return {"architecture": "Tadinex", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "residual_mult": mult, "layers": layers}


CONFIGS = {
    # the two mixers in turn; a window shorter than two pages; grouped heads on both sides
    "a": _model(211, 96, 1e-5, 4.0, 0.8, [
        _layer(_parallel(4, 2, 16, 11, 0.3, 10000.0, 8, (4.0, 64, 16.0, 2.0), 3, 8, 12, (0.9, 0.5, 0.99), 0.7, 1.2),
               _moe(5, 1, 2, 24, 1.2, (40, 2.5))),
        _layer(_delta(4, 2, 12, 20, 4), _dense(72)),
        _layer(_delta(3, 3, 16, 8, 2), None),
        _layer(_parallel(2, 2, 24, 40, 0.2, 500.0, 24, None, 1, 16, 16, (0.8,), 1.0, 0.5), _moe(4, 0, 1, 16, 3.0))]),
    # one head everywhere; a convolution of one tap (no inputs to keep); a multiplier of 1; a window of one token
    "b": _model(160, 64, 3e-6, 1.0, 1.0, [
        _layer(_delta(1, 1, 32, 32, 1), _moe(3, 2, 3, 20, 0.8)),
        _layer(_parallel(1, 1, 32, 1, 0.25, 1000.0, 16, None, 1, 24, 40, (0.95,), 0.4, 0.9), _dense(48)),
        _layer(_delta(2, 1, 8, 24, 5), None)]),
    # sizes at which the GPU takes its matrix-core attention and its few-row products
    "c": _model(300, 128, 1e-6, 8.0, 0.6, [
        _layer(_delta(4, 2, 64, 32, 3), _moe(8, 2, 2, 96, 1.25, (64, 1.75))),
        _layer(_parallel(4, 1, 64, 24, 0.11, 50000.0, 32, (16.0, 128, 32.0, 1.0), 2, 32, 64, (0.7, 0.995), 0.55, 1.15),
               _dense(256)),
        _layer(_delta(2, 2, 32, 64, 4), _moe(4, 0, 2, 128, 2.0)),
        _layer(_parallel(2, 2, 32, 70, 0.2, 10000.0, 32, None, 4, 32, 32, (0.5, 0.9, 0.97, 1.0), 1.3, 0.8),
               _moe(6, 1, 4, 64, 1.0, (64, 1.0)))]),
    # sizes that are multiples of nothing the kernels like: every vector path has to step aside
    "e": _model(131, 100, 2e-6, 1.3, 0.9, [
        _layer(_parallel(5, 5, 12, 7, 0.4, 777.0, 4, (2.0, 40, 8.0, 1.0), 3, 10, 6, (0.6, 0.8, 0.9), 0.9, 0.9),
               _moe(7, 3, 2, 36, 1.1, (10, 0.7))),
        _layer(_delta(6, 2, 10, 14, 3), _dense(52)),
        _layer(_delta(3, 1, 20, 12, 2), _moe(2, 1, 1, 10, 2.2))]),
}

PAGE_SIZE = {"a": 8, "b": 16, "c": 16, "e": 16}


def all_experts(cfg):
    """The configuration with every output of the router chosen for every token: what remains of routing are the
    weights, which do not jump.  (With fewer, two scores that nearly tie pick another expert under bfloat16's rounding
    of the router's input, and the outputs then differ by an expert, not by rounding.)"""
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if layer["mlp"] and layer["mlp"]["kind"] == "moe":
            router = layer["mlp"]["router"]
            router["top"] = router["experts"] + router.get("identity", 0)
    return cfg


def tame(tensors, seed=0):
    """Vectors that the random mode draws around 1 and that mean something else: gains stored as their distance from
    one, biases, sinks, corrections and decay rates around 0, convolution weights of a size that keeps the recurrences
    lively."""
    g = torch.Generator().manual_seed(1000 + seed)
    for name, t in tensors.items():
        draw = lambda std: torch.randn(t.shape, generator=g) * std
        if name.endswith((".norm1", ".norm2", "final.norm")):
            t.copy_(draw(0.3))
        elif name.endswith((".dt_bias", ".sink", ".A_log")):
            t.copy_(draw(0.5))
        elif name.endswith(".correction"):
            t.copy_(draw(0.05))
        elif name.endswith(".conv"):
            t.copy_(draw(0.5))


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
