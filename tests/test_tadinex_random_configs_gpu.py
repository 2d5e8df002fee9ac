"""Seeded random Tadinex configurations through trace replay on the GPU, against the plain implementation: the two
mixers in any order and number, delta rules with any grouping of heads, key and value widths of every kind and
convolutions of one to five taps, windowed attention with windows from one token to beyond the prompts, rotations of
all or a part of a head with and without stretched frequencies, decaying attention with any number of heads, dense
feed-forwards, experts with and without identity experts and a shared expert, layers without a feed-forward, layer
multipliers of every kind, widths and vocabularies that are no multiple of anything.  float32 routes as the
configuration says; bfloat16 chooses every expert (see ``tadinex_models.all_experts``), and where a model errs more
than the usual bound under bfloat16's rounding alone (the same replay with the torch twins of the kernels, which round
at the same places), the kernels may err up to twice that."""

import copy
import random

import pytest
import torch

import tadinex_models as M
from test_trace_run import collect, make_trace

pytestmark = pytest.mark.gpu


def random_mixer(rng):
    if rng.random() < 0.5:
        kv = rng.choice([1, 2, 3])
        return {"type": "delta", "mixer": {"conv": rng.choice([1, 2, 3, 4, 5]), "dim": rng.choice([8, 20, 32, 48, 64, 128]),
                                           "heads": kv * rng.choice([1, 2, 4]), "kv_heads": kv,
                                           "vdim": rng.choice([8, 12, 32, 64, 80, 128])}}
    dim = rng.choice([8, 16, 24, 32, 48, 64, 96, 128])
    dims = rng.choice([d for d in (4, 8, 16, 32, 64, dim) if d <= dim])
    rot = {"base": rng.choice([100.0, 10000.0, 250000.0]), "dims": dims}
    if rng.random() < 0.6:
        rot["scaling"] = {"factor": rng.choice([2.0, 8.0, 40.0]), "original": rng.choice([16, 64, 1024]),
                          "fast": rng.choice([8.0, 32.0]), "slow": rng.choice([1.0, 2.0])}
    kv = rng.choice([1, 2, 3])
    r_heads = rng.choice([1, 2, 3, 5])
    return {"type": "parallel", "mixer": {
        "left": {"dim": dim, "vdim": dim, "heads": kv * rng.choice([1, 2, 4]), "kv_heads": kv,
                 "mask": {"size": rng.choice([1, 2, 7, 16, 17, 31, 40, 64, 200])}, "rot": rot,
                 "scale": rng.choice([0.05, 0.125, 0.3, dim ** -0.5])},
        "left_scale": rng.choice([0.3, 0.6, 1.0, 1.4]),
        "right": {"dim": rng.choice([8, 20, 32, 64, 128]), "vdim": rng.choice([8, 12, 32, 64, 80]), "heads": r_heads,
                  "decay": [rng.choice([0.3, 0.6, 0.9, 0.97, 0.999, 1.0]) for _ in range(r_heads)]},
        "right_scale": rng.choice([0.4, 0.9, 1.0, 1.2])}}


def random_mlp(rng):
    pick = rng.random()
    if pick < 0.2:
        return None
    if pick < 0.4:
        return {"kind": "dense", "ff": rng.choice([24, 50, 64, 136, 256])}
    experts, identity = rng.choice([1, 2, 3, 4, 8, 12]), rng.choice([0, 0, 1, 2, 5])
    mlp = {"kind": "moe", "router": {"experts": experts, "identity": identity,
                                     "top": rng.choice([t for t in (1, 2, 3, 4, 6) if t <= experts + identity])},
           "expert": {"ff": rng.choice([8, 24, 32, 50, 64]), "limit": rng.choice([0.5, 1.0, 2.0, 7.0])}}
    if rng.random() < 0.6:
        mlp["shared"] = {"ff": rng.choice([8, 32, 50, 128]), "limit": rng.choice([0.5, 1.5, 3.0])}
    return mlp


def random_config(seed):
    rng = random.Random(4000 + seed)
    shapes = [dict(random_mixer(rng), mlp=random_mlp(rng)) for _ in range(rng.choice([2, 3, 4]))]
    layers = [copy.deepcopy(rng.choice(shapes)) for _ in range(rng.choice([2, 3, 4, 5, 6]))]
    return {"architecture": "Tadinex", "vocab": rng.choice([97, 257, 500, 1001]),
            "width": rng.choice([40, 72, 100, 128, 136, 192, 200, 264]), "norm": {"eps": rng.choice([1e-5, 1e-6, 3e-4])},
            "embedding": {"scale": rng.choice([1.0, 3.0, 12.0])}, "residual_mult": rng.choice([0.5, 0.7, 1.0, 1.2]),
            "layers": layers}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_configuration_replays_like_the_plain_implementation(tmp_path, seed, dtype):
    from simple_inference_amd.replay import TraceReplayer

    cfg = random_config(seed)
    if dtype == "bfloat16":
        cfg = M.all_experts(cfg)
    print("configuration", seed, cfg, flush=True)
    folder = M.write_model(tmp_path, cfg, seed=300 + seed, std=0.07, spread=0.3)
    steps, prompts, most = make_trace(cfg["vocab"], lengths=(50, 33, 71, 20, 64))
    page = (8, 16, 32, 64)[seed % 4]
    rp = TraceReplayer(folder, dtype, most, block_size=page, max_live=4)
    got = collect(steps, lambda st: rp.step(st["entries"], st["end"]).float().cpu().numpy())
    backend = "hip-f32" if dtype == "float32" else "hip-bf16"
    rounded = None
    if dtype == "bfloat16":     # what rounding at the same places costs this model, without this package's kernels
        from twins import TwinKernels
        twin = TraceReplayer(folder, dtype, most, block_size=page, max_live=4, device="cpu", kernels=TwinKernels())
        rounded = collect(steps, lambda st: twin.step(st["entries"], st["end"]).float().numpy())
    for r, toks in prompts.items():
        ref = M.plain_logits(folder, toks)
        mine = torch.stack([torch.as_tensor(got[r][p]) for p in range(len(toks))])
        bound = M.TOLERANCE[backend]
        if rounded is not None:
            theirs = torch.stack([torch.as_tensor(rounded[r][p]) for p in range(len(toks))])
            bound = max(bound, 2 * M.err(theirs, ref, backend))
        assert M.err(mine, ref, backend) <= bound, (r, M.err(mine, ref, backend), bound)
    assert all(rp.cache.free_pages(g) == -(-most // page) for g in range(len(rp.cache.groups))) and not rp.ids
    assert rp.cache.slots.free_slots == 4
