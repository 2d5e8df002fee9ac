"""Seeded random Famepel configurations through trace replay on the GPU, against the plain implementation: the three
mixers in any order and number, state-space mixers with any grouping of heads and of the norm and convolutions of one
to five taps, forget-gate recurrences with key and value widths of every kind, latent attention with latents narrower
and wider than its heads, rotations of all or a part of the shared key part with and without stretched frequencies,
layers that read an earlier layer's latent, experts with and without groups (any number kept), layers without a
feed-forward, widths and vocabularies that are no multiple of anything.  float32 routes as the configuration says;
bfloat16 chooses every expert (see ``famepel_models.all_experts``), and where a model errs more than the usual bound
under bfloat16's rounding alone (the same replay with the torch twins of the kernels, which round at the same
places), the kernels may err up to twice that."""

import copy
import random

import pytest
import torch

import famepel_models as M
from test_trace_run import collect, make_trace

pytestmark = pytest.mark.gpu


def random_mixer(rng):
    pick = rng.random()
    if pick < 0.35:
        groups = rng.choice([1, 2, 3])
        heads = groups * rng.choice([1, 2, 4])
        vdim = rng.choice([8, 12, 16, 32, 40, 64])
        parts = rng.choice([p for p in (1, 2, 3, 4, heads) if (heads * vdim) % p == 0])
        return {"type": "mamba2", "mixer": {"conv": rng.choice([1, 2, 3, 4, 5]), "groups": groups, "heads": heads,
                                            "norm_groups": parts, "state": rng.choice([8, 16, 24, 50, 64, 128]), "vdim": vdim}}
    if pick < 0.6:
        return {"type": "hgrn2", "mixer": {"dim": rng.choice([8, 20, 32, 48, 64, 128]), "heads": rng.choice([1, 2, 3, 6]),
                                           "vdim": rng.choice([8, 12, 32, 64, 80, 128])}}
    rot_dim = rng.choice([4, 8, 16, 24, 32, 64])
    dims = rng.choice([d for d in (4, 8, 16, 32, 64, rot_dim) if d <= rot_dim])
    rot = {"base": rng.choice([100.0, 10000.0, 250000.0]), "dims": dims}
    if rng.random() < 0.6:
        rot["scaling"] = {"factor": rng.choice([2.0, 8.0, 40.0]), "original": rng.choice([16, 64, 1024]),
                          "fast": rng.choice([8.0, 32.0]), "slow": rng.choice([1.0, 2.0])}
    dim = rng.choice([8, 16, 24, 32, 64, 128])
    return {"type": "latent_attention",
            "mixer": {"dim": dim, "heads": rng.choice([1, 2, 3, 4, 8]), "kv_rank": rng.choice([16, 24, 40, 64, 96, 160]),
                      "q_rank": rng.choice([8, 20, 48, 80]), "rot": rot, "rot_dim": rot_dim,
                      "scale": rng.choice([0.05, 0.125, 0.3, (dim + rot_dim) ** -0.5]),
                      "vdim": dim if rng.random() < 0.5 else rng.choice([8, 16, 24, 48, 72, 128])}}


def random_mlp(rng):
    if rng.random() < 0.2:
        return None
    experts = rng.choice([2, 3, 4, 8, 12, 20])
    router = {"experts": experts, "scale": rng.choice([0.5, 1.0, 1.5, 2.5])}
    most = experts
    if rng.random() < 0.7:
        count = rng.choice([c for c in (1, 2, 3, 4, experts) if experts % c == 0])
        keep = rng.randint(1, count)
        router["groups"] = {"count": count, "keep": keep}
        most = experts // count * keep
    router["top"] = rng.choice([t for t in (1, 2, 3, 4, 6) if t <= most])
    return {"kind": "moe", "router": router, "expert": {"ff": rng.choice([8, 24, 32, 50, 64])}}


def random_config(seed):
    rng = random.Random(3000 + seed)
    shapes = [dict(random_mixer(rng), mlp=random_mlp(rng)) for _ in range(rng.choice([2, 3, 4]))]
    layers = [copy.deepcopy(rng.choice(shapes)) for _ in range(rng.choice([2, 3, 4, 5, 6]))]
    owner = {}
    for i, layer in enumerate(layers):      # a later layer of the same shape may read the first one's latent
        if layer["type"] != "latent_attention":
            continue
        key = repr(sorted(layer["mixer"].items()))
        if key in owner and rng.random() < 0.6:
            layer["mixer"]["kv_from"] = owner[key]
        owner.setdefault(key, i)
    return {"architecture": "Famepel", "vocab": rng.choice([97, 257, 500, 1001]),
            "width": rng.choice([40, 72, 100, 128, 136, 192, 200, 264]), "norm": {"eps": rng.choice([1e-5, 1e-6, 3e-4])},
            "embedding": {"scale": rng.choice([1.0, 3.0, 12.0])}, "layers": layers}


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
