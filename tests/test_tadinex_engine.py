"""The Tadinex design through the engine's own step function, cache manager, state slots, scheduler and entry point,
against the plain implementation: every way of cutting the work must give the logits of the whole sequence.

The same tests run on the CPU with the torch twins of the kernels (they test configuration, plan, parts, cache
manager, state slots and batch layout) and on the GPU with the HIP kernels in float32 and bfloat16.  The bfloat16
runs route every token to all experts (see ``tadinex_models.all_experts``); routing to fewer is tested in float32.
"""

import copy

import pytest
import torch

import tadinex_models as M
from helpers import random_tokens
from test_mogisun_engine import cut, replay

BACKENDS = [
    pytest.param("twins"),
    pytest.param("twins-bf16"),
    pytest.param("hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip-bf16", marks=pytest.mark.gpu),
]
FLOAT_BACKENDS = [pytest.param("twins"), pytest.param("hip-f32", marks=pytest.mark.gpu)]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for i, name in enumerate(M.CONFIGS):
        out[name] = M.write_model(tmp_path_factory.mktemp(f"tadinex_{name}"), name, seed=5 + i)
        out[name + "-all"] = M.write_model(tmp_path_factory.mktemp(f"tadinex_{name}_all"), M.all_experts(M.CONFIGS[name]),
                                           seed=5 + i)
    return out


def folder_for(folders, name, backend):
    return folders[name + "-all"] if "bf16" in backend else folders[name]


def check(got, prompts, folder, backend):
    for req, rows in got.items():
        ref = M.plain_logits(folder, prompts[req])
        pos = sorted(rows)
        assert M.err(torch.stack([rows[p] for p in pos]), ref[pos], backend) <= M.TOLERANCE[backend], req


def test_configuration_reads_every_size_and_refuses_what_it_does_not_know():
    from simple_inference_amd.config import ConfigError, TadinexConfig
    for name, cfg in M.CONFIGS.items():
        parsed = TadinexConfig.from_dict(cfg)
        assert parsed.to_dict() == TadinexConfig.from_dict(parsed.to_dict()).to_dict() == cfg
        assert parsed.vocab == cfg["vocab"] and parsed.width == cfg["width"] and len(parsed.layers) == len(cfg["layers"])
        assert parsed.embedding_scale == cfg["embedding"]["scale"] and parsed.norm_eps == cfg["norm"]["eps"]
        assert parsed.residual_mult == cfg["residual_mult"]
    a = TadinexConfig.from_dict(M.CONFIGS["a"])
    assert a.layers[0].mixer.left.rot.scaling.factor == 4.0 and a.layers[3].mixer.left.rot.scaling is None
    assert a.layers[0].mixer.left.window == 11 and a.layers[0].mixer.right.decay == (0.9, 0.5, 0.99)
    assert a.layers[0].mlp.identity == 1 and a.layers[3].mlp.identity == 0 and a.layers[3].mlp.shared_ff is None
    assert a.layers[2].mlp is None and a.layers[1].mlp.ff == 72 and a.layers[1].mixer.kv_heads == 2

    def broken(change):
        cfg = copy.deepcopy(M.CONFIGS["a"])
        change(cfg)
        with pytest.raises(ConfigError):
            TadinexConfig.from_dict(cfg)
    broken(lambda c: c["layers"][1].update(type="lstm"))
    broken(lambda c: c["layers"][0]["mlp"].update(kind="glu"))
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=7))      # five experts and one identity expert
    broken(lambda c: c["layers"][0]["mlp"]["expert"].pop("limit"))
    broken(lambda c: c["layers"][1]["mixer"].update(kv_heads=3))
    broken(lambda c: c["layers"][1]["mixer"].pop("conv"))
    broken(lambda c: c["layers"][0]["mixer"]["left"].update(vdim=20))     # the values are the keys
    broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18))
    broken(lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5]))
    broken(lambda c: c["layers"][0]["mixer"].pop("left_scale"))
    broken(lambda c: c.pop("width"))


def test_plan_gives_the_mixers_side_by_side_pages_and_a_state_and_the_delta_rule_a_state(folders):
    runner, cache = M.make_runner(folders["a"], "twins", 8, 16)
    layout = runner.model.cache_layout()
    assert layout.run_kv == [(0, 0), None, None, (1, 0)] and layout.kv_slabs == [1, 1]
    need = layout.kv_groups[0]
    assert (need.num_kv_heads, need.head_dim, need.value_dim, need.window) == (2, 16, 16, 11)
    assert layout.kv_groups[1].window == 40
    assert layout.run_state == [0, 1, 2, 3]
    assert layout.states[0].shape == (3, 8, 12) and layout.states[3].shape == (1, 16, 16)
    # the matrices, and behind them the convolution's kept inputs: (taps - 1) rows of q, k and v channels
    assert layout.states[1].shape == (4 * 12 * 20 + (2 * 2 * 12 + 4 * 20) * 3,)
    assert layout.states[2].shape == (3 * 16 * 8 + (2 * 3 * 16 + 3 * 8) * 1,)
    runner, cache = M.make_runner(folders["b"], "twins", 16, 16)
    assert runner.model.cache_layout().states[0].shape == (32 * 32,)      # one tap: nothing to keep


def test_the_residual_after_every_layer_is_the_plain_one(folders):
    """Layer by layer: the engine's model is cut off behind layer i and its residual read through a head and a last
    norm that pass it on unchanged."""
    from simple_inference_amd.parts.context import ResidualStream
    name = "a"
    runner, cache = M.make_runner(folders[name], "twins", 8, 16)
    toks = random_tokens(211, 37, seed=3)
    cfg, w = M.read_model(folders[name])
    layers, _ = M.plain.layer_streams(cfg, w, toks)
    model = runner.model
    seen = []
    for layer in model.layers:
        block = layer.block
        original = block.forward

        def spy(stream, ctx, cache_, original=original):
            original(stream, ctx, cache_)
            probe = ResidualStream(stream.residual.clone(), stream.raw_delta)
            probe.scale = stream.scale
            seen.append(probe.settle(ctx.kernels).clone())
        block.forward = spy
    replay(runner, cache, [([(1, toks, [0])], [1])])
    assert len(seen) == len(cfg["layers"])
    for i, x in enumerate(seen):
        assert M.rel_err(x, layers[i]) < 2e-5, i


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c", "e"])
def test_whole_prompt_then_token_by_token(folders, backend, name):
    folder = folder_for(folders, name, backend)
    runner, cache = M.make_runner(folder, backend, M.PAGE_SIZE[name], 40)
    toks = random_tokens(M.CONFIGS[name]["vocab"], 130, seed=7)
    n0 = 61        # the decoded tokens pass page borders of every configuration
    schedule = [([(1, toks[:n0], list(range(n0)))], [])] + [([(1, [t], [0])], []) for t in toks[n0:]]
    got = replay(runner, cache, schedule)
    check(got, {1: toks}, folder, backend)
    # and all of it token by token, from the first token on
    cache.release(1)
    got = replay(runner, cache, [([(2, [t], [0])], []) for t in toks[:50]])
    check(got, {2: toks[:50]}, folder, backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name,sizes", [("a", [2, 5, 23, 1, 24, 3]), ("b", [19, 2, 2, 40, 1, 7]), ("c", [50, 17, 2, 33, 64]),
                                        ("e", [7, 2, 45, 1, 16])])
def test_portions_cut_anywhere_down_to_two_tokens(folders, backend, name, sizes):
    """Portions shorter than the convolution's reach and than the window, portions that end in the middle of a page:
    the convolution's kept inputs, the states and the pages must carry over every cut."""
    folder = folder_for(folders, name, backend)
    runner, cache = M.make_runner(folder, backend, M.PAGE_SIZE[name], 40)
    toks = random_tokens(M.CONFIGS[name]["vocab"], 141, seed=8)
    got = replay(runner, cache, [([(1, part, list(range(len(part))))], []) for part in cut(toks, sizes)])
    check(got, {1: toks}, folder, backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "c", "e"])
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(folders, backend, name):
    """Up to three live requests of very different lengths: portions beside single tokens, requests left out of
    steps, requests that end and whose pages and state slots the next ones get (a state or a convolution's inputs
    left behind by the slot's last holder would show in the first tokens of the next).  The pool holds far less
    than all."""
    folder = folder_for(folders, name, backend)
    vocab = M.CONFIGS[name]["vocab"]
    lengths = [90, 7, 133, 41, 1, 66, 30]
    prompts = {i + 1: random_tokens(vocab, n, seed=100 + i) for i, n in enumerate(lengths)}
    plans = {r: cut(t[:-4], [11 + r, 2, 29]) + [[x] for x in t[-4:]] if len(t) > 4 else [[x] for x in t]
             for r, t in prompts.items()}
    waiting, live, schedule = list(prompts), [], []
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, ends = [], []
        for r in list(live):
            if (len(schedule) + r) % 5 == 4 and len(live) > 1:
                continue
            part = plans[r].pop(0)
            entries.append((r, part, list(range(len(part)))))
            if not plans[r]:
                ends.append(r)
                live.remove(r)
        schedule.append((entries, ends))
    page = M.PAGE_SIZE[name]
    pool = sum(sorted(-(-n // page) for n in lengths)[-3:]) + 1
    runner, cache = M.make_runner(folder, backend, page, pool, max_running=3)
    got = replay(runner, cache, schedule)
    check(got, prompts, folder, backend)
    assert all(cache.free_pages(g) == pool for g in range(len(cache.groups))) and not cache.slots.slot_of
    # each alone gives the same (float32: to the last bits of the sums' order)
    if backend in ("twins", "hip-f32"):
        for r in (3, 6):
            solo = replay(runner, cache, [([(50 + r, prompts[r], list(range(len(prompts[r]))))], [50 + r])])
            for p, row in solo[50 + r].items():
                assert M.rel_err(row, got[r][p]) < 2e-5


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(folders, backend):
    name = "c"
    folder = folder_for(folders, name, backend)
    runner, cache = M.make_runner(folder, backend, 16, 24)
    toks = random_tokens(300, 330, seed=9)
    wanted = {5, 15, 16, 47, 48, 49, 50, 99, 100, 149, 150, 200, 249, 250, 299, 300, 329}
    schedule = [([(1, toks[:3], [0, 1, 2])], [])] + [([(1, [t], [0] if 3 + i in wanted else [])], [])
                                                    for i, t in enumerate(toks[3:])]
    got = replay(runner, cache, schedule)
    assert set(got[1]) == wanted | {0, 1, 2}
    check(got, {1: toks}, folder, backend)


def _long_memory(tensors):
    """Weights with which a token far back still weighs in the last logits: the delta rule's decays are slowed down
    (a state that forgot nothing at all would hold the far token as one of hundreds of equal shares, so the decays are
    set to keep about a third over the distance).  The windows have long passed it: only the states can carry it."""
    for name, t in tensors.items():
        if name.endswith(".mix.A_log"):
            t.fill_(-6.0)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["c", "e"])
def test_a_far_token_reaches_the_last_logits_however_the_prompt_is_cut(folders, backend, tmp_path, name):
    """Two prompts that differ in one token hundreds of positions back: the last logits differ by far more than the
    tolerance, and by what the plain implementation says, in whole prompts, portions and decoding: a state's share
    that got lost on the way would show."""
    cfg = M.all_experts(M.CONFIGS[name]) if "bf16" in backend else M.CONFIGS[name]
    vocab = cfg["vocab"]
    folder = M.write_model(tmp_path / "far", cfg, seed=77, change=_long_memory)
    base = random_tokens(vocab, 420, seed=10)
    for place in (16, 31, 0):
        other = list(base)
        other[place] = (other[place] + 1) % vocab
        ref = [M.plain_logits(folder, p)[-1] for p in (base, other)]
        assert M.rel_err(ref[0], ref[1]) > 2e-4      # the far token matters: four times the float32 tolerance and more
        for sizes, tail in (([420], 0), ([37, 2, 161], 40)):
            rows = []
            for prompt in (base, other):
                runner, cache = M.make_runner(folder, backend, 16, 30)
                steps = [([(1, part, [])], []) for part in cut(prompt[:420 - tail - 1], sizes)]
                steps += [([(1, [t], [])], []) for t in prompt[420 - tail - 1:-1]] + [([(1, prompt[-1:], [0])], [])]
                rows.append(replay(runner, cache, steps)[1][419])
            for row, want in zip(rows, ref):
                assert M.err(row, want, backend) <= M.TOLERANCE[backend]
            if "bf16" not in backend:
                assert M.rel_err(rows[0], rows[1]) > 1e-4


@pytest.mark.parametrize("backend", FLOAT_BACKENDS)
@pytest.mark.parametrize("name", ["a", "c"])
def test_the_window_gives_its_pages_back_and_sees_exactly_its_keys(folders, backend, tmp_path, name):
    """Two prompts that differ in one token: the last logits of a model whose only memory is the window (the states'
    writes are switched off) differ if the token lies just inside the window and are equal to the last bit if it
    lies just outside, in a whole prompt, in portions and in decoding; pages behind the window go back to the pool."""
    cfg = copy.deepcopy(M.CONFIGS[name])
    cfg["layers"] = [layer for layer in cfg["layers"] if layer["type"] == "parallel"]
    windows = [layer["mixer"]["left"]["mask"]["size"] for layer in cfg["layers"]]
    for layer, w in zip(cfg["layers"], windows):
        layer["mixer"]["left"]["mask"]["size"] = max(windows)     # one window, so that its edge is the model's
        layer["mixer"]["right_scale"] = 0.0                        # what the state remembers is not added
    window, depth = max(windows), len(cfg["layers"])
    vocab = cfg["vocab"]
    folder = M.write_model(tmp_path / "edge", cfg, seed=55)
    n = 150
    base = random_tokens(vocab, n, seed=12)
    reach = depth * (window - 1)            # every layer lets a token see window - 1 further back
    for back, seen in ((reach, True), (reach + 1, False)):
        other = list(base)
        other[n - 1 - back] = (other[n - 1 - back] + 1) % vocab
        ref = [M.plain_logits(folder, p)[-1] for p in (base, other)]
        assert (M.rel_err(ref[0], ref[1]) > 1e-6) == seen
        for sizes, tail in (([n], 0), ([9, 2, 31], 30)):
            rows = []
            for prompt in (base, other):
                runner, cache = M.make_runner(folder, backend, M.PAGE_SIZE[name], 30)
                steps = [([(1, part, [])], []) for part in cut(prompt[:n - tail - 1], sizes)]
                steps += [([(1, [t], [])], []) for t in prompt[n - tail - 1:-1]] + [([(1, prompt[-1:], [0])], [])]
                rows.append(replay(runner, cache, steps)[1][n - 1])
                held = len([p for p in cache.table(0, 1) if p >= 0])
                assert held <= -(-(window + max(sizes)) // M.PAGE_SIZE[name]) + 1
            for row, want in zip(rows, ref):
                assert M.rel_err(row, want) < 5e-5
            assert (M.rel_err(rows[0], rows[1]) > 1e-6) == seen


@pytest.mark.parametrize("backend", FLOAT_BACKENDS)
@pytest.mark.parametrize("name", ["b", "e"])
def test_a_state_slot_starts_from_zero_for_its_next_holder(folders, backend, name):
    """One slot: the second request gets the slot, the matrices and the convolution's kept inputs that the first one
    left; its first tokens, which the convolution pads with zeros, must not see them."""
    vocab = M.CONFIGS[name]["vocab"]
    runner, cache = M.make_runner(folders[name], backend, 16, 8, max_running=1)
    a, b = random_tokens(vocab, 40, seed=41), random_tokens(vocab, 25, seed=42)
    got = replay(runner, cache, [([(1, a, [39])], [1]), ([(2, b[:2], [0, 1])], []), ([(2, b[2:10], [0, 7])], []),
                                 ([(2, b[10:], [14])], [2])])
    check(got, {1: a, 2: b}, folders[name], backend)
    assert cache.slots.free_slots == 1


@pytest.mark.parametrize("backend", FLOAT_BACKENDS)
def test_greedy_generation_through_the_engine_and_its_scheduler(folders, backend):
    from simple_inference_amd import Engine, EngineConfig, SamplingParams
    name = "c"
    if backend == "twins":
        from twins import TwinKernels
        kernels, device = TwinKernels(), "cpu"
    else:
        from simple_inference_amd.kernels import HipKernels
        kernels, device = HipKernels(), "cuda:0"
    eng = Engine.from_folder(folders[name], EngineConfig(
        device=device, dtype="float32", max_seq_len=128, block_size=16, max_running=3, chunk_tokens=24, eos_id=-1,
        num_kv_blocks=20), kernels)
    assert "Tadinex" in eng.describe()
    prompts = [random_tokens(300, n, seed=300 + n) for n in (50, 3, 27, 41)]   # four requests for three slots
    reqs = [eng.add_request(p, params=SamplingParams(temperature=0.0, max_new_tokens=9)) for p in prompts]
    eng.run()
    cfg, w = M.read_model(folders[name])
    for req, prompt in zip(reqs, prompts):
        toks = list(prompt)
        assert len(req.generated) == 9
        for got in req.generated:
            logits = M.plain.forward(cfg, w, toks)[-1]
            want = int(torch.argmax(logits))
            assert got == want or float(logits[want] - logits[got]) < 1e-4 * float(logits.abs().max())
            toks.append(got)
    eng.cache.check()
    assert not eng.cache.lengths


def test_trace_replay_of_a_model_folder_on_the_cpu(folders):
    from simple_inference_amd.replay import TraceReplayer
    from twins import TwinKernels
    name = "a"
    rp = TraceReplayer(folders[name], "float32", 192, device="cpu", kernels=TwinKernels(), max_live=3)
    assert rp.describe().startswith("Tadinex")
    a, b = random_tokens(211, 70, seed=31), random_tokens(211, 33, seed=32)
    out = rp.step([{"id": "x", "tokens": a[:40], "want": [39]}, {"id": "y", "tokens": b, "want": [0, 32]}], ["y"])
    out2 = rp.step([{"id": "x", "tokens": a[40:], "want": [29]}, {"id": "z", "tokens": b[:2], "want": [1]}], ["x", "z"])
    ra, rb = M.plain_logits(folders[name], a), M.plain_logits(folders[name], b)
    assert M.rel_err(out, torch.stack([ra[39], rb[0], rb[32]])) < 5e-5
    assert M.rel_err(out2, torch.stack([ra[69], rb[1]])) < 5e-5
    assert not rp.ids and rp.cache.free_pages() == 12 and rp.cache.slots.free_slots == 3


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["a", "c"])
def test_bfloat16_generation_from_replayed_graphs_is_the_eager_one(folders, name):
    """The serving path: bfloat16, decode steps replayed from graphs, the host running ahead.  The tokens are those
    of eager steps, and each is the plain implementation's best token or ties with it within bfloat16's reach."""
    from simple_inference_amd import Engine, EngineConfig, SamplingParams
    folder = folders[name + "-all"]
    vocab = M.CONFIGS[name]["vocab"]
    prompts = [random_tokens(vocab, n, seed=400 + n) for n in (45, 70, 9)]
    runs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, EngineConfig(
            device="cuda:0", dtype="bfloat16", max_seq_len=256, block_size=16, max_running=4, chunk_tokens=64,
            eos_id=-1, use_graphs=graphs, run_ahead=graphs))
        reqs = [eng.add_request(p, params=SamplingParams(temperature=0.0, max_new_tokens=40)) for p in prompts]
        eng.run()
        runs[graphs] = [list(r.generated) for r in reqs]
        if graphs:
            assert eng.graphs is not None and eng.stats["graph_fallbacks"] == 0
    assert runs[True] == runs[False]
    cfg, w = M.read_model(folder)
    for prompt, generated in zip(prompts, runs[True]):
        toks = list(prompt)
        for got in generated:
            logits = M.plain.forward(cfg, w, toks)[-1]
            want = int(torch.argmax(logits))
            assert got == want or float(logits[want] - logits[got]) < 5e-2 * float(logits.abs().max())
            toks.append(got)
