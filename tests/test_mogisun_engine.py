"""The Mogisun design through the engine's own step function, cache manager, state slots, scheduler and entry point,
against the plain implementation: every way of cutting the work must give the logits of the whole sequence.

The same tests run on the CPU with the torch twins of the kernels (they test configuration, plan, parts, cache
manager, state slots and batch layout) and on the GPU with the HIP kernels in float32 and bfloat16.  The bfloat16
runs route every token to all experts (see ``mogisun_models.all_experts``); routing to fewer is tested in float32.
"""

import json

import pytest
import torch

import mogisun_models as M
from helpers import random_tokens
from simple_inference_amd.engine import StepEntry

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
        out[name] = M.write_model(tmp_path_factory.mktemp(f"mogisun_{name}"), name, seed=5 + i)
        out[name + "-all"] = M.write_model(tmp_path_factory.mktemp(f"mogisun_{name}_all"), M.all_experts(M.CONFIGS[name]),
                                           seed=5 + i)
    return out


def folder_for(folders, name, backend):
    return folders[name + "-all"] if "bf16" in backend else folders[name]


def replay(runner, cache, schedule):
    """schedule: steps of (entries, ends); an entry is (req, tokens, want).  Returns {req: {position: logits}}."""
    got, fed = {}, {}
    for entries, ends in schedule:
        batch = []
        for req, tokens, want in entries:
            if req not in cache.lengths:
                cache.admit(req)
                fed[req] = 0
            batch.append(StepEntry(req, tokens, want))
        logits = runner.run(batch)
        r = 0
        for req, tokens, want in entries:
            for w in want:
                got.setdefault(req, {})[fed[req] + w] = logits[r].float().cpu()
                r += 1
            fed[req] += len(tokens)
        for req in ends:
            cache.release(req)
        cache.check()
    return got


def check(got, prompts, folder, backend):
    for req, rows in got.items():
        ref = M.plain_logits(folder, prompts[req])
        pos = sorted(rows)
        assert M.err(torch.stack([rows[p] for p in pos]), ref[pos], backend) <= M.TOLERANCE[backend], req


def cut(tokens, sizes):
    parts, k, j = [], 0, 0
    while k < len(tokens):
        n = min(sizes[j % len(sizes)], len(tokens) - k)
        parts.append(tokens[k:k + n])
        k += n
        j += 1
    return parts


# ---------------------------------------------------------------------------------------------------------------
def test_configuration_reads_every_size_and_refuses_what_it_does_not_know():
    from simple_inference_amd.config import ConfigError, MogisunConfig, architecture_of
    cfg = MogisunConfig.from_dict(M.CONFIGS["c"])
    assert architecture_of(M.CONFIGS["c"]).name == "Mogisun"
    assert (cfg.vocab, cfg.width, cfg.norm_eps, cfg.logit_scale, cfg.logit_softcap) == (300, 128, 1e-6, 1.0, 20.0)
    assert (cfg.loop.start, cfg.loop.stop, cfg.loop.times) == (1, 3, 2)
    a, g = cfg.layers[0].mixer, cfg.layers[3].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.q_temp.coef, a.q_temp.every) == (4, 1, 64, 64, 0.12, 0.3, 16)
    assert (g.heads, g.dim, g.vdim, g.tau, g.rank) == (2, 64, 32, 8.0, 24)
    m = cfg.layers[0].mlp
    assert (m.experts, m.top, m.ff, m.shared_ff) == (6, 2, 64, 64) and cfg.layers[3].mlp.shared_ff is None
    assert MogisunConfig.from_dict(cfg.to_dict()) == cfg
    assert [i for i, _ in cfg.run_order()] == [0, 1, 2, 1, 2, 3]
    assert [e for _, e in cfg.run_order()] == [False, True, False, True, False, False]
    b = MogisunConfig.from_dict(M.CONFIGS["b"])
    assert b.loop is None and b.layers[0].mixer.q_temp is None
    assert MogisunConfig.from_dict(M.CONFIGS["a"]).layers[2].mlp is None
    assert MogisunConfig.from_dict(M.CONFIGS["a"]).logit_softcap is None

    def changed(path, value):
        c = json.loads(json.dumps(M.CONFIGS["c"]))
        at = c
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        return c
    for path, value in [(("layers", 0, "type"), "recurrent"), (("layers", 1, "mlp", "kind"), "routed"),
                        (("layers", 0, "mixer", "kv_heads"), 3), (("layers", 0, "mlp", "router", "top"), 7),
                        (("layers", 1, "mixer", "tau"), 0), (("loop", "stop"), 5), (("loop", "start"), 3),
                        (("loop", "times"), 0), (("norm", "eps"), 0), (("logit_softcap",), -1.0),
                        (("layers", 0, "mixer", "q_temp", "every"), 0)]:
        with pytest.raises(ConfigError):
            MogisunConfig.from_dict(changed(path, value))
    c = json.loads(json.dumps(M.CONFIGS["c"]))
    del c["layers"][0]["mixer"]["scale"]
    with pytest.raises(ConfigError, match="scale"):
        MogisunConfig.from_dict(c)


def test_plan_walks_the_loop_with_caches_and_states_of_its_own(folders):
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import build_model
    model, _ = build_model(M.CONFIGS["c"], EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    assert model.order == [0, 1, 2, 1, 2, 3] and len(model.layers) == 4
    assert model.entries == {1: 0, 3: 0} and len(model.stream_ops) == 1
    names = set(model.expected_tensors())
    assert {"embed", "head", "final.norm", "loop.in", "l0.mix.q.b", "l0.mix.g", "l0.mix.o.b", "l1.mix.a2.b", "l1.mix.norm",
            "l0.rg1", "l0.rg2.b", "l0.mlp.e5.down", "l0.mlp.router", "l0.mlp.shared.sg", "l3.mlp.e3.gate"} <= names
    assert "l3.mlp.shared.gate" not in names and "l0.mlp.e6.gate" not in names
    layout = model.cache_layout()
    # two shapes of softmax attention: two groups; the looped one has a slab for each walk.  A state per run of a
    # linear-attention layer.
    assert layout.run_kv == [(0, 0), None, (1, 0), None, (1, 1), None]
    assert layout.run_state == [None, 0, None, 1, None, 2]
    assert [s.shape for s in layout.states] == [(4, 32, 64), (4, 32, 64), (2, 64, 32)]
    model, _ = build_model(M.CONFIGS["b"], EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    assert model.entries == {} and "loop.in" not in model.expected_tensors()


def test_the_rank_of_the_decay_is_read_from_the_checkpoint(folders, tmp_path):
    with open(f"{folders['a']}/config.json") as f:
        assert all("rank" not in layer["mixer"] for layer in json.load(f)["layers"])
    runner, _ = M.make_runner(folders["a"], "twins", 8, 4)
    assert [runner.model.layers[i].mixer.rank for i in (0, 2)] == [5, 3]
    # a configuration that names another rank than the tensors have is refused
    other = json.loads(json.dumps(M.CONFIGS["a"]))
    kept = M.write_model(tmp_path / "kept", other, keep_rank=True)
    with open(f"{kept}/config.json") as f:
        cfg = json.load(f)
    cfg["layers"][0]["mixer"]["rank"] = 6
    with open(f"{kept}/config.json", "w") as f:
        json.dump(cfg, f)
    from simple_inference_amd.weights.loader import WeightError
    with pytest.raises(WeightError, match="l0.mix.a1"):
        M.make_runner(kept, "twins", 8, 4)


def test_the_residual_after_every_run_of_a_layer_is_the_plain_one(folders):
    from simple_inference_amd.parts.context import ResidualStream
    for name in ("c", "a"):
        runner, cache = M.make_runner(folders[name], "twins", M.PAGE_SIZE[name], 32)
        toks = random_tokens(M.CONFIGS[name]["vocab"], 45, seed=3)
        cfg, w = M.read_model(folders[name])
        want = M.plain.residuals(cfg, w, toks)
        cache.admit(1)
        ctx = runner.build_context([StepEntry(1, toks, [])])
        caches = cache.layer_caches(ctx.block_tables)
        model = runner.model
        first = model.embedding.forward(ctx)
        stream = ResidualStream(first.clone())
        for e, li in enumerate(model.order):
            if e in model.entries:
                model.stream_ops[model.entries[e]].forward(stream, ctx, first)
            model.layers[li].block.forward(stream, ctx, caches[e])
            stream.settle(runner.kernels)
            assert M.rel_err(stream.residual, want[e]) < 1e-5, (name, e)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c", "d", "e"])
def test_whole_prompt_then_token_by_token(folders, backend, name):
    folder = folder_for(folders, name, backend)
    runner, cache = M.make_runner(folder, backend, M.PAGE_SIZE[name], 40)
    toks = random_tokens(M.CONFIGS[name]["vocab"], 130, seed=7)
    n0 = 61        # the decoded tokens pass page borders and steps of the query temperature of every configuration
    schedule = [([(1, toks[:n0], list(range(n0)))], [])] + [([(1, [t], [0])], []) for t in toks[n0:]]
    got = replay(runner, cache, schedule)
    check(got, {1: toks}, folder, backend)
    # and all of it token by token, from the first token on
    cache.release(1)
    got = replay(runner, cache, [([(2, [t], [0])], []) for t in toks[:50]])
    check(got, {2: toks[:50]}, folder, backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name,sizes", [("a", [2, 5, 23, 1, 24, 3]), ("b", [19, 2, 2, 40, 1, 7]), ("c", [50, 17, 2, 33, 64]),
                                        ("d", [3, 2, 2, 31]), ("e", [7, 2, 45, 1, 16])])
def test_portions_cut_anywhere_down_to_two_tokens(folders, backend, name, sizes):
    folder = folder_for(folders, name, backend)
    runner, cache = M.make_runner(folder, backend, M.PAGE_SIZE[name], 40)
    toks = random_tokens(M.CONFIGS[name]["vocab"], 141, seed=8)
    got = replay(runner, cache, [([(1, part, list(range(len(part))))], []) for part in cut(toks, sizes)])
    check(got, {1: toks}, folder, backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(folders, backend, name):
    """Up to three live requests of very different lengths: portions beside single tokens, requests left out of
    steps, requests that end and whose pages and state slots the next ones get (a state left behind by the slot's
    last holder would show in the first token of the next).  The pool holds far less than all."""
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


def _far_memory(tensors):
    """Weights with which a token far back still weighs in the last logits: the linear layers' decays are pushed
    close to 1, so that their states keep what they were given hundreds of tokens ago."""
    for name, t in tensors.items():
        if name.endswith(".mix.a2.b"):
            t.fill_(9.0)


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_far_token_reaches_the_last_logits_however_the_prompt_is_cut(folders, backend, tmp_path):
    """Two prompts that differ in one token hundreds of positions back, at a page's first or last place: the last
    logits differ by a hundred times the float32 tolerance, and by what the plain implementation says, in whole
    prompts, portions and decoding: a key or a state's share that got lost on the way would show."""
    cfg = M.all_experts(M.CONFIGS["c"]) if "bf16" in backend else M.CONFIGS["c"]
    folder = M.write_model(tmp_path / "far", cfg, seed=77, change=_far_memory)
    base = random_tokens(300, 420, seed=10)
    for place in (16, 31, 0):
        other = list(base)
        other[place] = (other[place] + 1) % 300
        ref = [M.plain_logits(folder, p)[-1] for p in (base, other)]
        assert M.rel_err(ref[0], ref[1]) > 5e-3      # the far token matters
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
                assert M.rel_err(rows[0], rows[1]) > 4e-3


@pytest.mark.parametrize("backend", FLOAT_BACKENDS)
def test_a_state_slot_starts_from_zero_for_its_next_holder(folders, backend):
    """One slot: the second request gets the slot, and the state rows, that the first one left."""
    name = "b"
    runner, cache = M.make_runner(folders[name], backend, 16, 8, max_running=1)
    a, b = random_tokens(160, 40, seed=41), random_tokens(160, 25, seed=42)
    got = replay(runner, cache, [([(1, a, [39])], [1]), ([(2, b[:10], [9])], []), ([(2, b[10:], [14])], [2])])
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
    assert "Mogisun" in eng.describe()
    prompts = [random_tokens(300, n, seed=300 + n) for n in (50, 3, 27, 41)]   # four requests for three slots
    reqs = [eng.add_request(p, params=SamplingParams(temperature=0.0, max_new_tokens=9)) for p in prompts]
    eng.run()
    cfg, w = M.read_model(folders[name])
    for req, prompt in zip(reqs, prompts):
        toks = list(prompt)
        assert len(req.generated) == 9
        for got in req.generated:
            logits = M.plain.logits(cfg, w, toks)[-1]
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
    assert rp.describe().startswith("Mogisun")
    a, b = random_tokens(211, 70, seed=31), random_tokens(211, 33, seed=32)
    out = rp.step([{"id": "x", "tokens": a[:40], "want": [39]}, {"id": "y", "tokens": b, "want": [0, 32]}], ["y"])
    out2 = rp.step([{"id": "x", "tokens": a[40:], "want": [29]}, {"id": "z", "tokens": b[:2], "want": [1]}], ["x", "z"])
    ra, rb = M.plain_logits(folders[name], a), M.plain_logits(folders[name], b)
    assert M.rel_err(out, torch.stack([ra[39], rb[0], rb[32]])) < 5e-5
    assert M.rel_err(out2, torch.stack([ra[69], rb[1]])) < 5e-5
    assert not rp.ids and rp.cache.free_pages() == 12 and rp.cache.slots.free_slots == 3


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["b", "c"])
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
            logits = M.plain.logits(cfg, w, toks)[-1]
            want = int(torch.argmax(logits))
            assert got == want or float(logits[want] - logits[got]) < 5e-2 * float(logits.abs().max())
            toks.append(got)
