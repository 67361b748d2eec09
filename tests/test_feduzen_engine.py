"""The Feduzen design through the engine's own step function, cache manager, scheduler and entry point, against the
plain implementation: every way of cutting the work must give the logits of the whole sequence.

The same tests run on the CPU with the torch twins of the kernels (they test configuration, plan, parts, cache
manager and batch layout) and on the GPU with the HIP kernels in float32 and bfloat16.
"""

import json

import pytest
import torch

import feduzen_models as F
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
    return {name: F.write_model(tmp_path_factory.mktemp(f"feduzen_{name}"), name, seed=5 + i)
            for i, name in enumerate(F.CONFIGS)}


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
        ref = F.plain_logits(folder, prompts[req])
        pos = sorted(rows)
        assert F.rel_err(torch.stack([rows[p] for p in pos]), ref[pos]) <= F.TOLERANCE[backend], req


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
    from simple_inference_amd.config import ConfigError, FeduzenConfig, architecture_of
    cfg = FeduzenConfig.from_dict(F.CONFIGS["b"])
    assert architecture_of(F.CONFIGS["b"]).name == "Feduzen"
    assert (cfg.vocab, cfg.width, cfg.embedding_scale, cfg.norm_eps) == (160, 128, 0.6, 3e-6)
    m = cfg.layers[1].mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.chunk, m.rot.dims, m.rot.base) == (2, 1, 64, 64, 0.09, 37, 16, 20000.0)
    assert (m.rot.scaling.factor, m.rot.scaling.low, m.rot.scaling.high, m.rot.scaling.original) == (2.0, 1.0, 8.0, 64)
    assert [cfg.owner_of(i) for i in range(4)] == [0, 1, 1, 0] and cfg.layers[0].mlp.ff == 72
    assert FeduzenConfig.from_dict(cfg.to_dict()) == cfg
    assert FeduzenConfig.from_dict(F.CONFIGS["a"]).layers[1].mlp is None
    d = FeduzenConfig.from_dict(F.CONFIGS["d"]).layers[0].mixer
    assert d.chunk is None and d.rot is None

    def changed(path, value):
        c = json.loads(json.dumps(F.CONFIGS["b"]))
        at = c
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        return c
    for path, value in [(("layers", 0, "type"), "recurrent"), (("layers", 0, "mlp", "kind"), "routed"),
                        (("layers", 2, "weights_of"), 2), (("layers", 2, "weights_of"), 0),   # another layer's shape
                        (("layers", 1, "mixer", "heads"), 3), (("layers", 0, "mixer", "rot", "dims"), 18),
                        (("layers", 0, "mixer", "mask", "size"), 0), (("norm", "eps"), 0)]:
        with pytest.raises(ConfigError):
            FeduzenConfig.from_dict(changed(path, value))
    c = json.loads(json.dumps(F.CONFIGS["b"]))
    del c["layers"][0]["mixer"]["scale"]
    with pytest.raises(ConfigError, match="scale"):
        FeduzenConfig.from_dict(c)


def test_plan_runs_a_shared_layer_again_with_a_cache_of_its_own(folders):
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import build_model
    model, cfg = build_model(F.CONFIGS["b"], EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    assert model.order == [0, 1, 1, 0] and len(model.layers) == 2
    names = set(model.expected_tensors())
    assert {"embed", "head", "final.norm", "l0.mix.q.b", "l1.mix.k.norm", "l1.mix.sink", "l0.mlp.up", "l1.norm2"} <= names
    assert not any(n.startswith(("l2.", "l3.")) for n in names)
    layout = model.cache_layout()
    # two shapes of mixer: two groups, each with a slab for every run of its layers
    assert len(layout.kv_groups) == 2 and layout.kv_slabs == [2, 2]
    assert layout.run_kv == [(0, 0), (1, 0), (1, 1), (0, 1)]
    assert {(g.head_dim, g.value_dim, g.chunk) for g in layout.kv_groups} == {(16, 48, 20), (64, 64, 37)}
    assert cfg.num_parameters() == sum(torch.Size(s.shape).numel() for s in model.expected_tensors().values())
    # a layer without a feed-forward has neither its tensors nor its norm
    model, _ = build_model(F.CONFIGS["a"], EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    assert "l1.norm1" in model.expected_tensors() and "l1.norm2" not in model.expected_tensors()
    assert "l1.mlp.up" not in model.expected_tensors() and model.order == [0, 1, 0]


def test_the_residual_after_every_layer_is_the_plain_one(folders):
    """Layer by layer, in float32 on the CPU: what the block adds is the norm of the sublayer's output."""
    from twins import TwinKernels
    from simple_inference_amd.parts.context import ResidualStream
    name = "b"
    runner, cache = F.make_runner(folders[name], "twins", F.PAGE_SIZE[name], 32)
    toks = random_tokens(F.CONFIGS[name]["vocab"], 45, seed=3)
    cfg, w = F.read_model(folders[name])
    _, want = F.plain.forward(cfg, w, toks, keep_layers=True)
    cache.admit(1)
    ctx = runner.build_context([StepEntry(1, toks, [])])
    caches = cache.layer_caches(ctx.block_tables)
    model = runner.model
    stream = ResidualStream(model.embedding.forward(ctx))
    for e, li in enumerate(model.order):
        model.layers[li].block.forward(stream, ctx, caches[e])
        assert stream.raw_delta is None
        assert F.rel_err(stream.residual, want[e]) < 1e-5, e


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_whole_prompt_then_token_by_token(folders, backend, name):
    runner, cache = F.make_runner(folders[name], backend, F.PAGE_SIZE[name], 40)
    toks = random_tokens(F.CONFIGS[name]["vocab"], 130, seed=7)
    n0 = 61        # the decoded tokens pass the borders of pages and of blocks of every configuration
    schedule = [([(1, toks[:n0], list(range(n0)))], [])] + [([(1, [t], [0])], []) for t in toks[n0:]]
    got = replay(runner, cache, schedule)
    check(got, {1: toks}, folders[name], backend)
    # and all of it token by token, from the first token on
    cache.release(1)
    got = replay(runner, cache, [([(2, [t], [0])], []) for t in toks[:50]])
    check(got, {2: toks[:50]}, folders[name], backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name,sizes", [("a", [2, 5, 23, 1, 24, 3]), ("b", [19, 2, 2, 40, 1, 7]), ("c", [50, 17, 2, 33, 64])])
def test_portions_cut_anywhere_down_to_two_tokens(folders, backend, name, sizes):
    runner, cache = F.make_runner(folders[name], backend, F.PAGE_SIZE[name], 40)
    toks = random_tokens(F.CONFIGS[name]["vocab"], 141, seed=8)
    got = replay(runner, cache, [([(1, part, list(range(len(part))))], []) for part in cut(toks, sizes)])
    check(got, {1: toks}, folders[name], backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(folders, backend, name):
    """Up to four live requests of very different lengths: portions beside single tokens, requests left out of
    steps, requests that end and whose pages and slots the next ones get.  The pool holds far less than all."""
    vocab = F.CONFIGS[name]["vocab"]
    lengths = [90, 7, 133, 41, 1, 66, 30]
    prompts = {i + 1: random_tokens(vocab, n, seed=100 + i) for i, n in enumerate(lengths)}
    plans = {r: cut(t[:-4], [11 + r, 2, 29]) + [[x] for x in t[-4:]] if len(t) > 4 else [[x] for x in t]
             for r, t in prompts.items()}
    waiting, live, schedule = list(prompts), [], []
    while waiting or live:
        while waiting and len(live) < 4:
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
    page = F.PAGE_SIZE[name]
    pool = sum(sorted(-(-n // page) for n in lengths)[-4:]) + 1
    runner, cache = F.make_runner(folders[name], backend, page, pool, max_running=4)
    got = replay(runner, cache, schedule)
    check(got, prompts, folders[name], backend)
    assert all(cache.free_pages(g) == pool for g in range(len(cache.groups))) and not cache.slots.slot_of
    # each alone gives the same (float32: to the last bits of the sums' order)
    if backend in ("twins", "hip-f32"):
        for r in (3, 6):
            solo = replay(runner, cache, [([(50 + r, prompts[r], list(range(len(prompts[r]))))], [50 + r])])
            for p, row in solo[50 + r].items():
                assert F.rel_err(row, got[r][p]) < 2e-5


@pytest.mark.parametrize("backend", FLOAT_BACKENDS)
def test_a_block_mask_gives_pages_back_and_keeps_what_is_still_seen(folders, backend):
    """Blocks of 24 positions over pages of 8: once a step starts in a new block, the pages of the blocks before go
    back to the pool (and are handed to another request at once), and nothing that is still seen goes with them."""
    name = "a"
    runner, cache = F.make_runner(folders[name], backend, 8, 9, max_running=2)
    a, b = random_tokens(211, 100, seed=21), random_tokens(211, 60, seed=22)
    schedule, ka, kb = [], 0, 0
    for na, nb in [(23, 5), (2, 19), (30, 1), (1, 1), (20, 24), (24, 10)]:
        schedule.append(([(1, a[ka:ka + na], list(range(na))), (2, b[kb:kb + nb], list(range(nb)))], []))
        ka, kb = ka + na, kb + nb
    got = replay(runner, cache, schedule)
    check(got, {1: a[:ka], 2: b[:kb]}, folders[name], backend)
    # request 1's last step began at 76, in the block from 72: the nine pages below went back, and it holds the four
    # that reach from 72 to its end at 100
    assert [p >= 0 for p in cache.table(0, 1)] == [False] * 9 + [True] * 4
    assert [p >= 0 for p in cache.table(0, 2)] == [False] * 6 + [True] * 2
    # 100 + 60 positions would be 21 pages; the pool has 9
    assert cache.free_pages(0) == 9 - 4 - 2


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding_over_many_blocks(folders, backend):
    name = "c"
    runner, cache = F.make_runner(folders[name], backend, 16, 8)
    toks = random_tokens(300, 330, seed=9)
    wanted = {5, 49, 50, 51, 99, 100, 149, 150, 200, 249, 250, 299, 300, 329}
    schedule = [([(1, toks[:3], [0, 1, 2])], [])] + [([(1, [t], [0] if 3 + i in wanted else [])], [])
                                                    for i, t in enumerate(toks[3:])]
    got = replay(runner, cache, schedule)
    assert set(got[1]) == wanted | {0, 1, 2}
    check(got, {1: toks}, folders[name], backend)


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_far_token_decides_the_logits_only_inside_its_block(folders, backend):
    """Two prompts that differ in one far token.  While the last token's block still holds the differing place the
    logits differ; once it lies one position before the block's start they must not differ by a bit of float32,
    whatever the portions were."""
    name = "c"            # blocks of 50 positions in every layer
    toks = random_tokens(300, 150, seed=10)
    for place, reaches in [(100, True), (99, False), (0, False)]:
        other = list(toks)
        other[place] = (other[place] + 1) % 300
        rows = []
        for prompt in (toks, other):
            runner, cache = F.make_runner(folders[name], backend, 16, 12)
            got = replay(runner, cache, [([(1, part, [len(part) - 1])], []) for part in cut(prompt, [37, 2, 61])])
            rows.append(got[1][149])
        if reaches:
            assert F.rel_err(rows[0], rows[1]) > 1e-3
        else:
            assert torch.equal(rows[0], rows[1]) or F.rel_err(rows[0], rows[1]) < (1e-6 if "bf16" not in backend else 2e-2)


@pytest.mark.parametrize("backend", FLOAT_BACKENDS)
def test_greedy_generation_through_the_engine_and_its_scheduler(folders, backend):
    from simple_inference_amd import Engine, EngineConfig, SamplingParams
    name = "b"
    if backend == "twins":
        from twins import TwinKernels
        kernels, device = TwinKernels(), "cpu"
    else:
        from simple_inference_amd.kernels import HipKernels
        kernels, device = HipKernels(), "cuda:0"
    eng = Engine.from_folder(folders[name], EngineConfig(
        device=device, dtype="float32", max_seq_len=128, block_size=16, max_running=3, chunk_tokens=24, eos_id=-1,
        num_kv_blocks=20), kernels)
    assert "Feduzen" in eng.describe()
    prompts = [random_tokens(160, n, seed=300 + n) for n in (50, 3, 27, 41)]   # four requests for three slots
    reqs = [eng.add_request(p, params=SamplingParams(temperature=0.0, max_new_tokens=9)) for p in prompts]
    eng.run()
    cfg, w = F.read_model(folders[name])
    for req, prompt in zip(reqs, prompts):
        toks = list(prompt)
        assert len(req.generated) == 9
        for got in req.generated:
            logits = F.plain.forward(cfg, w, toks)[-1]
            want = int(torch.argmax(logits))
            assert got == want or float(logits[want] - logits[got]) < 1e-4 * float(logits.abs().max())
            toks.append(got)
    eng.cache.check()
    assert not eng.cache.lengths


def test_trace_replay_of_a_model_folder_on_the_cpu(folders):
    from simple_inference_amd.replay import TraceReplayer
    from twins import TwinKernels
    name = "a"
    rp = TraceReplayer(folders[name], "float32", 192, device="cpu", kernels=TwinKernels())
    assert rp.describe().startswith("Feduzen")
    a, b = random_tokens(211, 70, seed=31), random_tokens(211, 33, seed=32)
    out = rp.step([{"id": "x", "tokens": a[:40], "want": [39]}, {"id": "y", "tokens": b, "want": [0, 32]}], ["y"])
    out2 = rp.step([{"id": "x", "tokens": a[40:], "want": [29]}, {"id": "z", "tokens": b[:2], "want": [1]}], ["x", "z"])
    ra, rb = F.plain_logits(folders[name], a), F.plain_logits(folders[name], b)
    assert F.rel_err(out, torch.stack([ra[39], rb[0], rb[32]])) < 3e-5
    assert F.rel_err(out2, torch.stack([ra[69], rb[1]])) < 3e-5
    assert not rp.ids and rp.cache.free_pages() == 12


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["b", "c"])
def test_bfloat16_generation_from_replayed_graphs_is_the_eager_one(folders, name):
    """The serving path: bfloat16, decode steps replayed from graphs, the host running ahead.  The tokens are those
    of eager steps, and each is the plain implementation's best token or ties with it within bfloat16's reach."""
    from simple_inference_amd import Engine, EngineConfig, SamplingParams
    vocab = F.CONFIGS[name]["vocab"]
    prompts = [random_tokens(vocab, n, seed=400 + n) for n in (45, 70, 9)]
    runs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folders[name], EngineConfig(
            device="cuda:0", dtype="bfloat16", max_seq_len=256, block_size=16, max_running=4, chunk_tokens=64,
            eos_id=-1, use_graphs=graphs, run_ahead=graphs))
        reqs = [eng.add_request(p, params=SamplingParams(temperature=0.0, max_new_tokens=40)) for p in prompts]
        eng.run()
        runs[graphs] = [list(r.generated) for r in reqs]
        if graphs:
            assert eng.graphs is not None and eng.stats["graph_fallbacks"] == 0
    assert runs[True] == runs[False]
    cfg, w = F.read_model(folders[name])
    for prompt, generated in zip(prompts, runs[True]):
        toks = list(prompt)
        for got in generated:
            logits = F.plain.forward(cfg, w, toks)[-1]
            want = int(torch.argmax(logits))
            assert got == want or float(logits[want] - logits[got]) < 4e-2 * float(logits.abs().max())
            toks.append(got)
