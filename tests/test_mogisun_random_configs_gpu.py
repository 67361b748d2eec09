"""Seeded random Mogisun configurations through trace replay on the GPU, against the plain implementation: softmax
and linear attention in any order, head and value sizes of every kind (equal and unequal, multiples of 16 and not),
any grouping of heads, with and without a query temperature, decays that forget at once and that last, ranks of any
size, dense and routed feed-forwards with any number of experts and choices, with and without a shared expert,
layers without a feed-forward, loops anywhere (also none, also over everything, walked once to three times), with
and without a cap on the logits, widths and vocabularies that are no multiple of anything.  float32 routes as the
configuration says; bfloat16 chooses every expert (see ``mogisun_models.all_experts``), and where a deep or narrow
model errs more than the usual bound under bfloat16's rounding alone (the same replay with the torch twins of the
kernels, which round at the same places), the kernels may err up to twice that."""

import random

import pytest
import torch

import mogisun_models as M
from test_trace_run import collect, make_trace

pytestmark = pytest.mark.gpu


def random_layer(rng):
    if rng.random() < 0.5:
        dim = rng.choice([16, 24, 32, 40, 64, 80, 128])
        kv = rng.choice([1, 2, 3])
        mixer = {"dim": dim, "vdim": dim if rng.random() < 0.5 else rng.choice([8, 16, 24, 48, 72, 128]),
                 "heads": kv * rng.choice([1, 2, 3, 5]), "kv_heads": kv,
                 "scale": rng.choice([0.05, 0.125, 0.3, dim ** -0.5])}
        if rng.random() < 0.7:
            mixer["q_temp"] = {"coef": rng.choice([0.1, 0.5, 1.0]), "every": rng.choice([1, 3, 16, 30, 64, 1000])}
        kind = "attention"
    else:
        mixer = {"dim": rng.choice([8, 20, 32, 48, 64, 128]), "vdim": rng.choice([8, 12, 32, 64, 80, 128]),
                 "heads": rng.choice([1, 2, 3, 6]), "tau": rng.choice([0.5, 1.0, 4.0, 16.0, 64.0]),
                 "rank": rng.choice([1, 4, 7, 16, 32])}
        kind = "gla"
    pick = rng.random()
    if pick < 0.2:
        mlp = None
    elif pick < 0.55:
        mlp = {"kind": "dense", "ff": rng.choice([56, 96, 150, 192])}
    else:
        experts = rng.choice([2, 3, 8, 12, 20])
        mlp = {"kind": "moe", "router": {"experts": experts, "top": rng.choice([t for t in (1, 2, 3, 4) if t <= experts])},
               "expert": {"ff": rng.choice([8, 24, 32, 50, 64])}}
        if rng.random() < 0.6:
            mlp["shared"] = {"ff": rng.choice([16, 40, 64])}
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def random_config(seed):
    rng = random.Random(2000 + seed)
    shapes = [random_layer(rng) for _ in range(rng.choice([2, 3]))]
    n = rng.choice([2, 3, 4, 5])
    cfg = {"architecture": "Mogisun", "vocab": rng.choice([97, 257, 500, 1001]),
           "width": rng.choice([40, 72, 100, 128, 136, 192, 200, 264]), "norm": {"eps": rng.choice([1e-5, 1e-6, 3e-4])},
           "logit_scale": rng.choice([0.5, 1.0, 2.5]), "layers": [dict(rng.choice(shapes)) for _ in range(n)]}
    if rng.random() < 0.7:
        cfg["logit_softcap"] = rng.choice([4.0, 15.0, 50.0])
    if rng.random() < 0.8:
        start = rng.randrange(n)
        cfg["loop"] = {"start": start, "stop": rng.randrange(start + 1, n + 1), "times": rng.choice([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
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
