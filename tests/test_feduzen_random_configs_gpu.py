"""Seeded random Feduzen configurations through trace replay on the GPU, against the plain implementation: head
and value sizes of every kind (equal and unequal, multiples of 16 and not), any grouping of heads, full, partial and
no rotation, blocks from one position to longer than any request, layers of several shapes, layers without a
feed-forward, every pattern of shared weights, widths and vocabularies that are no multiple of anything."""

import random

import pytest
import torch

import feduzen_models as F
from test_trace_run import collect, make_trace

pytestmark = pytest.mark.gpu


def random_mixer(rng, seed):
    dim = rng.choice([16, 24, 32, 40, 64, 80, 96, 128])
    vdim = dim if rng.random() < 0.5 else rng.choice([8, 16, 24, 48, 64, 72, 128])
    kv = rng.choice([1, 2, 3])
    heads = kv * rng.choice([1, 2, 3, 5])
    m = {"dim": dim, "vdim": vdim, "heads": heads, "kv_heads": kv, "scale": rng.choice([0.05, 0.125, 0.3, dim ** -0.5])}
    if rng.random() < 0.9:
        m["mask"] = {"size": rng.choice([1, 3, 16, 30, 47, 64, 100, 1000])}
    if rng.random() < 0.9:
        dims = rng.choice([2, 8, 16, dim // 2 // 2 * 2, dim])
        rot = {"dims": min(dims, dim), "base": rng.choice([100.0, 10000.0, 50000.0])}
        if rng.random() < 0.6:
            rot["scaling"] = {"factor": rng.choice([2.0, 8.0]), "low": 1.0, "high": rng.choice([2.0, 4.0]),
                              "original": rng.choice([16, 64, 256])}
        m["rot"] = rot
    return m


def random_config(seed):
    rng = random.Random(1000 + seed)
    shapes = [(random_mixer(rng, seed), rng.choice([None, 56, 96, 150, 192])) for _ in range(rng.choice([1, 2]))]
    layers, owners = [], []
    for i in range(rng.choice([2, 3, 4, 5])):
        if owners and rng.random() < 0.5:
            j = rng.choice(owners)
            layers.append(dict(layers[j], weights_of=j))
        else:
            mixer, ff = rng.choice(shapes)
            layers.append({"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None})
            owners.append(i)
    return {"architecture": "Feduzen", "vocab": rng.choice([97, 257, 500, 1001]),
            "width": rng.choice([40, 72, 100, 128, 136, 192, 200, 264]), "embedding": {"scale": rng.choice([0.5, 1.0, 4.0])},
            "norm": {"eps": rng.choice([1e-5, 1e-6, 3e-4])}, "layers": layers}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_random_configuration_replays_like_the_plain_implementation(tmp_path, seed, dtype):
    from simple_inference_amd.replay import TraceReplayer

    cfg = random_config(seed)
    print("configuration", seed, cfg, flush=True)
    folder = F.write_model(tmp_path, cfg, seed=300 + seed, std=0.07, spread=0.3)
    steps, prompts, most = make_trace(cfg["vocab"], lengths=(50, 33, 71, 20, 64))
    page = (8, 16, 32, 64)[seed % 4]
    rp = TraceReplayer(folder, dtype, most, block_size=page, max_live=4)
    got = collect(steps, lambda st: rp.step(st["entries"], st["end"]).float().cpu().numpy())
    tol = F.TOLERANCE["hip-f32" if dtype == "float32" else "hip-bf16"]
    for r, toks in prompts.items():
        ref = F.plain_logits(folder, toks)
        mine = torch.stack([torch.as_tensor(got[r][p]) for p in range(len(toks))])
        assert F.rel_err(mine, ref) <= tol, (r, F.rel_err(mine, ref))
    assert all(rp.cache.free_pages(g) == -(-most // page) for g in range(len(rp.cache.groups))) and not rp.ids
