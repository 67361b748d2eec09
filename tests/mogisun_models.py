"""Small Mogisun configurations for the tests, their model folders, and runners over them.

The configurations differ from one another in every size and option: softmax attention with one key/value head per
query head, with several query heads a key/value head and with one key/value head for all; values narrower and
wider than the keys; with and without a query temperature; linear attention with key and value widths that differ,
with one head, with decays that forget within a few tokens (tau 1) and that last (tau 16), with ranks that are no
multiple of anything; experts with top 1, 2 and 3, with and without a shared expert; layers without a feed-forward;
no loop, a loop from the first layer, a loop walked once and three times; with and without a cap on the logits.
"""

from __future__ import annotations

import copy
import json

import torch
from safetensors import safe_open

import plain_mogisun as plain


def _att(heads, kv, dim, vdim, scale, temp=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv, "scale": scale, "vdim": vdim}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m}


def _gla(heads, dim, vdim, tau, rank):
    return {"type": "gla", "mixer": {"dim": dim, "heads": heads, "tau": tau, "vdim": vdim, "rank": rank}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=None):
    d = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def _layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


CONFIGS = {
    # a loop from the first layer, walked three times; top 1 without a shared expert; a layer without a feed-forward
    "a": {"architecture": "Mogisun", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "logit_scale": 0.7,
          "loop": {"start": 0, "stop": 2, "times": 3},
          "layers": [_layer(_gla(3, 24, 40, 4.0, 5), _moe(5, 1, 40)),
                     _layer(_att(4, 2, 32, 16, 0.3, (0.5, 7)), _dense(80)),
                     _layer(_gla(1, 8, 8, 1.0, 3), None)]},
    # no loop; values wider than keys; top 3 of 8 with a shared expert; no query temperature; capped logits
    "b": {"architecture": "Mogisun", "vocab": 160, "width": 128, "norm": {"eps": 3e-6}, "logit_scale": 3.0,
          "logit_softcap": 5.0,
          "layers": [_layer(_att(6, 3, 16, 48, 0.21), _moe(8, 3, 24, 72)),
                     _layer(_gla(2, 64, 64, 1.5, 8), _dense(136))]},
    # sizes at which the GPU takes its matrix-core attention and its few-row products; a loop in the middle walked twice
    "c": {"architecture": "Mogisun", "vocab": 300, "width": 128, "norm": {"eps": 1e-6}, "logit_scale": 1.0,
          "logit_softcap": 20.0, "loop": {"start": 1, "stop": 3, "times": 2},
          "layers": [_layer(_att(4, 1, 64, 64, 0.12, (0.3, 16)), _moe(6, 2, 64, 64)),
                     _layer(_gla(4, 32, 64, 16.0, 16), _dense(192)),
                     _layer(_att(4, 4, 32, 32, 0.2, (0.1, 50)), _dense(64)),
                     _layer(_gla(2, 64, 32, 8.0, 24), _moe(4, 2, 128))]},
    # a loop over all layers walked once; every query head its own key/value head
    "d": {"architecture": "Mogisun", "vocab": 97, "width": 48, "norm": {"eps": 1e-5},
          "loop": {"start": 0, "stop": 2, "times": 1},
          "layers": [_layer(_att(2, 2, 24, 24, 0.25, (1.0, 3)), None),
                     _layer(_gla(2, 16, 24, 2.0, 4), _moe(3, 2, 16, 8))]},
    # sizes that are multiples of nothing the kernels like: every vector path has to step aside
    "e": {"architecture": "Mogisun", "vocab": 131, "width": 100, "norm": {"eps": 2e-6}, "logit_scale": 1.3,
          "logit_softcap": 9.0, "loop": {"start": 1, "stop": 2, "times": 2},
          "layers": [_layer(_att(5, 5, 20, 12, 0.4, (0.2, 5)), _moe(7, 2, 36, 20)),
                     _layer(_gla(3, 12, 20, 3.0, 7), _dense(52)),
                     _layer(_att(3, 1, 12, 28, 0.3), _moe(2, 1, 10))]},
}

PAGE_SIZE = {"a": 8, "b": 16, "c": 16, "d": 4, "e": 16}


def all_experts(cfg):
    """The configuration with every expert chosen for every token: what remains of routing is the softmax over the
    logits, which does not jump.  (With fewer, two logits that nearly tie pick another expert under bfloat16's
    rounding of the router's input, and the outputs then differ by an expert, not by rounding.)"""
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if layer["mlp"] and layer["mlp"]["kind"] == "moe":
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return cfg


def write_model(folder, name_or_config, seed=0, std=0.08, spread=0.3, keep_rank=False, change=None):
    """config.json + model.safetensors with the package's random mode: matrices N(0, std), vectors (gains, biases)
    1 + N(0, spread).  The written config.json does not name the rank of the decays' low-rank pairs (the loader
    reads it from the tensors) unless ``keep_rank``.  ``change(tensors)`` may edit the tensors before they are
    written."""
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import build_model
    from simple_inference_amd.weights import random_tensors, write_model_folder

    cfg = copy.deepcopy(CONFIGS[name_or_config] if isinstance(name_or_config, str) else name_or_config)
    model, mcfg = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    tensors = random_tensors(model.expected_tensors(), seed, std, spread, "bfloat16")
    if change is not None:
        change(tensors)
    out = mcfg.to_dict()
    if not keep_rank:
        for layer in out["layers"]:
            layer["mixer"].pop("rank", None)
    write_model_folder(folder, out, tensors)
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
    return plain.logits(cfg, w, tokens).float()


def make_runner(folder, backend, page_size, num_pages, max_seq_len=1024, max_running=4):
    """(StepRunner, CacheManager) on 'twins' (CPU, float32), 'twins-bf16', 'hip-f32' or 'hip-bf16'."""
    from simple_inference_amd.cache import CacheManager
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import StepRunner, model_from_folder

    if backend.startswith("twins"):
        from twins import TwinKernels
        kernels, device, dtype = TwinKernels(), "cpu", "bfloat16" if backend.endswith("bf16") else "float32"
    else:
        from simple_inference_amd.kernels import HipKernels
        kernels, device = HipKernels(), "cuda:0"
        dtype = {"hip-f32": "float32", "hip-bf16": "bfloat16"}[backend]
    ecfg = EngineConfig(device=device, dtype=dtype, max_seq_len=max_seq_len, block_size=page_size,
                        num_kv_blocks=num_pages, max_running=max_running)
    model, _ = model_from_folder(folder, ecfg, kernels)
    cache = CacheManager(model.cache_layout(), page_size=page_size, num_pages=num_pages, max_running=max_running,
                         dtype=ecfg.torch_dtype, device=device)
    return StepRunner(model, cache, kernels, device, max_seq_len), cache


# float32: max |a - b| / max |b| over the logits; what differs is the order of additions (and the decays' powers
# over a long sequence).  bfloat16: 8 bits of mantissa through every product, with norms, softmax, the state and the
# residual in float32.  A row's error is the root mean square of a - b against the root mean square of all of b.
# Where a linear-attention head's output nearly cancels, its norm divides by a small number and the rounding of q, k
# and v weighs many times more than elsewhere, at that one position (at a sequence's first token the output is
# (q . k) v, whose norm keeps only the sign of q . k): so all rows but one (or but one in ten) must lie within the
# tolerance, and every row must be finite.  What happens at single places (a portion's first token, a page's border)
# is held to the float32 tolerance by the float32 runs of the same tests.
TOLERANCE = {"twins": 5e-5, "hip-f32": 5e-5, "twins-bf16": 4e-2, "hip-bf16": 4e-2}


def rel_err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


def rms_err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    rows = (a - b).reshape(-1, b.shape[-1]).pow(2).mean(-1).sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30)
    kept = rows.sort().values[:max(1, rows.numel() - max(1, rows.numel() // 10))]     # all but one row, or but a tenth
    return float(kept.max()) if bool(torch.isfinite(rows).all()) else float("inf")


def err(a, b, backend):
    return rms_err(a, b) if "bf16" in backend else rel_err(a, b)
