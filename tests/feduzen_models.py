"""Small Feduzen configurations for the tests, their model folders, and runners over them.

The configurations differ from one another in every size and option: head counts and groupings (one key/value
head per query head, several query heads a key/value head), value heads narrower and wider than the keys, full and
partial rotation with and without frequency scaling, score scales that are not 1/sqrt(dim), block masks whose size
is no multiple of a page, layers without a feed-forward, layers that differ from one another (two cache groups),
and layers that run another layer's weights once more.
"""

from __future__ import annotations

import copy
import json

import torch
from safetensors import safe_open

import plain_feduzen as plain


def _mixer(heads, kv, dim, vdim, scale, size=None, rot=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv, "scale": scale, "vdim": vdim}
    if size is not None:
        m["mask"] = {"size": size}
    if rot is not None:
        m["rot"] = rot
    return m


def _layer(mixer, ff=None, weights_of=None):
    d = {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


_ROT_FULL = {"dims": 32, "base": 10000.0}
_ROT_PART = {"dims": 8, "base": 3000.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 16}}
_ROT_16 = {"dims": 16, "base": 20000.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 8.0, "original": 64}}

_A0 = _mixer(3, 3, 32, 16, 0.3, 24, _ROT_FULL)
_B0 = _mixer(4, 2, 16, 48, 0.21, 20, _ROT_PART)
_B1 = _mixer(2, 1, 64, 64, 0.09, 37, _ROT_16)
_C0 = _mixer(6, 2, 32, 32, 0.2, 50, _ROT_16)
_D0 = _mixer(2, 2, 24, 24, 0.25)

CONFIGS = {
    # values narrower than keys, every query head its own key/value head, full rotation without scaling, a layer
    # without a feed-forward, a layer run twice
    "a": {"architecture": "Feduzen", "vocab": 211, "width": 96, "embedding": {"scale": 1.7}, "norm": {"eps": 1e-5},
          "layers": [_layer(_A0, 80), _layer(_A0, None), _layer(_A0, 80, weights_of=0)]},
    # values wider than keys, partial rotation with scaling, layers of two shapes (two cache groups), the shared
    # layers not in the order of their owners
    "b": {"architecture": "Feduzen", "vocab": 160, "width": 128, "embedding": {"scale": 0.6}, "norm": {"eps": 3e-6},
          "layers": [_layer(_B0, 72), _layer(_B1, 136), _layer(_B1, 136, weights_of=1), _layer(_B0, 72, weights_of=0)]},
    # sizes at which the GPU takes its matrix-core attention and its few-row products (multiples of 64 and 16)
    "c": {"architecture": "Feduzen", "vocab": 300, "width": 128, "embedding": {"scale": 2.5}, "norm": {"eps": 1e-6},
          "layers": [_layer(_C0, 192), _layer(_C0, 192), _layer(_C0, 192, weights_of=1)]},
    # no block mask and no rotation
    "d": {"architecture": "Feduzen", "vocab": 97, "width": 48, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
          "layers": [_layer(_D0, 64), _layer(_D0, 64)]},
}

PAGE_SIZE = {"a": 8, "b": 16, "c": 16, "d": 4}


def write_model(folder, name_or_config, seed=0, std=0.08, spread=0.3):
    """config.json + model.safetensors with the package's random mode: matrices N(0, std), vectors (gains, biases,
    sinks) 1 + N(0, spread)."""
    from simple_inference_amd.config import EngineConfig
    from simple_inference_amd.engine import build_model
    from simple_inference_amd.weights import random_tensors, write_model_folder

    cfg = copy.deepcopy(CONFIGS[name_or_config] if isinstance(name_or_config, str) else name_or_config)
    model, mcfg = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    tensors = random_tensors(model.expected_tensors(), seed, std, spread, "bfloat16")
    write_model_folder(folder, mcfg.to_dict(), tensors)
    return folder


def read_model(folder):
    with open(f"{folder}/config.json") as f:
        cfg = json.load(f)
    w = {}
    with safe_open(f"{folder}/model.safetensors", framework="pt") as f:
        for k in f.keys():
            w[k] = f.get_tensor(k)
    return cfg, w


def plain_logits(folder, tokens):
    cfg, w = read_model(folder)
    return plain.forward(cfg, w, tokens).float()


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


# max |a - b| / max |b| over the logits.  float32: order of additions only.  bfloat16: 8 bits of mantissa through
# every product, with norms, softmax and the residual in float32.
TOLERANCE = {"twins": 3e-5, "hip-f32": 3e-5, "twins-bf16": 4e-2, "hip-bf16": 4e-2}


def rel_err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
