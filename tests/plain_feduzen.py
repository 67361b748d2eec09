"""A plain, slow implementation of the Feduzen design: whole sequences, no cache, one function per mechanism.

It shares no code with the package: it reads a configuration dictionary and a dictionary of tensors by their
checkpoint names and computes everything in float64 (or whatever dtype its tensors are given in).  The tests
compare the engine with it.

Notation.  ``x`` is the residual stream ``[T, width]`` of one sequence whose tokens stand at positions
``0 .. T-1``.  A layer is ``x += N1(mixer(x))`` and, if it has a feed-forward, ``x += N2(ff(x))``: each norm is
applied to its sublayer's result, and mixer and feed-forward get the stream un-normed.
"""

from __future__ import annotations

import math

import torch


def rms_norm(x, gain, eps):
    """``x / sqrt(mean(x^2) + eps) * gain`` over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain


def embed(tokens, table, scale):
    return table[torch.as_tensor(tokens, dtype=torch.long)] * scale


def rotary_frequencies(dims, base, scaling=None):
    """``f_i = base^(-2i/dims)`` for ``i < dims/2``; with ``scaling`` every frequency is changed by its wavelength
    ``l = 2 pi / f``: kept below ``original/high``, divided by ``factor`` above ``original/low``, blended between."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
            original = float(scaling["original"])
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x, positions, dims, base, scaling=None):
    """Rotates the first ``dims`` elements of every head of ``x [T, heads, dim]``: element ``i`` with ``i + dims/2``."""
    if not dims:
        return x
    f = torch.tensor(rotary_frequencies(dims, base, scaling), dtype=torch.float64)
    a = torch.as_tensor(positions, dtype=torch.float64)[:, None] * f[None, :]
    c, s = a.cos().to(x.dtype)[:, None, :], a.sin().to(x.dtype)[:, None, :]
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def chunk_mask(n, size):
    """``[n, n]`` bool: key ``j`` is seen from ``i`` iff ``j <= i`` and ``j // size == i // size`` (``size`` None:
    plain causal)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if size:
        seen &= (i // size) == (j // size)
    return seen


def softmax_with_sink(scores, sink):
    """Softmax over the last axis with ``exp(sink)`` added to the denominator and to nothing else."""
    m = torch.maximum(scores.max(-1, keepdim=True).values, sink)
    e = torch.exp(scores - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - m))


def attention(x, w, prefix, mixer, eps):
    """The mixer of one layer on one whole sequence ``x [T, width]``."""
    T = x.shape[0]
    H, G, D, Dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    g = lambda name: w[f"{prefix}.mix.{name}"].to(x.dtype)
    q = (x @ g("q").T + g("q.b")).view(T, H, D)
    k = (x @ g("k").T + g("k.b")).view(T, G, D)
    v = (x @ g("v").T + g("v.b")).view(T, G, Dv)
    q = rms_norm(q, g("q.norm"), eps)
    k = rms_norm(k, g("k.norm"), eps)
    rot = mixer.get("rot")
    if rot:
        pos = list(range(T))
        q = rotate(q, pos, rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate(k, pos, rot["dims"], rot["base"], rot.get("scaling"))
    seen = chunk_mask(T, (mixer.get("mask") or {}).get("size"))
    out = torch.empty(T, H, Dv, dtype=x.dtype)
    for h in range(H):
        kv = h // (H // G)
        s = (q[:, h] @ k[:, kv].T) * mixer["scale"]
        s = s.masked_fill(~seen, float("-inf"))
        p = softmax_with_sink(s, g("sink")[h])
        out[:, h] = p @ v[:, kv]
    return out.reshape(T, H * Dv) @ g("o").T


def dense_feed_forward(x, w, prefix):
    up = x @ w[f"{prefix}.mlp.up"].to(x.dtype).T
    return torch.relu(up) ** 2 @ w[f"{prefix}.mlp.down"].to(x.dtype).T


def owner_of(layers, i):
    """The layer whose tensors layer ``i`` uses."""
    seen = set()
    while layers[i].get("weights_of") is not None:
        if i in seen:
            raise ValueError("weights_of goes in a circle")
        seen.add(i)
        i = int(layers[i]["weights_of"])
    return i


def forward(config, w, tokens, dtype=torch.float64, keep_layers=False):
    """Logits ``[T, vocab]`` of one whole sequence (and the residual stream after every layer, if asked)."""
    eps = float(config["norm"]["eps"])
    x = embed(tokens, w["embed"].to(dtype), float(config["embedding"]["scale"]))
    after = []
    for i, layer in enumerate(config["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"unknown layer type {layer['type']!r}")
        p = f"l{owner_of(config['layers'], i)}"
        x = x + rms_norm(attention(x, w, p, layer["mixer"], eps), w[f"{p}.norm1"].to(dtype), eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")
            x = x + rms_norm(dense_feed_forward(x, w, p), w[f"{p}.norm2"].to(dtype), eps)
        after.append(x)
    logits = rms_norm(x, w["final.norm"].to(dtype), eps) @ w["head"].to(dtype).T
    return (logits, torch.stack(after)) if keep_layers else logits
