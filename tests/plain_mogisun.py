"""A plain, slow implementation of the Mogisun design: whole sequences, no cache, one function per mechanism.

It shares no code with the package: it reads a configuration dictionary and a dictionary of tensors by their
checkpoint names and computes everything in float64 (or whatever dtype its tensors are given in).  The tests
compare the engine with it.

Notation.  ``x [T, width]`` is the residual stream of one sequence whose tokens stand at positions ``0 .. T-1``;
``N(y) = y / sqrt(mean(y^2) + eps)``.  A layer is ``h = N(x) w1; x += sigma(R1 h + r1) * mixer(h)`` and, if it has
a feed-forward, ``h = N(x) w2; x += sigma(R2 h + r2) * ff(h)``.  Some run of layers is walked several times with
the same weights; before every walk the stream is mixed with the embedding output: ``x = J [x; x0]``.
"""

from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    """``x / sqrt(mean(x^2) + eps)`` over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def swiglu(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


# ---------------------------------------------------------------------------------------------------------
# mixers
# ---------------------------------------------------------------------------------------------------------

def query_temperature(positions, coef, every):
    """``1 + coef * ln(floor((p + 1) / every) + 1)`` for every position."""
    return torch.tensor([1.0 + coef * math.log((int(p) + 1) // int(every) + 1) for p in positions], dtype=torch.float64)


def attention(h, w, prefix, mixer, eps):
    """Causal softmax attention with grouped key/value heads, unit-RMS q and k, a query temperature that grows
    with the position, and a sigmoid gate per head on the output."""
    T = h.shape[0]
    H, G, D, Dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = (h @ w[prefix + "q"].T + w[prefix + "q.b"]).view(T, H, D)
    k = (h @ w[prefix + "k"].T + w[prefix + "k.b"]).view(T, G, D)
    v = (h @ w[prefix + "v"].T + w[prefix + "v.b"]).view(T, G, Dv)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    temp = mixer.get("q_temp")
    if temp:
        q = q * query_temperature(range(T), temp["coef"], temp["every"]).to(q.dtype)[:, None, None]
    gate = torch.sigmoid(h @ w[prefix + "g"].T)                         # [T, H]
    seen = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * mixer["scale"]
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, -1) @ v[:, g]
    out = out * gate[:, :, None]
    return out.reshape(T, H * Dv) @ w[prefix + "o"].T + w[prefix + "o.b"]


def decay(h, w, prefix, mixer):
    """Per key channel, ``sigma(z)^(1/tau)`` with ``z = A2 (A1 h) + a``: ``[T, heads, dim]``."""
    z = (h @ w[prefix + "a1"].T) @ w[prefix + "a2"].T + w[prefix + "a2.b"]
    return torch.exp(torch.nn.functional.logsigmoid(z) / mixer["tau"]).view(h.shape[0], mixer["heads"], mixer["dim"])


def linear_recurrence(q, k, v, alpha, state=None):
    """``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` for one head, token by token.
    ``q, k, alpha [T, D]``, ``v [T, Dv]``; returns ``(o [T, Dv], S [D, Dv])``."""
    T, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=q.dtype) if state is None else state.clone()
    out = []
    for t in range(T):
        S = alpha[t][:, None] * S + k[t][:, None] * v[t][None, :]
        out.append(S.T @ q[t])
    return torch.stack(out), S


def gla(h, w, prefix, mixer, eps):
    """Gated linear attention: a matrix state per head that decays per key channel."""
    T = h.shape[0]
    H, D, Dv = mixer["heads"], mixer["dim"], mixer["vdim"]
    q = (h @ w[prefix + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[prefix + "k"].T).view(T, H, D)
    v = (h @ w[prefix + "v"].T).view(T, H, Dv)
    alpha = decay(h, w, prefix, mixer)
    o = torch.stack([linear_recurrence(q[:, a], k[:, a], v[:, a], alpha[:, a])[0] for a in range(H)], dim=1)
    o = unit_rms(o, eps) * w[prefix + "norm"]
    o = o.reshape(T, H * Dv) * silu(h @ w[prefix + "g"].T)
    return o @ w[prefix + "o"].T


# ---------------------------------------------------------------------------------------------------------
# feed-forwards
# ---------------------------------------------------------------------------------------------------------

def route(h, router, top):
    """The ``top`` experts with the largest logits and the softmax over their logits alone."""
    logits = h @ router.T
    best, which = torch.topk(logits, top, dim=-1)
    return which, torch.softmax(best, -1)


def mixture(h, w, prefix, mlp):
    which, weight = route(h, w[prefix + "router"], mlp["router"]["top"])
    y = torch.zeros(h.shape[0], w[prefix + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, p in zip(which[t].tolist(), weight[t]):
            y[t] += p * swiglu(h[t], w[f"{prefix}e{e}.gate"], w[f"{prefix}e{e}.up"], w[f"{prefix}e{e}.down"])
    if mlp.get("shared"):
        s = swiglu(h, w[prefix + "shared.gate"], w[prefix + "shared.up"], w[prefix + "shared.down"])
        y = y + torch.sigmoid(h @ w[prefix + "shared.sg"].T) * s
    return y


def feed_forward(h, w, prefix, mlp):
    if mlp["kind"] == "dense":
        return swiglu(h, w[prefix + "gate"], w[prefix + "up"], w[prefix + "down"])
    if mlp["kind"] == "moe":
        return mixture(h, w, prefix, mlp)
    raise ValueError(mlp["kind"])


# ---------------------------------------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------------------------------------

def layer(x, w, i, spec, eps):
    p = f"l{i}."
    h = unit_rms(x, eps) * w[p + "norm1"]
    mix = {"attention": attention, "gla": gla}[spec["type"]](h, w, p + "mix.", spec["mixer"], eps)
    x = x + torch.sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"]) * mix
    if spec.get("mlp"):
        h = unit_rms(x, eps) * w[p + "norm2"]
        x = x + torch.sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"]) * feed_forward(h, w, p + "mlp.", spec["mlp"])
    return x


def run_order(cfg):
    """``(layer index, whether a walk of the repeated run starts here)`` in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    out = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        out += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return out + [(i, False) for i in range(loop["stop"], n)]


def residuals(cfg, w, tokens):
    """The residual stream after every run of a layer: ``[runs, T, width]``."""
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x, eps, out = x0, cfg["norm"]["eps"], []
    for i, enters in run_order(cfg):
        if enters:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        x = layer(x, w, i, cfg["layers"][i], eps)
        out.append(x)
    return torch.stack(out)


def logits(cfg, w, tokens):
    x = residuals(cfg, w, tokens)[-1]
    z = (unit_rms(x, cfg["norm"]["eps"]) * w["final.norm"]) @ w["head"].T * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
