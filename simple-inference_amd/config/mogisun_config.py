"""Typed configuration of the Mogisun design, read from its own config.json keys.

A Mogisun config.json names the design in ``architecture`` and describes every layer in ``layers``: the kind of its
mixer (``type``: ``attention`` or ``gla``), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``:
``dense``, ``moe`` or null).  ``loop`` names a run of layers that is walked ``times`` times with the same weights;
``logit_scale`` and ``logit_softcap`` shape the output.  Every size and constant comes from here or, where the file
has no key for it (the rank of a decay's low-rank pair), from the checkpoint's tensors; what the file does not
mention is not there (no loop, no temperature, no shared expert, no cap).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple, Union

from .model_config import ConfigError


def _need(d: Mapping[str, Any], key: str, where: str):
    if not isinstance(d, Mapping) or key not in d:
        raise ConfigError(f"config.json lacks {where}.{key}")
    return d[key]


def _positive_int(v, what: str) -> int:
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{what} must be a positive integer, got {v!r}")
    return v


def _positive(v, what: str) -> float:
    try:
        f = float(v)
    except (TypeError, ValueError):
        raise ConfigError(f"{what} must be a number, got {v!r}") from None
    if not f > 0:
        raise ConfigError(f"{what} must be positive, got {v!r}")
    return f


@dataclass(frozen=True)
class QueryTemperature:
    coef: float
    every: int

    def to_dict(self) -> dict:
        return {"coef": self.coef, "every": self.every}


@dataclass(frozen=True)
class SoftmaxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp: Optional[QueryTemperature]

    @classmethod
    def from_dict(cls, d, where):
        heads = _positive_int(_need(d, "heads", where), f"{where}.heads")
        kv = _positive_int(_need(d, "kv_heads", where), f"{where}.kv_heads")
        if heads % kv:
            raise ConfigError(f"{where}: heads {heads} is not a multiple of kv_heads {kv}")
        temp = d.get("q_temp")
        if temp is not None:
            temp = QueryTemperature(float(_need(temp, "coef", f"{where}.q_temp")),
                                    _positive_int(_need(temp, "every", f"{where}.q_temp"), f"{where}.q_temp.every"))
        return cls(heads, kv, _positive_int(_need(d, "dim", where), f"{where}.dim"),
                   _positive_int(_need(d, "vdim", where), f"{where}.vdim"),
                   _positive(_need(d, "scale", where), f"{where}.scale"), temp)

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.q_temp is not None:
            d["q_temp"] = self.q_temp.to_dict()
        return d


@dataclass(frozen=True)
class LinearAttention:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: Optional[int] = None    # of the decay's low-rank pair; None: whatever the checkpoint's tensors have

    @classmethod
    def from_dict(cls, d, where):
        rank = d.get("rank")
        return cls(_positive_int(_need(d, "heads", where), f"{where}.heads"),
                   _positive_int(_need(d, "dim", where), f"{where}.dim"),
                   _positive_int(_need(d, "vdim", where), f"{where}.vdim"),
                   _positive(_need(d, "tau", where), f"{where}.tau"),
                   _positive_int(rank, f"{where}.rank") if rank is not None else None)

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "tau": self.tau, "vdim": self.vdim}
        if self.rank is not None:
            d["rank"] = self.rank
        return d


@dataclass(frozen=True)
class DenseMlp:
    ff: int

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class MoeMlp:
    experts: int
    top: int
    ff: int
    shared_ff: Optional[int]

    @classmethod
    def from_dict(cls, d, where):
        router = _need(d, "router", where)
        experts = _positive_int(_need(router, "experts", f"{where}.router"), f"{where}.router.experts")
        top = _positive_int(_need(router, "top", f"{where}.router"), f"{where}.router.top")
        if top > experts:
            raise ConfigError(f"{where}.router.top {top} exceeds its {experts} experts")
        ff = _positive_int(_need(_need(d, "expert", where), "ff", f"{where}.expert"), f"{where}.expert.ff")
        shared = d.get("shared")
        shared_ff = _positive_int(_need(shared, "ff", f"{where}.shared"), f"{where}.shared.ff") if shared else None
        return cls(experts, top, ff, shared_ff)

    def to_dict(self) -> dict:
        d = {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass(frozen=True)
class MogisunLayer:
    type: str
    mixer: Union[SoftmaxAttention, LinearAttention]
    mlp: Union[DenseMlp, MoeMlp, None]

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None, "type": self.type}


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int

    def to_dict(self) -> dict:
        return {"start": self.start, "stop": self.stop, "times": self.times}


_MIXERS = {"attention": SoftmaxAttention, "gla": LinearAttention}


@dataclass(frozen=True)
class MogisunConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[MogisunLayer, ...]
    loop: Optional[Loop]
    logit_scale: float
    logit_softcap: Optional[float]
    architecture: str = "Mogisun"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "MogisunConfig":
        vocab = _positive_int(_need(d, "vocab", "config"), "vocab")
        width = _positive_int(_need(d, "width", "config"), "width")
        eps = _positive(_need(_need(d, "norm", "config"), "eps", "norm"), "norm.eps")
        entries = _need(d, "layers", "config")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError("config.json's layers must be a list with at least one layer")
        layers = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(e, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"{where}.type {kind!r} is not implemented (known: {', '.join(sorted(_MIXERS))})")
            mixer = _MIXERS[kind].from_dict(_need(e, "mixer", where), f"{where}.mixer")
            mlp = e.get("mlp")
            if mlp is not None:
                mk = _need(mlp, "kind", f"{where}.mlp")
                if mk == "dense":
                    mlp = DenseMlp(_positive_int(_need(mlp, "ff", f"{where}.mlp"), f"{where}.mlp.ff"))
                elif mk == "moe":
                    mlp = MoeMlp.from_dict(mlp, f"{where}.mlp")
                else:
                    raise ConfigError(f"{where}.mlp.kind {mk!r} is not implemented (known: 'dense', 'moe')")
            layers.append(MogisunLayer(str(kind), mixer, mlp))
        loop = d.get("loop")
        if loop is not None:
            start, stop, times = (_need(loop, k, "loop") for k in ("start", "stop", "times"))
            for v, what in ((start, "start"), (stop, "stop")):
                if isinstance(v, bool) or not isinstance(v, int):
                    raise ConfigError(f"loop.{what} must be an integer, got {v!r}")
            if not 0 <= start < stop <= len(layers):
                raise ConfigError(f"loop runs layers {start} .. {stop - 1}, which are not among the {len(layers)} layers")
            loop = Loop(start, stop, _positive_int(times, "loop.times"))
        cap = d.get("logit_softcap")
        return cls(vocab, width, eps, tuple(layers), loop,
                   _positive(d.get("logit_scale", 1.0), "logit_scale"),
                   _positive(cap, "logit_softcap") if cap is not None else None,
                   str(d.get("architecture", "Mogisun")))

    def run_order(self):
        """``(layer, whether a walk of the loop starts with this run)`` for every run, in order."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        lp = self.loop
        runs = [(i, False) for i in range(lp.start)]
        for _ in range(lp.times):
            runs += [(i, i == lp.start) for i in range(lp.start, lp.stop)]
        return runs + [(i, False) for i in range(lp.stop, n)]

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers],
             "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        return d
