"""Typed configuration of the Feduzen design, read from its own config.json keys.

A Feduzen config.json names the design in ``architecture`` and describes every layer in ``layers``: the kind of
its mixer (``type``), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, or null).  An entry
with ``weights_of: j`` stands for one more run of layer ``j``'s tensors (the checkpoint holds none under its index)
that keeps separate keys and values; its description has to repeat layer ``j``'s, and is checked against it.
Every size and constant comes from here; nothing is derived from another model's habits (the score scale, the
value width and the rotated width are all given, not implied by the head size).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .model_config import ConfigError


def _need(d: Mapping[str, Any], key: str, where: str):
    if not isinstance(d, Mapping) or key not in d:
        raise ConfigError(f"config.json lacks {where}.{key}")
    return d[key]


def _positive_int(v, what: str) -> int:
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{what} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class FrequencyScaling:
    """Rescaling of rotary frequencies by wavelength (the rule of Llama 3.1), under this design's key names."""

    factor: float
    low: float
    high: float
    original: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "FrequencyScaling":
        out = cls(float(_need(d, "factor", where)), float(_need(d, "low", where)), float(_need(d, "high", where)),
                  int(_need(d, "original", where)))
        if out.factor <= 0 or out.original <= 0 or out.low <= 0 or out.high <= 0:
            raise ConfigError(f"{where}: factor, low, high and original must be positive")
        if out.high == out.low:
            raise ConfigError(f"{where}: high must differ from low")
        return out

    def as_rope_scaling(self) -> dict:
        """In the words of the rotary part's ``scaling`` parameter."""
        return {"rope_type": "llama3", "factor": self.factor, "low_freq_factor": self.low,
                "high_freq_factor": self.high, "original_max_position_embeddings": self.original}

    def to_dict(self) -> dict:
        return {"factor": self.factor, "high": self.high, "low": self.low, "original": self.original}


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[FrequencyScaling] = None

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int            # width of a query / key head
    vdim: int           # width of a value head
    scale: float        # scores are (q . k) * scale
    chunk: Optional[int]   # keys are seen only inside the query's block of this many positions (None: all before)
    rot: Optional[Rotation]

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "AttentionMixer":
        heads = _positive_int(_need(d, "heads", where), f"{where}.heads")
        kv = _positive_int(_need(d, "kv_heads", where), f"{where}.kv_heads")
        dim = _positive_int(_need(d, "dim", where), f"{where}.dim")
        vdim = _positive_int(_need(d, "vdim", where), f"{where}.vdim")
        if heads % kv:
            raise ConfigError(f"{where}: heads {heads} is not a multiple of kv_heads {kv}")
        scale = float(_need(d, "scale", where))
        mask = d.get("mask")
        chunk = None
        if mask is not None:
            chunk = _positive_int(_need(mask, "size", f"{where}.mask"), f"{where}.mask.size")
        rot = None
        r = d.get("rot")
        if r is not None:
            dims = int(_need(r, "dims", f"{where}.rot"))
            if dims < 0 or dims % 2 or dims > dim:
                raise ConfigError(f"{where}.rot.dims must be even and at most dim {dim}, got {dims}")
            base = float(_need(r, "base", f"{where}.rot"))
            if not base > 0:
                raise ConfigError(f"{where}.rot.base must be positive, got {base}")
            s = r.get("scaling")
            if dims:
                rot = Rotation(dims, base, FrequencyScaling.from_dict(s, f"{where}.rot.scaling") if s is not None else None)
        return cls(heads, kv, dim, vdim, scale, chunk, rot)

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.chunk is not None:
            d["mask"] = {"size": self.chunk}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class DenseFeedForward:
    ff: int

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class FeduzenLayer:
    type: str
    mixer: AttentionMixer
    mlp: Optional[DenseFeedForward]
    weights_of: Optional[int] = None   # the layer whose tensors this one uses (None: its own)

    def to_dict(self) -> dict:
        d = {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None, "type": self.type}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class FeduzenConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[FeduzenLayer, ...]
    architecture: str = "Feduzen"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "FeduzenConfig":
        vocab = _positive_int(_need(d, "vocab", "config"), "vocab")
        width = _positive_int(_need(d, "width", "config"), "width")
        scale = float(_need(_need(d, "embedding", "config"), "scale", "embedding"))
        eps = float(_need(_need(d, "norm", "config"), "eps", "norm"))
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        entries = _need(d, "layers", "config")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError("config.json's layers must be a list with at least one layer")
        layers = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(e, "type", where)
            if kind != "attention":
                raise ConfigError(f"{where}.type {kind!r} is not implemented (known: 'attention')")
            mixer = AttentionMixer.from_dict(_need(e, "mixer", where), f"{where}.mixer")
            mlp = e.get("mlp")
            if mlp is not None:
                mk = _need(mlp, "kind", f"{where}.mlp")
                if mk != "dense":
                    raise ConfigError(f"{where}.mlp.kind {mk!r} is not implemented (known: 'dense')")
                mlp = DenseFeedForward(_positive_int(_need(mlp, "ff", f"{where}.mlp"), f"{where}.mlp.ff"))
            owner = e.get("weights_of")
            if owner is not None:
                if isinstance(owner, bool) or not isinstance(owner, int) or not 0 <= owner < len(entries) or owner == i:
                    raise ConfigError(f"{where}.weights_of must name another layer, got {owner!r}")
            layers.append(FeduzenLayer(str(kind), mixer, mlp, owner))
        cfg = cls(vocab, width, scale, eps, tuple(layers), str(d.get("architecture", "Feduzen")))
        for i, layer in enumerate(layers):
            j = cfg.owner_of(i)
            if j != i and (layers[j].mixer, layers[j].mlp, layers[j].type) != (layer.mixer, layer.mlp, layer.type):
                raise ConfigError(f"layers[{i}] uses the weights of layer {j} but describes another layer")
        return cfg

    def owner_of(self, i: int) -> int:
        """The layer whose tensors layer ``i`` uses (itself, unless ``weights_of`` leads elsewhere)."""
        seen = set()
        while self.layers[i].weights_of is not None:
            if i in seen:
                raise ConfigError(f"weights_of of layer {i} leads in a circle")
            seen.add(i)
            i = self.layers[i].weights_of
        return i

    def num_parameters(self) -> int:
        total = 2 * self.vocab * self.width + self.width
        for i, layer in enumerate(self.layers):
            if self.owner_of(i) != i:
                continue
            m = layer.mixer
            q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            total += (q + k + v) * (self.width + 1) + 2 * m.dim + m.heads + self.width * m.heads * m.vdim + self.width
            if layer.mlp is not None:
                total += 2 * self.width * layer.mlp.ff + self.width
        return total

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers], "norm": {"eps": self.norm_eps},
                "vocab": self.vocab, "width": self.width}
