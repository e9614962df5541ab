"""NoresunConfig: the keys of a Noresun config.json, typed and checked.

    {"architecture": "Noresun", "vocab": V, "width": H, "postln_alpha": a, "norm": {"eps": e},
     "embedding": {"scale": s, "bigram": {"buckets": B, "mul_prev": p, "mul_cur": c}},
     "layers": [{"type": "attention" | "mingru", "mixer": {...}, "mlp": {"kind": "moe", "expert": {"ff": F},
                 "router": {"experts": E, "top": k}} | null}, ...]}

An "attention" mixer gives heads, kv_heads, dim, vdim, scale, mask {size}, rot {base, dims, scaling {factor, low, high,
original}} and optionally kv_from: j, the layer whose keys and values it reads instead of making its own; a "mingru"
mixer gives width.  Every size and every constant that differs between models of the design is read from here; the
order and kind of the layers is data.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError
from .novosun import _positive_ints, _take


@dataclass(frozen=True)
class RotSpec:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]] = None      # factor, low, high, original

    @classmethod
    def from_dict(cls, raw, where):
        base, dims = _take(raw, ("base", "dims"), where)
        _positive_ints((dims,), where)
        if dims % 2 or not float(base) > 0:
            raise ConfigError(f"{where}: dims must be even and base positive")
        scaling = raw.get("scaling")
        if scaling is not None:
            scaling = tuple(float(v) for v in _take(scaling, ("factor", "low", "high", "original"), where + ".scaling"))
            if not (scaling[0] > 0 and scaling[3] > 0 and 0 < scaling[1] < scaling[2]):
                raise ConfigError(f"{where}.scaling: factor and original positive, 0 < low < high")
        return cls(float(base), dims, scaling)

    def to_dict(self):
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return out


@dataclass(frozen=True)
class SigmoidAttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotSpec
    window: Optional[int] = None
    kv_from: Optional[int] = None

    @classmethod
    def from_dict(cls, raw, where):
        heads, kv_heads, dim, vdim, scale, rot = _take(raw, ("heads", "kv_heads", "dim", "vdim", "scale", "rot"), where)
        _positive_ints((heads, kv_heads, dim, vdim), where)
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if max(dim, vdim) > 256:
            raise ConfigError(f"{where}: head sizes of at most 256 are supported")
        if not float(scale) > 0:
            raise ConfigError(f"{where}: scale must be positive")
        rot = RotSpec.from_dict(rot, where + ".rot")
        if rot.dims > dim:
            raise ConfigError(f"{where}: {rot.dims} turning coordinates in heads of {dim}")
        window = None
        if raw.get("mask") is not None:
            (window,) = _take(raw["mask"], ("size",), where + ".mask")
            _positive_ints((window,), where + ".mask")
        kv_from = raw.get("kv_from")
        if kv_from is not None and (not isinstance(kv_from, int) or isinstance(kv_from, bool) or kv_from < 0):
            raise ConfigError(f"{where}: kv_from must be the index of a layer")
        return cls(heads, kv_heads, dim, vdim, float(scale), rot, window, kv_from)

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
               "rot": self.rot.to_dict()}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class MinGRUSpec:
    width: int

    @classmethod
    def from_dict(cls, raw, where):
        (width,) = _take(raw, ("width",), where)
        _positive_ints((width,), where)
        return cls(width)

    def to_dict(self):
        return {"width": self.width}


@dataclass(frozen=True)
class ExpertsSpec:
    ff: int
    experts: int
    top: int

    @classmethod
    def from_dict(cls, raw, where):
        if raw.get("kind") != "moe":
            raise ConfigError(f"{where}: feed-forward kind {raw.get('kind')!r} is not moe")
        expert, router = _take(raw, ("expert", "router"), where)
        (ff,) = _take(expert, ("ff",), where + ".expert")
        experts, top = _take(router, ("experts", "top"), where + ".router")
        _positive_ints((ff, experts, top), where)
        if top > experts or top > 16:
            raise ConfigError(f"{where}: {top} of {experts} experts: at most all of them, and at most 16")
        return cls(ff, experts, top)

    def to_dict(self):
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class LayerSpec:
    type: str                                 # "attention" or "mingru"
    attention: Optional[SigmoidAttentionSpec] = None
    mingru: Optional[MinGRUSpec] = None
    mlp: Optional[ExpertsSpec] = None

    @classmethod
    def from_dict(cls, raw, where):
        kind, mixer = _take(raw, ("type", "mixer"), where)
        mlp = raw.get("mlp")
        mlp = None if mlp is None else ExpertsSpec.from_dict(mlp, where + ".mlp")
        if kind == "attention":
            return cls(kind, attention=SigmoidAttentionSpec.from_dict(mixer, where + ".mixer"), mlp=mlp)
        if kind == "mingru":
            return cls(kind, mingru=MinGRUSpec.from_dict(mixer, where + ".mixer"), mlp=mlp)
        raise ConfigError(f"{where}: layer type {kind!r} is neither attention nor mingru")

    def to_dict(self):
        mixer = self.attention.to_dict() if self.type == "attention" else self.mingru.to_dict()
        return {"type": self.type, "mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class PairTableSpec:
    buckets: int
    mul_prev: int
    mul_cur: int

    @classmethod
    def from_dict(cls, raw, where):
        values = _take(raw, ("buckets", "mul_prev", "mul_cur"), where)
        _positive_ints(values[:1], where)
        if any((not isinstance(v, int)) or isinstance(v, bool) or v < 0 for v in values[1:]):
            raise ConfigError(f"{where}: multipliers must be integers >= 0")
        return cls(*values)

    def to_dict(self):
        return {"buckets": self.buckets, "mul_prev": self.mul_prev, "mul_cur": self.mul_cur}


@dataclass(frozen=True)
class NoresunConfig:
    vocab: int
    width: int
    layers: Tuple[LayerSpec, ...]
    norm_eps: float
    postln_alpha: float
    embedding_scale: float
    bigram: Optional[PairTableSpec] = None
    # config.json names no longest context; this bounds the block tables and the rotary tables.
    max_positions: int = 1 << 17

    architecture = "Noresun"

    @classmethod
    def from_dict(cls, raw):
        if raw.get("architecture", raw.get("model_type")) not in ("Noresun", "noresun") and "Noresun" not in (raw.get("architectures") or []):
            raise ConfigError(f"architecture {raw.get('architecture')!r} is not Noresun")
        vocab, width, layers, norm, alpha, embedding = _take(raw, ("vocab", "width", "layers", "norm", "postln_alpha", "embedding"), "config.json")
        _positive_ints((vocab, width), "config.json")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a list of at least one layer")
        if not isinstance(norm, dict) or "eps" not in norm or not float(norm["eps"]) >= 0:
            raise ConfigError("config.json: norm.eps must be a number >= 0")
        (scale,) = _take(embedding, ("scale",), "embedding")
        bigram = embedding.get("bigram")
        bigram = None if bigram is None else PairTableSpec.from_dict(bigram, "embedding.bigram")
        limit = raw.get("max_positions", cls.max_positions)
        _positive_ints((limit,), "config.json max_positions")
        specs = tuple(LayerSpec.from_dict(layer, f"layers[{i}]") for i, layer in enumerate(layers))
        for i, spec in enumerate(specs):
            a = spec.attention
            if a is None or a.kv_from is None:
                continue
            source = specs[a.kv_from].attention if a.kv_from < i else None
            if source is None or source.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from: layer {a.kv_from} is no earlier attention layer with keys of its own")
            if (source.kv_heads, source.dim, source.vdim, source.rot) != (a.kv_heads, a.dim, a.vdim, a.rot):
                raise ConfigError(f"layers[{i}].mixer: key heads, head sizes and rotation must equal layer {a.kv_from}'s")
        return cls(vocab, width, specs, float(norm["eps"]), float(alpha), float(scale), bigram, limit)

    def to_dict(self):
        embedding = {"scale": self.embedding_scale}
        if self.bigram is not None:
            embedding["bigram"] = self.bigram.to_dict()
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "postln_alpha": self.postln_alpha,
               "norm": {"eps": self.norm_eps}, "embedding": embedding, "layers": [layer.to_dict() for layer in self.layers]}
        if self.max_positions != type(self).max_positions:
            out["max_positions"] = self.max_positions
        return out
