"""ZovozenConfig: the keys of a Zovozen config.json, typed and checked.

    {"architecture": "Zovozen", "vocab": V, "width": H, "norm": {"eps": e},
     "layers": [{"type": "parallel",
                 "mixer": {"left": {...}, "right": {...}, "left_scale": a, "right_scale": b},
                 "mlp": {"kind": "dense", "ff": F}
                      | {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": k, "identity": n,
                         "groups": {"count": c, "keep": m}}, "shared": {"ff": F2}} | null}, ...]}

`left` is attention whose scores are mixed over the heads: heads, kv_heads, dim, vdim, scale, optionally mask {size}
(blocks of that many positions that see only themselves) and rot {base, dims, scaling {factor}}.  `right` is a matrix
memory with exponential gates: heads, dim, vdim, gate_cap.  Every size and every constant that differs between models of
the design is read from here; the order and kind of the layers is data.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError
from .novosun import _positive_ints, _take


def _count(value, where, least=0):
    if not isinstance(value, int) or isinstance(value, bool) or value < least:
        raise ConfigError(f"{where} must be an integer >= {least}")
    return value


@dataclass(frozen=True)
class TurnSpec:
    """Rotary positions: `dims` turning coordinates a head, frequencies base^(-2i/dims) divided by `factor`."""
    base: float
    dims: int
    factor: float = 1.0

    @classmethod
    def from_dict(cls, raw, where):
        base, dims = _take(raw, ("base", "dims"), where)
        _positive_ints((dims,), where)
        if dims % 2 or not float(base) > 0:
            raise ConfigError(f"{where}: dims must be even and base positive")
        factor = 1.0
        if raw.get("scaling") is not None:
            (factor,) = _take(raw["scaling"], ("factor",), where + ".scaling")
            if not float(factor) > 0:
                raise ConfigError(f"{where}.scaling.factor must be positive")
        return cls(float(base), dims, float(factor))

    def to_dict(self):
        out = {"base": self.base, "dims": self.dims}
        if self.factor != 1.0:
            out["scaling"] = {"factor": self.factor}
        return out


@dataclass(frozen=True)
class TalkingAttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[TurnSpec] = None
    chunk: Optional[int] = None

    @classmethod
    def from_dict(cls, raw, where):
        heads, kv_heads, dim, vdim, scale = _take(raw, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
        _positive_ints((heads, kv_heads, dim, vdim), where)
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if not float(scale) > 0:
            raise ConfigError(f"{where}: scale must be positive")
        rot = None if raw.get("rot") is None else TurnSpec.from_dict(raw["rot"], where + ".rot")
        if rot is not None and rot.dims > dim:
            raise ConfigError(f"{where}: {rot.dims} turning coordinates in heads of {dim}")
        chunk = None
        if raw.get("mask") is not None:
            (chunk,) = _take(raw["mask"], ("size",), where + ".mask")
            _positive_ints((chunk,), where + ".mask")
        return cls(heads, kv_heads, dim, vdim, float(scale), rot, chunk)

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        return out


@dataclass(frozen=True)
class MatrixMemorySpec:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, raw, where):
        heads, dim, vdim, cap = _take(raw, ("heads", "dim", "vdim", "gate_cap"), where)
        _positive_ints((heads, dim, vdim), where)
        if not float(cap) > 0:
            raise ConfigError(f"{where}: gate_cap must be positive")
        return cls(heads, dim, vdim, float(cap))

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class PairSpec:
    left: TalkingAttentionSpec
    right: MatrixMemorySpec
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw, where):
        left, right, ls, rs = _take(raw, ("left", "right", "left_scale", "right_scale"), where)
        return cls(TalkingAttentionSpec.from_dict(left, where + ".left"), MatrixMemorySpec.from_dict(right, where + ".right"),
                   float(ls), float(rs))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale, "right_scale": self.right_scale}


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str                                  # "dense" or "moe"
    ff: int                                    # dense: the inner size; moe: an expert's
    experts: int = 0                           # experts with matrices
    top: int = 0
    identity: int = 0                          # further router outputs whose expert is the input itself
    groups: Optional[Tuple[int, int]] = None   # (count, keep)
    shared_ff: Optional[int] = None

    @classmethod
    def from_dict(cls, raw, where):
        kind = raw.get("kind")
        if kind == "dense":
            (ff,) = _take(raw, ("ff",), where)
            _positive_ints((ff,), where)
            return cls(kind, ff)
        if kind != "moe":
            raise ConfigError(f"{where}: feed-forward kind {kind!r} is neither dense nor moe")
        expert, router = _take(raw, ("expert", "router"), where)
        (ff,) = _take(expert, ("ff",), where + ".expert")
        experts, top = _take(router, ("experts", "top"), where + ".router")
        _positive_ints((ff, experts, top), where)
        identity = _count(router.get("identity", 0), where + ".router.identity")
        outputs = experts + identity
        groups = None
        if router.get("groups") is not None:
            count, keep = _take(router["groups"], ("count", "keep"), where + ".router.groups")
            _positive_ints((count, keep), where + ".router.groups")
            if outputs % count or keep > count:
                raise ConfigError(f"{where}.router.groups: {outputs} router outputs in {count} equal groups of which {keep} are kept")
            if keep * (outputs // count) < top:
                raise ConfigError(f"{where}.router: {top} experts cannot be chosen from {keep} groups of {outputs // count}")
            groups = (count, keep)
        if top > outputs or top > 16:
            raise ConfigError(f"{where}: {top} of {outputs} router outputs: at most all of them, and at most 16")
        shared = None
        if raw.get("shared") is not None:
            (shared,) = _take(raw["shared"], ("ff",), where + ".shared")
            _positive_ints((shared,), where + ".shared")
        return cls(kind, ff, experts, top, identity, groups, shared)

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        router = {"experts": self.experts, "top": self.top, "identity": self.identity}
        if self.groups is not None:
            router["groups"] = {"count": self.groups[0], "keep": self.groups[1]}
        out = {"kind": "moe", "expert": {"ff": self.ff}, "router": router}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class LayerSpec:
    type: str                                 # "parallel"
    mixer: PairSpec
    mlp: Optional[FeedForwardSpec] = None

    @classmethod
    def from_dict(cls, raw, where):
        kind, mixer = _take(raw, ("type", "mixer"), where)
        if kind != "parallel":
            raise ConfigError(f"{where}: layer type {kind!r} is not parallel")
        mlp = raw.get("mlp")
        return cls(kind, PairSpec.from_dict(mixer, where + ".mixer"), None if mlp is None else FeedForwardSpec.from_dict(mlp, where + ".mlp"))

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class ZovozenConfig:
    vocab: int
    width: int
    layers: Tuple[LayerSpec, ...]
    norm_eps: float
    # config.json names no longest context; this bounds the block tables and the rotary tables.
    max_positions: int = 1 << 17

    architecture = "Zovozen"

    @classmethod
    def from_dict(cls, raw):
        if raw.get("architecture", raw.get("model_type")) not in ("Zovozen", "zovozen") and "Zovozen" not in (raw.get("architectures") or []):
            raise ConfigError(f"architecture {raw.get('architecture')!r} is not Zovozen")
        vocab, width, layers, norm = _take(raw, ("vocab", "width", "layers", "norm"), "config.json")
        _positive_ints((vocab, width), "config.json")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a list of at least one layer")
        if not isinstance(norm, dict) or "eps" not in norm or not float(norm["eps"]) >= 0:
            raise ConfigError("config.json: norm.eps must be a number >= 0")
        limit = raw.get("max_positions", cls.max_positions)
        _positive_ints((limit,), "config.json max_positions")
        return cls(vocab, width, tuple(LayerSpec.from_dict(layer, f"layers[{i}]") for i, layer in enumerate(layers)), float(norm["eps"]), limit)

    def to_dict(self):
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": [layer.to_dict() for layer in self.layers]}
        if self.max_positions != type(self).max_positions:
            out["max_positions"] = self.max_positions
        return out
