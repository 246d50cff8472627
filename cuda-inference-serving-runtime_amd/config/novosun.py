"""NovosunConfig: the keys of a Novosun config.json, typed and checked.

    {"architecture": "Novosun", "vocab": V, "width": H, "residual_mult": m, "norm": {"eps": e},
     "layers": [{"type": "gla" | "parallel", "mixer": {...}, "mlp": {"kind": "dense", "ff": F, "limit": L} | null}, ...]}

A "gla" mixer gives heads, dim, vdim and tau; a "parallel" mixer gives "left" (heads, kv_heads, dim, vdim, scale: softmax
attention) and "right" (heads, vdim, state, groups, conv, norm_groups: a state-space layer).  Every size and every
constant that differs between models of the design is read from here; the order and kind of the layers is data.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError


def _take(raw, keys, where):
    missing = [k for k in keys if k not in raw]
    if missing:
        raise ConfigError(f"{where} lacks {missing}")
    return [raw[k] for k in keys]


def _positive_ints(values, where):
    if any((not isinstance(v, int)) or isinstance(v, bool) or v <= 0 for v in values):
        raise ConfigError(f"{where}: sizes must be positive integers")


@dataclass(frozen=True)
class GLASpec:
    heads: int
    dim: int
    vdim: int
    tau: float

    @classmethod
    def from_dict(cls, raw, where):
        heads, dim, vdim, tau = _take(raw, ("heads", "dim", "vdim", "tau"), where)
        _positive_ints((heads, dim, vdim), where)
        if not float(tau) > 0:
            raise ConfigError(f"{where}: tau must be positive")
        return cls(heads, dim, vdim, float(tau))

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}


@dataclass(frozen=True)
class AttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float

    @classmethod
    def from_dict(cls, raw, where):
        heads, kv_heads, dim, vdim, scale = _take(raw, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
        _positive_ints((heads, kv_heads, dim, vdim), where)
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if max(dim, vdim) > 256:
            raise ConfigError(f"{where}: head sizes of at most 256 are supported")
        if not float(scale) > 0:
            raise ConfigError(f"{where}: scale must be positive")
        return cls(heads, kv_heads, dim, vdim, float(scale))

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}


@dataclass(frozen=True)
class SSDSpec:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, raw, where):
        values = _take(raw, ("heads", "vdim", "state", "groups", "conv", "norm_groups"), where)
        _positive_ints(values, where)
        heads, vdim, state, groups, conv, norm_groups = values
        if heads % groups:
            raise ConfigError(f"{where}: {heads} heads do not divide into {groups} groups")
        if (heads * vdim) % norm_groups:
            raise ConfigError(f"{where}: {heads * vdim} channels do not divide into {norm_groups} norm_groups")
        if conv > 16:
            raise ConfigError(f"{where}: convolutions of at most 16 taps are supported")
        return cls(*values)

    def to_dict(self):
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class MLPSpec:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, raw, where):
        if raw.get("kind", "dense") != "dense":
            raise ConfigError(f"{where}: feed-forward kind {raw.get('kind')!r} is not dense")
        ff, limit = _take(raw, ("ff", "limit"), where)
        _positive_ints((ff,), where)
        if not float(limit) > 0:
            raise ConfigError(f"{where}: limit must be positive")
        return cls(ff, float(limit))

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class LayerSpec:
    type: str                                # "gla" or "parallel"
    gla: Optional[GLASpec] = None
    left: Optional[AttentionSpec] = None
    right: Optional[SSDSpec] = None
    mlp: Optional[MLPSpec] = None

    @classmethod
    def from_dict(cls, raw, where):
        kind, mixer = _take(raw, ("type", "mixer"), where)
        mlp = raw.get("mlp")
        mlp = None if mlp is None else MLPSpec.from_dict(mlp, where + ".mlp")
        if kind == "gla":
            return cls(kind, gla=GLASpec.from_dict(mixer, where + ".mixer"), mlp=mlp)
        if kind == "parallel":
            left, right = _take(mixer, ("left", "right"), where + ".mixer")
            return cls(kind, left=AttentionSpec.from_dict(left, where + ".mixer.left"),
                       right=SSDSpec.from_dict(right, where + ".mixer.right"), mlp=mlp)
        raise ConfigError(f"{where}: layer type {kind!r} is neither gla nor parallel")

    def to_dict(self):
        mixer = self.gla.to_dict() if self.type == "gla" else {"left": self.left.to_dict(), "right": self.right.to_dict()}
        return {"type": self.type, "mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class NovosunConfig:
    vocab: int
    width: int
    layers: Tuple[LayerSpec, ...]
    norm_eps: float
    residual_mult: float
    # The design has no position encoding and config.json names no longest context; this bounds the block tables only.
    max_positions: int = 1 << 17

    architecture = "Novosun"

    @classmethod
    def from_dict(cls, raw):
        if raw.get("architecture", raw.get("model_type")) not in ("Novosun", "novosun") and "Novosun" not in (raw.get("architectures") or []):
            raise ConfigError(f"architecture {raw.get('architecture')!r} is not Novosun")
        vocab, width, layers, norm, mult = _take(raw, ("vocab", "width", "layers", "norm", "residual_mult"), "config.json")
        _positive_ints((vocab, width), "config.json")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a list of at least one layer")
        if not isinstance(norm, dict) or "eps" not in norm or not float(norm["eps"]) >= 0:
            raise ConfigError("config.json: norm.eps must be a number >= 0")
        limit = raw.get("max_positions", cls.max_positions)
        _positive_ints((limit,), "config.json max_positions")
        return cls(vocab, width, tuple(LayerSpec.from_dict(layer, f"layers[{i}]") for i, layer in enumerate(layers)),
                   float(norm["eps"]), float(mult), limit)

    def to_dict(self):
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "residual_mult": self.residual_mult,
               "norm": {"eps": self.norm_eps}, "layers": [layer.to_dict() for layer in self.layers]}
        if self.max_positions != type(self).max_positions:
            out["max_positions"] = self.max_positions
        return out
