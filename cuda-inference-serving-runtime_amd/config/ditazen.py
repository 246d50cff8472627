"""DitazenConfig: the keys of a Ditazen config.json, typed and checked.

    {"architecture": "Ditazen", "vocab": V, "width": H, "logit_scale": s, "norm": {"eps": e},
     "layers": [{"type": "latent_attention" | "latent_attention_2" | "delta", "mixer": {...},
                 "mlp": {"kind": "dense", "ff": F} | null, "weights_of": j (optional)}, ...]}

A latent-attention mixer gives heads, dim, rot_dim, vdim, kv_rank, scale and `rot` (base, dims, optionally `scaling`:
factor, original, fast, slow); "latent_attention" looks back over `mask.size` tokens, "latent_attention_2" makes its
queries through a latent of `q_rank` (or of whatever the file holds, if config.json does not say) and sees every
earlier token.  A delta mixer gives heads, kv_heads, dim, vdim and conv (taps).  A layer with `weights_of`: j runs
with layer j's tensors and a cache or state of its own.  Every size and every constant that differs between models of
the design is read from here; the order and kind of the layers is data.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError
from .novosun import _take, _positive_ints

LATENT_TYPES = ("latent_attention", "latent_attention_2")


@dataclass(frozen=True)
class RotarySpec:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]] = None     # factor, original, fast, slow

    @classmethod
    def from_dict(cls, raw, where):
        base, dims = _take(raw, ("base", "dims"), where)
        _positive_ints((dims,), where)
        if dims % 2 or not float(base) > 1:
            raise ConfigError(f"{where}: an even number of dims and a base above 1")
        scaling = raw.get("scaling")
        if scaling is not None:
            scaling = tuple(float(v) for v in _take(scaling, ("factor", "original", "fast", "slow"), where + ".scaling"))
            if not all(v > 0 for v in scaling):
                raise ConfigError(f"{where}.scaling: factor, original, fast and slow must be positive")
        return cls(float(base), dims, scaling)

    def to_dict(self):
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return out


@dataclass(frozen=True)
class LatentSpec:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: RotarySpec
    q_rank: Optional[int] = None      # None: the file decides (second kind), or no query latent (first kind)
    window: Optional[int] = None

    @classmethod
    def from_dict(cls, raw, where, second):
        heads, dim, rot_dim, vdim, kv_rank, scale, rot = _take(raw, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"), where)
        _positive_ints((heads, dim, rot_dim, vdim, kv_rank), where)
        if not float(scale) > 0:
            raise ConfigError(f"{where}: scale must be positive")
        rot = RotarySpec.from_dict(rot, where + ".rot")
        if rot.dims > rot_dim:
            raise ConfigError(f"{where}: rot.dims {rot.dims} exceeds rot_dim {rot_dim}")
        if kv_rank + rot_dim > 640:
            raise ConfigError(f"{where}: kv_rank + rot_dim of at most 640 is supported")
        q_rank = raw.get("q_rank") if second else None
        if q_rank is not None:
            _positive_ints((q_rank,), where + ".q_rank")
        window = None
        if raw.get("mask") is not None:
            (window,) = _take(raw["mask"], ("size",), where + ".mask")
            _positive_ints((window,), where + ".mask.size")
        elif not second:
            raise ConfigError(f"{where} lacks mask.size")
        return cls(heads, dim, rot_dim, vdim, kv_rank, float(scale), rot, q_rank, window)

    def to_dict(self):
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
               "scale": self.scale, "rot": self.rot.to_dict()}
        if self.q_rank is not None:
            out["q_rank"] = self.q_rank
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class DeltaSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, raw, where):
        values = _take(raw, ("heads", "kv_heads", "dim", "vdim", "conv"), where)
        _positive_ints(values, where)
        heads, kv_heads, dim, _, conv = values
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if conv > 16 or dim > 256:
            raise ConfigError(f"{where}: convolutions of at most 16 taps and heads of at most 256 are supported")
        return cls(*values)

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class DenseSpec:
    ff: int
    act: str = "gelu"

    @classmethod
    def from_dict(cls, raw, where):
        if raw.get("kind", "dense") != "dense":
            raise ConfigError(f"{where}: feed-forward kind {raw.get('kind')!r} is not dense")
        (ff,) = _take(raw, ("ff",), where)
        _positive_ints((ff,), where)
        act = raw.get("act", "gelu")
        if act not in ("gelu", "gelu_erf", "gelu_tanh"):
            raise ConfigError(f"{where}: activation {act!r} is neither gelu nor gelu_tanh")
        return cls(ff, act)

    def to_dict(self):
        out = {"kind": "dense", "ff": self.ff}
        if self.act != "gelu":
            out["act"] = self.act
        return out


@dataclass(frozen=True)
class DitazenLayer:
    type: str
    latent: Optional[LatentSpec] = None
    delta: Optional[DeltaSpec] = None
    mlp: Optional[DenseSpec] = None
    weights_of: Optional[int] = None

    @classmethod
    def from_dict(cls, raw, where):
        kind, mixer = _take(raw, ("type", "mixer"), where)
        mlp = raw.get("mlp")
        mlp = None if mlp is None else DenseSpec.from_dict(mlp, where + ".mlp")
        owner = raw.get("weights_of")
        if owner is not None and (not isinstance(owner, int) or isinstance(owner, bool) or owner < 0):
            raise ConfigError(f"{where}: weights_of must name a layer")
        if kind in LATENT_TYPES:
            return cls(kind, latent=LatentSpec.from_dict(mixer, where + ".mixer", kind == "latent_attention_2"), mlp=mlp, weights_of=owner)
        if kind == "delta":
            return cls(kind, delta=DeltaSpec.from_dict(mixer, where + ".mixer"), mlp=mlp, weights_of=owner)
        raise ConfigError(f"{where}: layer type {kind!r} is none of {LATENT_TYPES + ('delta',)}")

    def to_dict(self):
        out = {"type": self.type, "mixer": (self.latent or self.delta).to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out

    def same_weights(self, other):
        return (self.type, self.latent, self.delta, self.mlp) == (other.type, other.latent, other.delta, other.mlp)


@dataclass(frozen=True)
class DitazenConfig:
    vocab: int
    width: int
    layers: Tuple[DitazenLayer, ...]
    norm_eps: float
    logit_scale: float
    # config.json names no longest context; this bounds the block tables and the tables of cosines and sines.
    max_positions: int = 1 << 17

    architecture = "Ditazen"

    @classmethod
    def from_dict(cls, raw):
        if raw.get("architecture", raw.get("model_type")) not in ("Ditazen", "ditazen") and "Ditazen" not in (raw.get("architectures") or []):
            raise ConfigError(f"architecture {raw.get('architecture')!r} is not Ditazen")
        vocab, width, layers, norm = _take(raw, ("vocab", "width", "layers", "norm"), "config.json")
        _positive_ints((vocab, width), "config.json")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a list of at least one layer")
        if not isinstance(norm, dict) or "eps" not in norm or not float(norm["eps"]) >= 0:
            raise ConfigError("config.json: norm.eps must be a number >= 0")
        limit = raw.get("max_positions", cls.max_positions)
        _positive_ints((limit,), "config.json max_positions")
        typed = [DitazenLayer.from_dict(layer, f"layers[{i}]") for i, layer in enumerate(layers)]
        for i, layer in enumerate(typed):
            j, seen = layer.weights_of, {i}
            if j is None:
                continue
            while j is not None and j < len(typed) and j not in seen and typed[j].weights_of is not None:
                seen.add(j)                   # (a layer that names a layer that names another: the one that has the tensors)
                j = typed[j].weights_of
            if j is None or j >= len(typed) or j in seen:
                raise ConfigError(f"layers[{i}]: weights_of {layer.weights_of} must lead to another layer that has tensors of its own")
            if not layer.same_weights(typed[j]):
                raise ConfigError(f"layers[{i}]: its entry differs from that of layer {j}, whose weights it uses")
            typed[i] = DitazenLayer(layer.type, layer.latent, layer.delta, layer.mlp, j)
        typed = tuple(typed)
        return cls(vocab, width, typed, float(norm["eps"]), float(raw.get("logit_scale", 1.0)), limit)

    def to_dict(self):
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "logit_scale": self.logit_scale,
               "norm": {"eps": self.norm_eps}, "layers": [layer.to_dict() for layer in self.layers]}
        if self.max_positions != type(self).max_positions:
            out["max_positions"] = self.max_positions
        return out
