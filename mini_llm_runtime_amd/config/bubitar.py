"""The Bubitar decoder's configuration.

Its config.json is nested and lists the layers one by one, each with a mixer of its own kind and
sizes:

    {"architecture": "Bubitar", "vocab": V, "width": W, "norm": {"eps": e},
     "token_side": {"dim": s},
     "layers": [{"type": "retention",
                 "mixer": {"heads": H, "dim": d, "vdim": dv, "decay": [g_0 .. g_H-1],
                           "rot": {"base": b, "dims": r}},
                 "mlp": {"kind": "dense", "ff": F, "limit": c} | null},
                {"type": "latent_attention",
                 "mixer": {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "kv_rank": R, "scale": c,
                           "rot": {"base": b, "dims": r,
                                   "scaling": {"factor": f, "original": n, "fast": a, "slow": z}},
                           "kv_from": j},
                 "mlp": ...}, ...]}

`kv_from` (optional) names an earlier latent-attention layer whose cached latents and rotated key
part this layer reads instead of making its own.  Nothing here is a size of one particular model.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar, Mapping, Optional

from .model_config import ConfigError, ModelConfig, positive_float, positive_int, require_keys


def _mapping(data: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = data.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where}: {key!r} must be an object, found {value!r}")
    return value


@dataclass(frozen=True)
class RotaryScaling:
    """Frequencies stretched by `factor` where a turn is longer than `original` / `slow` positions,
    kept where it is shorter than `original` / `fast`, blended linearly (over the dimension index)
    between; cosines and sines are multiplied by 0.1 ln(factor) + 1."""

    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "RotaryScaling":
        require_keys(data, ("factor", "original", "fast", "slow"), where)
        return cls(
            factor=positive_float(data, "factor"),
            original=positive_float(data, "original"),
            fast=positive_float(data, "fast"),
            slow=positive_float(data, "slow"),
        )

    def to_dict(self) -> dict[str, Any]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class Rotary:
    base: float
    dims: int
    scaling: Optional[RotaryScaling] = None

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "Rotary":
        require_keys(data, ("base", "dims"), where)
        scaling = data.get("scaling")
        if scaling is not None and not isinstance(scaling, Mapping):
            raise ConfigError(f"{where}: 'scaling' must be an object or null")
        out = cls(
            base=positive_float(data, "base"),
            dims=positive_int(data, "dims"),
            scaling=None if scaling is None else RotaryScaling.from_dict(scaling, where + ".scaling"),
        )
        if out.dims % 2:
            raise ConfigError(f"{where}: dims must be even")
        return out

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = self.scaling.to_dict()
        return out


@dataclass(frozen=True)
class BubitarRetention:
    """Linear attention with a fixed decay per head and a matrix state per head."""

    heads: int
    dim: int
    vdim: int
    decay: tuple[float, ...]
    rot: Rotary

    kind: ClassVar[str] = "retention"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "BubitarRetention":
        require_keys(data, ("heads", "dim", "vdim", "decay", "rot"), where)
        decay = data["decay"]
        if not isinstance(decay, (list, tuple)) or not all(
            isinstance(g, (int, float)) and not isinstance(g, bool) and 0 <= g <= 1 for g in decay
        ):
            raise ConfigError(f"{where}: 'decay' must list one number within 0..1 per head")
        out = cls(
            heads=positive_int(data, "heads"),
            dim=positive_int(data, "dim"),
            vdim=positive_int(data, "vdim"),
            decay=tuple(float(g) for g in decay),
            rot=Rotary.from_dict(_mapping(data, "rot", where), where + ".rot"),
        )
        if len(out.decay) != out.heads:
            raise ConfigError(f"{where}: {len(out.decay)} decays for {out.heads} heads")
        if out.rot.dims > out.dim:
            raise ConfigError(f"{where}: more rotated dimensions than a head has")
        return out

    def to_dict(self) -> dict[str, Any]:
        return {
            "heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay), "rot": self.rot.to_dict(),
        }


@dataclass(frozen=True)
class BubitarLatentAttention:
    """Attention whose keys and values are made from one cached latent vector per token."""

    heads: int
    dim: int  # unrotated query/key dimensions per head
    rot_dim: int  # rotated ones; the rotated key part is shared by all heads
    vdim: int
    kv_rank: int
    scale: float
    rot: Rotary
    kv_from: Optional[int] = None

    kind: ClassVar[str] = "latent_attention"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "BubitarLatentAttention":
        require_keys(data, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"), where)
        source = data.get("kv_from")
        if source is not None and (isinstance(source, bool) or not isinstance(source, int) or source < 0):
            raise ConfigError(f"{where}: 'kv_from' must be a layer index or absent")
        out = cls(
            heads=positive_int(data, "heads"),
            dim=positive_int(data, "dim"),
            rot_dim=positive_int(data, "rot_dim"),
            vdim=positive_int(data, "vdim"),
            kv_rank=positive_int(data, "kv_rank"),
            scale=positive_float(data, "scale"),
            rot=Rotary.from_dict(_mapping(data, "rot", where), where + ".rot"),
            kv_from=source,
        )
        if out.rot.dims > out.rot_dim:
            raise ConfigError(f"{where}: more rotated dimensions than the rotated part has")
        return out

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
            "scale": self.scale, "rot": self.rot.to_dict(),
        }
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


_MIXERS = {c.kind: c for c in (BubitarRetention, BubitarLatentAttention)}


@dataclass(frozen=True)
class BubitarFeedForward:
    """down(g sigmoid(1.702 g) (u + 1)) with g = min(gate(x), limit), u = clamp(up(x), -limit, limit)."""

    ff: int
    limit: float

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "BubitarFeedForward":
        require_keys(data, ("kind", "ff", "limit"), where)
        if data["kind"] != "dense":
            raise ConfigError(f"{where}: kind must be 'dense', found {data['kind']!r}")
        return cls(ff=positive_int(data, "ff"), limit=positive_float(data, "limit"))

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class BubitarLayer:
    mixer: Any  # BubitarRetention or BubitarLatentAttention
    mlp: Optional[BubitarFeedForward]

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.mixer.kind, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class BubitarConfig(ModelConfig):
    architecture: ClassVar[str] = "Bubitar"
    model_type: ClassVar[str] = "bubitar"

    vocab: int
    width: int
    norm_eps: float
    token_side_dim: int
    layers: tuple[BubitarLayer, ...]

    def __post_init__(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.token_side_dim <= 0:
            raise ConfigError("BubitarConfig: vocab, width and token_side.dim must be > 0")
        if not self.layers:
            raise ConfigError("BubitarConfig: a model needs at least one layer")
        if not self.norm_eps >= 0:
            raise ConfigError("BubitarConfig: norm.eps must be >= 0")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            source = getattr(m, "kv_from", None)
            if source is None:
                continue
            other = self.layers[source].mixer if source < i else None
            if not isinstance(other, BubitarLatentAttention) or other.kv_from is not None:
                raise ConfigError(f"layers[{i}]: kv_from must name an earlier latent-attention layer that makes its own cache")
            if (other.kv_rank, other.rot_dim, other.rot) != (m.kv_rank, m.rot_dim, m.rot):
                raise ConfigError(f"layers[{i}]: kv_rank, rot_dim and rotation must equal those of layer {source}")

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "BubitarConfig":
        require_keys(data, ("vocab", "width", "norm", "token_side", "layers"), "BubitarConfig")
        norm = _mapping(data, "norm", "BubitarConfig")
        require_keys(norm, ("eps",), "BubitarConfig.norm")
        eps = norm["eps"]
        if isinstance(eps, bool) or not isinstance(eps, (int, float)) or not eps >= 0:
            raise ConfigError(f"norm.eps must be a number >= 0, found {eps!r}")
        side = _mapping(data, "token_side", "BubitarConfig")
        require_keys(side, ("dim",), "BubitarConfig.token_side")
        listed = data["layers"]
        if not isinstance(listed, (list, tuple)):
            raise ConfigError("BubitarConfig: 'layers' must be a list")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{where} must be an object")
            require_keys(entry, ("type", "mixer"), where)
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}: unknown mixer type {entry['type']!r}; known: {', '.join(sorted(_MIXERS))}")
            mixer = _MIXERS[entry["type"]].from_dict(_mapping(entry, "mixer", where), where + ".mixer")
            mlp = entry.get("mlp")
            if mlp is not None and not isinstance(mlp, Mapping):
                raise ConfigError(f"{where}: 'mlp' must be an object or null")
            layers.append(BubitarLayer(mixer, None if mlp is None else BubitarFeedForward.from_dict(mlp, where + ".mlp")))
        return cls(
            vocab=positive_int(data, "vocab"),
            width=positive_int(data, "width"),
            norm_eps=float(eps),
            token_side_dim=positive_int(side, "dim"),
            layers=tuple(layers),
        )

    def to_dict(self) -> dict[str, Any]:
        return {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "norm": {"eps": self.norm_eps},
            "token_side": {"dim": self.token_side_dim},
            "layers": [layer.to_dict() for layer in self.layers],
        }
