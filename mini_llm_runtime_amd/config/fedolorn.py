"""The Fedolorn decoder's configuration.

Its config.json is nested and lists the layers one by one, each with its own sizes:

    {"architecture": "Fedolorn", "vocab": V, "width": W, "norm": {"eps": e},
     "embedding": {"scale": s},
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": c,
                           "mask": {"size": C}},
                 "mlp": {"kind": "dense", "ff": F}
                      | {"kind": "moe", "expert": {"ff": F},
                         "router": {"experts": E, "top": k, "scale": r,
                                    "groups": {"count": n, "keep": m}}}
                      | null}, ...]}

Nothing here is a size of one particular model: every layer may differ from the next.
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
class FedolornAttention:
    """Gated attention without position encoding whose mask is cut into runs of `mask_size`
    positions (None: plain causal)."""

    heads: int
    kv_heads: int
    dim: int  # width of a query and key head
    vdim: int  # width of a value head
    scale: float
    mask_size: Optional[int]

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "FedolornAttention":
        require_keys(data, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
        mask = data.get("mask")
        size = None
        if mask is not None:
            if not isinstance(mask, Mapping):
                raise ConfigError(f"{where}: 'mask' must be an object or null")
            require_keys(mask, ("size",), where + ".mask")
            size = positive_int(mask, "size")
        out = cls(
            heads=positive_int(data, "heads"),
            kv_heads=positive_int(data, "kv_heads"),
            dim=positive_int(data, "dim"),
            vdim=positive_int(data, "vdim"),
            scale=positive_float(data, "scale"),
            mask_size=size,
        )
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
        return out

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
        }
        if self.mask_size is not None:
            out["mask"] = {"size": self.mask_size}
        return out


@dataclass(frozen=True)
class FedolornFeedForward:
    """kind "dense": one feed-forward of `ff` inner features.  kind "moe": `experts` of them,
    `top` per token; the experts are cut into `groups_count` contiguous blocks, and only those of the
    `groups_keep` highest-scoring blocks are eligible."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0
    groups_count: int = 1
    groups_keep: int = 1

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "FedolornFeedForward":
        require_keys(data, ("kind",), where)
        kind = data["kind"]
        if kind == "dense":
            require_keys(data, ("ff",), where)
            return cls(kind="dense", ff=positive_int(data, "ff"))
        if kind != "moe":
            raise ConfigError(f"{where}: kind must be 'dense' or 'moe', found {kind!r}")
        expert = _mapping(data, "expert", where)
        router = _mapping(data, "router", where)
        require_keys(expert, ("ff",), where + ".expert")
        require_keys(router, ("experts", "top", "scale"), where + ".router")
        groups = router.get("groups")
        count = keep = 1
        if groups is not None:
            if not isinstance(groups, Mapping):
                raise ConfigError(f"{where}.router: 'groups' must be an object or null")
            require_keys(groups, ("count", "keep"), where + ".router.groups")
            count, keep = positive_int(groups, "count"), positive_int(groups, "keep")
        out = cls(
            kind="moe",
            ff=positive_int(expert, "ff"),
            experts=positive_int(router, "experts"),
            top=positive_int(router, "top"),
            router_scale=positive_float(router, "scale"),
            groups_count=count,
            groups_keep=keep,
        )
        if out.experts % out.groups_count:
            raise ConfigError(f"{where}: the experts do not divide into {out.groups_count} equal groups")
        if out.groups_keep > out.groups_count:
            raise ConfigError(f"{where}: more groups kept than there are")
        if out.top > out.groups_keep * (out.experts // out.groups_count):
            raise ConfigError(f"{where}: the kept groups hold fewer experts than a token uses")
        return out

    def to_dict(self) -> dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {
            "kind": "moe",
            "expert": {"ff": self.ff},
            "router": {
                "experts": self.experts, "top": self.top, "scale": self.router_scale,
                "groups": {"count": self.groups_count, "keep": self.groups_keep},
            },
        }


@dataclass(frozen=True)
class FedolornLayer:
    mixer: FedolornAttention
    mlp: Optional[FedolornFeedForward]

    def to_dict(self) -> dict[str, Any]:
        return {"type": "attention", "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class FedolornConfig(ModelConfig):
    architecture: ClassVar[str] = "Fedolorn"
    model_type: ClassVar[str] = "fedolorn"

    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: tuple[FedolornLayer, ...]

    def __post_init__(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("FedolornConfig: vocab and width must be > 0")
        if not self.layers:
            raise ConfigError("FedolornConfig: a model needs at least one layer")
        if not self.norm_eps >= 0:
            raise ConfigError("FedolornConfig: norm.eps must be >= 0")

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "FedolornConfig":
        require_keys(data, ("vocab", "width", "norm", "layers"), "FedolornConfig")
        norm = _mapping(data, "norm", "FedolornConfig")
        require_keys(norm, ("eps",), "FedolornConfig.norm")
        eps = norm["eps"]
        if isinstance(eps, bool) or not isinstance(eps, (int, float)) or not eps >= 0:
            raise ConfigError(f"norm.eps must be a number >= 0, found {eps!r}")
        embedding = data.get("embedding") or {}
        scale = positive_float(embedding, "scale") if "scale" in embedding else 1.0
        listed = data["layers"]
        if not isinstance(listed, (list, tuple)):
            raise ConfigError("FedolornConfig: 'layers' must be a list")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{where} must be an object")
            require_keys(entry, ("type", "mixer"), where)
            if entry["type"] != "attention":
                raise ConfigError(f"{where}: unknown mixer type {entry['type']!r}")
            mixer = FedolornAttention.from_dict(_mapping(entry, "mixer", where), where + ".mixer")
            mlp = entry.get("mlp")
            if mlp is not None and not isinstance(mlp, Mapping):
                raise ConfigError(f"{where}: 'mlp' must be an object or null")
            layers.append(
                FedolornLayer(mixer, None if mlp is None else FedolornFeedForward.from_dict(mlp, where + ".mlp"))
            )
        return cls(
            vocab=positive_int(data, "vocab"),
            width=positive_int(data, "width"),
            norm_eps=float(eps),
            embedding_scale=scale,
            layers=tuple(layers),
        )

    def to_dict(self) -> dict[str, Any]:
        return {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "norm": {"eps": self.norm_eps},
            "embedding": {"scale": self.embedding_scale},
            "layers": [layer.to_dict() for layer in self.layers],
        }
