"""Zotunex's configuration: the keys of its config.json.

The file is nested: `norm.eps`, `embedding.scale`, and `layers`, a list with one entry a layer: `type` (the mixer's
kind, "attention" or "latent_attention"), `mixer` (its sizes and constants) and `mlp` (`{kind: "dense", ff}`,
`{kind: "moe", router: {experts, top, scale}, expert: {ff, limit}, shared: {ff, limit} or absent}`, or null for a
layer without a feed-forward). Every size and constant of a model is read from there or from a tensor's shape; the
design's own constants are in the code of its parts.
"""
from dataclasses import dataclass
from typing import Any, ClassVar, Dict, Optional

from ..config.model_config import REQUIRED, ConfigError, ModelConfig

MIXERS = ("attention", "latent_attention")
MLP_KINDS = ("dense", "moe")


def _need(d, key: str, kind, where: str, positive: bool = True):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Zotunex: required key '{where}.{key}' is missing")
    v = d[key]
    if kind is int and (isinstance(v, bool) or not isinstance(v, int)):
        raise ConfigError(f"key '{where}.{key}' must be an integer, got {v!r}")
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"key '{where}.{key}' must be a number, got {v!r}")
        v = float(v)
    if positive and not v > 0:
        raise ConfigError(f"key '{where}.{key}' must be positive, got {v!r}")
    return v


def _rotation(rot, where: str, most: int) -> None:
    """`rot` = {base, dims, scaling: {factor} or absent}: `dims` even and at most `most`."""
    _need(rot, "base", float, where)
    dims = _need(rot, "dims", int, where)
    if dims % 2 or dims > most:
        raise ConfigError(f"key '{where}.dims' ({dims}) must be even and at most {most}")
    if rot.get("scaling") is not None:
        _need(rot["scaling"], "factor", float, where + ".scaling")


@dataclass(frozen=True)
class ZotunexConfig(ModelConfig):
    architecture: ClassVar[str] = "Zotunex"
    model_type: ClassVar[str] = "zotunex"

    vocab: int = REQUIRED
    width: int = REQUIRED
    layers: list = REQUIRED
    norm: dict = REQUIRED
    embedding: Optional[dict] = None
    # not a key of the design, which has no longest request: the most positions the engine's tables are made for
    max_positions: int = 1 << 17
    init_std: float = 0.05
    torch_dtype: str = "bfloat16"

    @staticmethod
    def _coerce(f, value):
        if f.name == "layers":
            if not isinstance(value, list) or not value:
                raise ConfigError(f"key 'layers' must be a list with one entry a layer, got {type(value).__name__}")
            return value
        if f.name in ("norm", "embedding"):
            if not isinstance(value, dict):
                raise ConfigError(f"key '{f.name}' must be an object, got {value!r}")
            return value
        return ModelConfig._coerce(f, value)

    # ---------------------------------------------------------------- what the nested keys say

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    @property
    def embedding_scale(self) -> float:
        return float((self.embedding or {}).get("scale", 1.0))

    def validate(self) -> None:
        for key in ("vocab", "width", "max_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"key '{key}' must be positive, got {getattr(self, key)}")
        _need(self.norm, "eps", float, "norm")
        if self.embedding is not None and "scale" in self.embedding:
            _need(self.embedding, "scale", float, "embedding", positive=False)
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"key '{where}' must be an object")
            if layer.get("type") not in MIXERS:
                raise ConfigError(f"key '{where}.type' must be one of {MIXERS}, got {layer.get('type')!r}")
            m, at = layer.get("mixer"), where + ".mixer"
            for key in ("heads", "dim") + (("vdim",) if layer["type"] != "attention" else ()):
                _need(m, key, int, at)
            _need(m, "scale", float, at)
            if layer["type"] == "attention":
                groups = _need(m, "kv_heads", int, at) if "kv_heads" in m else m["heads"]
                if m["heads"] % groups:
                    raise ConfigError(f"key '{at}.heads' ({m['heads']}) must be a multiple of kv_heads ({groups})")
                if m.get("vdim", m["dim"]) != m["dim"]:
                    raise ConfigError(f"key '{at}.vdim' ({m['vdim']}) must equal dim ({m['dim']}): the values are the keys")
                if m.get("rot") is not None:
                    _rotation(m["rot"], at + ".rot", m["dim"])
            else:
                _need(m, "kv_rank", int, at)
                rot_dim = _need(m, "rot_dim", int, at)
                if rot_dim % 2:
                    raise ConfigError(f"key '{at}.rot_dim' ({rot_dim}) must be even")
                _rotation(m.get("rot"), at + ".rot", rot_dim)
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            at = where + ".mlp"
            if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                raise ConfigError(f"key '{at}.kind' must be one of {MLP_KINDS}")
            if mlp["kind"] == "dense":
                _need(mlp, "ff", int, at)
                continue
            experts = _need(mlp.get("router"), "experts", int, at + ".router")
            top = _need(mlp.get("router"), "top", int, at + ".router")
            if top > experts:
                raise ConfigError(f"key '{at}.router.top' ({top}) exceeds the experts ({experts})")
            if "scale" in mlp["router"]:
                _need(mlp["router"], "scale", float, at + ".router")
            _need(mlp.get("expert"), "ff", int, at + ".expert")
            _need(mlp.get("expert"), "limit", float, at + ".expert")
            if mlp.get("shared") is not None:
                _need(mlp["shared"], "ff", int, at + ".shared")
                _need(mlp["shared"], "limit", float, at + ".shared")

    def to_dict(self) -> Dict[str, Any]:
        d = super().to_dict()
        d["architecture"] = self.architecture
        d["model_type"] = self.model_type
        return {k: v for k, v in d.items() if v is not None}
