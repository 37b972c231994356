"""Tadolix's configuration: the keys of its config.json.

The file is nested: `norm.eps`, `embedding.scale`, `canon.taps`, `streams`, `loop.{start, stop, times}` and
`layers`, a list with one entry a layer: `type` (the mixer's kind, "parallel" or "rglru"), `mixer` (its sizes and
constants) and `mlp` (`{kind: "dense", ff}`, or null for a layer without a feed-forward). A "parallel" mixer has
`left` (the attention: `heads`, `kv_heads`, `dim`, `vdim`, `scale`, `softcap`, `bias_max`, `mask.size`), `right`
(the gated recurrence: `width`) and the two factors `left_scale`, `right_scale`; an "rglru" mixer has `width`,
`blocks` and `conv` (its taps). Every size and constant of a model is read from there or from a tensor's shape;
the design's own constants are in the code of its parts.
"""
from dataclasses import dataclass
from typing import Any, ClassVar, Dict, Optional

from ..config.model_config import REQUIRED, ConfigError, ModelConfig

MIXERS = ("parallel", "rglru")
MLP_KINDS = ("dense",)


def _need(d, key: str, kind, where: str, positive: bool = True):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Tadolix: required key '{where}.{key}' is missing")
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


@dataclass(frozen=True)
class TadolixConfig(ModelConfig):
    architecture: ClassVar[str] = "Tadolix"
    model_type: ClassVar[str] = "tadolix"

    vocab: int = REQUIRED
    width: int = REQUIRED
    layers: list = REQUIRED
    norm: dict = REQUIRED
    embedding: Optional[dict] = None
    canon: Optional[dict] = None
    streams: Optional[int] = None      # absent: one stream and the plain residual sum
    loop: Optional[dict] = None
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
        if f.name in ("norm", "embedding", "canon", "loop"):
            if value is not None and not isinstance(value, dict):
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

    @property
    def taps(self) -> int:
        return int((self.canon or {}).get("taps", 0))

    def run_order(self):
        """The layers in the order they run: those of the loop `times` times in a row."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        start, stop, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))

    def validate(self) -> None:
        for key in ("vocab", "width", "max_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"key '{key}' must be positive, got {getattr(self, key)}")
        if self.streams is not None and (isinstance(self.streams, bool) or not isinstance(self.streams, int)
                                         or self.streams <= 0):
            raise ConfigError(f"key 'streams' must be a positive integer, got {self.streams!r}")
        _need(self.norm, "eps", float, "norm")
        if self.embedding is not None and "scale" in self.embedding:
            _need(self.embedding, "scale", float, "embedding", positive=False)
        if self.canon is not None:
            _need(self.canon, "taps", int, "canon")
        if self.loop is not None:
            start = _need(self.loop, "start", int, "loop", positive=False)
            stop = _need(self.loop, "stop", int, "loop", positive=False)
            _need(self.loop, "times", int, "loop")
            if not 0 <= start <= stop <= len(self.layers):
                raise ConfigError(f"key 'loop': layers {start} to {stop} of {len(self.layers)}")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"key '{where}' must be an object")
            if layer.get("type") not in MIXERS:
                raise ConfigError(f"key '{where}.type' must be one of {MIXERS}, got {layer.get('type')!r}")
            m = layer.get("mixer")
            if layer["type"] == "parallel":
                left, right = (m or {}).get("left"), (m or {}).get("right")
                for key in ("heads", "dim", "vdim"):
                    _need(left, key, int, where + ".mixer.left")
                groups = _need(left, "kv_heads", int, where + ".mixer.left") if "kv_heads" in left else left["heads"]
                if left["heads"] % groups:
                    raise ConfigError(f"key '{where}.mixer.left.heads' ({left['heads']}) must be a multiple of "
                                      f"kv_heads ({groups})")
                if "scale" in left:
                    _need(left, "scale", float, where + ".mixer.left")
                if left.get("softcap") is not None:
                    _need(left, "softcap", float, where + ".mixer.left")
                _need(left, "bias_max", int, where + ".mixer.left")
                if "bias_rows" in left:
                    _need(left, "bias_rows", int, where + ".mixer.left")
                if left.get("mask") is not None:
                    _need(left["mask"], "size", int, where + ".mixer.left.mask")
                _need(right, "width", int, where + ".mixer.right")
                for key in ("left_scale", "right_scale"):
                    if key in m:
                        _need(m, key, float, where + ".mixer", positive=False)
            else:
                width = _need(m, "width", int, where + ".mixer")
                blocks = _need(m, "blocks", int, where + ".mixer")
                _need(m, "conv", int, where + ".mixer")
                if width % blocks:
                    raise ConfigError(f"key '{where}.mixer.width' ({width}) must be a multiple of blocks ({blocks})")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"key '{where}.mlp.kind' must be one of {MLP_KINDS}, got {mlp.get('kind')!r}")
                _need(mlp, "ff", int, where + ".mlp")

    def to_dict(self) -> Dict[str, Any]:
        d = super().to_dict()
        d["architecture"] = self.architecture
        d["model_type"] = self.model_type
        return {k: v for k, v in d.items() if v is not None}
