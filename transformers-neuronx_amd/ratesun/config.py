"""Ratesun's configuration: the keys of its config.json.

The file is nested: `norm.eps`, `canon.taps`, `embedding.bigram.{buckets, mul_prev, mul_cur}`, `token_side.dim`,
and `layers`, a list with one entry a layer: `type` (the mixer's kind), `mixer` (its sizes and constants) and
`mlp` (`{kind, ff}`, or null for a layer without a feed-forward). Every size and constant of a model is read
from there or from a tensor's shape; the design's own constants are in the code of its parts.
"""
from dataclasses import dataclass, field
from typing import Any, ClassVar, Dict, List, Optional

from ..config.model_config import REQUIRED, ConfigError, ModelConfig

MIXERS = ("latent_attention",)
MLP_KINDS = ("dense",)


def _need(d: Dict, key: str, kind, where: str, positive: bool = True):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Ratesun: required key '{where}.{key}' is missing")
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
class RatesunConfig(ModelConfig):
    architecture: ClassVar[str] = "Ratesun"
    model_type: ClassVar[str] = "ratesun"

    vocab: int = REQUIRED
    width: int = REQUIRED
    layers: list = REQUIRED
    norm: dict = REQUIRED
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    canon: Optional[dict] = None
    embedding: Optional[dict] = None
    token_side: Optional[dict] = None
    # not a key of the design, which has no longest request: the most positions the engine's tables are made for
    max_positions: int = 1 << 17
    init_std: float = 0.05
    torch_dtype: str = "bfloat16"

    @staticmethod
    def _coerce(f, value):
        if f.name in ("layers",):
            if not isinstance(value, list) or not value:
                raise ConfigError(f"key 'layers' must be a list with one entry a layer, got {type(value).__name__}")
            return value
        if f.name in ("norm", "canon", "embedding", "token_side"):
            if not isinstance(value, dict):
                raise ConfigError(f"key '{f.name}' must be an object, got {value!r}")
            return value
        return ModelConfig._coerce(f, value)

    # ---------------------------------------------------------------- what the nested keys say

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    @property
    def taps(self) -> int:
        return int(self.canon["taps"]) if self.canon else 0

    @property
    def bigram(self) -> Optional[dict]:
        return (self.embedding or {}).get("bigram")

    @property
    def side_dim(self) -> int:
        return int(self.token_side["dim"]) if self.token_side else 0

    def validate(self) -> None:
        for key in ("vocab", "width", "max_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"key '{key}' must be positive, got {getattr(self, key)}")
        _need(self.norm, "eps", float, "norm")
        if self.canon is not None:
            _need(self.canon, "taps", int, "canon")
        if self.bigram is not None:
            for key in ("buckets", "mul_prev", "mul_cur"):
                _need(self.bigram, key, int, "embedding.bigram", positive=key == "buckets")
        if self.token_side is not None:
            _need(self.token_side, "dim", int, "token_side")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"key '{where}' must be an object")
            if layer.get("type") not in MIXERS:
                raise ConfigError(f"key '{where}.type' must be one of {MIXERS}, got {layer.get('type')!r}")
            m = layer.get("mixer")
            for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"):
                _need(m, key, int, where + ".mixer")
            if "scale" in m:
                _need(m, "scale", float, where + ".mixer")
            rot = m.get("rot")
            _need(rot, "base", float, where + ".mixer.rot")
            dims = _need(rot, "dims", int, where + ".mixer.rot") if "dims" in rot else m["rot_dim"]
            if dims % 2 or dims > m["rot_dim"]:
                raise ConfigError(f"key '{where}.mixer.rot.dims' ({dims}) must be even and at most rot_dim ({m['rot_dim']})")
            if m.get("mask") is not None:
                _need(m["mask"], "size", int, where + ".mixer.mask")
            src = m.get("kv_from")
            if src is not None:
                if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < i:
                    raise ConfigError(f"key '{where}.mixer.kv_from' must name an earlier layer, got {src!r}")
                other = self.layers[src]["mixer"]
                if other.get("kv_from") is not None:
                    raise ConfigError(f"key '{where}.mixer.kv_from' names layer {src}, which has no latent of its own")
                for key in ("kv_rank", "rot_dim"):
                    if other[key] != m[key]:
                        raise ConfigError(f"key '{where}.mixer.{key}' ({m[key]}) differs from that of layer {src}, "
                                          f"whose latent it reads ({other[key]})")
                if other["rot"] != m["rot"]:
                    raise ConfigError(f"key '{where}.mixer.rot' differs from that of layer {src}, whose latent it reads")
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
