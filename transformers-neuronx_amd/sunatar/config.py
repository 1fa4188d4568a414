"""Sunatar's configuration: the keys of its config.json.

The file is nested: `norm.eps`, `embedding.scale`, and `layers`, a list with one entry a layer: `type` (the
mixer's kind, "attention" or "mlstm"), `mixer` (its sizes and constants) and `mlp` (`{kind: "moe", router:
{experts, top}, expert: {ff}, shared: {ff} or absent}`, or null for a layer without a feed-forward). Every size
and constant of a model is read from there or from a tensor's shape; the design's own constants are in the code
of its parts.
"""
from dataclasses import dataclass
from typing import Any, ClassVar, Dict, Optional

from ..config.model_config import REQUIRED, ConfigError, ModelConfig

MIXERS = ("attention", "mlstm")
MLP_KINDS = ("moe",)


def _need(d, key: str, kind, where: str, positive: bool = True):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Sunatar: required key '{where}.{key}' is missing")
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
class SunatarConfig(ModelConfig):
    architecture: ClassVar[str] = "Sunatar"
    model_type: ClassVar[str] = "sunatar"

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
        mixed = None        # the first layer that blends values: the others' value projections are as wide as its
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"key '{where}' must be an object")
            if layer.get("type") not in MIXERS:
                raise ConfigError(f"key '{where}.type' must be one of {MIXERS}, got {layer.get('type')!r}")
            m = layer.get("mixer")
            for key in ("heads", "dim", "vdim"):
                _need(m, key, int, where + ".mixer")
            if layer["type"] == "attention":
                groups = _need(m, "kv_heads", int, where + ".mixer") if "kv_heads" in m else m["heads"]
                if m["heads"] % groups:
                    raise ConfigError(f"key '{where}.mixer.heads' ({m['heads']}) must be a multiple of kv_heads ({groups})")
                if "scale" in m:
                    _need(m, "scale", float, where + ".mixer")
                rot = m.get("rot")
                if rot is not None:
                    _need(rot, "base", float, where + ".mixer.rot")
                    dims = _need(rot, "dims", int, where + ".mixer.rot") if "dims" in rot else m["dim"]
                    if dims % 2 or dims > m["dim"]:
                        raise ConfigError(f"key '{where}.mixer.rot.dims' ({dims}) must be even and at most dim ({m['dim']})")
                    if rot.get("scaling") is not None:
                        for key in ("factor", "low", "high", "original"):
                            _need(rot["scaling"], key, float, where + ".mixer.rot.scaling")
                        if rot["scaling"]["high"] == rot["scaling"]["low"]:
                            raise ConfigError(f"key '{where}.mixer.rot.scaling': high and low must differ")
                if m.get("mask") is not None:
                    _need(m["mask"], "size", int, where + ".mixer.mask")
                if "v_mix" in m and not isinstance(m["v_mix"], bool):
                    raise ConfigError(f"key '{where}.mixer.v_mix' must be true or false, got {m['v_mix']!r}")
                if m.get("v_mix"):
                    mine = (groups, m["vdim"])
                    if mixed is None:
                        mixed = (i, mine)
                    elif mixed[1] != mine:
                        raise ConfigError(f"key '{where}.mixer': its values ({mine[0]} heads of {mine[1]}) are blended with "
                                          f"those of layer {mixed[0]} ({mixed[1][0]} heads of {mixed[1][1]}); kv_heads and "
                                          f"vdim must agree")
            else:
                _need(m, "gate_cap", float, where + ".mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"key '{where}.mlp.kind' must be one of {MLP_KINDS}, got {mlp.get('kind')!r}")
                experts = _need(mlp.get("router"), "experts", int, where + ".mlp.router")
                top = _need(mlp.get("router"), "top", int, where + ".mlp.router")
                if top > experts:
                    raise ConfigError(f"key '{where}.mlp.router.top' ({top}) exceeds the experts ({experts})")
                _need(mlp.get("expert"), "ff", int, where + ".mlp.expert")
                if mlp.get("shared") is not None:
                    _need(mlp["shared"], "ff", int, where + ".mlp.shared")

    def to_dict(self) -> Dict[str, Any]:
        d = super().to_dict()
        d["architecture"] = self.architecture
        d["model_type"] = self.model_type
        return {k: v for k, v in d.items() if v is not None}
