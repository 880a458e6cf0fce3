"""Configuration of the Napadra decoder, from its config.json keys.

The file is nested: `layers` lists the layers in their order, each with its `type` (which mixer: "attention" or
"mlstm"), the mixer's sizes and constants under `mixer` and its feed-forward under `mlp` (null: the layer has
none); `norm.eps`, `residual_mult`, `streams`, `vocab` and `width` hold for the whole model.  Every size and
constant a model may choose is read from here; nothing is assumed equal between layers.
"""
from __future__ import annotations

import dataclasses
from typing import Any

from .base import ConfigError, ModelConfig


def _number(where: str, raw: dict, key: str, kind=int, positive: bool = True, default=None):
    if not isinstance(raw, dict) or raw.get(key) is None:
        if default is not None:
            return default
        raise ConfigError(f"config.json: {where} lacks {key!r}")
    value = raw[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or (kind is int and value != int(value)):
        raise ConfigError(f"config.json: {where}.{key} should be {kind.__name__}, found {value!r}")
    value = kind(value)
    if positive and not value > 0:
        raise ConfigError(f"config.json: {where}.{key} must be positive, found {value!r}")
    return value


@dataclasses.dataclass(frozen=True)
class NapadraConfig(ModelConfig):
    vocab: int
    width: int
    streams: int
    residual_mult: float
    norm: dict
    layers: list
    max_positions: int = 1 << 20      # positions are not bounded by the design: the bound is this engine's own

    MIXERS = ("attention", "mlstm")

    def validate(self) -> None:
        for key in ("vocab", "width", "streams", "max_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, found {getattr(self, key)}")
        if self.width % 2:
            raise ConfigError(f"width {self.width} is odd; the position vector pairs a sine with a cosine")
        _number("norm", self.norm, "eps", float, positive=False)
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config.json: `layers` must be a list with at least one layer")
        for index, layer in enumerate(self.layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict) or layer.get("type") not in self.MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {', '.join(self.MIXERS)}")
            mixer = layer.get("mixer")
            for key in ("heads", "dim", "vdim"):
                _number(f"{where}.mixer", mixer, key)
            if layer["type"] == "attention":
                heads, kv_heads = mixer["heads"], _number(f"{where}.mixer", mixer, "kv_heads")
                if heads % kv_heads:
                    raise ConfigError(f"{where}: {heads} query heads is not a multiple of {kv_heads} kv heads")
                _number(f"{where}.mixer", mixer, "scale", float)
                if mixer.get("mask") is not None:
                    _number(f"{where}.mixer.mask", mixer["mask"], "size")
                source = mixer.get("kv_from")
                if source is not None:
                    if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < index:
                        raise ConfigError(f"{where}.mixer.kv_from must name an earlier layer, found {source!r}")
                    other = self.layers[source]
                    if other.get("type") != "attention" or other["mixer"].get("kv_from") is not None:
                        raise ConfigError(f"{where}.mixer.kv_from = {source}: that layer has no keys and values of its own")
                    for key in ("kv_heads", "dim", "vdim"):
                        if other["mixer"].get(key) != mixer[key]:
                            raise ConfigError(f"{where} reads layer {source}'s keys and values but differs from it in {key}")
            else:
                _number(f"{where}.mixer", mixer, "gate_cap", float)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind must be dense")
                _number(f"{where}.mlp", mlp, "ff")
                _number(f"{where}.mlp", mlp, "limit", float)

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    def to_dict(self) -> dict[str, Any]:
        out = super().to_dict()
        out.pop("architectures")
        out.pop("max_positions")
        return {"architecture": self.architecture, **out}
