"""Configuration of the Dolidra decoder, from its config.json keys.

The file is nested: `layers` lists the layers in their order, each with its `type` (which mixer: "attention", the
differential one, or "attention_2", the gated one with normalised queries and keys), the mixer's sizes and
constants under `mixer` and its feed-forward under `mlp` (null: the layer has none; `kind` "dense" or "moe");
`loop` (start, stop, times) names a run of layers that is gone through several times; `token_side.dim` is the
width of the per-layer token input; `norm.eps`, `vocab` and `width` hold for the whole model.  Every size and
constant a model may choose is read from here; nothing is assumed equal between layers.
"""
from __future__ import annotations

import dataclasses
from typing import Any

from .base import ConfigError, ModelConfig
from .napadra import _number


@dataclasses.dataclass(frozen=True)
class DolidraConfig(ModelConfig):
    vocab: int
    width: int
    norm: dict
    layers: list
    loop: dict | None = None
    token_side: dict | None = None
    max_positions: int = 1 << 20      # positions are not bounded by the design: the bound is this engine's own

    MIXERS = ("attention", "attention_2")

    def validate(self) -> None:
        for key in ("vocab", "width", "max_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, found {getattr(self, key)}")
        _number("norm", self.norm, "eps", float, positive=False)
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config.json: `layers` must be a list with at least one layer")
        for index, layer in enumerate(self.layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict) or layer.get("type") not in self.MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {', '.join(self.MIXERS)}")
            mixer = layer.get("mixer")
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _number(f"{where}.mixer", mixer, key)
            if mixer["heads"] % mixer["kv_heads"]:
                raise ConfigError(f"{where}: {mixer['heads']} query heads is not a multiple of {mixer['kv_heads']} kv heads")
            _number(f"{where}.mixer", mixer, "scale", float)
            mask = mixer.get("mask")
            if mask is not None:
                _number(f"{where}.mixer.mask", mask, "size")
                if mask.get("keep_first") is not None:
                    _number(f"{where}.mixer.mask", mask, "keep_first", positive=False)
            rot = mixer.get("rot")
            if rot is not None:
                dims = _number(f"{where}.mixer.rot", rot, "dims")
                _number(f"{where}.mixer.rot", rot, "base", float)
                if dims % 2 or dims > mixer["dim"]:
                    raise ConfigError(f"{where}.mixer.rot.dims must be even and at most the head size, found {dims}")
                if rot.get("scaling") is not None:
                    for key in ("factor", "low", "high", "original"):
                        _number(f"{where}.mixer.rot.scaling", rot["scaling"], key, float)
                    if rot["scaling"]["high"] == rot["scaling"]["low"]:
                        raise ConfigError(f"{where}.mixer.rot.scaling: high and low must differ")
            if layer["type"] == "attention":
                _number(f"{where}.mixer", mixer, "diff", float, positive=False)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                    raise ConfigError(f"config.json: {where}.mlp.kind must be dense or moe")
                if mlp["kind"] == "dense":
                    _number(f"{where}.mlp", mlp, "ff")
                else:
                    _number(f"{where}.mlp.expert", mlp.get("expert"), "ff")
                    experts = _number(f"{where}.mlp.router", mlp.get("router"), "experts")
                    top = _number(f"{where}.mlp.router", mlp.get("router"), "top")
                    if top > experts:
                        raise ConfigError(f"{where}.mlp.router: top {top} of {experts} experts")
                    if mlp.get("shared") is not None:
                        _number(f"{where}.mlp.shared", mlp["shared"], "ff")
        if self.loop is not None:
            start = _number("loop", self.loop, "start", positive=False)
            stop = _number("loop", self.loop, "stop", positive=False)
            _number("loop", self.loop, "times")
            if not 0 <= start <= stop <= len(self.layers):
                raise ConfigError(f"loop: layers {start}..{stop} of {len(self.layers)}")
        if self.token_side is not None:
            _number("token_side", self.token_side, "dim")

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    def run_order(self) -> list[int]:
        """Layer indices in the order they run."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        start, stop, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))

    def to_dict(self) -> dict[str, Any]:
        out = super().to_dict()
        out.pop("architectures")
        out.pop("max_positions")
        return {"architecture": self.architecture, **out}
