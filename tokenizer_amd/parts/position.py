"""Position encodings applied to queries and keys before the keys go into the cache."""
from __future__ import annotations

import math

import torch

from .base import POSITIONS, PositionEncoding, Repeatable, Runtime, StoreEpilogue
from .spec import PositionSpec


@POSITIONS.register("none")
class NoPosition(PositionEncoding):
    """No encoding: the projection bias is added and keys and values are stored as they are."""
    graph_safe = True


    def __init__(self, spec: PositionSpec, runtime: Runtime):
        self.runtime = runtime

    def table(self):
        return None

    def repeatable(self):
        return Repeatable(("none",), ())

    def epilogue(self):
        # A subclass that encodes in its own way inherits this method but not the promise: it has to offer an
        # epilogue of its own (or none).
        if type(self).encode_and_store is not NoPosition.encode_and_store:
            return None
        return StoreEpilogue(self.table())

    def encode_and_store(self, qkv, bias, n_q, n_kv, head_dim, ctx, cache, value_dim=None):
        """`value_dim`: the size of a value head where it is not `head_dim`.  `n_kv` 0: the rows hold query heads
        alone and nothing is stored."""
        slots = ctx.slots[cache.group] if cache.writes and n_kv else None
        extra = {} if value_dim is None or value_dim == head_dim else {"value_dim": value_dim}
        if n_kv == 0 and self.table() is None and bias is None:
            return                              # nothing to add, rotate or store
        self.runtime.ops.rope_store(qkv, bias, ctx.positions, self.table(), slots,
                                    cache.k_pages if slots is not None else None,
                                    cache.v_pages if slots is not None else None, n_q, n_kv, head_dim, **extra)


@POSITIONS.register("rope_half_split")
class RotaryHalfSplit(NoPosition):
    """Rotation of the two halves of a head against each other (qwen-infer/src/model.rs:131-172).

    inv_freq[i] = 1 / theta^(2i/d) is computed in float64 and kept as float32; the angle of
    position p is p * inv_freq[i] in float32; the table holds cos then sin of the d/2 angles for
    every position up to `max_positions`.  Keys are stored after the rotation.
    """

    _tables: dict[tuple, torch.Tensor] = {}

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        if spec.head_dim % 2:
            raise ValueError(f"rope needs an even head size, found {spec.head_dim}")
        d = spec.head_dim
        key = (d, float(spec.theta), spec.max_positions, str(runtime.device))
        if key not in self._tables:               # the layers of a model share one table
            inv_freq = torch.tensor([1.0 / (float(spec.theta) ** (i / d)) for i in range(0, d, 2)],
                                    dtype=torch.float64).to(torch.float32)
            positions = torch.arange(spec.max_positions, dtype=torch.float32)
            angles = positions[:, None] * inv_freq[None, :]
            self._tables[key] = torch.cat([angles.cos(), angles.sin()], dim=1).contiguous().to(runtime.device)
        self.cos_sin = self._tables[key]
        self.max_positions = spec.max_positions

    def table(self):
        return self.cos_sin

    def repeatable(self):
        return Repeatable(("rope_half_split", self.max_positions), (self.cos_sin,))


def scaled_rates(theta: float, dims: int, scaling: dict | None) -> torch.Tensor:
    """float32 [dims / 2]: the rates f_i = theta^(-2i/dims), worked out in float64.  `scaling` (factor, low, high,
    original) slows the long waves: with wavelength l = 2 pi / f a rate stays as it is where l < original / high,
    becomes f / factor where l > original / low, and in between is (1 - s) f / factor + s f with
    s = (original / l - low) / (high - low)."""
    rates = []
    for i in range(dims // 2):
        f = float(theta) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[key]) for key in ("factor", "low", "high", "original"))
            wave = 2.0 * math.pi / f
            if wave > original / low:
                f = f / factor
            elif wave >= original / high:
                s = (original / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        rates.append(f)
    return torch.tensor(rates, dtype=torch.float64).to(torch.float32)


@POSITIONS.register("rope_partial")
class RotaryPartial(PositionEncoding):
    """Rotation of the first `dims` coordinates of every query and key head (options `dims`, even and at most the
    head size; `scaling`, see `scaled_rates`): coordinate i < dims / 2 is paired with coordinate i + dims / 2 and the
    pair turns by the angle position * f_i; the coordinates from `dims` on pass unchanged.  There is no table of
    positions: the kernel forms the angle in float32 from the position and the rate and takes its accurate sine and
    cosine, so positions are bounded by nothing here.  Keys are stored after the rotation.

    The same kernel adds the projection's bias before and, for mixers that ask for it, normalises all query rows
    at once and all key rows at once (an RMS norm with a weight over the whole projection) before the rotation."""
    graph_safe = True

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        self.runtime = runtime
        self.dims = int(spec.options.get("dims", spec.head_dim))
        if self.dims % 2 or not 0 <= self.dims <= spec.head_dim:
            raise ValueError(f"a rotation over {self.dims} of {spec.head_dim} coordinates")
        self.rates = scaled_rates(spec.theta, self.dims, spec.options.get("scaling")).to(runtime.device).contiguous()

    def encode_and_store(self, qkv, bias, n_q, n_kv, head_dim, ctx, cache, value_dim=None, value_heads=None,
                         q_norm=None, k_norm=None, eps=0.0):
        """Rows of `qkv`: n_q query heads and n_kv key heads of `head_dim`, then `value_heads` (n_kv if None) value
        heads of `value_dim`; whatever lies behind them in a row is left alone."""
        slots = ctx.slots[cache.group] if cache.writes and n_kv else None
        self.runtime.ops.norm_rotate_store(qkv, bias, ctx.positions, self.rates, self.dims, slots,
                                           cache.k_pages if slots is not None else None,
                                           cache.v_pages if slots is not None else None, n_q, n_kv,
                                           n_kv if value_heads is None else value_heads, head_dim,
                                           head_dim if value_dim is None else value_dim, q_norm, k_norm, eps)
