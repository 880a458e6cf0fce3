"""Several residual streams with learned reads, writes and mixing (hyper-connections), and the frame around them.

Instead of one residual x a model keeps S copies x_1 .. x_S [tokens, S, width], all equal to the embedding
output at the start.  A sub-layer reads u = sum_s r[s] x_s, runs y = f(norm(u)), and all streams change at once:
x_t <- sum_s M[s, t] x_s + c[t] * (g . y), with r, c (float [S]) and M (float [S, S], indexed [from, to]) the
sub-layer's own tensors `in`, `out`, `mix`, g an optional scale per coordinate (layer scale) and a constant
multiplier folded into c.  At the end the streams are added up.  With S = 1, r = c = M = 1 this is the plain
pre-norm layer.

As in the pre-norm block the write of one sub-layer and the read and norm of the next are one kernel
(`Ops.streams_step`): a sub-layer hands its output on as a `StreamWrite` still to be applied.

A token shift, if the layer has one, stands between the mixer's norm and the mixer: row t becomes
h_t + (h_(t-1) - h_t) * mu with the unshifted h_(t-1) of the same sequence (zeros before position 0).  The last
unshifted row of a step is per-request state (`CacheNeed.block_state_shape`), so a prompt cut anywhere and
decoding go on from it.
"""
from __future__ import annotations

import dataclasses

import torch

from .base import BLOCKS, FRAMES, Block
from .model import DecoderModel
from .spec import CacheNeed, LayerSpec, TensorSpec


@dataclasses.dataclass
class StreamWrite:
    """A sub-layer's output that is not in the streams yet: x_t <- sum_s mix[s, t] x_s + out[t] * scale * y."""
    y: torch.Tensor               # [tokens, width] in the compute dtype
    mix: torch.Tensor             # float32 [S, S]
    out: torch.Tensor             # float32 [S] (the residual multiplier is in it)
    scale: torch.Tensor | None    # float32 [width] or None


class _Connection:
    def __init__(self, tensors, prefix: str, streams: int, multiplier: float):
        self.read = tensors[f"{prefix}.in"].to(torch.float32).contiguous()
        self.out = (tensors[f"{prefix}.out"].to(torch.float32) * multiplier).contiguous()
        self.mix = tensors[f"{prefix}.mix"].to(torch.float32).contiguous()
        if self.read.numel() != streams or tuple(self.mix.shape) != (streams, streams):
            raise ValueError(f"{prefix}: the connection's tensors do not fit {streams} streams")


@BLOCKS.register("hyper_streams")
class HyperStreamsBlock(Block):
    """Pre-norm sub-layers around S residual streams.  Options of the layer: `streams`, `residual_mult` (every
    write is multiplied by it), `layer_scale` (tensors `ls1`, `ls2` [width]), `token_shift` (tensor `shift` [width]).
    Tensors: `hc1.in|out|mix` for the mixer, `hc2.*` for the feed-forward."""
    graph_safe = True

    @staticmethod
    def tensor_specs(layer: LayerSpec) -> dict[str, TensorSpec]:
        s, width = int(layer.options["streams"]), int(layer.options["width"])
        out = {}
        for q, part in ((1, layer.mixer), (2, layer.feed_forward)):
            if part is None:
                continue
            out.update({f"hc{q}.in": TensorSpec((s,), init="ones", role="vector"),
                        f"hc{q}.out": TensorSpec((s,), init="ones", role="vector"),
                        f"hc{q}.mix": TensorSpec((s, s), init="eye", role="vector")})
            if layer.options.get("layer_scale"):
                out[f"ls{q}"] = TensorSpec((width,), init="ones", role="vector")
        if layer.mixer is not None and layer.options.get("token_shift"):
            out["shift"] = TensorSpec((width,), role="vector", std=0.5)
        return out

    @staticmethod
    def cache_need(layer: LayerSpec, need: CacheNeed) -> CacheNeed:
        if layer.mixer is None or not layer.options.get("token_shift"):
            return need
        return dataclasses.replace(need, block_state_shape=(int(layer.options["width"]),))

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward, layer: LayerSpec, tensors, runtime):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward
        self.runtime = runtime
        self.streams = int(layer.options["streams"])
        multiplier = float(layer.options.get("residual_mult", 1.0))
        scaled = bool(layer.options.get("layer_scale"))
        self.mixer_link = self.ff_link = self.mixer_scale = self.ff_scale = self.shift = None
        if mixer is not None:
            self.mixer_link = _Connection(tensors, "hc1", self.streams, multiplier)
            self.mixer_scale = tensors["ls1"].to(torch.float32).contiguous() if scaled else None
            if layer.options.get("token_shift"):
                self.shift = tensors["shift"].to(torch.float32).contiguous()
        if feed_forward is not None:
            self.ff_link = _Connection(tensors, "hc2", self.streams, multiplier)
            self.ff_scale = tensors["ls2"].to(torch.float32).contiguous() if scaled else None
        for norm in (mixer_norm, feed_forward_norm):
            if norm is not None and getattr(norm, "gain", None) is None:
                raise ValueError("the streams' kernels take a norm of one number (`gain`)")

    def _read(self, streams, write, link, norm, dtype):
        tokens, width = streams.shape[0], streams.shape[2]
        out = torch.empty((tokens, width), dtype=dtype, device=streams.device)
        return self.runtime.ops.streams_step(streams, write, link.read, norm.gain, norm.eps, out)

    def forward(self, streams, write, ctx, cache):
        ops, dtype = self.runtime.ops, self.runtime.dtype
        if self.mixer is not None:
            if self.shift is None:
                h = self._read(streams, write, self.mixer_link, self.mixer_norm, dtype)
            else:
                if cache.block_state is None:
                    raise ValueError("a layer with a token shift needs its state in the request's slot")
                if getattr(ops, "fuses_single_shift", False) and ctx.q_tiles.numel() == 0:
                    # One token per request: read, norm, shift and the new state in one kernel.
                    h = torch.empty((streams.shape[0], streams.shape[2]), dtype=dtype, device=streams.device)
                    ops.streams_step(streams, write, self.mixer_link.read, self.mixer_norm.gain, self.mixer_norm.eps, h,
                                     shift=(self.shift, cache.block_state, ctx))
                else:
                    plain = self._read(streams, write, self.mixer_link, self.mixer_norm, torch.float32)
                    h = torch.empty(plain.shape, dtype=dtype, device=plain.device)
                    ops.token_shift(plain, self.shift, cache.block_state, ctx.cu_q, ctx.first_position, ctx.state_slots,
                                    ctx.entry_of_token, h)
            y = self.mixer.forward(h, ctx, cache)
            write = StreamWrite(y, self.mixer_link.mix, self.mixer_link.out, self.mixer_scale)
        if self.feed_forward is not None:
            h = self._read(streams, write, self.ff_link, self.feed_forward_norm, dtype)
            y = self.feed_forward.forward(h, ctx)
            write = StreamWrite(y, self.ff_link.mix, self.ff_link.out, self.ff_scale)
        return write


@FRAMES.register("stream_decoder")
class StreamDecoder(DecoderModel):
    """The decoder frame over S residual streams: the embedding output, with a position vector added if the
    model's options name one (`embedding_position` "sinusoidal": entry 2i is sin(p b^(-2i/width)), entry 2i+1 the
    cosine, b = `position_base`), fills every stream; the layers' blocks work on [tokens, S, width]; the streams'
    sum goes through the final norm to the head."""

    def __init__(self, spec, tensors, runtime):
        super().__init__(spec, tensors, runtime)
        self.n_streams = int(spec.options.get("streams", 1))
        self.rates = None
        kind = spec.options.get("embedding_position")
        if kind == "sinusoidal":
            width, base = spec.hidden_size, float(spec.options.get("position_base", 10000.0))
            # (The rates in float64, kept as float32; the angle is position * rate in float32.)
            self.rates = torch.tensor([base ** (-2.0 * i / width) for i in range(width // 2)],
                                      dtype=torch.float64).to(torch.float32).to(runtime.device)
        elif kind is not None:
            raise ValueError(f"unknown embedding position {kind!r}")
        if getattr(self.final_norm, "gain", None) is None:
            raise ValueError("the streams' kernels take a norm of one number (`gain`)")
        self.ones = torch.ones(self.n_streams, dtype=torch.float32, device=runtime.device)
        self.graph_safe = all(getattr(b, "graph_safe", False) and getattr(b.mixer, "graph_safe", False)
                              and (b.feed_forward is None or getattr(b.feed_forward, "graph_safe", False))
                              for b in self.blocks)
        self.repeat_layers = False         # the blocks make no promise of equal calls (they keep state)

    def embed(self, ctx) -> torch.Tensor:
        streams = torch.empty((ctx.n_tokens, self.n_streams, self.spec.hidden_size), dtype=torch.float32,
                              device=self.runtime.device)
        return self.runtime.ops.embedding_streams(ctx.token_ids, self.embedding, ctx.positions, self.rates, streams)

    def logits(self, streams, write, ctx) -> torch.Tensor:
        wanted = torch.empty((ctx.want_rows.numel(), self.spec.hidden_size), dtype=self.runtime.dtype,
                             device=streams.device)
        self.runtime.ops.streams_step(streams, write, self.ones, self.final_norm.gain, self.final_norm.eps, wanted,
                                      rows=ctx.want_rows)
        return self.runtime.ops.linear(wanted, self.head, out_dtype=torch.float32)
