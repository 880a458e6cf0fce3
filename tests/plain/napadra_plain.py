"""Plain, slow Napadra decoder: whole sequences, no cache, one function per mechanism.

Written from the design's equations in this file's own notation; it shares no code with `tokenizer_amd`.
Everything runs on the CPU in the dtype given (float64 by default).  A model is a config dict (the keys of
its config.json) and a dict of tensors by name.
"""
from __future__ import annotations

import json
import math
import os

import torch


def load_folder(folder: str, dtype=torch.float64):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    tensors = {k: (v if v.dtype in (torch.int32, torch.int64) else v.to(dtype))
               for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, tensors


# ------------------------------------------------------------------ small pieces
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over the root of (its mean square + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose scale is one number for every coordinate."""
    return unit_rms(x, eps) * g.reshape(())


def sinusoid(positions: torch.Tensor, width: int, base: float = 10000.0) -> torch.Tensor:
    """[n, width]: column 2i is sin(p * base^(-2i/width)), column 2i+1 the cosine of the same angle."""
    pairs = torch.arange(width // 2, dtype=torch.float64)
    rates = base ** (-2.0 * pairs / width)
    angles = positions.to(torch.float64)[:, None] * rates[None, :]
    out = torch.zeros((positions.numel(), width), dtype=torch.float64)
    out[:, 0::2] = angles.sin()
    out[:, 1::2] = angles.cos()
    return out


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """Row t becomes h[t] + (h[t-1] - h[t]) * mu, with the unshifted rows on the right and zeros before row 0."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * mu


def distance_slopes(n_heads: int) -> torch.Tensor:
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)], dtype=torch.float64)


def chunk_visible(n: int, chunk: int | None) -> torch.Tensor:
    """[n, n] bool: query i sees key j when j <= i and both lie in the same chunk counted from position 0."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if chunk is not None:
        ok = ok & (i // chunk == j // chunk)
    return ok


def sink_softmax(scores: torch.Tensor, visible: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """Softmax over the visible keys whose denominator holds exp(sink) once more.  scores [H, n, n], sink [H]."""
    scores = scores.masked_fill(~visible, -math.inf)
    top = torch.maximum(scores.max(dim=-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(scores - top)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink[:, None, None] - top))


def keys_and_values(h: torch.Tensor, mixer: dict, w: dict):
    """[G, n, dim] keys and [G, n, vdim] values of an attention layer that has projections of its own."""
    n, g = h.shape[0], mixer["kv_heads"]
    k = (h @ w["k"].t()).reshape(n, g, mixer["dim"]).transpose(0, 1)
    v = (h @ w["v"].t()).reshape(n, g, mixer["vdim"]).transpose(0, 1)
    return k, v


def attention(h: torch.Tensor, mixer: dict, w: dict, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Grouped-query attention without rotation: scaled scores minus slope * distance, chunked, with a sink."""
    n, heads, g = h.shape[0], mixer["heads"], mixer["kv_heads"]
    q = (h @ w["q"].t()).reshape(n, heads, mixer["dim"]).transpose(0, 1)
    per = heads // g
    k = k.repeat_interleave(per, dim=0)
    v = v.repeat_interleave(per, dim=0)
    scores = (q @ k.transpose(1, 2)) * mixer["scale"]
    distance = (torch.arange(n)[:, None] - torch.arange(n)[None, :]).to(h.dtype)
    scores = scores - distance_slopes(heads).to(h.dtype)[:, None, None] * distance[None]
    chunk = (mixer.get("mask") or {}).get("size")
    weights = sink_softmax(scores, chunk_visible(n, chunk), w["sink"])
    mixed = (weights @ v).transpose(0, 1).reshape(n, heads * mixer["vdim"])
    return mixed @ w["o"].t()


def capped(x: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(x / cap)


def mlstm(h: torch.Tensor, mixer: dict, w: dict, eps: float) -> torch.Tensor:
    """Matrix memory with exponential gates and a running maximum that starts at 0, token by token."""
    n, heads, dim, vdim, cap = h.shape[0], mixer["heads"], mixer["dim"], mixer["vdim"], mixer["gate_cap"]
    q = (h @ w["q"].t()).reshape(n, heads, dim) * dim ** -0.5
    k = (h @ w["k"].t()).reshape(n, heads, dim)
    v = (h @ w["v"].t()).reshape(n, heads, vdim)
    log_in = capped(h @ w["i"].t() + w["i.b"], cap)                                  # [n, heads]
    log_keep = torch.nn.functional.logsigmoid(capped(h @ w["f"].t() + w["f.b"], cap))
    memory = torch.zeros((heads, dim, vdim), dtype=h.dtype)
    norm = torch.zeros((heads, dim), dtype=h.dtype)
    top = torch.zeros(heads, dtype=h.dtype)
    out = torch.zeros((n, heads, vdim), dtype=h.dtype)
    for t in range(n):
        new_top = torch.maximum(log_keep[t] + top, log_in[t])
        keep = torch.exp(log_keep[t] + top - new_top)
        take = torch.exp(log_in[t] - new_top)
        memory = keep[:, None, None] * memory + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        norm = keep[:, None] * norm + take[:, None] * k[t]
        top = new_top
        read = torch.einsum("hdv,hd->hv", memory, q[t])
        floor = torch.maximum((norm * q[t]).sum(dim=-1).abs(), torch.exp(-top)) + 1e-6
        out[t] = read / floor[:, None]
    out = unit_rms(out, eps).reshape(n, heads * vdim) * w["norm"]
    out = out * torch.sigmoid(h @ w["g"].t())
    return out @ w["o"].t()


def feed_forward(h: torch.Tensor, mlp: dict, w: dict) -> torch.Tensor:
    limit = mlp["limit"]
    gate = torch.clamp(h @ w["gate"].t(), max=limit)
    up = torch.clamp(h @ w["up"].t(), min=-limit, max=limit)
    return (gate * torch.sigmoid(1.702 * gate) * (up + 1.0)) @ w["down"].t()


def strip(tensors: dict, prefix: str) -> dict:
    return {name[len(prefix):]: t for name, t in tensors.items() if name.startswith(prefix)}


# ------------------------------------------------------------------ the model
def forward(cfg: dict, tensors: dict, tokens, layers_out: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence from position 0.  `layers_out` receives the sum of the streams after
    every layer."""
    dtype = tensors["embed"].dtype
    n, width, eps, m = len(tokens), cfg["width"], cfg["norm"]["eps"], cfg["residual_mult"]
    x = tensors["embed"][torch.tensor(tokens, dtype=torch.long)] + sinusoid(torch.arange(n), width).to(dtype)
    streams = [x.clone() for _ in range(cfg["streams"])]
    kept: dict[int, tuple] = {}

    def sublayer(streams, hc: dict, run):
        u = sum(hc["in"][s] * streams[s] for s in range(len(streams)))
        y = run(u)
        return [sum(hc["mix"][s, t] * streams[s] for s in range(len(streams))) + m * hc["out"][t] * y
                for t in range(len(streams))]

    for index, layer in enumerate(cfg["layers"]):
        w = strip(tensors, f"l{index}.")
        mix_w = strip(w, "mix.")

        def mixer(u):
            h = token_shift(scalar_norm(u, w["norm1"], eps), w["shift"])
            if layer["type"] == "attention":
                source = layer["mixer"].get("kv_from")
                if source is None:
                    kept[index] = keys_and_values(h, layer["mixer"], mix_w)
                    source = index
                y = attention(h, layer["mixer"], mix_w, *kept[source])
            elif layer["type"] == "mlstm":
                y = mlstm(h, layer["mixer"], mix_w, eps)
            else:
                raise ValueError(layer["type"])
            return y * w["ls1"]

        streams = sublayer(streams, strip(w, "hc1."), mixer)
        if layer.get("mlp") is not None:
            streams = sublayer(streams, strip(w, "hc2."),
                               lambda u: feed_forward(scalar_norm(u, w["norm2"], eps), layer["mlp"], strip(w, "mlp.")) * w["ls2"])
        if layers_out is not None:
            layers_out.append(sum(streams))
    return scalar_norm(sum(streams), tensors["final.norm"], eps) @ tensors["head"].t()


def greedy_generate(cfg: dict, tensors: dict, prompt, n_new: int) -> list[int]:
    tokens, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(forward(cfg, tensors, tokens)[-1].argmax())
        out.append(nxt)
        tokens.append(nxt)
    return out
