"""Plain, slow Dolidra decoder: whole sequences, no cache, one function per mechanism.

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


def weighted_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ rotation
def rotation_rates(rot: dict) -> torch.Tensor:
    """The rates f_i = base^(-2i/n), i < n/2, of a rotation over n coordinates; with `scaling` the long waves are
    slowed: wavelength l = 2 pi / f; f stays where l < original/high, becomes f/factor where l > original/low, and
    in between is the mix (1 - s) f/factor + s f with s = (original/l - low) / (high - low)."""
    n = int(rot["dims"])
    rates = [float(rot["base"]) ** (-2.0 * i / n) for i in range(n // 2)]
    scaling = rot.get("scaling")
    if scaling:
        factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for f in rates:
            wave = 2.0 * math.pi / f
            if wave < original / high:
                out.append(f)
            elif wave > original / low:
                out.append(f / factor)
            else:
                s = (original / wave - low) / (high - low)
                out.append((1.0 - s) * f / factor + s * f)
        rates = out
    return torch.tensor(rates, dtype=torch.float64)


def rotate(x: torch.Tensor, positions: torch.Tensor, rates: torch.Tensor) -> torch.Tensor:
    """x [n, heads, d]: coordinates i and i + m (m = len(rates)) of every head turn by the angle p * rates[i]; the
    coordinates from 2m on pass through."""
    m = rates.numel()
    if m == 0:
        return x
    angles = positions.to(torch.float64)[:, None] * rates[None, :]
    cos, sin = angles.cos().to(x.dtype)[:, None, :], angles.sin().to(x.dtype)[:, None, :]
    a, b, rest = x[..., :m], x[..., m:2 * m], x[..., 2 * m:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)


# ------------------------------------------------------------------ masks
def visible(n: int, size: int | None, keep_first: int = 0) -> torch.Tensor:
    """[n, n] bool: query i sees key j when j <= i and (i - j < size or j < keep_first); no size: every j <= i."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if size is not None:
        seen = seen & ((i - j < size) | (j < keep_first))
    return seen


def masked_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, seen: torch.Tensor) -> torch.Tensor:
    """q [n, d], k [n, d], v [n, dv] of one head: softmax over the visible keys of scale * q.k, times v."""
    scores = (q @ k.T) * scale
    scores = scores.masked_fill(~seen, float("-inf"))
    return torch.softmax(scores, dim=-1) @ v


# ------------------------------------------------------------------ mixers
def differential_attention(h: torch.Tensor, w: dict, mixer: dict, eps: float) -> torch.Tensor:
    """Two attention maps per head over the same values; the second is taken off the first with one learned
    factor for the layer, the difference is brought to unit RMS per head and scaled by (1 - diff)."""
    n = h.shape[0]
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    q = (h @ w["q"].T + w["q.b"]).reshape(n, H, 2, d)
    k = (h @ w["k"].T + w["k.b"]).reshape(n, G, 2, d)
    v = (h @ w["v"].T + w["v.b"]).reshape(n, G, dv)
    positions = torch.arange(n)
    rot = mixer.get("rot")
    if rot:
        rates = rotation_rates(rot)
        q = rotate(q.reshape(n, 2 * H, d), positions, rates).reshape(n, H, 2, d)
        k = rotate(k.reshape(n, 2 * G, d), positions, rates).reshape(n, G, 2, d)
    mask = mixer.get("mask") or {}
    seen = visible(n, mask.get("size"))
    diff = float(mixer["diff"])
    lam = torch.exp((w["lq1"] * w["lk1"]).sum()) - torch.exp((w["lq2"] * w["lk2"]).sum()) + diff
    out = []
    for head in range(H):
        g = head // (H // G)
        first = masked_softmax_attention(q[:, head, 0], k[:, g, 0], v[:, g], float(mixer["scale"]), seen)
        second = masked_softmax_attention(q[:, head, 1], k[:, g, 1], v[:, g], float(mixer["scale"]), seen)
        out.append(unit_rms(first - lam * second, eps) * (1.0 - diff))
    return torch.cat(out, dim=-1) @ w["o"].T


def gated_window_attention(h: torch.Tensor, w: dict, mixer: dict, eps: float) -> torch.Tensor:
    """Queries and keys normalised over their whole projection, rotated; a window that also keeps the sequence's
    first positions; each head's output times a sigmoid gate read from the mixer's input."""
    n = h.shape[0]
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    q = weighted_norm(h @ w["q"].T, w["q.norm"], eps).reshape(n, H, d)
    k = weighted_norm(h @ w["k"].T, w["k.norm"], eps).reshape(n, G, d)
    v = (h @ w["v"].T).reshape(n, G, dv)
    positions = torch.arange(n)
    rot = mixer.get("rot")
    if rot:
        rates = rotation_rates(rot)
        q, k = rotate(q, positions, rates), rotate(k, positions, rates)
    mask = mixer.get("mask") or {}
    seen = visible(n, mask.get("size"), int(mask.get("keep_first", 0)))
    gate = torch.sigmoid(h @ w["g"].T)                       # [n, H]
    out = []
    for head in range(H):
        g = head // (H // G)
        mixed = masked_softmax_attention(q[:, head], k[:, g], v[:, g], float(mixer["scale"]), seen)
        out.append(mixed * gate[:, head:head + 1])
    return torch.cat(out, dim=-1) @ w["o"].T


# ------------------------------------------------------------------ feed-forwards
def gated_ff(h: torch.Tensor, w: dict, act) -> torch.Tensor:
    return (act(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def routed_ff(h: torch.Tensor, w: dict, mlp: dict) -> torch.Tensor:
    """Every token goes to the `top` experts with the largest router logits; their outputs are added with the
    softmax of those logits alone as weights; an expert that every token uses is added on top."""
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    logits = h @ w["router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(logits[t], top).indices
        weights = torch.softmax(logits[t, chosen], dim=-1)
        for e, p in zip(chosen.tolist(), weights):
            one = {name: w[f"e{e}.{name}"] for name in ("gate", "up", "down")}
            out[t] += p * gated_ff(h[t:t + 1], one, silu)[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, {name: w[f"shared.{name}"] for name in ("gate", "up", "down")}, silu)
    assert logits.shape[-1] == experts
    return out


def token_side_input(x: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor, w: dict, layer: int, dim: int, eps: float):
    """What a layer adds from the token itself: its slice of the token's side row, gated by the stream."""
    e = table[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return weighted_norm(y, w["norm"], eps)


# ------------------------------------------------------------------ the model
def _sub(tensors: dict, prefix: str) -> dict:
    lead = prefix + "."
    return {name[len(lead):]: value for name, value in tensors.items() if name.startswith(lead)}


def run_order(cfg: dict) -> list[int]:
    """Layer indices in the order they run: the looped run `times` times, the others once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def forward(cfg: dict, tensors: dict, tokens, return_layers: bool = False):
    """Logits [n, vocab] of one whole sequence (and, if asked, the stream after every layer run)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(cfg["norm"]["eps"])
    x = tensors["embed"][tokens]
    side = cfg.get("token_side")
    after = []
    for index in run_order(cfg):
        layer, w = cfg["layers"][index], _sub(tensors, f"l{index}")
        mix = _sub(w, "mix")
        h = weighted_norm(x, w["norm1"], eps)
        if layer["type"] == "attention":
            y = differential_attention(h, mix, layer["mixer"], eps)
        elif layer["type"] == "attention_2":
            y = gated_window_attention(h, mix, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + weighted_norm(y, w["norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = weighted_norm(x, w["norm2"], eps)
            y = gated_ff(h, _sub(w, "mlp"), gelu_tanh) if mlp["kind"] == "dense" else routed_ff(h, _sub(w, "mlp"), mlp)
            x = x + weighted_norm(y, w["norm2b"], eps)
        if side:
            x = x + token_side_input(x, tokens, tensors["side.embed"], _sub(w, "side"), index, int(side["dim"]), eps)
        after.append(x)
    logits = weighted_norm(x, tensors["final.norm"], eps) @ tensors["head"].T
    return (logits, after) if return_layers else logits


def greedy_generate(cfg: dict, tensors: dict, prompt, n_new: int) -> list[int]:
    """The first maximum of the last position's logits, appended and run again from the start, `n_new` times."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        logits = forward(cfg, tensors, ids)[-1]
        out.append(int(torch.argmax(logits)))
        ids.append(out[-1])
    return out
