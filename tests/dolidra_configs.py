"""Tiny Dolidra configurations for the tests, and their model folders.  They differ in every size, constant and in the
order of their layers; head ratios, value sizes, windows, kept first positions, rotated coordinates, expert counts and
the looped run take values that make nothing equal by accident (and some the values 1 and 0)."""
import os

import torch


def _rot(dims, base=10000.0, scaling=None):
    rot = {"dims": dims, "base": base}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return rot


def _differential(heads, kv_heads, dim, vdim, size, scale, diff, rot=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if size is not None:
        mixer["mask"] = {"size": size}
    if rot is not None:
        mixer["rot"] = rot
    return "attention", mixer


def _gated(heads, kv_heads, dim, vdim, size, keep, scale, rot=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size is not None:
        mixer["mask"] = {"size": size, "keep_first": keep}
    if rot is not None:
        mixer["rot"] = rot
    return "attention_2", mixer


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def _layer(kind_mixer, mlp=None):
    return {"type": kind_mixer[0], "mixer": kind_mixer[1], "mlp": mlp}


DOLIDRA = {
    # name: (config.json keys, weight seed)
    # Layers 1 and 2 run twice (a loop that starts behind layer 0 and holds both kinds of attention), a token input of
    # six numbers, a rotation over half a head with all three ranges of the scaling, value heads wider and narrower
    # than key heads, a layer without feed-forward, a layer without mask and without rotation, one expert a token.
    "A": ({"architecture": "Dolidra", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "token_side": {"dim": 6},
           "loop": {"start": 1, "stop": 3, "times": 2},
           "layers": [_layer(_differential(4, 2, 16, 24, 20, 0.3, 0.3, _rot(8, 10000.0, (4.0, 1.0, 4.0, 64))), _dense(72)),
                      _layer(_gated(4, 2, 16, 8, 12, 5, 0.3, _rot(16, 5000.0)), _moe(5, 2, 24, shared=40)),
                      _layer(_differential(2, 2, 24, 24, 33, 0.25, 0.7, _rot(24, 300.0))),
                      _layer(_gated(6, 1, 8, 16, None, 0, 0.4), _moe(3, 1, 20))]}, 3),
    # No loop, no token input; more kept first positions than the window is long; a window of one position; three of four
    # experts; a differential layer that sees every earlier key.
    "B": ({"architecture": "Dolidra", "vocab": 300, "width": 96, "norm": {"eps": 1e-6},
           "layers": [_layer(_gated(3, 3, 32, 32, 17, 30, 0.2, _rot(16, 10000.0, (8.0, 1.0, 2.0, 100))), _dense(104)),
                      _layer(_differential(3, 1, 16, 32, 1, 0.3, 0.5, _rot(16, 1000.0)), _moe(4, 3, 16, shared=8)),
                      _layer(_differential(2, 1, 32, 16, None, 0.2, 0.4, _rot(32, 20000.0, (2.0, 1.0, 4.0, 32))), _dense(40))]}, 8),
    # Sizes that are no multiples of eight anywhere; the first layer alone runs three times; a window without kept positions.
    "C": ({"architecture": "Dolidra", "vocab": 97, "width": 52, "norm": {"eps": 2e-6}, "token_side": {"dim": 3},
           "loop": {"start": 0, "stop": 1, "times": 3},
           "layers": [_layer(_differential(3, 3, 12, 14, 11, 0.4, 0.2, _rot(6, 100.0)), _moe(6, 2, 10, shared=6)),
                      _layer(_gated(6, 3, 12, 14, 26, 0, 0.35, _rot(12, 10000.0)), _dense(50))]}, 13),
    # Key and value heads of one size in multiples of sixteen (the sizes the matrix-core attention kernels take), windows
    # and kept positions that cut tiles of sixteen tokens and pages of sixteen.
    "D": ({"architecture": "Dolidra", "vocab": 180, "width": 128, "norm": {"eps": 1e-6}, "token_side": {"dim": 8},
           "loop": {"start": 0, "stop": 2, "times": 2},
           "layers": [_layer(_differential(4, 2, 32, 32, 36, 0.2, 0.45, _rot(32, 500000.0)), _dense(96)),
                      _layer(_gated(4, 2, 64, 64, 48, 16, 0.125, _rot(16, 500000.0)), _moe(8, 2, 32, shared=64)),
                      _layer(_gated(2, 1, 16, 16, 19, 7, 0.25, _rot(16, 1000.0)), _dense(80)),
                      _layer(_differential(8, 1, 16, 16, 23, 0.25, 0.35, _rot(8, 1000.0)), _moe(4, 2, 48))]}, 34),
    # Windows of hundreds of positions with kept first positions far behind them.
    "E": ({"architecture": "Dolidra", "vocab": 260, "width": 128, "norm": {"eps": 1e-6}, "token_side": {"dim": 16},
           "loop": {"start": 1, "stop": 2, "times": 2},
           "layers": [_layer(_differential(4, 2, 32, 32, 300, 0.18, 0.6, _rot(32, 80000.0, (8.0, 1.0, 4.0, 1024))), _dense(96)),
                      _layer(_gated(4, 2, 32, 32, 260, 44, 0.18, _rot(8, 80000.0)), _moe(6, 2, 32, shared=32)),
                      _layer(_gated(2, 2, 64, 64, 520, 3, 0.125, _rot(64, 10000.0)), _dense(64))]}, 55),
}


def write_model(raw: dict, seed: int, folder: str, sharpen: float = 6.0, router: float = 0.4) -> str:
    """A model folder from the random-weights mode, with its matrices made `sharpen` times larger, so that attention
    weights are peaked: a key too many or too few, a window one position off or a lost kept key then moves the logits
    by much more than rounding does.  The routers stay soft (`router` times the drawn weights: several experts carry
    weight; a large factor makes the choice decisive instead, far from the near ties that rounding tips), the vectors behind the
    differential factor are made large enough for it to differ from layer to layer, and the embedding is of the size
    of what the layers add."""
    import tokenizer_amd as ta
    from safetensors.torch import load_file, save_file
    from tokenizer_amd.config import DolidraConfig

    ta.write_random_model(DolidraConfig.from_dict(raw), seed, folder, norm_spread=0.3)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for name, tensor in tensors.items():
        if name == "embed":
            tensors[name] = (tensor.float() * 50.0).to(torch.bfloat16)
        elif name.endswith((".lq1", ".lk1", ".lq2", ".lk2")):
            tensors[name] = (tensor.float() * 4.0).to(torch.bfloat16)
        elif name.endswith(".router"):
            tensors[name] = (tensor.float() * router).to(torch.bfloat16)
        elif tensor.dim() == 2 and name not in ("head", "side.embed"):
            tensors[name] = (tensor.float() * sharpen).to(torch.bfloat16)
    save_file(tensors, path)
    return folder


def random_config(seed: int) -> dict:
    """A Dolidra configuration drawn from a seed: the number and order of layers, both kinds of attention, head counts and
    groupings, key and value sizes (some in sixteens, some odd multiples of two), windows, kept positions, rotated
    coordinates with and without scaling, dense and routed feed-forwards, layers without one, a loop or none, a token
    input or none."""
    import random
    rng = random.Random(seed)
    width = rng.choice([32, 40, 64, 72, 96, 128])
    layers = []
    for _ in range(rng.randint(1, 4)):
        kv_heads = rng.choice([1, 1, 2, 3])
        heads = kv_heads * rng.choice([1, 2, 4])
        dim = rng.choice([8, 12, 16, 16, 32, 32, 48, 64])
        vdim = dim if rng.random() < 0.6 else rng.choice([8, 10, 16, 24, 40])
        size = rng.choice([None, 1, 2, 7, 16, 17, 31, 36, 64, 100])
        rot = None
        if rng.random() < 0.85:
            dims = rng.choice([dim, dim, dim // 2, max(2, dim // 4 // 2 * 2), 2])
            scaling = None
            if rng.random() < 0.5:
                scaling = (rng.choice([2.0, 4.0, 8.0]), 1.0, rng.choice([2.0, 4.0]), rng.choice([16, 64, 256, 1024]))
            rot = _rot(dims, rng.choice([100.0, 10000.0, 500000.0]), scaling)
        scale = rng.choice([dim ** -0.5, 0.2, 0.35])
        if rng.random() < 0.5:
            mixer = _differential(heads, kv_heads, dim, vdim, size, scale, rng.choice([0.0, 0.2, 0.5, 0.8]), rot)
        else:
            mixer = _gated(heads, kv_heads, dim, vdim, size, rng.choice([0, 1, 5, 16, 20, 33, 70]), scale, rot)
        kind = rng.random()
        if kind < 0.15:
            mlp = None
        elif kind < 0.55:
            mlp = _dense(rng.choice([24, 50, 64, 100]))
        else:
            experts = rng.choice([1, 2, 4, 6, 9])
            mlp = _moe(experts, rng.randint(1, min(experts, 3)), rng.choice([8, 10, 24, 32]), rng.choice([None, None, 6, 16]))
        layers.append(_layer(mixer, mlp))
    raw = {"architecture": "Dolidra", "vocab": rng.choice([97, 128, 211, 300]), "width": width,
           "norm": {"eps": rng.choice([1e-5, 1e-6, 3e-6])}, "layers": layers}
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        raw["loop"] = {"start": start, "stop": rng.randint(start, len(layers)), "times": rng.randint(1, 3)}
    if rng.random() < 0.7:
        raw["token_side"] = {"dim": rng.choice([1, 3, 4, 8, 16, 24])}
    return raw
