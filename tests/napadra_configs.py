"""Tiny Napadra configurations for the tests, and their model folders.  They differ in every size, constant and in
the order of their layers; streams, head ratios and value sizes take values that make nothing equal by accident."""
import os

import torch


def _attention(heads, kv_heads, dim, vdim, chunk, scale, kv_from=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk}, "scale": scale}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return mixer


def _layer(kind, mixer, ff=None, limit=1.0):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


NAPADRA = {
    # name: (config.json keys, weight seed)
    # Value heads wider than key heads, a chunk that straddles pages of 16, a layer that reads layer 0's keys and values.
    "P": ({"architecture": "Napadra", "vocab": 211, "width": 64, "streams": 2, "residual_mult": 0.8, "norm": {"eps": 1e-5},
           "layers": [_layer("attention", _attention(4, 2, 16, 24, 20, 0.3), ff=72, limit=0.7),
                      _layer("mlstm", {"heads": 2, "dim": 16, "vdim": 24, "gate_cap": 9.0}),
                      _layer("attention", _attention(4, 2, 16, 24, 20, 0.3, kv_from=0), ff=40, limit=1.5)]}, 3),
    # One stream, as many key/value heads as query heads, a recurrent layer first, an attention layer without feed-forward.
    "Q": ({"architecture": "Napadra", "vocab": 300, "width": 96, "streams": 1, "residual_mult": 1.0, "norm": {"eps": 1e-6},
           "layers": [_layer("mlstm", {"heads": 3, "dim": 8, "vdim": 32, "gate_cap": 4.0}, ff=104),
                      _layer("attention", _attention(3, 3, 32, 32, 33, 0.2)),
                      _layer("mlstm", {"heads": 1, "dim": 40, "vdim": 8, "gate_cap": 20.0})]}, 8),
    # Four streams, eight query heads on one key/value head, value heads narrower than key heads, chunks of 7 and 48,
    # two layers that read another's keys and values.
    "R": ({"architecture": "Napadra", "vocab": 150, "width": 128, "streams": 4, "residual_mult": 0.5, "norm": {"eps": 3e-6},
           "layers": [_layer("attention", _attention(8, 1, 16, 8, 7, 0.25), ff=64, limit=2.0),
                      _layer("attention", _attention(2, 2, 48, 16, 48, 0.1), ff=136),
                      _layer("attention", _attention(8, 1, 16, 8, 5, 0.25, kv_from=0)),
                      _layer("mlstm", {"heads": 4, "dim": 24, "vdim": 16, "gate_cap": 12.0}, ff=48, limit=0.4),
                      _layer("attention", _attention(2, 2, 48, 16, 64, 0.1, kv_from=1), ff=32)]}, 21),
    # Sizes that are no multiples of eight anywhere (the bfloat16 products fill such a K up), three streams.
    "S": ({"architecture": "Napadra", "vocab": 97, "width": 52, "streams": 3, "residual_mult": 0.9, "norm": {"eps": 2e-6},
           "layers": [_layer("attention", _attention(3, 3, 12, 14, 11, 0.4), ff=50, limit=1.2),
                      _layer("mlstm", {"heads": 3, "dim": 12, "vdim": 20, "gate_cap": 7.0}, ff=30, limit=0.8),
                      _layer("attention", _attention(6, 3, 12, 14, 26, 0.3, kv_from=0))]}, 13),
    # Key and value heads of one size (the matrix-core attention kernels in bfloat16), chunks that cut tiles of sixteen tokens.
    "T": ({"architecture": "Napadra", "vocab": 180, "width": 64, "streams": 2, "residual_mult": 0.7, "norm": {"eps": 1e-6},
           "layers": [_layer("attention", _attention(4, 2, 16, 16, 19, 0.25), ff=48, limit=1.0),
                      _layer("attention", _attention(4, 2, 16, 16, 23, 0.25, kv_from=0), ff=48, limit=1.0),
                      _layer("mlstm", {"heads": 2, "dim": 32, "vdim": 32, "gate_cap": 10.0}),
                      _layer("attention", _attention(2, 1, 64, 64, 40, 0.125), ff=80, limit=3.0)]}, 34),
    # Chunks of hundreds of positions: several waves share a tile's keys, single tokens' keys are cut over workgroups.
    "U": ({"architecture": "Napadra", "vocab": 260, "width": 128, "streams": 2, "residual_mult": 0.6, "norm": {"eps": 1e-6},
           "layers": [_layer("attention", _attention(4, 2, 32, 32, 300, 0.18), ff=96, limit=1.5),
                      _layer("mlstm", {"heads": 2, "dim": 64, "vdim": 64, "gate_cap": 15.0}),
                      _layer("attention", _attention(4, 2, 32, 32, 1024, 0.18, kv_from=0), ff=96, limit=1.5),
                      _layer("attention", _attention(2, 2, 64, 64, 520, 0.125))]}, 55),
}


def write_model(raw: dict, seed: int, folder: str, sharpen: float = 6.0) -> str:
    """A model folder from the random-weights mode, with its matrices made `sharpen` times larger, so that attention
    weights are peaked and gates far from their middle: a key too many or too few, a lost state or a left-out sink
    then moves the logits by much more than rounding does."""
    import tokenizer_amd as ta
    from safetensors.torch import load_file, save_file
    from tokenizer_amd.config import NapadraConfig

    ta.write_random_model(NapadraConfig.from_dict(raw), seed, folder, norm_spread=0.3)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for name, tensor in tensors.items():
        if tensor.dim() == 2 and ".hc" not in name and name not in ("embed", "head"):
            tensors[name] = (tensor.float() * sharpen).to(torch.bfloat16)
        if name == "embed":
            tensors[name] = (tensor.float() * 20.0).to(torch.bfloat16)      # of the size of the position vector
    save_file(tensors, path)
    return folder
