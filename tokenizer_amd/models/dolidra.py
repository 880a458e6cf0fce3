"""Dolidra as a `ModelSpec`: a decoder whose sub-layers are normalised before and after (x + norm_b(f(norm(x)))), with
a per-layer token input behind the feed-forward, a run of layers gone through several times with the same weights
(each pass with a cache of its own), two kinds of attention (differential attention under a sliding window with
rotated queries and keys; gated attention with queries and keys normalised over the whole projection, partly
rotated, under a window that keeps the sequence's first positions), and dense (tanh-GELU) or routed (SiLU experts,
softmax over the chosen logits, a shared expert) gated feed-forwards.

Tensor names: `embed`, `side.embed`, `head`, `final.norm`; layer i's start with `l<i>.`: `norm1`, `norm1b`, `norm2`,
`norm2b`, `mix.*` (the mixer's), `mlp.*` (gate|up|down, or e<j>.gate|up|down, router, shared.gate|up|down),
`side.gate|proj|norm`.
"""
from __future__ import annotations

from ..config.dolidra import DolidraConfig
from ..config.registry import register_architecture
from ..parts.spec import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec, ScheduleEntry

_DIFFERENTIAL_NAMES = (("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("o_proj.weight", "o"),
                       ("q_proj.bias", "q.b"), ("k_proj.bias", "k.b"), ("v_proj.bias", "v.b"))
_GATED_NAMES = (("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("o_proj.weight", "o"),
                ("q_norm", "q.norm"), ("k_norm", "k.norm"), ("gate_proj.weight", "g"))
_DENSE_NAMES = (("gate_proj.weight", "gate"), ("up_proj.weight", "up"), ("down_proj.weight", "down"))


def _position(rot: dict | None, head_dim: int, max_positions: int) -> PositionSpec | None:
    if not rot:
        return None
    return PositionSpec("rope_partial", head_dim=head_dim, theta=float(rot["base"]), max_positions=max_positions,
                        options={"dims": int(rot["dims"]), "scaling": rot.get("scaling")})


def dolidra_spec(cfg: DolidraConfig) -> ModelSpec:
    width, eps = cfg.width, cfg.eps
    norm = NormSpec("rmsnorm", width, eps, options={"tensor_name": ""})     # the weight is the tensor the prefix names
    side_dim = int(cfg.token_side["dim"]) if cfg.token_side else 0
    layers = []
    for index, layer in enumerate(cfg.layers):
        prefix, raw = f"l{index}", layer["mixer"]
        mask = raw.get("mask") or {}
        # A query sees itself and the size - 1 positions before it: a window of size - 1 behind the query.
        window = None if mask.get("size") is None else int(mask["size"]) - 1
        common = dict(hidden_size=width, n_heads=raw["heads"], n_kv_heads=raw["kv_heads"], head_dim=raw["dim"],
                      value_dim=raw["vdim"], scale=float(raw["scale"]), window=window, eps=eps,
                      position=_position(raw.get("rot"), raw["dim"], cfg.max_positions))
        if layer["type"] == "attention":
            mixer = MixerSpec("gqa_attention", qkv_bias=True, differential=float(raw["diff"]),
                              tensor_names=_DIFFERENTIAL_NAMES, **common)
        else:
            mixer = MixerSpec("gqa_attention", keep_first=int(mask.get("keep_first") or 0) if window is not None else 0,
                              qk_norm="whole", head_gate=True, tensor_names=_GATED_NAMES, **common)
        mlp = layer.get("mlp")
        if mlp is None:
            feed_forward = None
        elif mlp["kind"] == "dense":
            feed_forward = FeedForwardSpec("gated_dense", hidden_size=width, intermediate_size=mlp["ff"],
                                           activation="gelu_tanh", tensor_names=_DENSE_NAMES)
        else:
            feed_forward = FeedForwardSpec("routed_experts", hidden_size=width, intermediate_size=mlp["expert"]["ff"],
                                           activation="silu", n_experts=mlp["router"]["experts"], top_k=mlp["router"]["top"],
                                           shared_size=int((mlp.get("shared") or {}).get("ff") or 0))
        layers.append(LayerSpec(
            block="sandwich_norm", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm,
            feed_forward_norm=None if mlp is None else norm,
            mixer_prefix=f"{prefix}.mix", feed_forward_prefix=f"{prefix}.mlp", mixer_norm_prefix=f"{prefix}.norm1",
            feed_forward_norm_prefix=f"{prefix}.norm2", prefix=prefix,
            options={"width": width, "eps": eps, "vocab": cfg.vocab, "side_dim": side_dim,
                     "side_offset": index * side_dim, "side_width": len(cfg.layers) * side_dim,
                     "side_table": "side.embed"}))
    # A layer that runs several times keeps the keys and values of each pass apart: the first pass has the layer's
    # own cache unit, every further pass a unit of its own.
    schedule, extra, seen = [], [], set()
    for index in cfg.run_order():
        if index in seen:
            schedule.append(ScheduleEntry(index, unit=len(cfg.layers) + len(extra)))
            extra.append(index)
        else:
            schedule.append(ScheduleEntry(index))
            seen.add(index)
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=width, max_positions=cfg.max_positions,
        embedding_name="embed", layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
        final_norm_prefix="final.norm", tied_head=False, head_name="head", extra_cache_units=tuple(extra))


register_architecture("Dolidra", DolidraConfig, dolidra_spec)
