"""Napadra as a `ModelSpec`: several residual streams with learned read, write and mixing weights around every
sub-layer, one-number RMS norms, a token shift in front of every mixer, chunked attention without rotation (a
distance bias and a sink instead; some layers read an earlier layer's keys and values) beside matrix-memory
recurrent layers, a capped gated feed-forward, and a sinusoidal position vector added to the embedding.

Tensor names: `embed`, `head`, `final.norm`; layer i's start with `l<i>.`: `norm1`, `norm2`, `shift`, `ls1`, `ls2`,
`hc1.in|out|mix`, `hc2.in|out|mix`, `mix.*` (the mixer's) and `mlp.gate|up|down`.
"""
from __future__ import annotations

from ..config.napadra import NapadraConfig
from ..config.registry import register_architecture
from ..parts.spec import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, ScheduleEntry

_ATTENTION_NAMES = (("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("o_proj.weight", "o"),
                    ("sink", "sink"))
_FEED_FORWARD_NAMES = (("gate_proj.weight", "gate"), ("up_proj.weight", "up"), ("down_proj.weight", "down"))


def napadra_spec(cfg: NapadraConfig) -> ModelSpec:
    width, eps = cfg.width, cfg.eps
    norm = NormSpec("rmsnorm_scalar", width, eps)
    layers, schedule = [], []
    for index, layer in enumerate(cfg.layers):
        prefix, raw = f"l{index}", layer["mixer"]
        if layer["type"] == "attention":
            mask = raw.get("mask") or {}
            mixer = MixerSpec("gqa_attention", hidden_size=width, n_heads=raw["heads"], n_kv_heads=raw["kv_heads"],
                              head_dim=raw["dim"], value_dim=raw["vdim"], scale=float(raw["scale"]),
                              chunk=mask.get("size"), distance_bias=8.0, sink=True,
                              own_kv=raw.get("kv_from") is None, tensor_names=_ATTENTION_NAMES)
            schedule.append(ScheduleEntry(index, raw.get("kv_from")))
        else:
            mixer = MixerSpec("mlstm", hidden_size=width, n_heads=raw["heads"], head_dim=raw["dim"],
                              value_dim=raw["vdim"], gate_cap=float(raw["gate_cap"]), eps=eps)
            schedule.append(ScheduleEntry(index))
        mlp = layer.get("mlp")
        feed_forward = None if mlp is None else FeedForwardSpec(
            "gated_dense", hidden_size=width, intermediate_size=mlp["ff"], activation="capped_swish",
            act_alpha=1.702, act_limit=float(mlp["limit"]), act_up_shift=1.0, tensor_names=_FEED_FORWARD_NAMES)
        layers.append(LayerSpec(
            block="hyper_streams", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm,
            feed_forward_norm=None if mlp is None else norm,
            mixer_prefix=f"{prefix}.mix", feed_forward_prefix=f"{prefix}.mlp", mixer_norm_prefix=f"{prefix}.norm1",
            feed_forward_norm_prefix=f"{prefix}.norm2", prefix=prefix,
            options={"streams": cfg.streams, "residual_mult": float(cfg.residual_mult), "token_shift": True,
                     "layer_scale": True, "width": width}))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=width, max_positions=cfg.max_positions,
        embedding_name="embed", layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
        final_norm_prefix="final.norm", tied_head=False, head_name="head", frame="stream_decoder",
        options={"streams": cfg.streams, "embedding_position": "sinusoidal", "position_base": 10000.0})


register_architecture("Napadra", NapadraConfig, napadra_spec)
