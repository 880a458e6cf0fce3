"""Matrix-memory recurrent mixer (the mLSTM of xLSTM) with its state in the request's slot."""
from __future__ import annotations

import torch

from .base import MIXERS, Mixer, Runtime
from .spec import CacheNeed, MixerSpec, TensorSpec


@MIXERS.register("mlstm")
class MatrixLSTM(Mixer):
    """Per head: q = W_q h / sqrt(d), k = W_k h [d], v = W_v h [dv]; log gates i = cap(W_i h + b_i) and
    f = logsigmoid(cap(W_f h + b_f)) with cap(z) = c tanh(z / c), c = `gate_cap`.  With a running maximum m
    (0 before the first token): m' = max(f + m, i); C' = exp(f + m - m') C + exp(i - m') k v^T; n' likewise with k
    alone; o = C'^T q / (max(|n' . q|, exp(-m')) + 1e-6).  Each head's o is divided by its root mean square
    (`eps`), all heads times `norm`, times sigmoid(W_g h), then W_o.

    C, n and m of every head are the layer's per-request state (float32, `CacheNeed.state_shape`): one row
    [heads * d * dv | heads * d | heads] per slot, read as zeros by a step that starts at position 0.  Gates,
    decays, the maximum and the state are float32 in every dtype; the gates' pre-activations come out of their
    product in float32.  Tensors: q, k, v, g, o, i, i.b, f, f.b, norm.
    """
    graph_safe = True

    def __init__(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.spec, self.runtime = spec, runtime
        self.heads, self.d, self.dv = spec.n_heads, spec.head_dim, spec.value_dim or spec.head_dim
        self.cap, self.eps = float(spec.gate_cap), float(spec.eps)
        # One product for q, k, v and the output gate (compute dtype), one for the two log gates (float32 out).
        self.w_qkvg = torch.cat([tensors["q"], tensors["k"], tensors["v"], tensors["g"]], dim=0).contiguous()
        gates = torch.cat([tensors["i"], tensors["f"]], dim=0)
        bias = torch.cat([tensors["i.b"], tensors["f.b"]], dim=0).to(torch.float32)
        fill = (-gates.shape[0]) % 8           # the products' output widths are multiples of eight
        if fill:
            gates = torch.cat([gates, gates.new_zeros((fill, gates.shape[1]))], dim=0)
            bias = torch.cat([bias, bias.new_zeros(fill)], dim=0)
        self.w_gates, self.b_gates = gates.contiguous(), bias.contiguous()
        self.norm = tensors["norm"].to(torch.float32).contiguous()
        self.w_o = tensors["o"]

    @staticmethod
    def tensor_specs(spec: MixerSpec) -> dict[str, TensorSpec]:
        heads, d, dv, hidden = spec.n_heads, spec.head_dim, spec.value_dim or spec.head_dim, spec.hidden_size
        return {"q": TensorSpec((heads * d, hidden)), "k": TensorSpec((heads * d, hidden)),
                "v": TensorSpec((heads * dv, hidden)), "g": TensorSpec((heads * dv, hidden)),
                "o": TensorSpec((hidden, heads * dv)), "norm": TensorSpec((heads * dv,), init="ones", role="vector"),
                "i": TensorSpec((heads, hidden)), "i.b": TensorSpec((heads,), role="vector", std=1.0),
                "f": TensorSpec((heads, hidden)), "f.b": TensorSpec((heads,), role="vector", std=1.0)}

    @staticmethod
    def state_size(heads: int, d: int, dv: int) -> int:
        return heads * d * dv + heads * d + heads

    @staticmethod
    def cache_need(spec: MixerSpec) -> CacheNeed:
        dv = spec.value_dim or spec.head_dim
        return CacheNeed(kind="none", state_shape=(MatrixLSTM.state_size(spec.n_heads, spec.head_dim, dv),))

    def forward(self, x, ctx, cache):
        ops = self.runtime.ops
        if cache.state is None:
            raise ValueError("the recurrent mixer needs its state in the request's slot")
        qkvg = ops.linear(x, self.w_qkvg)
        gates = ops.linear(x, self.w_gates, self.b_gates, out_dtype=torch.float32)
        read = torch.empty((x.shape[0], self.heads * self.dv), dtype=torch.float32, device=x.device)
        ops.mlstm_scan(qkvg, gates, cache.state, ctx.cu_q, ctx.first_position, ctx.state_slots, read,
                       self.heads, self.d, self.dv, self.cap)
        mixed = torch.empty((x.shape[0], self.heads * self.dv), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(read, self.norm, qkvg, 2 * self.heads * self.d + self.heads * self.dv, self.eps,
                           self.heads, self.dv, mixed)
        return ops.linear(mixed, self.w_o)
