"""Recurrent mixers that keep a matrix of state S [dim, vdim] per head and request, through the recurrence kernel

    S <- diag(w) S - a (b^T S) + k v^T;   o = S^T r          (`ops.linear_state`; both terms read the old S)

`generalized_delta`: the delta rule with a decay and a removal rate per key channel,

    r, k, v = x . W^T  (heads x dim each);   gate = x . Wg^T
    w = exp(-decay_scale * sigmoid(tanh(x . W1^T) . W2^T + w0));   rate = sigmoid(x . Wa^T + ba)
    u = k / sqrt(sum over the head of k^2 + 1e-6);   a = rate * u,  b = u
    y = (o / rms(o over the head) * norm_weight * sigmoid(gate)) . Wo^T          norm_weight of all heads' size

`lightning_attention`: decayed linear attention, a constant decay per head,

    q, k, v = silu(x . W^T);   S <- decay_h S + k v^T;   o = S^T q
    y = (rmsnorm(o of all heads together) * norm_weight * sigmoid(x . Wg^T)) . Wo^T

State, decays, rates, unit keys, the recurrence and the norms are float32 in every run; nothing is kept in pages.
"""
from __future__ import annotations

import math
from typing import List, Sequence

import torch

from .. import ops
from .base import Mixer, ParamSpec, StateNeed, register_part
from .dense_mlp import stack_rows


class GeneralizedDelta(Mixer):
    graph_safe = True  # every launch reads the step's device arrays and the state only

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, decay_rank: int, norm_eps: float = 1e-6,
                 decay_scale: float = math.exp(-0.5), unit_eps: float = 1e-6, init_std: float = 0.02):
        if min(num_heads, head_dim, decay_rank) <= 0 or head_dim > 256:
            raise ValueError("heads, head_dim (at most 256) and decay_rank must be positive")
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.decay_rank, self.norm_eps, self.init_std = int(decay_rank), float(norm_eps), float(init_std)
        self.decay_scale, self.unit_eps = float(decay_scale), float(unit_eps)
        self.channels = self.num_heads * self.head_dim
        self.w_in = self.w_w1 = self.w_w2 = self.w_out = self.w0 = self.a_bias = self.norm_weight = None

    def param_specs(self) -> List[ParamSpec]:
        W, s, C = self.hidden_size, self.init_std, self.channels
        return ([ParamSpec(f"{n}.weight", (C, W), std=s) for n in ("r", "k", "v", "g", "a")] +
                [ParamSpec("a.bias", (C,), std=0.5), ParamSpec("w1.weight", (self.decay_rank, W), std=s),
                 ParamSpec("w2.weight", (C, self.decay_rank), std=0.5), ParamSpec("w0", (C,), std=0.5),
                 ParamSpec("norm.weight", (C,), init="ones"), ParamSpec("o.weight", (W, C), std=s)])

    def state_need(self) -> StateNeed:
        return StateNeed((self.channels * self.head_dim,), "float32")

    def bind(self, tensors, rt) -> None:
        self.w_in = stack_rows([tensors[f"{n}.weight"] for n in ("r", "k", "v", "g", "a")])
        self.w_w1 = tensors["w1.weight"].contiguous()
        self.w_w2 = tensors["w2.weight"].to(torch.float32).contiguous()  # the decay's second product is float32
        self.w0, self.a_bias = tensors["w0"].contiguous(), tensors["a.bias"].contiguous()
        self.norm_weight = tensors["norm.weight"].contiguous()
        self.w_out = tensors["o.weight"].contiguous()

    def forward(self, ctx, x, cache):
        rt, T, C, H, D = ctx.rt, x.shape[0], self.channels, self.num_heads, self.head_dim
        proj = rt.linear(x, self.w_in)  # r | k | v | gate | rate's logits
        r, k, v, gate, rate = (proj[:, i * C:(i + 1) * C] for i in range(5))
        low = rt.linear_f32(x, self.w_w1)
        ops.tanh_(low)
        w_logit = rt.linear_f32(low, self.w_w2)
        w, a, u = (rt.empty((T, C), torch.float32) for _ in range(3))
        ops.delta_operands(w_logit, self.w0, rate, self.a_bias, k, w, a, u, H, D, self.decay_scale, self.unit_eps)
        o = rt.empty((T, H, D), torch.float32)
        ops.linear_state(r, k, v, cache.state, ops.StepRows(ctx.seq_of_token, ctx.q_start, ctx.state_slots), o, H, D, D,
                         w_rows=w, a_rows=a, b_rows=u)
        y = rt.empty((T, C))
        ops.head_norm_gate(o, y, self.norm_eps, weight=self.norm_weight, gate=gate, weight_per_head=True,
                           gate_sigmoid=True)
        return rt.linear(y, self.w_out)


class LightningAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay: Sequence[float],
                 norm_eps: float = 1e-6, init_std: float = 0.02):
        if min(num_heads, head_dim, value_dim) <= 0 or head_dim > 256:
            raise ValueError("heads, head_dim (at most 256) and value_dim must be positive")
        if len(decay) != num_heads:
            raise ValueError(f"{len(decay)} decays for {num_heads} heads")
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.value_dim, self.norm_eps, self.init_std = int(value_dim), float(norm_eps), float(init_std)
        self.decay_values = [float(d) for d in decay]
        self.qk_dim, self.v_dim = self.num_heads * self.head_dim, self.num_heads * self.value_dim
        self.w_in = self.w_out = self.norm_weight = self.decay = None

    def param_specs(self) -> List[ParamSpec]:
        W, s = self.hidden_size, self.init_std
        return [ParamSpec("q.weight", (self.qk_dim, W), std=s), ParamSpec("k.weight", (self.qk_dim, W), std=s),
                ParamSpec("v.weight", (self.v_dim, W), std=s), ParamSpec("g.weight", (self.v_dim, W), std=s),
                ParamSpec("norm.weight", (self.v_dim,), init="ones"), ParamSpec("o.weight", (W, self.v_dim), std=s)]

    def state_need(self) -> StateNeed:
        return StateNeed((self.qk_dim * self.value_dim,), "float32")

    def bind(self, tensors, rt) -> None:
        self.w_in = stack_rows([tensors[f"{n}.weight"] for n in "qkvg"])
        self.norm_weight = tensors["norm.weight"].contiguous()
        self.w_out = tensors["o.weight"].contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(rt.device)

    def forward(self, ctx, x, cache):
        rt, T, H = ctx.rt, x.shape[0], self.num_heads
        proj = rt.linear(x, self.w_in)  # q | k | v | gate
        Q, V = self.qk_dim, self.v_dim
        q, k, v, gate = proj[:, :Q], proj[:, Q:2 * Q], proj[:, 2 * Q:2 * Q + V], proj[:, 2 * Q + V:]
        o = rt.empty((T, H, self.value_dim), torch.float32)
        ops.linear_state(q, k, v, cache.state, ops.StepRows(ctx.seq_of_token, ctx.q_start, ctx.state_slots), o, H,
                         self.head_dim, self.value_dim, w_head=self.decay, silu=True)
        y = rt.empty((T, V))
        # one norm over all heads together: "one head" of all heads' value columns
        ops.head_norm_gate(o.view(T, 1, V), y, self.norm_eps, weight=self.norm_weight, gate=gate, gate_sigmoid=True)
        return rt.linear(y, self.w_out)


register_part("mixer", "generalized_delta", GeneralizedDelta)
register_part("mixer", "lightning_attention", LightningAttention)
