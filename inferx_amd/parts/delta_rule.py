"""A recurrent mixer: the gated delta rule, a matrix of state per head that every token decays, corrects and reads.

    q|k|v|gate = x . [Wq; Wk; Wv; Wg]^T;   a|b = x . [Wa; Wb]^T  (float32)
    q, k, v    = silu(short_conv(.))                 causal, per channel, continued from the request's last inputs
    q, k       = unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q also times dim^(-1/2)
    g          = exp(-exp(A_log) softplus(a + dt_bias)),   beta = sigmoid(b)            one of each per head
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                        S [dim, vdim] float32
    y          = (o / rms(o) * norm_weight * silu(gate)) . Wo^T                         rms over a head's vdim

Options: `decay_rank` r > 0 gives a decay per head AND key channel through two products in a row,
g = exp(-exp(A_log_h) softplus(Wa2 (Wa1 x) + dt_bias)) laid out heads x dim (Wa1 [r, hidden], Wa2 [heads * dim, r],
dt_bias [heads * dim]), acting on the rows of S; `gate_rank` r > 0 makes the gate's logits Wg2 (Wg1 x) likewise;
`gate_activation` "sigmoid" gates with sigmoid(gate) instead of silu(gate).

Query head h reads the q/k head h / (heads / kv_heads).  State per request: the heads' matrices (a column's rows side by side, as the kernels read them) and the short
convolution's last inputs, both float32, in the request's state slot; nothing is kept in pages.  Decays, step
sizes, unit norms, the recurrence and the head norm are float32 in every run.
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import Mixer, ParamSpec, StateNeed, register_part
from .dense_mlp import stack_rows
from .short_conv import ShortConv


class GatedDeltaMixer(Mixer):
    graph_safe = True  # every launch reads the step's device arrays and the state only

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 conv_taps: int, norm_eps: float = 1e-6, init_std: float = 0.02, decay_rank: int = 0,
                 gate_rank: int = 0, gate_activation: str = "silu"):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if head_dim > 256:
            raise ValueError(f"head_dim {head_dim}: at most 256")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim, self.norm_eps = int(head_dim), int(value_dim), float(norm_eps)
        self.init_std = float(init_std)
        if decay_rank < 0 or gate_rank < 0 or gate_activation not in ("silu", "sigmoid"):
            raise ValueError("decay_rank and gate_rank must not be negative, the gate's activation silu or sigmoid")
        self.decay_rank, self.gate_rank, self.gate_sigmoid = int(decay_rank), int(gate_rank), gate_activation == "sigmoid"
        self.qk_dim, self.v_dim = self.num_kv_heads * self.head_dim, self.num_heads * self.value_dim
        self.conv = ShortConv(self.qk_dim, self.qk_dim, self.v_dim, self.head_dim, self.value_dim, conv_taps)
        self.matrix_floats = self.num_heads * self.head_dim * self.value_dim
        self.w_in = self.w_ab = self.w_out = self.a_log = self.dt_bias = self.norm_weight = None
        self.w_a2 = self.w_g2 = None

    def param_specs(self) -> List[ParamSpec]:
        W, s, H = self.hidden_size, self.init_std, self.num_heads
        decays = H * self.head_dim if self.decay_rank else H
        specs = [ParamSpec("q.weight", (self.qk_dim, W), std=s), ParamSpec("k.weight", (self.qk_dim, W), std=s),
                 ParamSpec("v.weight", (self.v_dim, W), std=s), ParamSpec("b.weight", (H, W), std=s),
                 ParamSpec("A_log", (H,), std=0.5), ParamSpec("dt_bias", (decays,), std=0.5),
                 ParamSpec("norm.weight", (self.value_dim,), init="ones"),
                 ParamSpec("o.weight", (W, self.v_dim), std=s)] + self.conv.param_specs()
        if self.gate_rank:
            specs += [ParamSpec("g1.weight", (self.gate_rank, W), std=s),
                      ParamSpec("g2.weight", (self.v_dim, self.gate_rank), std=0.3)]
        else:
            specs.append(ParamSpec("g.weight", (self.v_dim, W), std=s))
        if self.decay_rank:
            specs += [ParamSpec("a1.weight", (self.decay_rank, W), std=s),
                      ParamSpec("a2.weight", (decays, self.decay_rank), std=0.3)]
        else:
            specs.append(ParamSpec("a.weight", (H, W), std=s))
        return specs

    def state_need(self) -> StateNeed:
        return StateNeed((self.matrix_floats + self.conv.state_floats,), "float32")

    def bind(self, tensors, rt) -> None:
        # one product for q | k | v | the gate (or its inner part) | the decay's inner part
        first = [tensors[f"{n}.weight"] for n in "qkv"] + [tensors["g1.weight" if self.gate_rank else "g.weight"]]
        if self.decay_rank:
            first.append(tensors["a1.weight"])
            self.w_ab = tensors["b.weight"].contiguous()
            self.w_a2 = tensors["a2.weight"].contiguous()
        else:
            self.w_ab = stack_rows([tensors["a.weight"], tensors["b.weight"]])
        if self.gate_rank:
            self.w_g2 = tensors["g2.weight"].contiguous()
        self.w_in = stack_rows(first)
        self.w_out = tensors["o.weight"].contiguous()
        self.a_log = tensors["A_log"].to(torch.float32).contiguous()
        self.dt_bias = tensors["dt_bias"].to(torch.float32).contiguous()
        self.norm_weight = tensors["norm.weight"].contiguous()
        self.conv.bind(tensors)

    def forward(self, ctx, x, cache):
        rt, T = ctx.rt, x.shape[0]
        proj = rt.linear(x, self.w_in)        # q | k | v | gate (or its inner part) | the decay's inner part
        ab = rt.linear_f32(x, self.w_ab)      # the decay's and the step size's logits (or the latter alone), float32
        at = 2 * self.qk_dim + self.v_dim
        gate_width = self.gate_rank or self.v_dim
        gate = proj[:, at:at + gate_width]
        if self.gate_rank:
            gate = rt.linear(gate.contiguous(), self.w_g2)
        channel_logits = None
        if self.decay_rank:  # a decay per key channel: its logits through the second product, float32
            inner = proj[:, at + gate_width:at + gate_width + self.decay_rank].contiguous()
            channel_logits = rt.linear_f32(inner, self.w_a2)
            ops.channel_decays(channel_logits, self.a_log, self.dt_bias, self.num_heads, self.head_dim)  # in place
        q, k, v = rt.empty((T, self.qk_dim)), rt.empty((T, self.qk_dim)), rt.empty((T, self.v_dim))
        matrices, tail = cache.state[:, :self.matrix_floats], cache.state[:, self.matrix_floats:]
        self.conv.apply(ctx, proj, tail, q, k, v, silu=True)
        o = rt.empty((T, self.num_heads, self.value_dim), torch.float32)
        ops.delta_rule(q, k, v, ab, self.a_log, self.dt_bias, matrices,
                       ops.StepRows(ctx.seq_of_token, ctx.q_start, ctx.state_slots), o, self.num_heads,
                       self.num_kv_heads, self.head_dim, self.value_dim, channel_logits)
        y = rt.empty((T, self.v_dim))
        ops.head_norm_gate(o, y, self.norm_eps, weight=self.norm_weight, gate=gate, gate_sigmoid=self.gate_sigmoid)
        return rt.linear(y, self.w_out)


register_part("mixer", "gated_delta", GatedDeltaMixer)
