"""A recurrent mixer: a matrix memory with exponential gates (the mLSTM cell), a matrix of state per head that every
token scales, adds to and reads.

    q|k|v|gate = x . [Wq; Wk; Wv; Wg]^T;   a|b = x . [Wi; Wf]^T + [bi; bf]  (float32)
    i = cap tanh(a / cap),  f = logsigmoid(cap tanh(b / cap))            the gates' logarithms, one of each per head
    m' = max(f + m, i)                                                   a running maximum that starts at 0
    S <- exp(f + m - m') S + exp(i - m') k v^T;   n <- likewise with k alone
    o = S^T q' / (max(|n . q'|, exp(-m')) + 1e-6),   q' = q dim^(-1/2)
    y = (o / rms(o over the head) * norm_weight * sigmoid(gate)) . Wo^T   norm_weight of all heads' size

State per request, float32, in the request's state slot: the heads' matrices (a column's rows side by side, as the
kernels read them) with n as one more column (its value is always 1), then the maxima; nothing is kept in pages.
The chain of maxima runs first, in a launch of its own, so that the recurrence's blocks share nothing; the division
rides on the kernel that normalises the heads.  Gates, maxima, exponentials, the recurrence and the
head norm are float32 in every run.
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import Mixer, ParamSpec, StateNeed, register_part
from .dense_mlp import stack_rows


class MatrixMemoryMixer(Mixer):
    graph_safe = True  # every launch reads the step's device arrays and the state only

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, gate_cap: float,
                 norm_eps: float = 1e-6, init_std: float = 0.02):
        if min(num_heads, head_dim, value_dim) <= 0 or head_dim > 256 or gate_cap <= 0:
            raise ValueError("heads, head_dim (at most 256), value_dim and gate_cap must be positive")
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.value_dim, self.gate_cap = int(value_dim), float(gate_cap)
        self.norm_eps, self.init_std = float(norm_eps), float(init_std)
        self.qk_dim, self.v_dim = self.num_heads * self.head_dim, self.num_heads * self.value_dim
        self.state_floats = ops.matrix_memory_state_floats(self.num_heads, self.head_dim, self.value_dim)
        self.w_in = self.w_gates = self.b_gates = self.w_out = self.norm_weight = None

    def param_specs(self) -> List[ParamSpec]:
        W, s, H = self.hidden_size, self.init_std, self.num_heads
        return [ParamSpec("q.weight", (self.qk_dim, W), std=s), ParamSpec("k.weight", (self.qk_dim, W), std=s),
                ParamSpec("v.weight", (self.v_dim, W), std=s), ParamSpec("g.weight", (self.v_dim, W), std=s),
                ParamSpec("i.weight", (H, W), std=s), ParamSpec("i.bias", (H,), std=0.5),
                ParamSpec("f.weight", (H, W), std=s), ParamSpec("f.bias", (H,), std=0.5, mean=2.0),
                ParamSpec("norm.weight", (self.v_dim,), init="ones"), ParamSpec("o.weight", (W, self.v_dim), std=s)]

    def state_need(self) -> StateNeed:
        return StateNeed((self.state_floats,), "float32")

    def bind(self, tensors, rt) -> None:
        self.w_in = stack_rows([tensors[f"{n}.weight"] for n in "qkvg"])
        self.w_gates = stack_rows([tensors["i.weight"], tensors["f.weight"]])
        self.b_gates = torch.cat([tensors["i.bias"].to(torch.float32), tensors["f.bias"].to(torch.float32)]).contiguous()
        self.norm_weight = tensors["norm.weight"].contiguous()
        self.w_out = tensors["o.weight"].contiguous()

    def forward(self, ctx, x, cache):
        rt, T, H = ctx.rt, x.shape[0], self.num_heads
        proj = rt.linear(x, self.w_in)            # q | k | v | gate
        gates = rt.linear_f32(x, self.w_gates)    # the two gates' logits, float32
        Q, V = self.qk_dim, self.v_dim
        q, k, v, gate = proj[:, :Q], proj[:, Q:2 * Q], proj[:, 2 * Q:2 * Q + V], proj[:, 2 * Q + V:]
        o, nq = rt.empty((T, H, self.value_dim), torch.float32), rt.empty((T, H), torch.float32)
        work = rt.empty((T, H, 3), torch.float32)  # keep, take, exp(-m') per token and head
        ops.matrix_memory(q, k, v, gates, self.b_gates, self.gate_cap, cache.state,
                          ops.StepRows(ctx.seq_of_token, ctx.q_start, ctx.state_slots), o, nq, work, H, self.head_dim,
                          self.value_dim)
        y = rt.empty((T, V))
        ops.head_norm_gate(o, y, self.norm_eps, weight=self.norm_weight, gate=gate, weight_per_head=True,
                           gate_sigmoid=True, den_a=nq, den_b=work[:, :, 2])
        return rt.linear(y, self.w_out)


register_part("mixer", "matrix_memory", MatrixMemoryMixer)
