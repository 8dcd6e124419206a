"""Attention over a compressed cache: one latent row per token, from which every head's keys and values are linear
maps, and one rotated key part that all heads share.

    q        = x . Wq^T                          per head [dim plain | rot_dim rotated]
    d        = x . Wdkv^T                        rank + rot_dim numbers
    c        = rmsnorm(d[:rank]) * w_c           the latent (float32 sums); kr = rotate(d[rank:])
    k_h, v_h = Wuk_h c,  Wuv_h c                 never formed: the maps move to the query's side
    ql_h     = Wuk_h^T q_h[:dim]                 a product per head before the attention
    p_h      = softmax_j<=i((ql_h . c[j] + rotate(q_h[dim:]) . kr[j]) * scale)
    y        = concat_h(Wuv_h (sum_j p_h[j] c[j])) . Wo^T        a product per head after it

Only [c | kr] is kept per token (`CacheNeed` of one array, one "head" of rank + rot_dim numbers), whatever the
number of heads.  The rotation pairs element 2i with 2i + 1 over the first `rotary_dim` numbers of the rotated part
(the position encoding's table by pair; the rest of the part passes); with `pairing` "halves" it pairs element i with
i + rotary_dim / 2 instead.  Norm, angles, scores and softmax are float32.

Options: `window` W (a query reads its own row and the W - 1 before it; older pages are given back), and `gate`
(the heads' results times sigmoid(x . Wg^T), element by element, before the last product).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..config.spec import PartSpec
from .base import CacheArray, CacheNeed, Mixer, ParamSpec, build_part, register_part
from .dense_mlp import stack_rows


class LatentAttention(Mixer):
    graph_safe = True  # every launch reads the step's device arrays only

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int,
                 scale: Optional[float] = None, norm_eps: float = 1e-6, position: Optional[PartSpec] = None,
                 init_std: float = 0.02, pairing: str = "pairs", window: int = 0, gate: bool = False):
        if min(num_heads, head_dim, value_dim, kv_rank) <= 0 or rot_dim < 0:
            raise ValueError("heads, head_dim, value_dim and kv_rank must be positive, rot_dim not negative")
        if kv_rank > 1024 or rot_dim > 64 + 1024 - kv_rank:
            raise ValueError(f"kv_rank {kv_rank} with rot_dim {rot_dim}: a latent of at most 1024 numbers, with the "
                             "rotated part at most 1088")
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.rot_dim, self.value_dim, self.kv_rank = int(rot_dim), int(value_dim), int(kv_rank)
        self.q_dim = self.head_dim + self.rot_dim
        self.scale = float(scale) if scale is not None else self.q_dim ** -0.5
        self.norm_eps, self.init_std = float(norm_eps), float(init_std)
        if pairing not in ("pairs", "halves") or window < 0:
            raise ValueError(f"pairing {pairing!r} (pairs or halves), window {window} (not negative)")
        self.halves, self.window, self.has_gate = pairing == "halves", int(window), bool(gate)
        self.position = build_part("position", position) if position is not None else None
        if self.position is not None:
            dims = int(getattr(self.position, "rotary_dim", 0))
            if getattr(self.position, "begin", 0) != 0 or dims <= 0 or dims % 2 or dims > self.rot_dim:
                raise ValueError(f"the position encoding must rotate the first {dims} elements of a rotated part of "
                                 f"{self.rot_dim}: an even number within the part, from its start")
        self.w_in = self.w_uk = self.w_uv_t = self.w_out = self.norm_weight = None

    def cache_need(self) -> CacheNeed:
        return CacheNeed((CacheArray("latent", 1, self.kv_rank + self.rot_dim),), self.window)

    def subparts(self):
        return [self.position]

    def param_specs(self) -> List[ParamSpec]:
        W, s, H = self.hidden_size, self.init_std, self.num_heads
        return [ParamSpec("q.weight", (H * self.q_dim, W), std=s),
                ParamSpec("dkv.weight", (self.kv_rank + self.rot_dim, W), std=s),
                ParamSpec("dkv_norm.weight", (self.kv_rank,), init="ones"),
                ParamSpec("uk.weight", (H * self.head_dim, self.kv_rank), std=s),
                ParamSpec("uv.weight", (H * self.value_dim, self.kv_rank), std=s),
                ParamSpec("o.weight", (W, H * self.value_dim), std=s)] + (
                    [ParamSpec("g.weight", (H * self.value_dim, W), std=s)] if self.has_gate else [])

    def bind(self, tensors, rt) -> None:
        H = self.num_heads
        self.w_in = stack_rows([tensors["q.weight"], tensors["dkv.weight"]] +
                               ([tensors["g.weight"]] if self.has_gate else []))
        self.w_uk = tensors["uk.weight"].contiguous().view(H, self.head_dim, self.kv_rank)
        self.w_uv_t = tensors["uv.weight"].view(H, self.value_dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_out = tensors["o.weight"].contiguous()
        self.norm_weight = tensors["dkv_norm.weight"].contiguous()
        if self.position is not None:
            self.position.bind({}, rt)

    def forward(self, ctx, x, cache):
        rt, T, H = ctx.rt, x.shape[0], self.num_heads
        table = self.position.prepare(ctx) if self.position is not None else None
        proj = rt.linear(x, self.w_in)  # q of all heads | d
        q, dkv = proj[:, :H * self.q_dim], proj[:, H * self.q_dim:H * self.q_dim + self.kv_rank + self.rot_dim]
        latent = cache.arrays["latent"]
        ops.latent_prepare(q, dkv, self.norm_weight, self.norm_eps, table,
                           ctx.slots[cache.group] if cache.writes else None, latent, H, self.rot_dim, self.kv_rank,
                           self.halves)
        q3 = q.unflatten(1, (H, self.q_dim))
        q_lat = torch.bmm(q3[:, :, :self.head_dim].transpose(0, 1), self.w_uk)  # [H, T, rank]
        if ctx.one_token_each:  # (the slices of a token's keys meet in a contiguous [T, H, rank])
            o_lat = rt.empty((T, H, self.kv_rank)).transpose(0, 1)
        else:
            o_lat = rt.empty((H, T, self.kv_rank))
        self.attend(ctx, q_lat.transpose(0, 1), q3[:, :, self.head_dim:], cache, o_lat.transpose(0, 1))
        y = rt.empty((T, H * self.value_dim))
        torch.bmm(o_lat, self.w_uv_t, out=y.view(T, H, self.value_dim).transpose(0, 1))
        if self.has_gate:
            ops.sigmoid_gate(y, proj[:, H * self.q_dim + self.kv_rank + self.rot_dim:])
        return rt.linear(y, self.w_out)

    def attend(self, ctx, q_lat, q_rot, cache, out) -> None:
        latent, table = cache.arrays["latent"], ctx.block_tables[cache.group]
        if not ops.latent_mfma_fits(q_lat, q_rot, out, self.kv_rank, self.rot_dim):  # float32 runs, other sizes
            ops.latent_attention_plain(q_lat, q_rot, latent, table, ctx.seq_of_token, ctx.positions, out, self.kv_rank,
                                       self.rot_dim, self.scale, self.window)
            return
        rt, T, H = ctx.rt, q_lat.shape[0], self.num_heads
        splits, work = 1, None
        if ctx.one_token_each:
            splits = ops.latent_mfma_splits(T, H)
            if splits > 1:
                work = (rt.empty((T * H * splits, self.kv_rank), torch.float32), rt.empty((T * H * splits, 2), torch.float32))
        ops.latent_attention_mfma(q_lat, q_rot, latent, table, ctx.seq_of_token, ctx.positions, out, self.kv_rank,
                                  self.rot_dim, self.scale, ctx.one_token_each, splits, work, self.window)


register_part("mixer", "latent_attention", LatentAttention)
