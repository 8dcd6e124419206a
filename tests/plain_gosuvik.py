"""A plain, slow implementation of the Gosuvik design: float64 on the CPU, one function per mechanism, a whole
sequence at a time, recurrences token by token.  It shares no code with the engine; the tests compare the two.

    layer      : h += mixer(gnorm1(h));  h += feed_forward(gnorm2(h))      gnorm: RMS norm over `groups` runs of the width
    order      : layers [start, stop) run `times` times in a row with the same tensors, a cache or state per pass
    chan_delta : q, k, v = silu(conv(W x));  q, k unit vectors per head (q also / sqrt(dim));  beta = sigmoid(Wb x)
                 g = exp(-exp(A_h) softplus(Wa2 Wa1 x + dt))  per head AND key channel
                 S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
                 y = Wo (o / rms(o) * wn * sigmoid(Wg2 Wg1 x))
    latent     : q = Wq x (per head [dim plain | rot_dim rotated]);  d = Wdkv x;  c = rmsnorm(d[:rank]) * wc;
                 kr = rotate(d[rank:]);  k_h = Wuk_h c, v_h = Wuv_h c;  keys i - size < j <= i
                 p = softmax((q_plain . k_h + q_rot . kr) scale);  y = Wo (concat(p v_h) * sigmoid(Wgate x))
                 rotate: halves (i, i + dims / 2), stretched frequencies (blend of f and f / factor by a ramp over i),
                 cos and sin times 0.1 ln(factor) + 1
    pair       : ls * left + rs * right
      left     : q, k normed per head, rotated over the first `dims` numbers (frequencies / factor);  values turned by
                 their own position over all of vdim, the head's sum turned back by the query's position
                 p_j = exp(s_j) / (exp(sink_h) + sum exp(s));  window as above
      right    : i = cap tanh((Wi x + bi) / cap);  f = logsigmoid(cap tanh((Wf x + bf) / cap));  m' = max(f + m, i)
                 S <- e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k;  o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)
                 y = Wo (concat(o / rms(o)) * wn * sigmoid(Wg x))
    polynorm   : Wdown (a N(z) + b N(z^2) + c N(z^3) + e),  z = Wup x,  N(v) = v / rms(v)
    experts    : s = softmax(Wr x);  top-k, weights s / (sum of the chosen + 1e-20);  expert = Wdown (silu(Wg x) * Wu x)
"""
import math

import torch

F = torch.float64


def exact(x):
    return x


def bfloat16(x):
    """x rounded to bfloat16 (nearest even) and back: what keeping an activation in 16 bits does to it."""
    return x.to(torch.bfloat16).to(F)


def jittered(seed):
    """Another sample of what 16-bit storage does: x moved at random by up to one part in 512 (as much as the rounding
    itself), then rounded to bfloat16.  (An engine rounds at other places than this model; several samples show better
    how far rounding alone can move a badly conditioned position.)"""
    g = torch.Generator().manual_seed(seed)

    def store(x):
        return bfloat16(x * (1.0 + (torch.rand(x.shape, generator=g, dtype=F) * 2.0 - 1.0) / 512.0))
    return store


_S = exact  # what keeping an activation between two operations does to it (`forward(store=...)` sets it)


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, eps, groups):
    """Each of `groups` equal consecutive runs of the last dimension over its own root mean square, then the weight."""
    parts = x.view(*x.shape[:-1], groups, x.shape[-1] // groups)
    return rms_unit(parts, eps).reshape(x.shape) * w


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def rotate_halves(x, angles, gain=1.0):
    """x [T, ..., d] with d = 2 * angles.shape[1]: element i is paired with i + d / 2 and the pair turned by
    angles[t, i]; cos and sin are multiplied by `gain`."""
    half = angles.shape[1]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = (torch.cos(angles) * gain).view(shape), (torch.sin(angles) * gain).view(shape)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * cos - v * sin, v * cos + u * sin], dim=-1)


def rotate_first(x, angles, gain=1.0):
    """The first 2 * angles.shape[1] numbers of the last dimension rotated, the rest as they are."""
    d = 2 * angles.shape[1]
    return torch.cat([rotate_halves(x[..., :d], angles, gain), x[..., d:]], dim=-1)


def frequencies(rot):
    """(f_i for i < dims / 2, gain of cos and sin) of a rotation {"dims", "base", "scaling"}."""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])
    if "original" not in sc:            # every frequency slowed alike
        return f / factor, 1.0

    def turns_to_index(t):
        return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turns_to_index(sc["fast"])), 0)
    hi = min(math.ceil(turns_to_index(sc["slow"])), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def visible(positions, window):
    d = positions[:, None] - positions[None, :]
    seen = d >= 0
    if window:
        seen &= d < window
    return seen


def short_conv(u, w):
    """u [T, C], w [C, taps]: y[t] = sum_j w[:, j] u[t - taps + 1 + j], zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=F), u])
    return sum(padded[j:j + T] * w[:, j] for j in range(taps))


def channel_delta(x, w, m, eps):
    T = x.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = _S(silu(short_conv(_S(x @ w["q"].T), w["q.conv"]))).view(T, G, d)
    k = _S(silu(short_conv(_S(x @ w["k"].T), w["k.conv"]))).view(T, G, d)
    v = _S(silu(short_conv(_S(x @ w["v"].T), w["v.conv"]))).view(T, H, vd)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(x @ w["b"].T)                                              # [T, H]
    a = (_S(x @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(T, H, d)
    g = torch.exp(-torch.exp(w["A_log"])[None, :, None] * softplus(a))               # [T, H, d]
    gate = torch.sigmoid(_S(_S(x @ w["g1"].T) @ w["g2"].T)).view(T, H, vd)
    S = torch.zeros(H, d, vd, dtype=F)
    o = torch.zeros(T, H, vd, dtype=F)
    for t in range(T):
        for h in range(H):
            kk, qq = k[t, h // (H // G)], q[t, h // (H // G)]
            S[h] = g[t, h][:, None] * S[h]
            u = beta[t, h] * (v[t, h] - S[h].T @ kk)
            S[h] = S[h] + torch.outer(kk, u)
            o[t, h] = S[h].T @ qq
    y = _S(rms_unit(o, eps) * w["norm"] * gate)
    return y.reshape(T, H * vd) @ w["o"].T


def latent_attention(x, w, m, eps, positions):
    T = x.shape[0]
    H, d, r, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = _S(x @ w["q"].T).view(T, H, d + r)
    dkv = _S(x @ w["dkv"].T)
    c = _S(rms_unit(dkv[:, :rank], eps) * w["dkv.norm"])
    kr, q_rot = dkv[:, rank:], q[:, :, d:]
    rot = m.get("rot")
    if rot:
        f, gain = frequencies(rot)
        ang = positions.to(F)[:, None] * f[None, :]
        kr, q_rot = _S(rotate_first(kr, ang, gain)), _S(rotate_first(q_rot, ang, gain))
    k = _S(c @ w["uk"].T).view(T, H, d)
    v = _S(c @ w["uv"].T).view(T, H, vd)
    score = (torch.einsum("ihd,jhd->hij", q[:, :, :d], k) + torch.einsum("ihr,jr->hij", q_rot, kr)) * m["scale"]
    seen = visible(positions, (m.get("mask") or {}).get("size", 0))
    p = torch.softmax(score.masked_fill(~seen[None], -math.inf), dim=-1)
    o = torch.einsum("hij,jhv->ihv", p, v).reshape(T, H * vd)
    return _S(_S(o) * torch.sigmoid(_S(x @ w["g"].T))) @ w["o"].T


def sink_attention(x, w, m, eps, positions):
    T = x.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_unit(_S(x @ w["q"].T).view(T, H, d), eps) * w["q.norm"]
    k = rms_unit(_S(x @ w["k"].T).view(T, G, d), eps) * w["k.norm"]
    v = _S(x @ w["v"].T).view(T, G, vd)
    rot = m.get("rot")
    pos = positions.to(F)[:, None]
    if rot:
        f, gain = frequencies(rot)
        q, k = rotate_first(q, pos * f[None, :], gain), rotate_first(k, pos * f[None, :], gain)
    q, k = _S(q), _S(k)
    fv = float(rot["base"]) ** (-2.0 * torch.arange(vd // 2, dtype=F) / vd) if rot else None
    if rot:
        v = _S(rotate_halves(v, pos * fv[None, :]))
    kx, vx = k.repeat_interleave(H // G, dim=1), v.repeat_interleave(H // G, dim=1)
    score = torch.einsum("ihd,jhd->hij", q, kx) * m["scale"]
    seen = visible(positions, (m.get("mask") or {}).get("size", 0))
    score = score.masked_fill(~seen[None], -math.inf)
    top = torch.maximum(score.max(-1).values, w["sink"][:, None])                   # [H, T]
    e = torch.exp(score - top[..., None])
    p = e / (e.sum(-1) + torch.exp(w["sink"][:, None] - top))[..., None]
    o = torch.einsum("hij,jhv->ihv", p, vx)
    if rot:
        o = rotate_halves(o, -pos * fv[None, :])
    return _S(o).reshape(T, H * vd) @ w["o"].T


def matrix_memory(x, w, m, eps):
    T = x.shape[0]
    H, d, vd, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (_S(x @ w["q"].T) * d ** -0.5).view(T, H, d)
    k = _S(x @ w["k"].T).view(T, H, d)
    v = _S(x @ w["v"].T).view(T, H, vd)
    gi = cap * torch.tanh((x @ w["i"].T + w["i.b"]) / cap)                          # [T, H]
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((x @ w["f"].T + w["f.b"]) / cap))
    S, n, top = torch.zeros(H, d, vd, dtype=F), torch.zeros(H, d, dtype=F), torch.zeros(H, dtype=F)
    o = torch.zeros(T, H, vd, dtype=F)
    for t in range(T):
        new_top = torch.maximum(gf[t] + top, gi[t])
        keep, take = torch.exp(gf[t] + top - new_top), torch.exp(gi[t] - new_top)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        top = new_top
        below = torch.maximum(((n * q[t]).sum(-1)).abs(), torch.exp(-top)) + 1e-6
        o[t] = torch.einsum("hdv,hd->hv", S, q[t]) / below[:, None]
    y = _S(rms_unit(o, eps).reshape(T, H * vd) * w["norm"] * torch.sigmoid(_S(x @ w["g"].T)))
    return y @ w["o"].T


def pair(x, w, m, eps, positions):
    left = sink_attention(x, sub(w, "left."), m["left"], eps, positions)
    right = matrix_memory(x, sub(w, "right."), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def polynorm_mlp(x, w, eps):
    z = _S(x @ w["up"].T)
    a, b, c, e = (float(t) for t in w["act"])
    y = a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e
    return _S(y) @ w["down"].T


def route(x, w, f):
    """(experts [T, top], weights [T, top]) of every token."""
    s = torch.softmax(x @ w["router"].T, dim=-1)
    val, idx = torch.topk(s, f["router"]["top"], dim=-1)
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20)


def experts_mlp(x, w, f, chosen=None):
    idx, weight = route(x, w, f)
    if chosen is not None:                                                          # the experts from outside
        s = torch.softmax(x @ w["router"].T, dim=-1)
        idx = chosen
        val = torch.gather(s, 1, idx)
        weight = val / (val.sum(-1, keepdim=True) + 1e-20)
    out = torch.zeros(x.shape[0], w["e0.down"].shape[0], dtype=F)
    for t in range(x.shape[0]):
        for e, p in zip(idx[t].tolist(), weight[t]):
            mid = _S(silu(x[t] @ w[f"e{e}.gate"].T) * (x[t] @ w[f"e{e}.up"].T))
            out[t] += p * _S(mid @ w[f"e{e}.down"].T)
    return out


def sub(w, prefix):
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def layer_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    body = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + body * loop["times"] + list(range(loop["stop"], n))


def forward(cfg, weights, tokens, store=exact, experts=None, trace=None, chosen=None, scores=None):
    """Logits [T, vocab] of one sequence from its start.  `weights`: name -> tensor (any float type).  `store`: what
    keeping an activation does (`bfloat16` for a 16-bit engine).  `trace`: a list that receives the stream after every
    layer run.  `experts`: per (layer run with experts) the experts [T, top] to use instead of the router's choice;
    `chosen`: a list that receives the router's own choice per such run, `scores` one that receives the router's
    scores [T, experts]."""
    global _S
    _S = store
    try:
        w = {k: v.to(F) for k, v in weights.items()}
        eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
        positions = torch.arange(len(tokens))
        h = w["embed"][torch.as_tensor(tokens)]
        run = 0
        for i in layer_order(cfg):
            layer, lw = cfg["layers"][i], sub(w, f"l{i}.")
            x = _S(group_norm(h, lw["norm1"], eps, groups))
            mw, m = sub(lw, "mix."), layer["mixer"]
            if layer["type"] == "channel_delta":
                a = channel_delta(x, mw, m, eps)
            elif layer["type"] == "latent_attention":
                a = latent_attention(x, mw, m, eps, positions)
            else:
                a = pair(x, mw, m, eps, positions)
            h = h + a
            f = layer.get("mlp")
            if f:
                x = _S(group_norm(h, lw["norm2"], eps, groups))
                fw = sub(lw, "mlp.")
                if f["kind"] == "dense":
                    h = h + polynorm_mlp(x, fw, eps)
                else:
                    if chosen is not None:
                        chosen.append(route(x, fw, f)[0])
                    if scores is not None:
                        scores.append(torch.softmax(x @ fw["router"].T, dim=-1))
                    h = h + experts_mlp(x, fw, f, None if experts is None else experts[run])
                    run += 1
            if trace is not None:
                trace.append(h.clone())
        return _S(group_norm(h, w["final.norm"], eps, groups)) @ w["head"].T
    finally:
        _S = exact
