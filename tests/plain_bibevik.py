"""A plain, slow implementation of the Bibevik design: float64 on the CPU, one function per mechanism, a whole
sequence at a time, recurrences token by token.  It shares no code with the engine; the tests compare the two.

    layer      : x = norm(h);  h += mixer(x) + feed_forward(x)        one norm with ONE number as its weight
    latent     : q = Wq x (per head [dim plain | rot_dim rotated]);  d = Wdkv x;  c = rmsnorm(d[:rank]) * wc;
                 kr = rotate(d[rank:]);  k_h = Wuk_h c, v_h = Wuv_h c;  p = softmax_j<=i((q_plain . k_h + q_rot . kr) scale)
    delta      : r, k, v = W x;  w = exp(-e^(-1/2) sigmoid(W2 tanh(W1 x) + w0));  a = sigmoid(Wa x + ba);  u = k / |k|
                 S <- diag(w) S - (a u)(u^T S) + k v^T;  o = S^T r;  y = Wo (o / rms(o) * wn * sigmoid(Wg x))
    lightning  : q, k, v = silu(W x);  S <- decay_h S + k v^T;  o = S^T q;  y = Wo (rmsnorm(all heads of o) * wn * sigmoid(Wg x))
    glu        : g = min(Wg x, L);  u = clamp(Wu x, -L, L);  down(g sigmoid(1.702 g) (u + 1))
    experts    : s = sigmoid(Wr x);  a group's score is the sum of its two best;  the best `keep` groups stay;
                 top-k of what stays, weights s * scale;  a shared expert beside
"""
import math

import torch

F = torch.float64


def exact(x):
    return x


def bfloat16(x):
    """x rounded to bfloat16 (nearest even) and back: what keeping an activation in 16 bits does to it."""
    return x.to(torch.bfloat16).to(F)


_S = exact  # what keeping an activation between two operations does to it (`forward(store=...)` sets it)


def jittered(seed):
    """Another sample of what 16-bit storage does: x moved by up to one part in 512 at random (as much as the rounding itself), then rounded to
    bfloat16.  (An engine rounds at other places than this model; several samples show better how far rounding alone
    can move a badly conditioned position.)"""
    g = torch.Generator().manual_seed(seed)

    def store(x):
        return bfloat16(x * (1.0 + (torch.rand(x.shape, generator=g, dtype=F) * 2.0 - 1.0) / 512.0))
    return store


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    return rms_unit(x, eps) * g


def rotate_pairs(x, positions, dims, base):
    """x [T, ..., d]: elements (2i, 2i + 1), i < dims / 2, turned by positions * base^(-2i / dims)."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=F)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(F)[:, None] * freq[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_attention(x, w, m, eps, positions):
    T = x.shape[0]
    H, d, r, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = _S(x @ w["q"].T).view(T, H, d + r)
    dkv = _S(x @ w["dkv"].T)
    c = _S(rms_unit(dkv[:, :rank], eps) * w["dkv.norm"])
    rot = m.get("rot")
    kr, q_rot = dkv[:, rank:], q[:, :, d:]
    if rot is not None:
        kr = _S(rotate_pairs(kr, positions, rot["dims"], rot["base"]))
        q_rot = _S(rotate_pairs(q_rot, positions, rot["dims"], rot["base"]))
    k = _S(c @ w["uk"].T).view(T, H, d)
    v = _S(c @ w["uv"].T).view(T, H, vd)
    score = (torch.einsum("ihd,jhd->hij", q[:, :, :d], k) + torch.einsum("ihr,jr->hij", q_rot, kr)) * m["scale"]
    seen = positions[None, :] <= positions[:, None]
    score = score.masked_fill(~seen[None], -math.inf)
    p = torch.softmax(score, -1)
    o = _S(torch.einsum("hij,jhv->ihv", p, v).reshape(T, H * vd))
    return _S(o @ w["o"].T)


def general_delta(x, w, m, eps):
    T = x.shape[0]
    H, d = m["heads"], m["dim"]
    r, k, v = [_S(x @ w[n].T).view(T, H, d) for n in ("r", "k", "v")]
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(x @ w["w1"].T) @ w["w2"].T + w["w0"])).view(T, H, d)
    a = torch.sigmoid(_S(x @ w["a"].T) + w["a.b"]).view(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, d, d, dtype=F)
    o = torch.zeros(T, H, d, dtype=F)
    for t in range(T):
        old = S
        read = torch.einsum("hi,hij->hj", u[t], old)
        S = decay[t][:, :, None] * old - (a[t] * u[t])[:, :, None] * read[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hij,hi->hj", S, r[t])
    y = _S(rms_unit(o, eps).reshape(T, H * d) * w["norm"] * torch.sigmoid(_S(x @ w["g"].T)))
    return _S(y @ w["o"].T)


def lightning(x, w, m, eps):
    T = x.shape[0]
    H, d, vd = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q, k = silu(_S(x @ w["q"].T)).view(T, H, d), silu(_S(x @ w["k"].T)).view(T, H, d)
    v = silu(_S(x @ w["v"].T)).view(T, H, vd)
    decay = torch.tensor(m["decay"], dtype=F)
    S = torch.zeros(H, d, vd, dtype=F)
    o = torch.zeros(T, H, vd, dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hij,hi->hj", S, q[t])
    y = _S(rms_unit(o.reshape(T, H * vd), eps) * w["norm"] * torch.sigmoid(_S(x @ w["g"].T)))
    return _S(y @ w["o"].T)


def clamped_glu(x, gate, up, down, limit, gate_b=0.0, up_b=0.0, down_b=0.0):
    g = torch.clamp(x @ gate.T + gate_b, max=limit)
    u = torch.clamp(x @ up.T + up_b, -limit, limit)
    return _S(_S(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T + down_b)


def dense_ff(x, w, f):
    return clamped_glu(x, w["gate"], w["up"], w["down"], f["limit"], w["gate.b"], w["up.b"], w["down.b"])


def choose_experts(scores, top, groups, keep):
    """scores [T, E] -> chosen experts [T, top] (best first; of equal scores the lower index)."""
    T, E = scores.shape
    size = E // groups
    per_group = scores.view(T, groups, size)
    best_two = torch.sort(per_group, -1, descending=True).values[..., :min(2, size)].sum(-1)
    kept = torch.sort(best_two, dim=-1, descending=True, stable=True).indices[:, :keep]
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = scores.masked_fill(~allowed[:, :, None].expand(T, groups, size).reshape(T, E), -math.inf)
    return torch.sort(masked, dim=-1, descending=True, stable=True).indices[:, :top]


def router_scores(x, w):
    return torch.sigmoid(x @ w["router"].T)


def moe_ff(x, w, f, chosen=None):
    """`chosen`: experts per token from outside (the engine's choice, where a near tie went the other way)."""
    router, expert = f["router"], f["expert"]
    s = router_scores(x, w)
    groups = router.get("groups") or {"count": 1, "keep": 1}
    if chosen is None:
        chosen = choose_experts(s, router["top"], groups["count"], groups["keep"])
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e in chosen[t].tolist():
            y = clamped_glu(x[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], expert["limit"])
            out[t] += s[t, e] * router["scale"] * y[0]
    shared = f.get("shared")
    if shared:
        out = out + clamped_glu(x, w["shared.gate"], w["shared.up"], w["shared.down"], shared["limit"])
    return out


MIXERS = {"latent_attention": lambda x, w, m, eps, pos: latent_attention(x, w, m, eps, pos),
          "general_delta": lambda x, w, m, eps, pos: general_delta(x, w, m, eps),
          "lightning": lambda x, w, m, eps, pos: lightning(x, w, m, eps)}


def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F) for k, v in tensors.items() if k.startswith(prefix)}


def forward(config, tensors, tokens, chosen=None, keep_layers=False, keep_router=None, store=exact):
    """Logits [T, vocab] of one sequence from position 0; with `keep_layers` also the stream after every layer run.
    `chosen`: {layer run: experts [T, top]} from outside; `keep_router`: a dict that receives every routed layer
    run's scores [T, E].  `store=bfloat16`: a model of a 16-bit run, in which every activation kept between two
    operations is rounded (the stream, the norms' sums, scores, routers and recurrences stay as they are)."""
    global _S
    _S = store
    try:
        return _forward(config, tensors, tokens, chosen, keep_layers, keep_router)
    finally:
        _S = exact


def _forward(config, tensors, tokens, chosen, keep_layers, keep_router):
    eps = config["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(ids))
    h = tensors["embed"].to(F)[ids] * config.get("embedding", {}).get("scale", 1.0)
    after = []
    for i, layer in enumerate(config["layers"]):
        src = layer.get("weights_of", i)
        p = f"l{src}."
        x = _S(scalar_norm(h, tensors[p + "norm1"].to(F), eps))
        delta = MIXERS[layer["type"]](x, sub(tensors, p + "mix."), layer["mixer"], eps, positions)
        f = layer.get("mlp")
        if f is not None:
            w = sub(tensors, p + "mlp.")
            if f["kind"] == "dense":
                delta = delta + dense_ff(x, w, f)
            else:
                if keep_router is not None:
                    keep_router[i] = router_scores(x, w)
                delta = delta + moe_ff(x, w, f, None if chosen is None else chosen.get(i))
        h = h + delta
        after.append(h.clone())
    logits = _S(scalar_norm(h, tensors["final.norm"].to(F), eps)) @ tensors["head"].to(F).T
    return (logits, torch.stack(after)) if keep_layers else logits
