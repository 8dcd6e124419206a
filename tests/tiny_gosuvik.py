"""Tiny Gosuvik configurations that differ from each other in every size and option, and a folder of random weights
for each (norm weights drawn at random too, so that one taken for another, or left out, shows)."""
import json
import os

import torch


def rot(dims, base, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling is not None:
        r["scaling"] = scaling
    return r


def yarn(factor, original, fast, slow):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def latent(heads, dim, rot_dim, vdim, rank, scale, window, rotation, mlp):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if window:
        mixer["mask"] = {"size": window}
    if rotation is not None:
        mixer["rot"] = rotation
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def delta(heads, kv_heads, dim, vdim, conv, mlp):
    return {"type": "channel_delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def pair(left, right, left_scale, right_scale, mlp):
    heads, kv_heads, dim, vdim, scale, window, rotation = left
    a = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        a["mask"] = {"size": window}
    if rotation is not None:
        a["rot"] = rotation
    heads, dim, vdim, cap = right
    b = {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": a, "right": b, "left_scale": left_scale, "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def experts(ff, n, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n, "top": top}}


def config(vocab, width, eps, groups, layers, loop=None):
    cfg = {"architecture": "Gosuvik", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups},
           "layers": layers, "initializer_range": 0.08}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# A: all three mixers, the first two run twice, two groups in the norm, windows shorter than the prompts, grouped
# query heads in the delta layer and in the attention, values wider than keys, stretched rotations of both kinds, a
# rotation of fewer dimensions than the rotated part holds
A = config(320, 96, 1e-5, 2, [
    latent(3, 16, 8, 24, 40, 0.2, 20, rot(6, 10000.0, yarn(4.0, 16, 8.0, 1.0)), dense(64)),
    delta(4, 2, 16, 12, 3, experts(32, 6, 2)),
    pair((4, 2, 16, 24, 0.3, 9, rot(8, 100.0, {"factor": 2.0})), (2, 12, 20, 8.0), 0.7, 1.2, experts(32, 6, 2)),
], loop=(0, 2, 2))
# B: sizes that are no multiple of 4 or 16; three groups; no loop; a layer without feed-forward; no windows; one expert
# per token; a rotation over all of a head without stretching; one tap; one head in the memory; values narrower than keys
B = config(131, 72, 1e-6, 3, [
    pair((3, 3, 10, 6, 0.4, 0, rot(10, 50.0)), (1, 20, 7, 3.0), 1.0, 0.5, None),
    delta(1, 1, 20, 9, 1, dense(36)),
    latent(2, 12, 10, 20, 36, 0.3, 0, rot(10, 100.0, {"factor": 3.0}), experts(36, 5, 1)),
])
# C: one group (the plain norm), one head everywhere, the last two layers run three times, windows of two tokens and of
# one (a token sees itself only), no rotation in the latent layer, all experts chosen
C = config(97, 40, 1e-5, 1, [
    delta(1, 1, 16, 16, 2, experts(24, 2, 2)),
    latent(1, 16, 4, 16, 16, 0.25, 2, None, dense(24)),
    pair((1, 1, 8, 8, 0.5, 1, rot(4, 500.0, {"factor": 1.5})), (1, 8, 8, 30.0), 0.3, 0.3, dense(40)),
], loop=(1, 3, 3))
# D: sizes that the matrix-core attention and the chunked recurrence take (latents and rotated parts in multiples of 16
# and 32, heads of 32, 64 and 128 numbers), sixteen query heads on one latent, eight on two key heads
D = config(256, 128, 1e-5, 4, [
    delta(2, 1, 64, 40, 4, experts(32, 8, 3)),
    latent(16, 24, 32, 40, 64, 0.15, 33, rot(32, 1000.0, yarn(6.0, 32, 16.0, 2.0)), dense(96)),
    pair((8, 2, 32, 32, 0.2, 40, rot(16, 5000.0, {"factor": 2.0})), (2, 64, 24, 6.0), 0.8, 1.1, experts(32, 8, 2)),
    delta(1, 1, 128, 32, 4, None),
    delta(4, 4, 32, 16, 2, dense(64)),
], loop=(1, 2, 2))
# E: a width, a vocabulary and heads that are no multiple of 4 or 8 (groups of 30 numbers in the norm), short windows,
# the pair first, a loop over the whole model
E = config(77, 90, 1e-5, 3, [
    pair((2, 1, 12, 14, 0.3, 5, rot(4, 200.0, {"factor": 1.5})), (3, 10, 6, 2.0), 0.5, 1.5, experts(28, 3, 1)),
    delta(2, 1, 24, 10, 2, dense(50)),
    latent(2, 10, 6, 14, 22, 0.25, 7, rot(6, 300.0, yarn(2.0, 8, 4.0, 0.5)), experts(28, 3, 2)),
], loop=(0, 3, 2))
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E}


def make_folder(raw_config: dict, seed: int, out_dir: str, dtype: str = "bfloat16") -> str:
    from safetensors.torch import load_file, save_file
    from inferx_amd.config import config_from_dict
    from inferx_amd.weights import write_model_folder
    write_model_folder(config_from_dict(json.loads(json.dumps(raw_config))), seed, out_dir, dtype)
    path = os.path.join(out_dir, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(seed + 1)
    for name, t in tensors.items():
        last = name.split(".")[-1]
        if last.startswith("norm"):  # l<i>.norm1, final.norm, l<i>.mix.norm, l<i>.mix.dkv.norm, l<i>.mix.left.q.norm
            tensors[name] = (1.0 + 0.3 * torch.randn(t.shape, generator=g)).to(t.dtype)
    save_file(tensors, path)
    return out_dir


def read_folder(model_dir: str):
    """config dict and tensors (float64), through the safetensors library (not the framework's reader)."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    tensors = load_file(os.path.join(model_dir, "model.safetensors"))
    return cfg, {k: v.to(torch.float64) for k, v in tensors.items()}


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
