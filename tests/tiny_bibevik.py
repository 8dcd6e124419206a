"""Tiny Bibevik configurations that differ from each other in every size and option, and a folder of random weights
for each (norm weights and biases drawn at random too, so that one taken for another, or left out, shows)."""
import json
import os

import torch


def latent(heads, dim, rot_dim, vdim, rank, scale, rot, mlp, **more):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if rot is not None:
        mixer["rot"] = {"dims": rot[0], "base": rot[1]}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp, **more}


def delta(heads, dim, decay_rank, mlp, **more):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim, "decay_rank": decay_rank}, "mlp": mlp, **more}


def lightning(heads, dim, vdim, decay, mlp, **more):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}, "mlp": mlp, **more}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def experts(ff, limit, n, top, scale, groups=None, shared=None):
    router = {"experts": n, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}
    if shared is not None:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


def again(layer, j):
    """The same layer once more, with layer j's tensors."""
    return {**json.loads(json.dumps(layer)), "weights_of": j}


def config(vocab, width, eps, embed_scale, layers):
    return {"architecture": "Bibevik", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": embed_scale}, "layers": layers, "initializer_range": 0.08}


# A: all three mixers, two layers that run twice, three groups of which two are kept, a shared expert with a limit of
# its own, a rotation of fewer dimensions than the rotated part holds
_a0 = latent(3, 16, 8, 24, 40, 0.2, (6, 10000.0), dense(64, 1.5))
_a1 = lightning(2, 16, 24, [0.9, 0.6], experts(32, 1.0, 6, 2, 1.5, (3, 2), (48, 2.0)))
A = config(320, 96, 1e-5, 4.0, [_a0, _a1, again(_a0, 0), delta(3, 16, 5, experts(32, 0.8, 6, 2, 2.5, (2, 1))), again(_a1, 1)])
# B: sizes that are no multiple of 4 or 16; a layer without feed-forward; one expert per token; no groups; no shared
# expert; one head; a delta layer that runs twice; values wider than keys
_b1 = delta(1, 20, 3, dense(36, 0.7))
B = config(131, 72, 1e-6, 1.0, [
    latent(2, 12, 10, 20, 36, 0.3, (10, 100.0), None),
    _b1,
    lightning(3, 12, 20, [0.99, 0.5, 0.97], experts(36, 1.2, 5, 1, 1.0)),
    again(_b1, 1),
])
# C: one head everywhere, no rotation at all in one layer, every group kept, a decay of exactly one, all experts chosen
C = config(97, 40, 1e-5, 2.0, [
    latent(1, 16, 4, 16, 16, 0.25, None, experts(24, 1.0, 2, 2, 1.0, (2, 2), (8, 1.0))),
    lightning(1, 16, 16, [1.0], dense(24, 2.0)),
    latent(1, 8, 16, 8, 24, 0.5, (16, 500.0), dense(40, 1.0)),
    delta(1, 16, 2, None),
])
# D: wider heads (the state's rows spread over more registers), sixteen query heads on one latent, many experts in
# groups of two (a group's two best are all it has)
D = config(256, 128, 1e-5, 8.0, [
    delta(2, 128, 8, experts(32, 1.0, 16, 4, 2.0, (8, 3), (32, 1.5))),
    latent(16, 32, 16, 32, 64, 0.15, (16, 1000.0), dense(96, 1.0)),
    lightning(2, 128, 80, [0.95, 0.999], experts(32, 1.0, 16, 4, 0.5, (4, 2))),
])
# E: recurrent layers only (nothing is kept in pages), a width and a vocabulary that are no multiple of 8, groups of one
# expert, the embedding's scale left to its default
E = config(77, 90, 1e-5, 1.0, [
    lightning(3, 10, 14, [0.8, 0.9, 0.7], experts(28, 1.0, 6, 2, 1.0, (6, 3))),
    delta(2, 24, 4, experts(28, 1.0, 3, 1, 3.0, (1, 1))),
])
del E["embedding"]
# F: sizes that the matrix-core attention and the chunked recurrence take (latents and rotated parts in multiples of
# 16 and 32, heads of 32 and 64 numbers), two latent layers of different classes of size, one of them run twice
_f0 = latent(4, 16, 32, 24, 32, 0.2, (32, 10000.0), dense(48, 1.0))
F = config(200, 64, 1e-6, 3.0, [
    _f0,
    delta(2, 32, 4, experts(24, 1.0, 4, 2, 1.5, (2, 1), (16, 1.0))),
    latent(2, 24, 64, 16, 128, 0.12, (48, 300.0), None),
    lightning(2, 64, 32, [0.9, 0.99], dense(40, 1.5)),
    again(_f0, 0),
])
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E, "F": F}


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
        if last.startswith("norm"):  # l<i>.norm1, final.norm (one number each), l<i>.mix.norm, l<i>.mix.dkv.norm
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
