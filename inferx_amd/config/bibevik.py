"""Typed configuration of the Bibevik design: a decoder whose config.json lists its layers one by one, each with
one norm (a single number as its weight) whose result both a mixer and a feed-forward read,

    {"architecture": "Bibevik", "vocab": V, "width": W, "norm": {"eps": e}, "embedding": {"scale": s},
     "layers": [{"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale",
                                                       "rot": {"dims", "base"}}, "mlp": ...},
                {"type": "general_delta", "mixer": {"heads", "dim"}, "mlp": ...},
                {"type": "lightning", "mixer": {"heads", "dim", "vdim", "decay": [one per head]}, "mlp": ...},
                {"type": ..., "mixer": ..., "mlp": ..., "weights_of": j}]}      layer j's tensors, a cache of its own
     mlp: {"kind": "dense", "ff": F, "limit": L} | null |
          {"kind": "moe", "expert": {"ff", "limit"}, "shared": {"ff", "limit"} (optional),
           "router": {"experts", "top", "scale", "groups": {"count", "keep"}}}

Every size and constant is read from there, layer by layer; the width of the decay's inner product is the shape of
its tensor.  What the design fixes: the parallel layer; in latent attention a normalised latent and a rotated key
part shared by the heads, rotation of neighbouring pairs, causal softmax; in the delta mixer the decay
exp(-e^(-1/2) sigmoid(.)), unit keys with 1e-6 under the root, a norm per head and a sigmoid gate; in lightning
attention silu on q, k, v, one norm over all heads and a sigmoid gate; feed-forwards of the clamped form
g sigmoid(1.702 g) (u + 1) (dense ones with biases); a router of sigmoid scores whose groups are scored by their two
best experts, weights not renormalised.  Tensor names: `embed`, `head`, `final.norm`, and per layer `l<i>.` + `norm1`,
`mix.{q,dkv,dkv.norm,uk,uv,o}` | `mix.{r,k,v,g,a,a.b,w1,w2,w0,norm,o}` | `mix.{q,k,v,g,norm,o}`,
`mlp.{gate,up,down}[.b]` | `mlp.router`, `mlp.e<j>.{gate,up,down}`, `mlp.shared.{gate,up,down}`.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .pelalix import _number
from .registry import ConfigError, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, token_embedding

ARCHITECTURE = "Bibevik"
MIXER_TYPES = ("latent_attention", "general_delta", "lightning")
MLP_KINDS = ("dense", "moe")


@dataclass
class BibevikMixer:
    heads: int
    dim: int
    # latent attention
    rot_dim: int = 0
    vdim: int = 0
    kv_rank: int = 0
    scale: Optional[float] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    # lightning attention
    decay: List[float] = field(default_factory=list)
    # the delta mixer: width of the decay's inner product (from the checkpoint's shapes; 0: not known yet)
    decay_rank: int = 0


@dataclass
class BibevikMlp:
    kind: str
    ff: int
    limit: float
    experts: int = 0
    top: int = 0
    scale: float = 1.0
    groups: int = 1
    groups_keep: int = 1
    shared_ff: int = 0
    shared_limit: float = 0.0


@dataclass
class BibevikLayer:
    type: str
    mixer: BibevikMixer
    mlp: Optional[BibevikMlp] = None
    weights_of: Optional[int] = None


def _mixer(kind: str, m: Any, where: str) -> BibevikMixer:
    mixer = BibevikMixer(heads=_number(m, "heads", where, int), dim=_number(m, "dim", where, int))
    if kind == "latent_attention":
        mixer.rot_dim = _number(m, "rot_dim", where, int)
        mixer.vdim = _number(m, "vdim", where, int)
        mixer.kv_rank = _number(m, "kv_rank", where, int)
        mixer.scale = _number(m, "scale", where, float)
        rot = m.get("rot")
        if rot is not None:
            mixer.rot_dims = _number(rot, "dims", where + ".rot", int)
            mixer.rot_base = _number(rot, "base", where + ".rot", float)
    elif kind == "lightning":
        mixer.vdim = _number(m, "vdim", where, int, mixer.dim, required=False)
        decay = m.get("decay")
        if not isinstance(decay, list) or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"config.json: {where}.decay must be a list of numbers, one per head")
        mixer.decay = [float(d) for d in decay]
    elif kind == "general_delta":
        mixer.decay_rank = _number(m, "decay_rank", where, int, 0, required=False)
    return mixer


def _mlp(raw: Any, where: str) -> Optional[BibevikMlp]:
    if raw is None:
        return None
    kind = _number(raw, "kind", where, str)
    if kind not in MLP_KINDS:
        raise ConfigError(f"config.json: {where}.kind {kind!r} is not known (known: " + ", ".join(MLP_KINDS) + ")")
    if kind == "dense":
        return BibevikMlp(kind, ff=_number(raw, "ff", where, int), limit=_number(raw, "limit", where, float))
    router, expert = raw.get("router"), raw.get("expert")
    mlp = BibevikMlp(kind, ff=_number(expert, "ff", where + ".expert", int),
                     limit=_number(expert, "limit", where + ".expert", float),
                     experts=_number(router, "experts", where + ".router", int),
                     top=_number(router, "top", where + ".router", int),
                     scale=_number(router, "scale", where + ".router", float, 1.0, required=False))
    groups = router.get("groups")
    if groups is not None:
        mlp.groups = _number(groups, "count", where + ".router.groups", int)
        mlp.groups_keep = _number(groups, "keep", where + ".router.groups", int)
    shared = raw.get("shared")
    if shared is not None:
        mlp.shared_ff = _number(shared, "ff", where + ".shared", int)
        mlp.shared_limit = _number(shared, "limit", where + ".shared", float)
    return mlp


@dataclass
class BibevikConfig:
    vocab: int
    width: int
    layers: List[BibevikLayer]
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    eos_token_ids: List[int] = field(default_factory=list)
    initializer_range: float = 0.02

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "BibevikConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, lr in enumerate(layers_raw):
            where = f"layers[{i}]"
            kind = _number(lr, "type", where, str)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type {kind!r} is not a mixer of this design (known: "
                                  + ", ".join(MIXER_TYPES) + ")")
            layers.append(BibevikLayer(kind, _mixer(kind, lr.get("mixer"), where + ".mixer"),
                                       _mlp(lr.get("mlp"), where + ".mlp"),
                                       _number(lr, "weights_of", where, int, None, required=False)))
        eos = raw.get("eos_token_id")
        eos = [] if eos is None else (eos if isinstance(eos, list) else [eos])
        if any(isinstance(x, bool) or not isinstance(x, int) for x in eos):
            raise ConfigError("config.json: eos_token_id must be an integer or a list of integers")
        top = "the configuration"
        return cls(vocab=_number(raw, "vocab", top, int), width=_number(raw, "width", top, int), layers=layers,
                   norm_eps=_number(raw.get("norm", {}), "eps", "norm", float, 1e-6, required=False),
                   embedding_scale=_number(raw.get("embedding", {}), "scale", "embedding", float, 1.0, required=False),
                   eos_token_ids=list(eos),
                   initializer_range=_number(raw, "initializer_range", top, float, 0.02, required=False))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            m = l.mixer
            mixer: Dict[str, Any] = {"heads": m.heads, "dim": m.dim}
            if l.type == "latent_attention":
                mixer.update({"rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale})
                if m.rot_dims:
                    mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base}
            elif l.type == "lightning":
                mixer.update({"vdim": m.vdim, "decay": list(m.decay)})
            elif m.decay_rank:
                mixer["decay_rank"] = m.decay_rank
            mlp = None
            if l.mlp is not None:
                f = l.mlp
                if f.kind == "dense":
                    mlp = {"kind": "dense", "ff": f.ff, "limit": f.limit}
                else:
                    mlp = {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit},
                           "router": {"experts": f.experts, "top": f.top, "scale": f.scale,
                                      "groups": {"count": f.groups, "keep": f.groups_keep}}}
                    if f.shared_ff:
                        mlp["shared"] = {"ff": f.shared_ff, "limit": f.shared_limit}
            entry = {"type": l.type, "mixer": mixer, "mlp": mlp}
            if l.weights_of is not None:
                entry["weights_of"] = l.weights_of
            layers.append(entry)
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "layers": layers,
             "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
             "initializer_range": self.initializer_range}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else self.eos_token_ids
        return d

    def validate(self) -> None:
        def need(ok, msg):
            if not ok:
                raise ConfigError("config.json: " + msg)

        need(self.vocab > 0 and self.width > 0, "vocab and width must be positive")
        need(self.norm_eps > 0, "norm.eps must be positive")
        need(self.initializer_range > 0, "initializer_range must be positive")
        need(all(0 <= t < self.vocab for t in self.eos_token_ids), "eos_token_id names a token outside the vocabulary")
        for i, l in enumerate(self.layers):
            m, w = l.mixer, f"layers[{i}].mixer"
            need(l.type in MIXER_TYPES, f"layers[{i}].type {l.type!r} is not a mixer of this design")
            need(m.heads > 0 and 0 < m.dim <= 256, f"{w}: heads and dim (at most 256) must be positive")
            if l.type == "latent_attention":
                need(m.vdim > 0 and m.rot_dim >= 0 and 0 < m.kv_rank <= 1024 and m.kv_rank + m.rot_dim <= 1088,
                     f"{w}: vdim, kv_rank (at most 1024, with rot_dim at most 1088) must be positive")
                need(m.scale is not None and m.scale > 0, f"{w}.scale must be positive")
                need(m.rot_dims >= 0 and m.rot_dims % 2 == 0 and m.rot_dims <= m.rot_dim,
                     f"{w}.rot.dims must be even and at most rot_dim")
                need(m.rot_dims == 0 or m.rot_base > 0, f"{w}.rot.base must be positive")
            elif l.type == "lightning":
                need(m.vdim > 0, f"{w}.vdim must be positive")
                need(len(m.decay) == m.heads and all(0 < d <= 1 for d in m.decay),
                     f"{w}.decay must hold one number in (0, 1] per head")
            if l.weights_of is not None:
                j = l.weights_of
                need(0 <= j < len(self.layers) and j != i and self.layers[j].weights_of is None,
                     f"layers[{i}].weights_of must name another layer that has tensors of its own")
                other = self.layers[j]
                need(other.type == l.type and _same_sizes(other, l),
                     f"layers[{i}] uses the tensors of layer {j} and must be of its type and sizes")
            if l.mlp is not None:
                f, w = l.mlp, f"layers[{i}].mlp"
                need(f.kind in MLP_KINDS, f"{w}.kind {f.kind!r} is not known (known: " + ", ".join(MLP_KINDS) + ")")
                need(f.ff > 0 and f.limit > 0, f"{w}: ff and limit must be positive")
                if f.kind == "moe":
                    need(f.experts > 0, f"{w}.router.experts must be positive")
                    need(1 <= f.groups <= 64 and f.experts % f.groups == 0,
                         f"{w}.router.groups.count must divide the experts (at most 64 groups)")
                    need(1 <= f.groups_keep <= f.groups, f"{w}.router.groups.keep must be between 1 and groups.count")
                    need(1 <= f.top <= f.groups_keep * (f.experts // f.groups),
                         f"{w}.router.top must be at least 1 and fit into the kept groups")
                    need(f.shared_ff >= 0 and (f.shared_ff == 0 or f.shared_limit > 0),
                         f"{w}.shared: ff and limit must be positive")

    def resolve_shapes(self, shapes: Dict[str, Any]) -> None:
        """Sizes that config.json leaves to the tensors' shapes: the width of the decay's inner product of every
        delta layer (`shapes`: checkpoint name -> shape)."""
        for i, l in enumerate(self.layers):
            if l.type == "general_delta" and l.weights_of is None:
                shape = shapes.get(f"l{i}.mix.w1")
                if shape is not None:
                    l.mixer.decay_rank = int(shape[0])
        for l in self.layers:
            if l.type == "general_delta" and l.weights_of is not None:
                l.mixer.decay_rank = self.layers[l.weights_of].mixer.decay_rank

    def model_spec(self) -> ModelSpec:
        W, std, eps = self.width, self.initializer_range, self.norm_eps
        norm = lambda name: PartSpec("rmsnorm", {"width": W, "eps": eps, "scalar": True}, rename={"weight": name})
        layers, index_of, schedule = [], {}, []
        for i, l in enumerate(self.layers):
            if l.weights_of is not None:
                continue
            p, m = f"l{i}.", l.mixer
            plain = lambda names: {f"{n}.weight": n for n in names}
            if l.type == "latent_attention":
                position = PartSpec("rope", {"theta": m.rot_base, "rotary_dim": m.rot_dims}) if m.rot_dims else None
                mixer = PartSpec("latent_attention",
                                 {"hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
                                  "value_dim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "norm_eps": eps,
                                  "position": position, "init_std": std}, prefix=p + "mix.",
                                 rename={**plain(("q", "dkv", "uk", "uv", "o")), "dkv_norm.weight": "dkv.norm"})
            elif l.type == "general_delta":
                mixer = PartSpec("generalized_delta",
                                 {"hidden_size": W, "num_heads": m.heads, "head_dim": m.dim,
                                  "decay_rank": m.decay_rank or max(1, min(64, W // 16)), "norm_eps": eps,
                                  "init_std": std}, prefix=p + "mix.",
                                 rename={**plain(("r", "k", "v", "g", "a", "w1", "w2", "o")), "a.bias": "a.b",
                                         "norm.weight": "norm"})
            else:
                mixer = PartSpec("lightning_attention",
                                 {"hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
                                  "decay": list(m.decay), "norm_eps": eps, "init_std": std}, prefix=p + "mix.",
                                 rename={**plain(("q", "k", "v", "g", "o")), "norm.weight": "norm"})
            parts = {"norm": norm(p + "norm1"), "mixer": mixer}
            f = l.mlp
            if f is not None and f.kind == "dense":
                parts["feed_forward"] = PartSpec(
                    "dense_mlp", {"hidden_size": W, "width": f.ff, "bias": True, "limit": f.limit, "init_std": std},
                    prefix=p + "mlp.", rename={f"{n}_proj.weight": n for n in ("gate", "up", "down")}
                    | {f"{n}_proj.bias": n + ".b" for n in ("gate", "up", "down")})
            elif f is not None:
                rename = {"gate.weight": "router"}
                for e in range(f.experts):
                    rename.update({f"experts.{e}.{n}_proj.weight": f"e{e}.{n}" for n in ("gate", "up", "down")})
                rename.update({f"shared_expert.{n}_proj.weight": f"shared.{n}" for n in ("gate", "up", "down")})
                parts["feed_forward"] = PartSpec(
                    "moe", {"hidden_size": W, "num_experts": f.experts, "top_k": f.top, "expert_width": f.ff,
                            "shared_width": f.shared_ff, "shared_gated": False, "renormalize": False,
                            "routed_scale": f.scale, "activation": "clamped_glu", "limit": f.limit,
                            "shared_limit": f.shared_limit if f.shared_ff else None, "groups": f.groups,
                            "groups_keep": f.groups_keep, "score": "sigmoid", "group_score": "top2",
                            "init_std": std}, prefix=p + "mlp.", rename=rename)
            index_of[i] = len(layers)
            layers.append(LayerSpec("parallel", parts))
        for i, l in enumerate(self.layers):
            schedule.append(ScheduleEntry(index_of[i if l.weights_of is None else l.weights_of]))
        spec = ModelSpec(
            architecture=ARCHITECTURE, hidden_size=W, vocab_size=self.vocab, max_positions=0, layers=layers,
            schedule=schedule, embedding=token_embedding("embed", self.vocab, W, std, scale=self.embedding_scale),
            final_norm=norm("final.norm"), head=linear_head("head", self.vocab, W, std), init_std=std)
        spec.validate()
        return spec


def _same_sizes(a: BibevikLayer, b: BibevikLayer) -> bool:
    """Whether two layers agree in everything that shapes their tensors (the delta mixer's inner width aside, which
    only the owner's tensors give)."""
    ma, mb = copy.copy(a.mixer), copy.copy(b.mixer)
    ma.decay_rank = mb.decay_rank = 0
    return ma == mb and a.mlp == b.mlp


register_architecture(ARCHITECTURE, BibevikConfig)
