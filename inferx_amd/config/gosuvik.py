"""Typed configuration of the Gosuvik design: a pre-norm decoder whose config.json lists its layers one by one and may
run a stretch of them several times in a row,

    {"architecture": "Gosuvik", "vocab": V, "width": W, "norm": {"eps": e, "groups": g},
     "loop": {"start": a, "stop": b, "times": n},            layers a .. b-1 run n times, a cache or state per pass
     "layers": [{"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale",
                                                       "mask": {"size"}, "rot": ROT}, "mlp": MLP},
                {"type": "channel_delta", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"}, "mlp": MLP},
                {"type": "parallel", "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot": ROT},
                                               "right": {"heads", "dim", "vdim", "gate_cap"},
                                               "left_scale", "right_scale"}, "mlp": MLP}]}
     ROT: {"dims", "base", "scaling": {"factor"} | {"factor", "original", "fast", "slow"}}
     MLP: null | {"kind": "dense", "ff": F} | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}

Every size and constant is read from there, layer by layer; the inner widths of the delta mixer's decay and gate are
the shapes of their tensors.  What the design fixes: RMS norms over `groups` runs of the width before each branch;
in latent attention a normalised latent, a rotated key part shared by the heads, rotation of halves with stretched
frequencies, a window, a sigmoid gate on the heads' results; in the delta mixer short convolutions with silu, unit
queries and keys, a decay per key channel, a norm per head and a sigmoid gate; the pair of a windowed attention with
normed queries and keys, rotated values and a sink beside a matrix memory with capped gates; dense feed-forwards with
the PolyNorm activation; experts with silu gates chosen by a softmax router whose weights are renormalised.  Tensor
names: `embed`, `head`, `final.norm`, and per layer `l<i>.` + `norm1`, `norm2`, `mix.*`, `mlp.*`.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .pelalix import _number
from .registry import ConfigError, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, token_embedding

ARCHITECTURE = "Gosuvik"
MIXER_TYPES = ("latent_attention", "channel_delta", "parallel")
MLP_KINDS = ("dense", "moe")


def _rot(raw: Any, where: str) -> Optional[Dict[str, Any]]:
    """A rotation as the position encoding's parameters: theta, rotary_dim and how its frequencies are stretched."""
    if raw is None:
        return None
    out: Dict[str, Any] = {"theta": _number(raw, "base", where, float), "rotary_dim": _number(raw, "dims", where, int)}
    sc = raw.get("scaling")
    if sc is not None:
        w = where + ".scaling"
        scaling = {"factor": _number(sc, "factor", w, float)}
        if any(k in sc for k in ("original", "fast", "slow")):
            scaling.update(original=_number(sc, "original", w, float), fast=_number(sc, "fast", w, float),
                           slow=_number(sc, "slow", w, float))
        out["scaling"] = scaling
    return out


def _window(m: Any, where: str) -> int:
    mask = m.get("mask") if isinstance(m, dict) else None
    return 0 if mask is None else _number(mask, "size", where + ".mask", int)


def _mixer(kind: str, m: Any, where: str) -> Dict[str, Any]:
    if not isinstance(m, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    n = lambda key, typ=int, at=m, w=where: _number(at, key, w, typ)
    if kind == "latent_attention":
        return {"heads": n("heads"), "dim": n("dim"), "rot_dim": n("rot_dim"), "vdim": n("vdim"),
                "kv_rank": n("kv_rank"), "scale": n("scale", float), "window": _window(m, where),
                "rot": _rot(m.get("rot"), where + ".rot")}
    if kind == "channel_delta":
        return {"heads": n("heads"), "kv_heads": _number(m, "kv_heads", where, int, m.get("heads"), required=False),
                "dim": n("dim"), "vdim": n("vdim"), "conv": n("conv"),
                "decay_rank": _number(m, "decay_rank", where, int, 0, required=False),
                "gate_rank": _number(m, "gate_rank", where, int, 0, required=False)}
    left, right = m.get("left"), m.get("right")
    lw, rw = where + ".left", where + ".right"
    if not isinstance(left, dict) or not isinstance(right, dict):
        raise ConfigError(f"config.json: {where} needs the objects 'left' and 'right'")
    return {"left": {"heads": n("heads", int, left, lw),
                     "kv_heads": _number(left, "kv_heads", lw, int, left.get("heads"), required=False),
                     "dim": n("dim", int, left, lw), "vdim": n("vdim", int, left, lw),
                     "scale": n("scale", float, left, lw), "window": _window(left, lw),
                     "rot": _rot(left.get("rot"), lw + ".rot")},
            "right": {"heads": n("heads", int, right, rw), "dim": n("dim", int, right, rw),
                      "vdim": n("vdim", int, right, rw), "gate_cap": n("gate_cap", float, right, rw)},
            "left_scale": n("left_scale", float), "right_scale": n("right_scale", float)}


def _mlp(raw: Any, where: str) -> Optional[Dict[str, Any]]:
    if raw is None:
        return None
    kind = _number(raw, "kind", where, str)
    if kind not in MLP_KINDS:
        raise ConfigError(f"config.json: {where}.kind {kind!r} is not known (known: " + ", ".join(MLP_KINDS) + ")")
    if kind == "dense":
        return {"kind": kind, "ff": _number(raw, "ff", where, int)}
    return {"kind": kind, "ff": _number(raw.get("expert"), "ff", where + ".expert", int),
            "experts": _number(raw.get("router"), "experts", where + ".router", int),
            "top": _number(raw.get("router"), "top", where + ".router", int)}


@dataclass
class GosuvikLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]] = None


@dataclass
class GosuvikConfig:
    vocab: int
    width: int
    layers: List[GosuvikLayer]
    norm_eps: float = 1e-6
    norm_groups: int = 1
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    eos_token_ids: List[int] = field(default_factory=list)
    initializer_range: float = 0.02

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "GosuvikConfig":
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
            layers.append(GosuvikLayer(kind, _mixer(kind, lr.get("mixer"), where + ".mixer"),
                                       _mlp(lr.get("mlp"), where + ".mlp")))
        eos = raw.get("eos_token_id")
        eos = [] if eos is None else (eos if isinstance(eos, list) else [eos])
        if any(isinstance(x, bool) or not isinstance(x, int) for x in eos):
            raise ConfigError("config.json: eos_token_id must be an integer or a list of integers")
        top, norm, loop = "the configuration", raw.get("norm") or {}, raw.get("loop")
        cfg = cls(vocab=_number(raw, "vocab", top, int), width=_number(raw, "width", top, int), layers=layers,
                  norm_eps=_number(norm, "eps", "norm", float, 1e-6, required=False),
                  norm_groups=_number(norm, "groups", "norm", int, 1, required=False),
                  eos_token_ids=list(eos),
                  initializer_range=_number(raw, "initializer_range", top, float, 0.02, required=False))
        if loop is not None:
            cfg.loop_start, cfg.loop_stop = _number(loop, "start", "loop", int), _number(loop, "stop", "loop", int)
            cfg.loop_times = _number(loop, "times", "loop", int)
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        def rot(r):
            if r is None:
                return None
            out = {"dims": r["rotary_dim"], "base": r["theta"]}
            if "scaling" in r:
                out["scaling"] = dict(r["scaling"])
            return out

        def attention(m, keys):
            out = {k: m[k] for k in keys}
            if m["window"]:
                out["mask"] = {"size": m["window"]}
            if m["rot"] is not None:
                out["rot"] = rot(m["rot"])
            return out

        layers = []
        for l in self.layers:
            m = l.mixer
            if l.type == "latent_attention":
                mixer = attention(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"))
            elif l.type == "channel_delta":
                mixer = {k: m[k] for k in ("heads", "kv_heads", "dim", "vdim", "conv")}
                mixer.update({k: m[k] for k in ("decay_rank", "gate_rank") if m[k]})
            else:
                mixer = {"left": attention(m["left"], ("heads", "kv_heads", "dim", "vdim", "scale")),
                         "right": dict(m["right"]), "left_scale": m["left_scale"], "right_scale": m["right_scale"]}
            f = l.mlp
            mlp = None
            if f is not None:
                mlp = ({"kind": "dense", "ff": f["ff"]} if f["kind"] == "dense" else
                       {"kind": "moe", "expert": {"ff": f["ff"]}, "router": {"experts": f["experts"], "top": f["top"]}})
            layers.append({"type": l.type, "mixer": mixer, "mlp": mlp})
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "layers": layers,
             "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "initializer_range": self.initializer_range}
        if self.loop_times != 1 or self.loop_stop > self.loop_start:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else self.eos_token_ids
        return d

    def validate(self) -> None:
        def need(ok, msg):
            if not ok:
                raise ConfigError("config.json: " + msg)

        def rotation(r, within, w):
            if r is None:
                return
            need(r["theta"] > 0, f"{w}.rot.base must be positive")
            need(0 < r["rotary_dim"] <= within and r["rotary_dim"] % 2 == 0,
                 f"{w}.rot.dims must be even, positive and at most {within}")
            sc = r.get("scaling")
            if sc is not None:
                need(sc["factor"] > 0, f"{w}.rot.scaling.factor must be positive")
                if "original" in sc:
                    need(sc["original"] > 0 and sc["fast"] > 0 and sc["slow"] > 0 and r["theta"] != 1.0,
                         f"{w}.rot.scaling: original, fast and slow must be positive (and the base not 1)")

        need(self.vocab > 0 and self.width > 0, "vocab and width must be positive")
        need(self.norm_eps > 0, "norm.eps must be positive")
        need(self.norm_groups > 0 and self.width % self.norm_groups == 0, "norm.groups must divide the width")
        need(self.initializer_range > 0, "initializer_range must be positive")
        need(all(0 <= t < self.vocab for t in self.eos_token_ids), "eos_token_id names a token outside the vocabulary")
        need(0 <= self.loop_start <= self.loop_stop <= len(self.layers), "loop.start .. loop.stop must lie within the layers")
        need(self.loop_times >= 1, "loop.times must be at least 1")
        for i, l in enumerate(self.layers):
            m, w = l.mixer, f"layers[{i}].mixer"
            need(l.type in MIXER_TYPES, f"layers[{i}].type {l.type!r} is not a mixer of this design")
            if l.type == "latent_attention":
                need(min(m["heads"], m["dim"], m["vdim"], m["kv_rank"]) > 0 and m["rot_dim"] >= 0,
                     f"{w}: heads, dim, vdim and kv_rank must be positive")
                need(m["kv_rank"] <= 1024 and m["kv_rank"] + m["rot_dim"] <= 1088,
                     f"{w}: kv_rank at most 1024, with rot_dim at most 1088")
                need(m["scale"] > 0 and m["window"] >= 0, f"{w}: scale must be positive, mask.size not negative")
                rotation(m["rot"], m["rot_dim"], w)
            elif l.type == "channel_delta":
                need(min(m["heads"], m["kv_heads"], m["vdim"]) > 0 and 0 < m["dim"] <= 256,
                     f"{w}: heads, kv_heads, vdim and dim (at most 256) must be positive")
                need(m["heads"] % m["kv_heads"] == 0, f"{w}.heads must be a multiple of kv_heads")
                need(1 <= m["conv"] <= 64, f"{w}.conv must be between 1 and 64 taps")
            else:
                a, b = m["left"], m["right"]
                need(min(a["heads"], a["kv_heads"]) > 0 and 0 < a["dim"] <= 256 and 0 < a["vdim"] <= 256,
                     f"{w}.left: heads, kv_heads, dim and vdim (at most 256) must be positive")
                need(a["heads"] % a["kv_heads"] == 0, f"{w}.left.heads must be a multiple of kv_heads")
                need(a["scale"] > 0 and a["window"] >= 0, f"{w}.left: scale must be positive, mask.size not negative")
                need(a["rot"] is None or a["vdim"] % 2 == 0, f"{w}.left.vdim must be even where values are rotated")
                rotation(a["rot"], a["dim"], w + ".left")
                need(min(b["heads"], b["vdim"]) > 0 and 0 < b["dim"] <= 256 and b["gate_cap"] > 0,
                     f"{w}.right: heads, vdim, dim (at most 256) and gate_cap must be positive")
            f = l.mlp
            if f is not None:
                w = f"layers[{i}].mlp"
                need(f["kind"] in MLP_KINDS and f["ff"] > 0, f"{w}: a known kind and a positive ff")
                if f["kind"] == "moe":
                    need(1 <= f["top"] <= f["experts"], f"{w}.router.top must be between 1 and router.experts")

    def resolve_shapes(self, shapes: Dict[str, Any]) -> None:
        """Sizes that config.json leaves to the tensors' shapes: the inner widths of every delta layer's decay and
        gate (`shapes`: checkpoint name -> shape)."""
        for i, l in enumerate(self.layers):
            if l.type == "channel_delta":
                for key, name in (("decay_rank", "a1"), ("gate_rank", "g1")):
                    shape = shapes.get(f"l{i}.mix.{name}")
                    if shape is not None:
                        l.mixer[key] = int(shape[0])

    def layer_order(self) -> List[int]:
        """The layers in the order they run: those of the loop `times` times in a row."""
        n = len(self.layers)
        body = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + body * self.loop_times + list(range(self.loop_stop, n))

    def model_spec(self) -> ModelSpec:
        W, std, eps = self.width, self.initializer_range, self.norm_eps
        norm = lambda name: PartSpec("rmsnorm", {"width": W, "eps": eps, "groups": self.norm_groups},
                                     rename={"weight": name})
        plain = lambda names: {f"{n}.weight": n for n in names}
        position = lambda r: None if r is None else PartSpec("rope", dict(r))
        layers = []
        for i, l in enumerate(self.layers):
            p, m = f"l{i}.", l.mixer
            parts = {"mixer_norm": norm(p + "norm1")}
            if l.type == "latent_attention":
                parts["mixer"] = PartSpec(
                    "latent_attention",
                    {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
                     "value_dim": m["vdim"], "kv_rank": m["kv_rank"], "scale": m["scale"], "norm_eps": eps,
                     "position": position(m["rot"]), "pairing": "halves", "window": m["window"], "gate": True,
                     "init_std": std}, prefix=p + "mix.",
                    rename={**plain(("q", "dkv", "uk", "uv", "g", "o")), "dkv_norm.weight": "dkv.norm"})
            elif l.type == "channel_delta":
                rank = max(1, min(64, W // 16))
                parts["mixer"] = PartSpec(
                    "gated_delta",
                    {"hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
                     "value_dim": m["vdim"], "conv_taps": m["conv"], "norm_eps": eps, "init_std": std,
                     "decay_rank": m["decay_rank"] or rank, "gate_rank": m["gate_rank"] or rank,
                     "gate_activation": "sigmoid"}, prefix=p + "mix.",
                    rename={**plain(("q", "k", "v", "b", "o", "a1", "a2", "g1", "g2")), "norm.weight": "norm"})
            else:
                a, b = m["left"], m["right"]
                values = None if a["rot"] is None else PartSpec("rope", {"theta": a["rot"]["theta"], "rotary_dim": a["vdim"]})
                parts["mixer"] = PartSpec(
                    "attention",
                    {"hidden_size": W, "num_heads": a["heads"], "num_kv_heads": a["kv_heads"], "head_dim": a["dim"],
                     "value_dim": a["vdim"], "qkv_bias": False, "window": a["window"], "scale": a["scale"],
                     "position": position(a["rot"]), "value_position": values, "qk_norm": True, "qk_norm_eps": eps,
                     "sink": True, "init_std": std}, prefix=p + "mix.left.",
                    rename={f"{n}_proj.weight": n for n in "qkvo"} | {"q_norm.weight": "q.norm", "k_norm.weight": "k.norm"})
                parts["second_mixer"] = PartSpec(
                    "matrix_memory",
                    {"hidden_size": W, "num_heads": b["heads"], "head_dim": b["dim"], "value_dim": b["vdim"],
                     "gate_cap": b["gate_cap"], "norm_eps": eps, "init_std": std}, prefix=p + "mix.right.",
                    rename={**plain(("q", "k", "v", "g", "o", "i", "f")), "i.bias": "i.b", "f.bias": "f.b",
                            "norm.weight": "norm"})
                parts["mixer_gain"] = PartSpec("constant_gain", {"factor": m["left_scale"]})
                parts["second_mixer_gain"] = PartSpec("constant_gain", {"factor": m["right_scale"]})
            f = l.mlp
            if f is not None:
                parts["feed_forward_norm"] = norm(p + "norm2")
                if f["kind"] == "dense":
                    parts["feed_forward"] = PartSpec(
                        "polynorm_mlp", {"hidden_size": W, "width": f["ff"], "norm_eps": eps, "init_std": std},
                        prefix=p + "mlp.", rename={"up_proj.weight": "up", "down_proj.weight": "down"})
                else:
                    rename = {"gate.weight": "router"}
                    for e in range(f["experts"]):
                        rename.update({f"experts.{e}.{n}_proj.weight": f"e{e}.{n}" for n in ("gate", "up", "down")})
                    parts["feed_forward"] = PartSpec(
                        "moe", {"hidden_size": W, "num_experts": f["experts"], "top_k": f["top"],
                                "expert_width": f["ff"], "shared_width": 0, "renormalize": True, "init_std": std},
                        prefix=p + "mlp.", rename=rename)
            layers.append(LayerSpec("prenorm_branches", parts))
        spec = ModelSpec(
            architecture=ARCHITECTURE, hidden_size=W, vocab_size=self.vocab, max_positions=0, layers=layers,
            schedule=[ScheduleEntry(i) for i in self.layer_order()],
            embedding=token_embedding("embed", self.vocab, W, std), final_norm=norm("final.norm"),
            head=linear_head("head", self.vocab, W, std), init_std=std)
        spec.validate()
        return spec

    def copy(self) -> "GosuvikConfig":
        return copy.deepcopy(self)


register_architecture(ARCHITECTURE, GosuvikConfig)
