"""Host-side checks of the Gosuvik design: its configuration and tensor names, the order its layers run in, what its
parts keep between steps, and the plain implementation's own mechanisms on cases worked out by hand."""
import copy
import math

import pytest
import torch

import plain_gosuvik as pg
import tiny_gosuvik as tg

F = torch.float64


def test_configuration_is_read_layer_by_layer():
    from inferx_amd.config import ConfigError, config_from_dict
    cfg = config_from_dict(copy.deepcopy(tg.A))
    assert cfg.architecture == "Gosuvik" and (cfg.vocab, cfg.width, cfg.norm_eps, cfg.norm_groups) == (320, 96, 1e-5, 2)
    assert [l.type for l in cfg.layers] == ["latent_attention", "channel_delta", "parallel"]
    assert (cfg.loop_start, cfg.loop_stop, cfg.loop_times) == (0, 2, 2) and cfg.layer_order() == [0, 1, 0, 1, 2]
    m = cfg.layers[0].mixer
    assert (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"], m["window"]) == (3, 16, 8, 24, 40, 0.2, 20)
    assert m["rot"] == {"theta": 10000.0, "rotary_dim": 6, "scaling": {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0}}
    m = cfg.layers[1].mixer
    assert (m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]) == (4, 2, 16, 12, 3)
    m = cfg.layers[2].mixer
    assert m["left"]["rot"]["scaling"] == {"factor": 2.0} and m["left"]["window"] == 9 and m["left"]["kv_heads"] == 2
    assert m["right"] == {"heads": 2, "dim": 12, "vdim": 20, "gate_cap": 8.0} and (m["left_scale"], m["right_scale"]) == (0.7, 1.2)
    assert cfg.layers[0].mlp == {"kind": "dense", "ff": 64} and cfg.layers[1].mlp == {"kind": "moe", "ff": 32, "experts": 6, "top": 2}
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    assert config_from_dict(copy.deepcopy(tg.B)).layer_order() == [0, 1, 2]                 # no loop
    assert config_from_dict(copy.deepcopy(tg.C)).layer_order() == [0, 1, 2, 1, 2, 1, 2]
    assert config_from_dict(copy.deepcopy(tg.D)).layer_order() == [0, 1, 1, 2, 3, 4]
    for breaker, text in [
        (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
        (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
        (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
        (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "at most 8"),
        (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
        (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple of kv_heads"),
        (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "between 1 and router.experts"),
        (lambda c: c["layers"][2]["mixer"].pop("right"), "'left' and 'right'"),
        (lambda c: c["layers"][2]["mixer"]["right"].update(gate_cap=0.0), "gate_cap"),
        (lambda c: c["layers"][0]["mlp"].update(kind="relu"), "not known"),
        (lambda c: c["norm"].update(groups=5), "divide the width"),
        (lambda c: c["loop"].update(stop=4), "within the layers"),
        (lambda c: c["loop"].update(times=0), "at least 1"),
    ]:
        raw = copy.deepcopy(tg.A)
        breaker(raw)
        with pytest.raises(ConfigError) as err:
            config_from_dict(raw)
        assert text in str(err.value), str(err.value)


def test_tensor_names_and_what_keeps_what():
    from inferx_amd.config import config_from_dict
    from inferx_amd.parts import build_model
    cfg = config_from_dict(copy.deepcopy(tg.A))
    cfg.resolve_shapes({"l1.mix.a1": (5, 96), "l1.mix.g1": (7, 96)})  # the inner widths come from the tensors
    model = build_model(cfg.model_spec())
    names = model.expected_tensors()
    shape = lambda n: tuple(names[n].shape)
    assert shape("l0.norm1") == (96,) and shape("final.norm") == (96,) and shape("head") == (320, 96)
    assert shape("l0.mix.q") == (3 * 24, 96) and shape("l0.mix.dkv") == (48, 96) and shape("l0.mix.dkv.norm") == (40,)
    assert shape("l0.mix.uk") == (48, 40) and shape("l0.mix.uv") == (72, 40) and shape("l0.mix.g") == (72, 96)
    assert shape("l0.mlp.up") == (64, 96) and shape("l0.mlp.down") == (96, 64) and shape("l0.mlp.act") == (4,)
    assert shape("l1.mix.q") == (32, 96) and shape("l1.mix.v") == (48, 96) and shape("l1.mix.q.conv") == (32, 3)
    assert shape("l1.mix.v.conv") == (48, 3) and shape("l1.mix.b") == (4, 96) and shape("l1.mix.A_log") == (4,)
    assert shape("l1.mix.a1") == (5, 96) and shape("l1.mix.a2") == (64, 5) and shape("l1.mix.dt_bias") == (64,)
    assert shape("l1.mix.g1") == (7, 96) and shape("l1.mix.g2") == (48, 7) and shape("l1.mix.norm") == (12,)
    assert shape("l1.mlp.router") == (6, 96) and shape("l1.mlp.e5.gate") == (32, 96) and shape("l1.mlp.e0.down") == (96, 32)
    assert shape("l2.mix.left.q") == (64, 96) and shape("l2.mix.left.k") == (32, 96) and shape("l2.mix.left.v") == (48, 96)
    assert shape("l2.mix.left.q.norm") == (16,) and shape("l2.mix.left.sink") == (4,) and shape("l2.mix.left.o") == (96, 96)
    assert shape("l2.mix.right.q") == (24, 96) and shape("l2.mix.right.v") == (40, 96) and shape("l2.mix.right.i") == (2, 96)
    assert shape("l2.mix.right.f.b") == (2,) and shape("l2.mix.right.norm") == (40,) and shape("l2.mix.right.o") == (96, 40)
    # five layer runs; each keeps pages or state of its own
    plan = model.cache_plan()
    assert len(plan) == 5 and all(cache_from is None for _, cache_from in plan)
    need, state = plan[0][0]["mixer"]
    assert state is None and need.window == 20 and [(a.name, a.heads, a.width) for a in need.arrays] == [("latent", 1, 48)]
    need, state = plan[1][0]["mixer"]
    assert need is None and state.shape == (4 * 16 * 12 + 2 * (32 + 32 + 48),)
    need, state = plan[4][0]["mixer"]
    assert need.window == 9 and [(a.name, a.heads, a.width, a.transposed) for a in need.arrays] == [("k", 2, 16, False), ("v", 2, 24, True)]
    need, state = plan[4][0]["second_mixer"]
    assert need is None and state.shape == (2 * 12 * (20 + 1) + 2,)  # n is one more column; then the maxima
    assert model.graph_safe()


def test_stretched_frequencies_worked_out_by_hand():
    from inferx_amd.parts.rope import Rotary
    # eight numbers, base 16: f = 1, 1/2, 1/4, 1/8.  original 16, fast 8, slow 1: at(t) = 8 ln(16 / (2 pi t)) / (2 ln 16)
    at = lambda t: 8 * math.log(16 / (2 * math.pi * t)) / (2 * math.log(16))
    lo, hi = max(math.floor(at(8.0)), 0), min(math.ceil(at(1.0)), 7)
    assert (lo, hi) == (0, 2)
    ramp = [min(max((i - lo) / (hi - lo), 0.0), 1.0) for i in range(4)]
    want = [f / 4.0 * r + f * (1 - r) for f, r in zip([1, 0.5, 0.25, 0.125], ramp)]
    rot = {"dims": 8, "base": 16.0, "scaling": {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0}}
    f, gain = pg.frequencies(rot)
    assert torch.allclose(f, torch.tensor(want, dtype=F)) and gain == pytest.approx(0.1 * math.log(4.0) + 1.0)
    part = Rotary(16.0, 8, scaling=rot["scaling"])
    assert torch.allclose(part.frequencies().double(), f, rtol=1e-6) and part.gain == pytest.approx(gain)
    f, gain = pg.frequencies({"dims": 8, "base": 16.0, "scaling": {"factor": 2.0}})
    assert torch.allclose(f, torch.tensor([0.5, 0.25, 0.125, 0.0625], dtype=F)) and gain == 1.0
    assert torch.allclose(Rotary(16.0, 8, scaling={"factor": 2.0}).frequencies().double(), f)
    # halves are paired: a quarter turn of pair (0, 2) of four numbers
    x = torch.tensor([[1.0, 5.0, 0.0, 7.0]], dtype=F)
    y = pg.rotate_halves(x, torch.tensor([[math.pi / 2, 0.0]], dtype=F))
    assert torch.allclose(y, torch.tensor([[0.0, 5.0, 1.0, 7.0]], dtype=F), atol=1e-12)


def test_plain_mechanisms_on_cases_worked_out_by_hand():
    # the norm in groups: each run over its own root mean square
    x = torch.tensor([[3.0, 4.0, 0.0, 2.0]], dtype=F)
    y = pg.group_norm(x, torch.tensor([1.0, 1.0, 2.0, 2.0], dtype=F), 0.0, 2)
    assert torch.allclose(y, torch.tensor([[3 / math.sqrt(12.5), 4 / math.sqrt(12.5), 0.0, 2 * 2 / math.sqrt(2.0)]], dtype=F))
    # a window of 2: a token sees itself and the one before
    assert pg.visible(torch.arange(4), 2).tolist() == [[True, False, False, False], [True, True, False, False],
                                                      [False, True, True, False], [False, False, True, True]]
    # the short convolution: the last column is the present token's
    u = torch.tensor([[1.0], [2.0], [3.0]], dtype=F)
    assert pg.short_conv(u, torch.tensor([[10.0, 1.0]], dtype=F)).flatten().tolist() == [1.0, 12.0, 23.0]
    # PolyNorm of a row of equal numbers z: N(z) = N(z^2) = N(z^3) = 1 (eps 0), so the blend is a + b + c + e
    w = {"up": torch.eye(3, dtype=F), "down": torch.eye(3, dtype=F), "act": torch.tensor([0.5, 0.25, 2.0, -1.0], dtype=F)}
    assert torch.allclose(pg.polynorm_mlp(torch.full((1, 3), 2.0, dtype=F), w, 0.0), torch.full((1, 3), 1.75, dtype=F))
    # the router: softmax over all experts, the chosen weights divided by their sum
    idx, weight = pg.route(torch.tensor([[1.0, 0.0]], dtype=F), {"router": torch.tensor([[0.0, 0.0], [1.0, 0.0], [2.0, 0.0]], dtype=F)},
                           {"router": {"top": 2}})
    e1, e2 = math.exp(1.0), math.exp(2.0)
    assert idx.tolist() == [[2, 1]] and torch.allclose(weight, torch.tensor([[e2 / (e1 + e2), e1 / (e1 + e2)]], dtype=F))


def test_sink_and_memory_by_hand():
    # one token, one head: the softmax over its own key and the sink.  q = k = (1, 0) after the norm (weights 1, eps 0
    # would divide by rms = sqrt(1/2): q = k = (sqrt 2, 0)), score = 2 * scale; values pass (position 0 turns nothing)
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 0.5}
    eye = torch.eye(2, dtype=F)
    w = {"q": eye, "k": eye, "v": eye, "o": eye, "q.norm": torch.ones(2, dtype=F), "k.norm": torch.ones(2, dtype=F),
         "sink": torch.tensor([0.3], dtype=F)}
    y = pg.sink_attention(torch.tensor([[1.0, 0.0]], dtype=F), w, m, 0.0, torch.arange(1))
    p = math.exp(1.0) / (math.exp(1.0) + math.exp(0.3))
    assert torch.allclose(y, torch.tensor([[p, 0.0]], dtype=F))
    # the memory's first token: m' = max(f + 0, i); with i > f the write is k v^T whole and
    # o = (q . k) v / (max(|q . k|, exp(-i)) + 1e-6)
    m = {"heads": 1, "dim": 2, "vdim": 2, "gate_cap": 100.0}
    w = {"q": eye, "k": eye, "v": eye, "g": torch.zeros(2, 2, dtype=F), "o": eye, "norm": torch.ones(2, dtype=F),
         "i": torch.zeros(1, 2, dtype=F), "i.b": torch.tensor([1.0], dtype=F), "f": torch.zeros(1, 2, dtype=F),
         "f.b": torch.tensor([0.0], dtype=F)}
    x = torch.tensor([[3.0, 4.0]], dtype=F)
    gi = 100.0 * math.tanh(0.01)
    qk = 25.0 / math.sqrt(2.0)
    o = qk * x / (max(qk, math.exp(-gi)) + 1e-6)
    want = o / torch.sqrt((o * o).mean()) * 0.5                       # the head's norm, then sigmoid(0) = 1/2
    assert torch.allclose(pg.matrix_memory(x, w, m, 0.0), want)
