"""Host-side checks of the Bibevik design: its configuration and tensor names, what its parts keep between steps,
and the plain implementation's own mechanisms on cases worked out by hand."""
import copy
import math

import pytest
import torch

import plain_bibevik as pb
import tiny_bibevik as tb


def test_configuration_is_read_layer_by_layer():
    from inferx_amd.config import ConfigError, config_from_dict
    cfg = config_from_dict(copy.deepcopy(tb.A))
    assert cfg.architecture == "Bibevik" and cfg.vocab == 320 and cfg.width == 96 and cfg.embedding_scale == 4.0
    assert [l.type for l in cfg.layers] == ["latent_attention", "lightning", "latent_attention", "general_delta", "lightning"]
    assert [l.weights_of for l in cfg.layers] == [None, None, 0, None, 1]
    m = cfg.layers[0].mixer
    assert (m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, m.rot_dims, m.rot_base) == (3, 16, 8, 24, 40, 0.2, 6, 10000.0)
    assert cfg.layers[1].mixer.decay == [0.9, 0.6] and cfg.layers[1].mixer.vdim == 24
    f = cfg.layers[1].mlp
    assert (f.kind, f.ff, f.limit, f.experts, f.top, f.scale, f.groups, f.groups_keep, f.shared_ff, f.shared_limit) == \
        ("moe", 32, 1.0, 6, 2, 1.5, 3, 2, 48, 2.0)
    assert (cfg.layers[0].mlp.kind, cfg.layers[0].mlp.ff, cfg.layers[0].mlp.limit) == ("dense", 64, 1.5)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    assert config_from_dict(copy.deepcopy(tb.E)).embedding_scale == 1.0  # left out: the default
    for breaker, text in [
        (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
        (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
        (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
        (lambda c: c["layers"][1]["mixer"].update(decay=[0.9]), "one number in (0, 1] per head"),
        (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "divide the experts"),
        (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "fit into the kept groups"),
        (lambda c: c["layers"][2].update(weights_of=1), "of its type and sizes"),
        (lambda c: c["layers"][4].update(weights_of=2), "tensors of its own"),
        (lambda c: c["layers"][0]["mlp"].update(kind="relu"), "not known"),
    ]:
        raw = copy.deepcopy(tb.A)
        breaker(raw)
        with pytest.raises(ConfigError) as err:
            config_from_dict(raw)
        assert text in str(err.value), str(err.value)


def test_tensor_names_and_what_keeps_what():
    from inferx_amd.config import config_from_dict
    from inferx_amd.parts import build_model
    model = build_model(config_from_dict(copy.deepcopy(tb.A)).model_spec())
    names = model.expected_tensors()
    shape = lambda n: tuple(names[n].shape)
    assert shape("l0.norm1") == () and shape("final.norm") == () and shape("head") == (320, 96) and shape("embed") == (320, 96)
    assert shape("l0.mix.q") == (3 * 24, 96) and shape("l0.mix.dkv") == (48, 96) and shape("l0.mix.dkv.norm") == (40,)
    assert shape("l0.mix.uk") == (48, 40) and shape("l0.mix.uv") == (72, 40) and shape("l0.mix.o") == (96, 72)
    assert shape("l0.mlp.gate") == (64, 96) and shape("l0.mlp.gate.b") == (64,) and shape("l0.mlp.down.b") == (96,)
    assert shape("l1.mix.q") == (32, 96) and shape("l1.mix.v") == (48, 96) and shape("l1.mix.norm") == (48,)
    assert shape("l1.mlp.router") == (6, 96) and shape("l1.mlp.e5.up") == (32, 96) and shape("l1.mlp.shared.down") == (96, 48)
    assert shape("l3.mix.r") == (48, 96) and shape("l3.mix.w1") == (5, 96) and shape("l3.mix.w2") == (48, 5)
    assert shape("l3.mix.a.b") == (48,) and shape("l3.mix.w0") == (48,) and shape("l3.mix.norm") == (48,)
    assert not any(n.startswith(("l2.", "l4.")) for n in names), "a layer that uses another's tensors has none of its own"
    assert "l1.mlp.e0.gate.b" not in names and "l1.norm2" not in names
    plan = model.cache_plan()
    need, state = plan[0][0]["mixer"]
    assert [(a.name, a.heads, a.width) for a in need.arrays] == [("latent", 1, 48)] and state is None
    assert plan[2][0]["mixer"][0] is not None, "the second run of a layer keeps a cache of its own"
    assert plan[1][0]["mixer"][0] is None and plan[1][0]["mixer"][1].shape == (2 * 16 * 24,)
    assert plan[3][0]["mixer"][1].shape == (3 * 16 * 16,) and plan[3][0]["mixer"][1].dtype == "float32"
    assert model.graph_safe()


def test_plain_rotation_of_neighbouring_pairs_by_hand():
    x = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 5.0, 7.0]]], dtype=torch.float64)  # one token at position 3, one head
    out = pb.rotate_pairs(x, torch.tensor([3]), 4, 100.0)
    a0, a1 = 3.0, 3.0 * 100.0 ** (-2 / 4)
    want = [math.cos(a0), math.sin(a0), -2 * math.sin(a1), 2 * math.cos(a1), 5.0, 7.0]
    assert torch.allclose(out[0, 0], torch.tensor(want, dtype=torch.float64))


def test_plain_routing_by_two_best_of_a_group_by_hand():
    # groups of three: (0.9, 0.1, 0.1) sums to 1.0 by its two best, (0.6, 0.6, 0.0) to 1.2, (0.5, 0.4, 0.4) to 0.9
    s = torch.tensor([[0.9, 0.1, 0.1, 0.6, 0.6, 0.0, 0.5, 0.4, 0.4]], dtype=torch.float64)
    assert set(pb.choose_experts(s, 2, 3, 1)[0].tolist()) == {3, 4}      # the best single expert's group is dropped
    assert set(pb.choose_experts(s, 2, 3, 2)[0].tolist()) == {0, 3}      # two groups kept: 0.9 and one of the 0.6
    assert set(pb.choose_experts(s, 3, 1, 1)[0].tolist()) == {0, 3, 4}   # no groups: the three best
    assert set(pb.choose_experts(s, 2, 9, 2)[0].tolist()) == {0, 3}      # groups of one: a group's score is its expert's


def test_plain_clamped_unit_by_hand():
    x = torch.eye(2, dtype=torch.float64)
    gate = torch.tensor([[3.0, 0.0], [0.0, -2.0]], dtype=torch.float64)
    up = torch.tensor([[-5.0, 0.0], [0.0, 0.5]], dtype=torch.float64)
    down = torch.eye(2, dtype=torch.float64)
    out = pb.clamped_glu(x, gate, up, down, 1.0)
    sig = lambda z: 1.0 / (1.0 + math.exp(-z))
    # token 0: g = min(3, 1) = 1, u = clamp(-5) = -1 -> 1 * sig(1.702) * 0 = 0; token 1: g = -2 (no lower clamp), u = 0.5
    assert abs(float(out[0, 0])) < 1e-12 and abs(float(out[1, 1]) - (-2.0 * sig(-3.404) * 1.5)) < 1e-12


def test_plain_recurrences_first_steps_by_hand():
    eps = 1e-5
    # lightning attention, one head of two keys and one value: S1 = k1 v1, o1 = (q1 . k1) v1; S2 = d S1 + k2 v2
    silu = lambda z: z / (1.0 + math.exp(-z))
    W = {"q": torch.tensor([[1.0, 0.0], [0.0, 1.0]]), "k": torch.tensor([[0.0, 1.0], [1.0, 0.0]]),
         "v": torch.tensor([[2.0, 0.0]]), "g": torch.zeros(1, 2), "norm": torch.ones(1), "o": torch.ones(1, 1)}
    W = {k: v.double() for k, v in W.items()}
    x = torch.tensor([[1.0, 2.0], [3.0, -1.0]], dtype=torch.float64)
    m = {"heads": 1, "dim": 2, "vdim": 1, "decay": [0.5]}
    out = pb.lightning(x, W, m, eps)
    q1, k1, v1 = [silu(1.0), silu(2.0)], [silu(2.0), silu(1.0)], silu(2.0)
    q2, k2, v2 = [silu(3.0), silu(-1.0)], [silu(-1.0), silu(3.0)], silu(6.0)
    o1 = (q1[0] * k1[0] + q1[1] * k1[1]) * v1
    o2 = 0.5 * (q2[0] * k1[0] + q2[1] * k1[1]) * v1 + (q2[0] * k2[0] + q2[1] * k2[1]) * v2
    for got, o in zip(out[:, 0].tolist(), (o1, o2)):
        assert abs(got - o / math.sqrt(o * o + eps) * 0.5) < 1e-9  # one norm over the one column, gate sigmoid(0)
