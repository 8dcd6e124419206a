"""The Gosuvik design through the engine against the plain implementation (`plain_gosuvik.py`): whole prompts, last
tokens one by one (past every window), portions of changing size down to two tokens, mixed batches with few pages, in
float32 and in bfloat16, on tiny configurations that differ in every size and option; requests alone against in a
batch; pages and state slots that others left dirty; long decoding (from graphs, bit-equal to kernel by kernel); other
page sizes; greedy generation through `LLMEngine` and the command lines."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_gosuvik as pg
import replay_util as ru
import tiny_gosuvik as tg
from test_gpu_bibevik import ChosenExperts

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"A": (5, 9, 27, 70), "B": (7, 23, 40, 75), "C": (1, 2, 33, 70), "D": (3, 50, 90), "E": (4, 19, 45)}
# relative to the largest |logit| of the expected rows; fixed before the first run
TOL = {"float32": ru.FP32_TOL, "bfloat16": ru.BF16_TOL}
NAMES = sorted(tg.CONFIGS)
NEAR_TIE_16 = 5e-2  # how far apart (relatively) two scores may lie for a 16-bit run to take either


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in tg.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            d = tmp_path_factory.mktemp(f"gosuvik_{name}_{dtype}")
            tg.make_folder(cfg, seed=53, out_dir=str(d), dtype=dtype)
            out[(name, dtype)] = str(d)
    return out


def prompts_for(name):
    return {f"r{i}": tg.random_tokens(n, tg.CONFIGS[name]["vocab"], seed=900 + i) for i, n in enumerate(LENGTHS[name])}


def make_runner(folders, name, dtype, num_pages=64, page_size=16, max_requests=4, **kw):
    from inferx_amd.engine.runner import ModelRunner
    return ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=page_size, num_pages=num_pages,
                                      max_requests=max_requests, max_seq_len=num_pages * page_size, **kw)


def routed_runs(cfg):
    return [i for i in pg.layer_order(cfg) if (cfg["layers"][i].get("mlp") or {}).get("kind") == "moe"]


def expected_for(folders, name, dtype, prompts, chosen, what):
    """The plain logits of every request, and for bfloat16 how far rounding every stored activation to 16 bits moves
    each position's (relative to the largest logit).  bfloat16: with the engine's choice of experts, which may differ
    from the plain one at near ties only."""
    cfg, weights = tg.read_folder(folders[(name, dtype)])
    runs = routed_runs(cfg)
    out, gap = {}, {}
    for rid, toks in prompts.items():
        theirs = None
        if chosen is not None and runs:
            theirs = [torch.tensor([chosen.by_place[(rid, pos)][call] for pos in range(len(toks))])
                      for call in range(len(runs))]
        own, scores = [], []
        logits = pg.forward(cfg, weights, toks, experts=theirs, chosen=own, scores=scores)
        for call in range(len(runs) if theirs is not None else 0):
            for pos in range(len(toks)):  # with the engine's experts upstream, every choice is the plain one or a near tie
                mine, other = set(own[call][pos].tolist()), set(theirs[call][pos].tolist())
                if mine != other:
                    s = scores[call][pos]
                    lost, taken = max(float(s[e]) for e in mine - other), min(float(s[e]) for e in other - mine)
                    assert (lost - taken) / lost < NEAR_TIE_16, \
                        f"{what}: request {rid} position {pos} routed run {call}: the engine chose {sorted(other)}, " \
                        f"the plain implementation {sorted(mine)}: no near tie"
        if dtype == "bfloat16":
            exact = logits if theirs is not None else pg.forward(cfg, weights, toks, experts=own)
            # the largest of nine samples (a sequence's first token leaves a delta layer as sign(q . k) times its
            # normalised value: where q . k nearly cancels, rounding decides the sign, and few samples miss that)
            for store in [pg.bfloat16] + [pg.jittered(s) for s in range(8)]:
                stored = pg.forward(cfg, weights, toks, experts=theirs if theirs is not None else own, store=store)
                for pos, g in enumerate((stored - exact).abs().max(dim=1).values.tolist()):
                    gap[(rid, pos)] = max(g, gap.get((rid, pos), 0.0))
        out[rid] = logits
    scale = max(float(l.abs().max()) for l in out.values())
    return out, {place: g / scale for place, g in gap.items()}


def run_and_check(folders, name, dtype, steps, monkeypatch, what, prompts=None, only=None, **runner_kw):
    if dtype == "bfloat16":
        runner_kw.setdefault("use_graphs", False)
    runner = make_runner(folders, name, dtype, **runner_kw)
    chosen = ChosenExperts(runner, monkeypatch) if dtype == "bfloat16" else None
    got = ru.replay(runner, steps)
    every = prompts or prompts_for(name)
    expected, gap = expected_for(folders, name, dtype, {r: every[r] for r in (only or every)}, chosen, what)
    # bfloat16: a position that 16-bit storage alone moves by more than a third of the fixed tolerance may differ by
    # three times what that storage costs there; every position is compared in float32 with the fixed tolerance
    tol = TOL[dtype]
    touchy = {place: 3 * g for place, g in gap.items() if 3 * g > tol}
    worst = ru.compare(got, expected, tol, what, skip=touchy)
    scale = max(float(e.abs().max()) for e in expected.values())
    for (rid, pos), limit in touchy.items():
        err = float((got[(rid, pos)].double() - expected[rid][pos]).abs().max()) / scale
        assert err <= limit, f"{what}: request {rid} position {pos}: error {err:.3e}, 16-bit storage alone {limit / 3:.1e}"
    print(f"{what}: worst {worst:.2e} (tolerance {tol:.1e}; {len(touchy)} positions by their own)")
    return runner, got


WAYS = {"whole": lambda p: ru.whole(p), "tail": lambda p: ru.tail_decoded(p, 45), "portions": lambda p: ru.chunked(p)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("way", ["whole", "tail", "portions"])
def test_each_request_alone(folders, name, dtype, way, monkeypatch):
    """(`tail`: the last 45 tokens one by one, more than every window of these configurations, so that windows pass
    over decoded tokens and their pages are given back while decoding.)"""
    run_and_check(folders, name, dtype, WAYS[way](prompts_for(name)), monkeypatch, f"{way} {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_few_pages(folders, name, dtype, monkeypatch):
    """Up to four live requests, portions of some beside single tokens of others, in a pool with room for about two
    of the longer ones: pages and state slots are given back and used again."""
    prompts = prompts_for(name)
    for i in range(4):  # more requests than slots
        prompts[f"x{i}"] = tg.random_tokens(11 + 7 * i, tg.CONFIGS[name]["vocab"], seed=950 + i)
    max_tokens = 192
    steps = ru.mixed(prompts, seed=8, max_tokens=max_tokens)
    assert any(len(s["entries"]) > 1 and {len(e[1]) for e in s["entries"]} & {1} and
               max(len(e[1]) for e in s["entries"]) > 1 for s in steps), "no step mixes a portion with a single token"
    run_and_check(folders, name, dtype, steps, monkeypatch, f"mixed {name} {dtype}", prompts, num_pages=max_tokens // 16)
    owners = {}
    runner = make_runner(folders, name, dtype, num_pages=max_tokens // 16)
    ru.replay(runner, steps, page_owners=owners)
    assert any(len(who) > 1 for who in owners.values()), "no physical page was used by two requests"


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_a_batch_gives_what_each_request_gives_alone(folders, name):
    """float32: the logits of a request in a batch of unequal requests, cut into unequal portions, equal the logits of
    the same request run alone and whole, to rounding."""
    prompts = prompts_for(name)
    alone = ru.replay(make_runner(folders, name, "float32"), ru.whole(prompts))
    together = ru.replay(make_runner(folders, name, "float32"), ru.mixed(prompts, seed=5))
    scale = max(float(v.abs().max()) for v in alone.values())
    for key, row in alone.items():
        assert float((row - together[key]).abs().max()) <= 1e-5 * scale, f"{key} differs between alone and in a batch"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_slots_and_pages_that_others_left_dirty(folders, name, dtype, monkeypatch):
    """A request that starts in a state slot and on pages that hold another request's leftovers (made not-a-number
    here) gives the same logits: a sequence's first tokens read no state and no key beyond its own."""
    from inferx_amd.engine.runner import ModelRunner
    prompts = prompts_for(name)
    made = ModelRunner.from_directory

    def dirty(*a, **kw):  # every page and every state slot starts as not-a-number
        runner = made(*a, **kw)
        for arrays in runner.pages:
            for t in arrays.values():
                t.fill_(float("nan"))
        for state in runner._states:
            state.fill_(float("nan"))
        return runner
    monkeypatch.setattr(ModelRunner, "from_directory", dirty)
    second = {"r3": prompts["r3"], "r2": prompts["r2"], "r1": prompts["r1"]}  # one after the other in the one slot
    run_and_check(folders, name, dtype, ru.chunked(second, sizes=(3, 2, 5)), monkeypatch, f"dirty slots {name} {dtype}",
                  only=second, num_pages=8, max_requests=1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "D"])
def test_long_decoding(folders, name, dtype, monkeypatch):
    """A short prompt and 150 tokens one by one, two requests side by side that started at different times: kernel
    by kernel against the plain implementation, then replayed from graphs with the same bits."""
    vocab = tg.CONFIGS[name]["vocab"]
    prompts = {"a": tg.random_tokens(156, vocab, 1), "b": tg.random_tokens(140, vocab, 2)}
    steps = [{"entries": [("a", prompts["a"][:6], list(range(6)))], "end": []},
             {"entries": [("a", prompts["a"][6:16], list(range(10)))], "end": []},
             {"entries": [("a", prompts["a"][16:17], [0]), ("b", prompts["b"][:1], [0])], "end": []}]
    for i in range(1, 140):
        steps.append({"entries": [("a", prompts["a"][16 + i:17 + i], [0]), ("b", prompts["b"][i:i + 1], [0])],
                      "end": ["a", "b"] if i == 139 else []})
    _, plainly = run_and_check(folders, name, dtype, steps, monkeypatch, f"long decoding {name} {dtype}", prompts,
                               use_graphs=False)
    runner = make_runner(folders, name, dtype)
    got = ru.replay(runner, steps)
    assert runner._graphs, "no step was replayed from a graph"
    for key, row in plainly.items():
        assert torch.equal(row, got[key]), f"{key}: replayed from a graph differs from kernel by kernel"


@pytest.mark.parametrize("page_size", [8, 48])
def test_other_page_sizes(folders, page_size, monkeypatch):
    for dtype in ("float32", "bfloat16"):
        run_and_check(folders, "A", dtype, ru.chunked(prompts_for("A")), monkeypatch, f"pages of {page_size} {dtype}",
                      num_pages=24, page_size=page_size)


def test_windowed_pages_given_back_change_no_logit(folders):
    """The pages that a window has passed are given back while a request runs; kept until its end instead, the logits
    are the same bits."""
    prompts = prompts_for("A")
    steps = ru.chunked(prompts)
    back = ru.replay(make_runner(folders, "A", "bfloat16", use_graphs=False), steps)
    kept = ru.replay(make_runner(folders, "A", "bfloat16", use_graphs=False, release_window_pages=False), steps)
    for key, row in back.items():
        assert torch.equal(row, kept[key]), f"{key} depends on whether passed pages were given back"


def greedy_agrees(cfg, weights, prompt, out, what):
    seq = list(prompt)
    for i, token in enumerate(out):
        want = int(torch.argmax(pg.forward(cfg, weights, seq)[-1]))
        assert token == want, f"{what}: token {i} is {token}, the plain implementation says {want}"
        seq.append(token)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    cfg, weights = tg.read_folder(folders[(name, dtype)])
    prompts = [tg.random_tokens(n, cfg["vocab"], seed=n) for n in (5, 9, 17, 30, 3, 12)]
    # a token budget below the longest prompt: prompts come in portions beside decoding requests; four at a time
    engine = LLMEngine(folders[(name, dtype)], dtype, max_num_seqs=4, max_model_len=96, max_num_batched_tokens=16,
                       num_gpu_blocks_override=20)
    outs = engine.generate(prompts, SamplingParams(max_tokens=12))
    for prompt, out in zip(prompts, outs):
        assert len(out) == 12
        if dtype == "float32":
            greedy_agrees(cfg, weights, prompt, out, f"{name} {dtype}")


def test_command_lines(folders, tmp_path):
    """`bin/inferx-generate` and `bin/trace_run` choose the model class by config.json."""
    folder = folders[("A", "float32")]
    cfg, weights = tg.read_folder(folder)
    prompt = tg.random_tokens(7, cfg["vocab"], 4)
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "inferx-generate"), "--model", folder, "--dtype",
                        "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5", "--max-model-len",
                        "64", "--num-gpu-blocks-override", "8"], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    tokens = json.loads(p.stdout.strip().splitlines()[-1])["output_token_ids"]
    assert len(tokens) == 5
    greedy_agrees(cfg, weights, prompt, list(tokens), "inferx-generate")

    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:4], "want": [0, 3]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[4:], "want": [2]},
                                     {"id": "b", "tokens": prompt[:2], "want": []}], "end": ["a"]},
             {"step": 2, "entries": [{"id": "b", "tokens": prompt[2:3], "want": [0]}], "end": ["b"]}]
    out_dir = tmp_path / "logits"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out",
                        str(out_dir), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = pg.forward(cfg, weights, prompt).numpy()
    scale = float(np.abs(want).max())
    for step, rows in ((0, [0, 3]), (1, [6]), (2, [2])):
        got = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(len(rows), -1)
        assert float(np.abs(got - want[rows]).max()) <= ru.FP32_TOL * scale
