"""Decode and prefill throughput at the Qwen1.5-MoE-A2.7B shape, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of the whole batch through the engine (scheduler,
batch layout, upload, every kernel, greedy choice of the next tokens).  Prints ONE
JSON line: decoded tokens a second at the default batch (with the smallest and the
median time of single steps), the prefill of one 2,048-token prompt, the decode
step's HBM roofline fraction, and decode at batch 1 and 64.  Fractions are given
against the published peaks and against what two probe kernels measure on this
machine at the start of the run (a pure read of 4 GiB, pure matrix-core
products).  One GPU only.

Two further workloads at the Qwen2-57B-A14B shape, each with a JSON line of the same form:

    python bench.py --workload mixed [--layers L]   # 32 decodes at a context of 4,096 beside 2 prompt portions of 512
    python bench.py --workload long [--layers L]    # batch 8, prompts of 16,384 to 32,000 tokens in portions of
                                                    # 2,048, then --steps decode steps (default there: 256)

and a small mixed step at the Qwen1.5-MoE-A2.7B shape, which is launched kernel by kernel (only steps of one token
per request are replayed from HIP graphs): under `rocprofv3 --kernel-trace` it shows whether such steps wait for
the host:

    python bench.py --workload mixed-small          # 8 decodes at a context of 2,048 beside 1 prompt portion of 64

and a prompt portion on top of a context at either shape (chunked prefill under a token budget), through the step
function:

    python bench.py --workload portion --shape a27b|57b --prefill-tokens N --prefill-context C [--layers L]

and the Pelalix design (Dynamic Tanh norms, token shift, attention whose heads' scores are mixed, with sinks and gates)
beside the dense layers of the Qwen2-MoE architecture at equal sizes (the same width, heads, key/value heads, head size,
feed-forward width, vocabulary and layers), both through the step function, at a few sizes of real models' layers:

    python bench.py --workload pelalix [--sizes 2k,4k] [--layers L] [--batch B] [--prompt-len C] [--prefill-tokens N]
    python bench.py --workload dezudra [--sizes 1k,2k] [--layers L] [--batch B] [--prompt-len C] [--prefill-tokens N]
    python bench.py --workload bibevik [--sizes 1k,2k] [--only bibevik|dezudra]       # Bibevik beside Dezudra
    python bench.py --workload gosuvik [--sizes 1k,2k] [--only gosuvik|dezudra]       # Gosuvik beside Dezudra

and a whole batch through the engine's loop (scheduler, portions, decode graphs as they come, sampling) at the same
shape:

    python bench.py --workload offline              # 96 requests of 5 to 3,000 prompt tokens and 4 to 120 generated,
                                                    # 64 at a time, 4,096 tokens a step; with --scarce so few pages
                                                    # that sequences are preempted
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Qwen1.5-MoE-A2.7B's sizes
SHAPE = {
    "architectures": ["Qwen2MoeForCausalLM"], "num_hidden_layers": 24, "hidden_size": 2048,
    "num_attention_heads": 16, "num_key_value_heads": 16, "head_dim": 128, "num_experts": 60,
    "num_experts_per_tok": 4, "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632,
    "intermediate_size": 5632, "decoder_sparse_step": 1, "mlp_only_layers": [], "norm_topk_prob": False,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 8192,
    "use_sliding_window": False, "tie_word_embeddings": False,
}
# Qwen2-57B-A14B's sizes
SHAPE_57B = {
    "architectures": ["Qwen2MoeForCausalLM"], "num_hidden_layers": 28, "hidden_size": 3584,
    "num_attention_heads": 28, "num_key_value_heads": 4, "head_dim": 128, "num_experts": 64,
    "num_experts_per_tok": 8, "moe_intermediate_size": 2560, "shared_expert_intermediate_size": 20480,
    "intermediate_size": 18944, "decoder_sparse_step": 1, "mlp_only_layers": [], "norm_topk_prob": False,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 32768,
    "use_sliding_window": False, "tie_word_embeddings": False,
}
CONTEXT = 4096
PROMPT = 2048
PAGE = 16
PEAK_HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def decode_bytes(cfg, batch, context, elt, distinct=None):
    """Bytes one decode step has to read: every weight it uses once, and the cache of the live requests.
    `distinct`: experts that a step's tokens choose, per layer (measured); without it what an even router gives."""
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    if distinct is None:
        distinct = E * (1.0 - (1.0 - k / E) ** batch)  # expected number of experts a batch touches
    per_layer = (qd + 2 * kvd) * H + (qd + 2 * kvd) + H * qd + 2 * H  # attention + norms
    per_layer += E * H + distinct * 3 * mi * H + 3 * si * H + H      # router, routed, shared, shared gate
    weights = L * per_layer + H + cfg.vocab_size * H + batch * H     # final norm, head, embedding rows
    cache = L * 2 * kvd * context * batch
    return (weights + cache) * elt


def prefill_flops(cfg, tokens):
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    per_token = (qd + 2 * kvd) * H + H * qd + E * H + k * 3 * mi * H + 3 * si * H + H
    linear = 2.0 * tokens * L * per_token + 2.0 * cfg.vocab_size * H  # head on the last row only
    attention = L * 2.0 * 2.0 * qd * tokens * (tokens + 1) / 2.0     # causal half of QK^T and PV
    return linear + attention


def experts_hit(run_step, runner, steps=2):
    """How many experts the tokens of a step really choose, per layer: `steps` steps run without graphs, the
    grouping's offsets read back."""
    import torch
    from inferx_amd import ops
    seen, hit, graphs = [], [], runner.use_graphs
    real = ops.moe_route_dispatch, ops.moe_dispatch

    def spy_small(*a, **k):
        real[0](*a, **k)
        seen.append(a[8])

    def spy_wide(topk_e, offsets, *a, **k):
        real[1](topk_e, offsets, *a, **k)
        seen.append(offsets)
    try:
        runner.use_graphs = False
        ops.moe_route_dispatch, ops.moe_dispatch = spy_small, spy_wide
        for _ in range(steps):
            seen.clear()
            run_step()
            torch.cuda.synchronize()  # (the offsets of a layer are a buffer of their own until the step ends)
            hit += [int(((o[1:] - o[:-1]) > 0).sum()) for o in seen]
    finally:
        runner.use_graphs = graphs
        ops.moe_route_dispatch, ops.moe_dispatch = real
    return sum(hit) / len(hit) if hit else None


def step_bytes(cfg, tokens, cache_tokens, elt, distinct=None):
    """Bytes a step of `tokens` tokens has to read: every weight it uses once, and `cache_tokens` of cache.
    `distinct`: experts that the step's tokens choose, per layer (measured); without it what an even router gives."""
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    if distinct is None:
        distinct = E * (1.0 - (1.0 - k / E) ** tokens)
    per_layer = (qd + 2 * kvd) * H + (qd + 2 * kvd) + H * qd + 2 * H + E * H + distinct * 3 * mi * H + 3 * si * H + H
    return (L * per_layer + H + cfg.vocab_size * H + L * 2 * kvd * cache_tokens) * elt


def linear_flops(cfg, tokens, head_rows):
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    per_token = (qd + 2 * kvd) * H + H * qd + E * H + k * 3 * mi * H + 3 * si * H + H
    return 2.0 * tokens * L * per_token + 2.0 * head_rows * cfg.vocab_size * H


def attention_flops(cfg, new, before):
    """QK^T and PV of `new` tokens that follow `before` cached ones (causal)."""
    return cfg.num_hidden_layers * 2.0 * 2.0 * cfg.q_dim * (new * before + new * (new + 1) / 2.0)


def run_57b(args) -> int:
    """The two workloads at the Qwen2-57B-A14B shape (see the module's docstring)."""
    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.sampling import SamplingParams
    from inferx_amd.weights import random_tensors

    shape = SHAPE if args.workload == "mixed-small" else SHAPE_57B
    shape_name = "Qwen1.5-MoE-A2.7B shape" if args.workload == "mixed-small" else "Qwen2-57B-A14B shape"
    layers = args.layers or shape["num_hidden_layers"]
    raw = dict(shape)
    raw["num_hidden_layers"] = layers
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    elt = 2 if args.dtype == "bfloat16" else 4
    peak = PEAK_TFLOPS["bf16" if elt == 2 else "fp32"] * 1e12
    mixed = args.workload in ("mixed", "mixed-small")
    context = {"mixed": 8192, "mixed-small": 4096, "long": 32768}[args.workload]
    log(f"drawing random weights on the device ({layers} layers, {args.dtype})")
    t0 = time.time()
    model = build_model(cfg.model_spec())
    weights = {k: rt.place(v) for k, v in random_tensors(model, seed=0, dtype=args.dtype, device="cuda:0").items()}
    gen = torch.Generator().manual_seed(1234)
    rnd = lambda n: torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()
    base = {"metric": None, "value": None, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if elt == 2 else "fp32", "data": "synthetic: seeded random weights and token ids"}
    sizes = {"layers": layers, "layers_of_shape": shape["num_hidden_layers"], "hidden": cfg.hidden_size,
             "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
             "experts": cfg.num_experts, "top_k": cfg.num_experts_per_tok, "moe_intermediate": cfg.moe_intermediate_size,
             "shared_intermediate": cfg.shared_expert_intermediate_size, "vocab": cfg.vocab_size, "page_size": PAGE}

    if mixed:
        n_dec, dec_ctx, n_pre, portion, pre_ctx = (32, 4096, 2, 512, 2048) if args.workload == "mixed" else \
            (8, 2048, 1, 64, 0)
        pages = (n_dec * context + n_pre * context) // PAGE
        runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=n_dec + n_pre,
                             max_seq_len=context, model=model)
        log(f"model ready in {time.time() - t0:.1f}s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB on the device")
        dec = [f"d{i}" for i in range(n_dec)]
        pre = [f"p{i}" for i in range(n_pre)]
        for r in dec + pre:  # the contexts the step starts from
            runner.add_request(r)
            for s in range(0, dec_ctx if r in dec else pre_ctx, 2048):
                runner.run_entries([(r, rnd(2048), [])])
        total = args.warmup + args.steps
        assert pre_ctx + total * portion <= context and dec_ctx + total <= context, f"fewer steps: the context is {context}"
        entries = lambda: [(r, rnd(1), [0]) for r in dec] + [(r, rnd(portion), []) for r in pre]
        for _ in range(args.warmup):
            runner.run_entries(entries())
        batches = [entries() for _ in range(args.steps)]
        torch.cuda.synchronize()
        t = time.perf_counter()
        for e in batches:
            runner.run_entries(e)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / args.steps
        tokens = n_dec + n_pre * portion
        mid = args.warmup + args.steps // 2
        cache_tokens = n_dec * (dec_ctx + mid) + n_pre * (pre_ctx + mid * portion)
        flops = linear_flops(cfg, tokens, n_dec) + n_dec * attention_flops(cfg, 1, dec_ctx + mid) \
            + n_pre * attention_flops(cfg, portion, pre_ctx + mid * portion)
        gbs = step_bytes(cfg, tokens, cache_tokens, elt) / dt / 1e9
        line = dict(base, metric=f"{shape_name}, mixed step ({n_dec} decodes at context {dec_ctx} beside {n_pre} prompt "
                                 f"portions of {portion}) through the step function, tokens/s",
                    value=round(tokens / dt, 1), ms_per_step=round(dt * 1e3, 3),
                    config=dict(sizes, model=shape_name, global_batch=n_dec + n_pre, seq_len=context,
                                tokens_per_step=tokens, parallelism="single GPU"),
                    prefill=None,
                    compute={"flops_per_step": flops, "frac": round(flops / dt / peak, 5)},
                    roofline={"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                              "frac": round(gbs / PEAK_HBM_GBS, 5)}, points={})
        print(json.dumps(line), flush=True)
        return 0

    # ---- long context: batch 8, prompts of 16,384 to 32,000 tokens in portions of 2,048, then decoding ----
    batch, chunk = 8, 2048
    steps = args.steps
    lens = torch.randint(16384, 32001, (batch,), generator=gen).tolist()
    free, _ = torch.cuda.mem_get_info()
    per_page = cfg.num_hidden_layers * 2 * cfg.kv_dim * PAGE * elt
    pages = max(batch * context // PAGE, int(free * 0.85) // per_page)  # the pool fills what memory is left
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=batch, max_seq_len=context,
                         model=model)
    runner.capture_after = 1
    log(f"model ready in {time.time() - t0:.1f}s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB on the device, "
        f"{pages} pages ({pages * PAGE} tokens of cache)")
    engine = LLMEngine("", runner=runner, max_num_seqs=batch, max_model_len=context, max_num_batched_tokens=chunk)
    # (the first requests decode while the later prompts are still being read, about a hundred steps: room for those)
    slack = 8 * (32000 // chunk + 1) + 8
    params = SamplingParams(max_tokens=args.warmup + steps + slack, ignore_eos=True)
    assert max(lens) + args.warmup + steps + slack <= context, "fewer steps: the context is 32,768"
    ids = [engine.add_request(rnd(n), params) for n in lens]
    torch.cuda.synchronize()
    t = time.perf_counter()
    n_steps = 0
    while any(engine.scheduler.sequence(i).generated() == 0 for i in ids):
        engine.step()
        n_steps += 1
    torch.cuda.synchronize()
    t_pre = time.perf_counter() - t
    log(f"prompts of {lens}: {t_pre:.2f}s in {n_steps} steps")
    for _ in range(args.warmup):
        engine.step()
    torch.cuda.synchronize()
    before = engine.stats.tokens_out
    t = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t) / steps
    assert engine.stats.tokens_out - before == batch * steps, "a timed step was not a decode step of the whole batch"
    pre_flops = linear_flops(cfg, sum(lens), batch) + sum(attention_flops(cfg, n, 0) for n in lens)
    cache_tokens = sum(lens) + batch * (args.warmup + steps // 2 + batch)
    hit = experts_hit(engine.step, runner)
    gbs = step_bytes(cfg, batch, cache_tokens, elt, hit) / dt / 1e9
    line = dict(base, metric="Qwen2-57B-A14B shape, decode tok/s @ batch 8 after prompts of 16384-32000 tokens",
                value=round(batch / dt, 1), ms_per_step=round(dt * 1e3, 3),
                config=dict(sizes, model="Qwen2-57B-A14B shape", global_batch=batch, seq_len=context,
                            prompt_tokens=sum(lens), portion=chunk, cache_pages=pages, parallelism="single GPU"),
                prefill={"value": round(sum(lens) / t_pre, 1), "tokens": sum(lens), "ms": round(t_pre * 1e3, 1),
                         "frac": round(pre_flops / t_pre / peak, 5)},
                roofline={"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                          "frac": round(gbs / PEAK_HBM_GBS, 5),
                          "experts_hit_per_layer": round(hit, 1) if hit else None}, points={})
    print(json.dumps(line), flush=True)
    return 0


def run_portion(args) -> int:
    """One request's portion of --prefill-tokens tokens on top of --prefill-context tokens that it has read before
    (in portions of 2,048, untimed): the best of three, the logits of the last token only."""
    import torch
    from inferx_amd import ops
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors

    shape = SHAPE_57B if args.shape == "57b" else SHAPE
    shape_name = "Qwen2-57B-A14B shape" if args.shape == "57b" else "Qwen1.5-MoE-A2.7B shape"
    layers = args.layers or shape["num_hidden_layers"]
    raw = dict(shape, num_hidden_layers=layers, max_position_embeddings=65536)
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    elt = 2 if args.dtype == "bfloat16" else 4
    ceilings = ops.measured_ceilings("cuda:0")
    log(f"drawing random weights on the device ({layers} layers, {args.dtype})")
    model = build_model(cfg.model_spec())
    weights = {k: rt.place(v) for k, v in random_tensors(model, seed=0, dtype=args.dtype, device="cuda:0").items()}
    n, before = args.prefill_tokens, args.prefill_context
    cap = -(-(n + before + PAGE) // PAGE) * PAGE
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=cap // PAGE, max_requests=1, max_seq_len=cap,
                         model=model)
    gen = torch.Generator().manual_seed(1234)
    rnd = lambda m: torch.randint(0, cfg.vocab_size, (m,), generator=gen).tolist()
    times = []
    for _ in range(3):
        runner.add_request("p")
        for at in range(0, before, PROMPT):
            runner.run_entries([("p", rnd(min(PROMPT, before - at)), [])])
        toks = rnd(n)
        torch.cuda.synchronize()
        t = time.perf_counter()
        runner.run_entries([("p", toks, [n - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t)
        runner.end_request("p")
    sec = min(times[1:])
    flops = linear_flops(cfg, n, 1) + attention_flops(cfg, n, before)
    peak = PEAK_TFLOPS["bf16" if elt == 2 else "fp32"] * 1e12
    line = {"metric": f"{shape_name}: prompt portion of {n} tokens on a context of {before}, tokens/s",
            "value": round(n / sec, 1), "unit": "tokens/s", "n_gpus": 1, "steps": 2, "warmup": 1,
            "ms_per_step": round(sec * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if elt == 2 else "fp32", "data": "synthetic: seeded random weights and token ids",
            "config": {"model": shape_name, "global_batch": 1, "seq_len": n + before, "portion": n, "context": before,
                       "parallelism": "single GPU", "layers": layers, "layers_of_shape": shape["num_hidden_layers"],
                       "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                       "head_dim": cfg.head_dim, "experts": cfg.num_experts, "top_k": cfg.num_experts_per_tok,
                       "moe_intermediate": cfg.moe_intermediate_size,
                       "shared_intermediate": cfg.shared_expert_intermediate_size, "vocab": cfg.vocab_size,
                       "page_size": PAGE},
            "prefill": {"value": round(n / sec, 1), "tokens": n, "ms": round(sec * 1e3, 3),
                        "frac": round(flops / sec / peak, 5), "tflops": round(flops / sec / 1e12, 1)},
            "ceilings": ceilings}
    print(json.dumps(line), flush=True)
    return 0


def run_offline(args) -> int:
    """A finite batch of requests of mixed lengths through `LLMEngine.generate` (see the module's docstring)."""
    import random
    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.sampling import SamplingParams
    from inferx_amd.weights import random_tensors
    raw = dict(SHAPE)
    raw["num_hidden_layers"] = args.layers or SHAPE["num_hidden_layers"]
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    rnd = random.Random(0)
    n, live, budget, context = 96, 64, 4096, 4096
    lens = [rnd.choice([rnd.randint(5, 100), rnd.randint(100, 1000), rnd.randint(1000, 3000)]) for _ in range(n)]
    outs = [rnd.randint(4, 120) for _ in range(n)]
    gen = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, cfg.vocab_size, (m,), generator=gen).tolist() for m in lens]
    params = [SamplingParams(max_tokens=m, ignore_eos=True) for m in outs]
    log(f"drawing random weights on the device ({cfg.num_hidden_layers} layers, {args.dtype})")
    model = build_model(cfg.model_spec())
    weights = {k: rt.place(v) for k, v in random_tensors(model, 0, args.dtype, "cuda:0").items()}
    pages = 2200 if args.scarce else live * context // PAGE
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=live, max_seq_len=context,
                         model=model, max_step_tokens=budget)
    engine = LLMEngine("", runner=runner, max_num_seqs=live, max_model_len=context, max_num_batched_tokens=budget)
    engine.generate(prompts[:2], [SamplingParams(max_tokens=2, ignore_eos=True)] * 2)  # libraries' first calls
    steps0 = engine.stats.steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    got = engine.generate(prompts, params, with_reasons=True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    bad = [(r, len(o), m) for (o, r), m in zip(got, outs) if r != "max_tokens" or len(o) != m]
    if bad:
        raise SystemExit(f"bench.py: {len(bad)} requests ended otherwise than asked, e.g. {bad[:3]}")
    runner.cache.check()
    total = sum(lens) + sum(outs)
    print(json.dumps({
        "metric": f"Qwen1.5-MoE-A2.7B offline batch, prompt + generated tokens/s ({n} requests, {live} at a time)",
        "value": round(total / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": engine.stats.steps - steps0,
        "warmup": 0, "ms_per_step": round(dt * 1e3 / max(engine.stats.steps - steps0, 1), 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded random weights, token ids and lengths",
        "config": {"model": "Qwen1.5-MoE-A2.7B shape", "layers": cfg.num_hidden_layers,
                   "layers_of_shape": SHAPE["num_hidden_layers"], "requests": n, "max_num_seqs": live,
                   "max_num_batched_tokens": budget, "max_model_len": context, "pages": pages, "page_size": PAGE,
                   "parallelism": "single GPU"},
        "seconds": round(dt, 3), "prompt_tokens": sum(lens), "generated_tokens": sum(outs),
        "prompt_tokens_per_s": round(sum(lens) / dt, 1), "generated_tokens_per_s": round(sum(outs) / dt, 1),
        "preemptions": engine.stats.preemptions, "graphs_captured": len(runner._graphs)}))
    return 0


# Layer sizes for `--workload pelalix`: width, heads, key/value heads, head size, feed-forward width, vocabulary
PELALIX_SIZES = {
    "1k": dict(width=1024, heads=8, kv_heads=2, dim=128, ff=2816, vocab=32000),
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, ff=5632, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, ff=11008, vocab=32000),
}


class _SpecOnly:
    """A configuration that is nothing but a `ModelSpec` (what the runner reads of a configuration)."""

    eos_token_ids = ()

    def __init__(self, spec):
        self._spec = spec

    def model_spec(self):
        return self._spec


def _time_prefill_and_decode(args, rt, spec, vocab, gen):
    """(seconds for a prompt of args.prefill_tokens in one step, seconds per step of args.batch requests of one token
    each at contexts of args.prompt_len), through the step function, random weights drawn on the device."""
    import torch
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors

    B, C, N = args.batch, args.prompt_len, args.prefill_tokens
    model = build_model(spec)
    weights = {k: rt.place(v) for k, v in random_tensors(model, seed=0, dtype=args.dtype, device="cuda:0").items()}
    cap = -(-(max(C + args.warmup + args.steps + 8, N) + 16) // PAGE) * PAGE
    runner = ModelRunner(_SpecOnly(spec), weights, rt, page_size=PAGE, num_pages=(B + 1) * cap // PAGE,
                         max_requests=B + 1, max_seq_len=cap, model=model)
    runner.capture_after = 1
    toks = lambda n: torch.randint(0, vocab, (n,), generator=gen).tolist()
    times = []
    for _ in range(4):  # the prompt of N tokens in one step
        runner.add_request("p")
        prompt = toks(N)
        torch.cuda.synchronize()
        t = time.perf_counter()
        runner.run_entries([("p", prompt, [N - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t)
        runner.end_request("p")
    pre = min(times[1:])
    for r in range(B):  # B requests with C tokens behind them, then steps of one token each
        runner.add_request(r)
        for at in range(0, C, 2048):
            runner.run_entries([(r, toks(min(2048, C - at)), [])])
    step = lambda: runner.run_entries([(r, toks(1), [0]) for r in range(B)])
    for _ in range(max(args.warmup, 2)):
        step()
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dec = (time.perf_counter() - t) / args.steps
    for r in range(B):
        runner.end_request(r)
    del runner, weights, model
    torch.cuda.empty_cache()
    return pre, dec


# Layer sizes for `--workload dezudra`: width, heads, key/value heads, head size, experts, experts per token, an
# expert's width, vocabulary
DEZUDRA_SIZES = {
    "1k": dict(width=1024, heads=8, kv_heads=2, dim=128, experts=16, top=4, ff=704, vocab=32000),
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, experts=32, top=4, ff=1408, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, experts=64, top=8, ff=1408, vocab=32000),
}


def run_dezudra(args) -> int:
    """Prefill of one prompt and decode steps of a batch, through the step function, for the Dezudra design (layers
    in turn: the gated delta rule, differential attention with a window of 1,024 that keeps 4 first tokens; experts
    of squared relu chosen among 4 groups of which 2 are kept) and for the Qwen2-MoE architecture (attention with
    rotation, gated experts, no shared expert) at equal width, heads, head size, experts and experts per token.  One
    JSON line; per size and model milliseconds and tokens a second of both phases, and Dezudra's time over the
    other's."""
    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.runtime import Runtime

    L = args.layers or 4
    B, C, N = args.batch, args.prompt_len, args.prefill_tokens
    rt = Runtime(args.dtype, "cuda:0")
    gen = torch.Generator().manual_seed(1234)
    out = {}

    def specs(z):
        mlp = {"kind": "moe", "expert": {"ff": z["ff"]},
               "router": {"experts": z["experts"], "top": z["top"], "groups": {"count": 4, "keep": 2}}}
        delta = {"type": "delta", "mlp": mlp,
                 "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"], "conv": 4}}
        attention = {"type": "attention", "mlp": mlp,
                     "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"] // 2, "vdim": z["dim"],
                               "conv": 4, "scale": (z["dim"] // 2) ** -0.5, "diff": 0.5,
                               "rot": {"dims": z["dim"] // 2, "base": 10000.0}, "mask": {"size": 1024, "keep_first": 4}}}
        dez = {"architecture": "Dezudra", "vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6},
               "logit_scale": 1.0, "layers": [delta if i % 2 == 0 else attention for i in range(L)]}
        qwen = {"architectures": ["Qwen2MoeForCausalLM"], "num_hidden_layers": L, "hidden_size": z["width"],
                "num_attention_heads": z["heads"], "num_key_value_heads": z["kv_heads"], "head_dim": z["dim"],
                "num_experts": z["experts"], "num_experts_per_tok": z["top"], "moe_intermediate_size": z["ff"],
                "shared_expert_intermediate_size": 0, "intermediate_size": z["ff"], "vocab_size": z["vocab"],
                "rope_theta": 1e6, "rms_norm_eps": 1e-6, "max_position_embeddings": 0}
        return {"dezudra": config_from_dict(dez).model_spec(), "qwen2_moe": config_from_dict(qwen).model_spec()}

    for name in [n for n in args.sizes.split(",") if n]:
        z = DEZUDRA_SIZES[name]
        res = {}
        for which, spec in specs(z).items():
            log(f"{name}: {which}")
            pre, dec = _time_prefill_and_decode(args, rt, spec, z["vocab"], gen)
            res[which] = {"prefill_ms": round(pre * 1e3, 3), "prefill_tokens_s": round(N / pre, 1),
                          "decode_ms": round(dec * 1e3, 3), "decode_tokens_s": round(B / dec, 1)}
            log(f"{name}: {which}: {res[which]}")
        res["dezudra_over_qwen2_moe"] = {
            "prefill": round(res["dezudra"]["prefill_ms"] / res["qwen2_moe"]["prefill_ms"], 3),
            "decode": round(res["dezudra"]["decode_ms"] / res["qwen2_moe"]["decode_ms"], 3)}
        out[name] = dict(res, sizes=z)
    first = out[next(iter(out))]
    print(json.dumps({
        "metric": f"Dezudra decode tok/s @ batch {B} ({C}-token contexts), first size", "value": first["dezudra"]["decode_tokens_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["dezudra"]["decode_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic: seeded random weights and token ids",
        "config": {"model": "Dezudra beside Qwen2-MoE at equal sizes", "layers": L, "global_batch": B,
                   "seq_len": C, "prefill_tokens": N, "parallelism": "single GPU", "page_size": PAGE},
        "sizes": out}), flush=True)
    return 0


# Layer sizes for `--workload bibevik`: width, attention heads (per head `dim` plain and `rot` rotated query numbers, values
# of `dim`, a latent of `rank`), heads of the two recurrent mixers, experts, experts per token, an expert's width, vocabulary
BIBEVIK_SIZES = {
    "1k": dict(width=1024, heads=8, dim=128, rot=64, rank=512, delta_heads=16, delta_dim=64, experts=16, top=4, ff=704,
               vocab=32000),
    "2k": dict(width=2048, heads=16, dim=128, rot=64, rank=512, delta_heads=32, delta_dim=64, experts=32, top=4, ff=1408,
               vocab=32000),
    "4k": dict(width=4096, heads=32, dim=128, rot=64, rank=512, delta_heads=64, delta_dim=64, experts=64, top=8, ff=1408,
               vocab=32000),
}


def run_bibevik(args) -> int:
    """Prefill of one prompt and decode steps of a batch, through the step function, for the Bibevik design (layers
    in turn: the generalized delta rule, latent attention, lightning attention, latent attention; every layer with
    clamped gated experts chosen by sigmoid scores among 4 groups of which 2 are kept, and a shared expert) and for the
    Dezudra design (the gated delta rule and differential attention in turn, experts chosen among groups) at equal
    width, attention heads, experts and experts per token.  One JSON line; per size and model milliseconds and tokens
    a second of both phases, and Bibevik's time over the other's."""
    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.runtime import Runtime

    L = args.layers or 4
    B, C, N = args.batch, args.prompt_len, args.prefill_tokens
    rt = Runtime(args.dtype, "cuda:0")
    gen = torch.Generator().manual_seed(1234)
    out = {}

    def specs(z):
        H, D = z["heads"], z["dim"]
        mlp = {"kind": "moe", "expert": {"ff": z["ff"], "limit": 7.0}, "shared": {"ff": z["ff"], "limit": 7.0},
               "router": {"experts": z["experts"], "top": z["top"], "scale": 2.5, "groups": {"count": 4, "keep": 2}}}
        latent = {"type": "latent_attention", "mlp": mlp,
                  "mixer": {"heads": H, "dim": D, "rot_dim": z["rot"], "vdim": D, "kv_rank": z["rank"],
                            "scale": (D + z["rot"]) ** -0.5, "rot": {"dims": z["rot"], "base": 10000.0}}}
        delta = {"type": "general_delta", "mlp": mlp, "mixer": {"heads": z["delta_heads"], "dim": z["delta_dim"], "decay_rank": 64}}
        lightning = {"type": "lightning", "mlp": mlp,
                     "mixer": {"heads": H, "dim": D, "vdim": D, "decay": [1.0 - 2.0 ** (-5 - 3 * h / H) for h in range(H)]}}
        order = [delta, latent, lightning, latent]
        bib = {"architecture": "Bibevik", "vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6},
               "embedding": {"scale": 1.0}, "layers": [order[i % 4] for i in range(L)]}
        dmlp = {"kind": "moe", "expert": {"ff": z["ff"]},
                "router": {"experts": z["experts"], "top": z["top"], "groups": {"count": 4, "keep": 2}}}
        kv = max(1, H // 4)
        ddelta = {"type": "delta", "mlp": dmlp, "mixer": {"heads": H, "kv_heads": kv, "dim": D, "vdim": D, "conv": 4}}
        dattn = {"type": "attention", "mlp": dmlp,
                 "mixer": {"heads": H, "kv_heads": kv, "dim": D // 2, "vdim": D, "conv": 4, "scale": (D // 2) ** -0.5,
                           "diff": 0.5, "rot": {"dims": D // 2, "base": 10000.0}, "mask": {"size": 1024, "keep_first": 4}}}
        dez = {"architecture": "Dezudra", "vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6},
               "logit_scale": 1.0, "layers": [ddelta if i % 2 == 0 else dattn for i in range(L)]}
        return {"bibevik": config_from_dict(bib).model_spec(), "dezudra": config_from_dict(dez).model_spec()}

    for name in [n for n in args.sizes.split(",") if n]:
        z = BIBEVIK_SIZES[name]
        res = {}
        for which, spec in specs(z).items():
            if args.only and which != args.only:
                continue
            log(f"{name}: {which}")
            pre, dec = _time_prefill_and_decode(args, rt, spec, z["vocab"], gen)
            res[which] = {"prefill_ms": round(pre * 1e3, 3), "prefill_tokens_s": round(N / pre, 1),
                          "decode_ms": round(dec * 1e3, 3), "decode_tokens_s": round(B / dec, 1)}
            log(f"{name}: {which}: {res[which]}")
        if len(res) == 2:
            res["bibevik_over_dezudra"] = {
                "prefill": round(res["bibevik"]["prefill_ms"] / res["dezudra"]["prefill_ms"], 3),
                "decode": round(res["bibevik"]["decode_ms"] / res["dezudra"]["decode_ms"], 3)}
        out[name] = dict(res, sizes=z)
    first = out[next(iter(out))]
    mine = first.get("bibevik") or next(iter(v for v in first.values() if isinstance(v, dict) and "decode_ms" in v))
    print(json.dumps({
        "metric": f"Bibevik decode tok/s @ batch {B} ({C}-token contexts), first size", "value": mine["decode_tokens_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": mine["decode_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic: seeded random weights and token ids",
        "config": {"model": "Bibevik beside Dezudra at equal sizes", "layers": L, "global_batch": B,
                   "seq_len": C, "prefill_tokens": N, "parallelism": "single GPU", "page_size": PAGE},
        "sizes": out}), flush=True)
    return 0


# Layer sizes for `--workload gosuvik`: width, attention heads and key/value heads of `dim` numbers (the latent layers:
# per head `dim` plain and `rot` rotated query numbers, a latent of `rank`), the matrix memory's heads, windows,
# experts, experts per token, an expert's width, the dense feed-forward's width, vocabulary
GOSUVIK_SIZES = {
    "1k": dict(width=1024, heads=8, kv_heads=2, dim=128, rot=64, rank=512, memory_heads=4, window=1024, experts=16,
               top=4, ff=704, dense_ff=2816, vocab=32000),
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, rot=64, rank=512, memory_heads=8, window=1024, experts=32,
               top=4, ff=1408, dense_ff=5632, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, rot=64, rank=512, memory_heads=16, window=1024, experts=64,
               top=8, ff=1408, dense_ff=11008, vocab=32000),
}


def run_gosuvik(args) -> int:
    """Prefill of one prompt and decode steps of a batch, through the step function, for the Gosuvik design (layers
    in turn: the delta rule with a decay per key channel, latent attention with a window and a gate, the pair of a
    windowed attention with a sink and rotated values beside a matrix memory, latent attention again; norms in two
    groups; experts chosen by a softmax router, the second layer's feed-forward dense with the PolyNorm activation)
    and for the Dezudra design (the gated delta rule and differential attention with a window in turn, experts chosen
    among groups) at equal width, attention heads, head size, window, experts and experts per token.  One JSON line;
    per size and model milliseconds and tokens a second of both phases, and Gosuvik's time over the other's."""
    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.runtime import Runtime

    L = args.layers or 4
    B, C, N = args.batch, args.prompt_len, args.prefill_tokens
    rt = Runtime(args.dtype, "cuda:0")
    gen = torch.Generator().manual_seed(1234)
    out = {}

    def specs(z):
        H, G, D, W = z["heads"], z["kv_heads"], z["dim"], z["window"]
        moe = {"kind": "moe", "expert": {"ff": z["ff"]}, "router": {"experts": z["experts"], "top": z["top"]}}
        yarn = {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}
        latent = lambda mlp: {"type": "latent_attention", "mlp": mlp,
                              "mixer": {"heads": H, "dim": D, "rot_dim": z["rot"], "vdim": D, "kv_rank": z["rank"],
                                        "scale": (D + z["rot"]) ** -0.5, "mask": {"size": W},
                                        "rot": {"dims": z["rot"], "base": 10000.0, "scaling": yarn}}}
        delta = {"type": "channel_delta", "mlp": moe,
                 "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "conv": 4, "decay_rank": 64, "gate_rank": 64}}
        pair = {"type": "parallel", "mlp": moe,
                "mixer": {"left": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "mask": {"size": W},
                                   "rot": {"dims": D // 2, "base": 10000.0, "scaling": {"factor": 4.0}}},
                          "right": {"heads": z["memory_heads"], "dim": D, "vdim": D, "gate_cap": 15.0},
                          "left_scale": 0.5, "right_scale": 0.5}}
        order = [delta, latent({"kind": "dense", "ff": z["dense_ff"]}), pair, latent(moe)]
        gos = {"architecture": "Gosuvik", "vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6, "groups": 2},
               "layers": [order[i % 4] for i in range(L)]}
        dmlp = {"kind": "moe", "expert": {"ff": z["ff"]},
                "router": {"experts": z["experts"], "top": z["top"], "groups": {"count": 4, "keep": 2}}}
        ddelta = {"type": "delta", "mlp": dmlp, "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "conv": 4}}
        dattn = {"type": "attention", "mlp": dmlp,
                 "mixer": {"heads": H, "kv_heads": G, "dim": D // 2, "vdim": D, "conv": 4, "scale": (D // 2) ** -0.5,
                           "diff": 0.5, "rot": {"dims": D // 2, "base": 10000.0}, "mask": {"size": W, "keep_first": 4}}}
        dez = {"architecture": "Dezudra", "vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6},
               "logit_scale": 1.0, "layers": [ddelta if i % 2 == 0 else dattn for i in range(L)]}
        return {"gosuvik": config_from_dict(gos).model_spec(), "dezudra": config_from_dict(dez).model_spec()}

    for name in [n for n in args.sizes.split(",") if n]:
        z = GOSUVIK_SIZES[name]
        res = {}
        for which, spec in specs(z).items():
            if args.only and which != args.only:
                continue
            log(f"{name}: {which}")
            pre, dec = _time_prefill_and_decode(args, rt, spec, z["vocab"], gen)
            res[which] = {"prefill_ms": round(pre * 1e3, 3), "prefill_tokens_s": round(N / pre, 1),
                          "decode_ms": round(dec * 1e3, 3), "decode_tokens_s": round(B / dec, 1)}
            log(f"{name}: {which}: {res[which]}")
        if len(res) == 2:
            res["gosuvik_over_dezudra"] = {
                "prefill": round(res["gosuvik"]["prefill_ms"] / res["dezudra"]["prefill_ms"], 3),
                "decode": round(res["gosuvik"]["decode_ms"] / res["dezudra"]["decode_ms"], 3)}
        out[name] = dict(res, sizes=z)
    first = out[next(iter(out))]
    mine = first.get("gosuvik") or next(iter(v for v in first.values() if isinstance(v, dict) and "decode_ms" in v))
    print(json.dumps({
        "metric": f"Gosuvik decode tok/s @ batch {B} ({C}-token contexts), first size", "value": mine["decode_tokens_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": mine["decode_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic: seeded random weights and token ids",
        "config": {"model": "Gosuvik beside Dezudra at equal sizes", "layers": L, "global_batch": B,
                   "seq_len": C, "prefill_tokens": N, "parallelism": "single GPU", "page_size": PAGE},
        "sizes": out}), flush=True)
    return 0


def run_pelalix(args) -> int:
    """Prefill of one prompt and decode steps of a batch, through the step function, for the Pelalix design and for
    the Qwen2-MoE architecture's dense layers (attention with rotation, RMS norms, the same gated feed-forward) at
    equal sizes.  One JSON line; per size and model: milliseconds and tokens a second of both phases, the matrix
    flops and the bytes of a decode step against the published peaks, and Pelalix's time over the other's."""
    import dataclasses

    import torch
    from inferx_amd.config import ScheduleEntry, config_from_dict
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors

    L = args.layers or 4
    B, C, N = args.batch, args.prompt_len, args.prefill_tokens
    rt = Runtime(args.dtype, "cuda:0")
    elt = 2 if args.dtype == "bfloat16" else 4
    peak = PEAK_TFLOPS["bf16" if elt == 2 else "fp32"] * 1e12
    gen = torch.Generator().manual_seed(1234)
    out = {}

    def specs(z):
        pel = {"architecture": "Pelalix", "vocab": z["vocab"], "width": z["width"], "embedding": {"scale": 1.0},
               "norm": {"eps": 1e-6},
               "layers": [{"type": "attention",
                           "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"],
                                     "scale": z["dim"] ** -0.5, "v_mix": True},
                           "mlp": {"kind": "dense", "ff": z["ff"]}} for _ in range(L)]}
        # the other architecture wants one layer of experts: it is configured last and left out of the model
        qwen = {"architectures": ["Qwen2MoeForCausalLM"], "num_hidden_layers": L + 1, "hidden_size": z["width"],
                "num_attention_heads": z["heads"], "num_key_value_heads": z["kv_heads"], "head_dim": z["dim"],
                "num_experts": 2, "num_experts_per_tok": 1, "moe_intermediate_size": 64,
                "shared_expert_intermediate_size": 0, "intermediate_size": z["ff"], "mlp_only_layers": list(range(L)),
                "vocab_size": z["vocab"], "rope_theta": 1e6, "rms_norm_eps": 1e-6, "max_position_embeddings": 0}
        spec = config_from_dict(qwen).model_spec()
        dense = dataclasses.replace(spec, layers=spec.layers[:L], schedule=[ScheduleEntry(i) for i in range(L)])
        return {"pelalix": config_from_dict(pel).model_spec(), "qwen2_dense": dense}

    def measure(spec, z):
        pre, dec = _time_prefill_and_decode(args, rt, spec, z["vocab"], gen)
        W, H, G, d, ff, V = z["width"], z["heads"], z["kv_heads"], z["dim"], z["ff"], z["vocab"]
        per_token = W * (H * d + 2 * G * d) + H * d * W + 3 * W * ff
        flops = 2.0 * N * L * per_token + 2.0 * V * W + L * 2.0 * 2.0 * H * d * N * (N + 1) / 2.0
        bytes_dec = (L * per_token + V * W + L * 2 * G * d * (C + args.warmup + args.steps // 2) * B) * elt
        return {"prefill_ms": round(pre * 1e3, 3), "prefill_tokens_s": round(N / pre, 1),
                "prefill_tflops": round(flops / pre / 1e12, 1), "prefill_frac_of_peak": round(flops / pre / peak, 4),
                "decode_ms": round(dec * 1e3, 3), "decode_tokens_s": round(B / dec, 1),
                "decode_gbs": round(bytes_dec / dec / 1e9, 1), "decode_frac_of_peak": round(bytes_dec / dec / 1e9 / PEAK_HBM_GBS, 4)}

    for name in [n for n in args.sizes.split(",") if n]:
        z = PELALIX_SIZES[name]
        res = {}
        for which, spec in specs(z).items():
            log(f"{name}: {which}")
            res[which] = measure(spec, z)
            log(f"{name}: {which}: {res[which]}")
        res["pelalix_over_qwen2_dense"] = {
            "prefill": round(res["pelalix"]["prefill_ms"] / res["qwen2_dense"]["prefill_ms"], 3),
            "decode": round(res["pelalix"]["decode_ms"] / res["qwen2_dense"]["decode_ms"], 3)}
        out[name] = dict(res, sizes=z)
    first = out[next(iter(out))]
    print(json.dumps({
        "metric": f"Pelalix decode tok/s @ batch {B} ({C}-token contexts), first size", "value": first["pelalix"]["decode_tokens_s"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["pelalix"]["decode_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if elt == 2 else "fp32", "data": "synthetic: seeded random weights and token ids",
        "config": {"model": "Pelalix beside Qwen2 dense layers at equal sizes", "layers": L, "global_batch": B,
                   "seq_len": C, "prefill_tokens": N, "parallelism": "single GPU", "page_size": PAGE},
        "sizes": out}), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (32; 8 for mixed, 256 for long)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (4; 2 for mixed)")
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the configuration has (sizes of a layer are never reduced)")
    ap.add_argument("--scarce", action="store_true", help="offline: so few pages that sequences are preempted")
    ap.add_argument("--workload", default="decode",
                    choices=["decode", "mixed", "long", "mixed-small", "offline", "portion", "pelalix", "dezudra", "bibevik",
                             "gosuvik"],
                    help="decode, mixed-small: the Qwen1.5-MoE-A2.7B shape (decode is the default); mixed, long: the "
                         "Qwen2-57B-A14B shape")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prefill-tokens", type=int, default=PROMPT,
                    help="tokens of the prompt whose reading in one step is timed (2,048 is the default workload's)")
    ap.add_argument("--prefill-context", type=int, default=0,
                    help="portion: tokens that the request has read before the timed portion")
    ap.add_argument("--shape", default="a27b", choices=["a27b", "57b"], help="portion: whose layer sizes")
    ap.add_argument("--sizes", default="2k,4k", help="pelalix, dezudra, bibevik, gosuvik: which of the layer sizes " + ", ".join(PELALIX_SIZES))
    ap.add_argument("--only", default="", help="bibevik, gosuvik: time one of the two models only (by its name)")
    ap.add_argument("--prompt-len", type=int, default=PROMPT,
                    help="tokens of every request's prompt before it decodes (the context of the decode steps)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; --gpus N > 1 is not supported")
        return 2
    if args.steps is None:
        args.steps = {"decode": 32, "mixed": 8, "long": 256, "mixed-small": 24, "offline": 0, "portion": 2, "pelalix": 32, "dezudra": 32, "bibevik": 32, "gosuvik": 32}[args.workload]
    if args.warmup is None:
        args.warmup = {"decode": 4, "mixed": 2, "long": 4, "mixed-small": 4, "offline": 0, "portion": 1, "pelalix": 4, "dezudra": 4, "bibevik": 4, "gosuvik": 4}[args.workload]
    if args.workload == "offline":
        return run_offline(args)
    if args.workload == "portion":
        return run_portion(args)
    if args.workload == "pelalix":
        return run_pelalix(args)
    if args.workload == "dezudra":
        return run_dezudra(args)
    if args.workload == "bibevik":
        return run_bibevik(args)
    if args.workload == "gosuvik":
        return run_gosuvik(args)
    if args.workload != "decode":
        return run_57b(args)
    if args.layers is None:
        args.layers = SHAPE["num_hidden_layers"]

    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.sampling import SamplingParams
    from inferx_amd.weights import random_tensors

    raw = dict(SHAPE)
    raw["num_hidden_layers"] = args.layers
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    elt = 2 if args.dtype == "bfloat16" else 4
    from inferx_amd import ops
    ceilings = ops.measured_ceilings("cuda:0")  # before the weights take the memory
    log(f"measured on this machine: {ceilings}")
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    log(f"drawing random weights on the device ({args.layers} layers, {args.dtype})")
    t0 = time.time()
    model = build_model(cfg.model_spec())
    weights = random_tensors(model, seed=0, dtype=args.dtype, device="cuda:0")
    weights = {k: rt.place(v) for k, v in weights.items()}
    prompt_len = args.prompt_len
    # a request's prompt, the tokens it decodes while the later prompts are read (a step each portion), the steps
    reading = max_batch * -(-prompt_len // PROMPT)
    context_cap = max(CONTEXT, args.prefill_tokens, -(-(prompt_len + reading + 2 * args.steps + args.warmup + 3 * max_batch + 32) // PAGE) * PAGE)
    pages = max_batch * context_cap // PAGE
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=max_batch,
                         max_seq_len=context_cap, model=model)
    runner.capture_after = 1  # a steady batch: its shape is captured at the first step, whatever --warmup says
    torch.cuda.synchronize()
    log(f"model ready in {time.time() - t0:.1f}s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB on the device")
    gen = torch.Generator().manual_seed(1234)

    def prompt(n=None):
        return torch.randint(0, cfg.vocab_size, (n or prompt_len,), generator=gen).tolist()

    def run_decode(batch, steps, warmup, single=0):
        """`batch` requests with prompts of `prompt_len` tokens through the engine (scheduler, step function, sampler):
        first their prompts, then `warmup` untimed and `steps` timed decode steps of the whole batch; then `single`
        more steps, each timed on its own (the device is waited for after every one of them, so they are a little
        slower than steps that follow each other).  Returns the time of the `steps` and the list of single times."""
        engine = LLMEngine("", runner=runner, max_num_seqs=batch, max_model_len=context_cap,
                           max_num_batched_tokens=max(PROMPT, batch))
        # (requests decode while the later prompts are still being read: room for those tokens too)
        params = SamplingParams(max_tokens=warmup + steps + single + batch * -(-prompt_len // PROMPT) + 3 * batch + 16,
                                ignore_eos=True)
        ids = [engine.add_request(prompt(), params) for _ in range(batch)]
        while any(engine.scheduler.sequence(i).generated() == 0 for i in ids):  # the prompts, one a step
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        before = engine.stats.tokens_out
        t = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        assert engine.stats.tokens_out - before == batch * steps, "a timed step was not a decode step of the whole batch"
        hit = experts_hit(engine.step, runner) if single else None
        singles = []
        for _ in range(single):
            t = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            singles.append(time.perf_counter() - t)
        for i in ids:
            engine.cancel(i)
        while engine.has_unfinished():
            engine.step()
        assert runner.cache.pools[0].used_pages == 0
        return dt, singles, hit

    # ---- prefill of one 2,048-token prompt ---------------------------------
    prefill = None
    if not args.no_prefill:
        log("prefill")
        n_pre = args.prefill_tokens
        times = []
        for i in range(3):
            runner.add_request("p")
            toks = prompt(n_pre)
            torch.cuda.synchronize()
            t = time.perf_counter()
            runner.run_entries([("p", toks, [n_pre - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            runner.end_request("p")
        sec = min(times[1:])
        flops = prefill_flops(cfg, n_pre)
        prefill = {"value": round(n_pre / sec, 1), "tokens": n_pre, "ms": round(sec * 1e3, 3),
                   "frac": round(flops / sec / (PEAK_TFLOPS["bf16" if elt == 2 else "fp32"] * 1e12), 5),
                   "tflops": round(flops / sec / 1e12, 1),
                   "frac_measured": round(flops / sec / (ceilings["mfma_bf16_tflops"] * 1e12), 5) if elt == 2 else None}
        log(f"prefill {prefill}")

    # ---- decode ----------------------------------------------------------------
    log(f"decode at batch {args.batch}")
    dt, singles, hit_per_layer = run_decode(args.batch, args.steps, args.warmup, single=args.steps)
    singles.sort()
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    context = prompt_len + args.warmup + args.steps // 2
    gbs = decode_bytes(cfg, args.batch, context, elt, hit_per_layer) / (dt / args.steps) / 1e9
    pts = {}
    for b in points:
        log(f"decode at batch {b}")
        steps = max(8, args.steps // 2)
        d, _, _ = run_decode(b, steps, max(2, args.warmup // 2))
        pts[f"decode_b{b}"] = round(b * steps / d, 1)

    line = {
        "metric": f"Qwen1.5-MoE-A2.7B decode tok/s @ batch {args.batch} ({prompt_len}-token prompts)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "step_ms": {"min": round(singles[0] * 1e3, 3), "median": round(singles[len(singles) // 2] * 1e3, 3)},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if elt == 2 else "fp32", "data": "synthetic: seeded random weights and token ids",
        "config": {
            "model": "Qwen1.5-MoE-A2.7B shape", "global_batch": args.batch, "seq_len": context_cap, "prompt_len": prompt_len,
            "parallelism": "single GPU", "layers": args.layers, "layers_of_shape": SHAPE["num_hidden_layers"],
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "experts": cfg.num_experts, "top_k": cfg.num_experts_per_tok,
            "moe_intermediate": cfg.moe_intermediate_size, "shared_intermediate": cfg.shared_expert_intermediate_size,
            "vocab": cfg.vocab_size, "page_size": PAGE,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 5), "frac_measured": round(gbs / ceilings["hbm_read_gbs"], 5),
                     "experts_hit_per_layer": round(hit_per_layer, 1) if hit_per_layer else None},
        "ceilings": ceilings,
        "points": pts,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
