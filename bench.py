#!/usr/bin/python3
"""Benchmark of serving on one MI355X: decode throughput, prefill throughput, rooflines.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L] [--dtype bfloat16]
                    [--shape 7b|14b|32b] [--context N] [--new-tokens G] [--prefill-tokens T]
                    [--workload decode|serve|migurax|nebutar|fotovik|bafulorn] [--only decode|step|prefill] [--all]

The default run has the layer sizes of Qwen2.5-7B (28 layers, hidden 3584, 28 heads, 4 KV heads, head
size 128, intermediate 18944, vocabulary 152064) with random weights and goes through the whole engine
(scheduler, step function with decode steps replayed as HIP graphs and enqueued one ahead, sampler):
8 requests with 2048-token random prompts are prefilled by the engine and generate up to 256 tokens
each, greedily, with no stop token; after W untimed decode steps exactly K decode steps are timed.  It
prints ONE JSON line; ``value`` is decoded tokens per second.  Every figure of the line can be
recomputed from its own fields.  The same line carries

* ``roofline``: the bytes a decode step has to read (``bytes_per_step``: every weight it uses once,
  the embedding rows of the batch, and the cache of the live requests at their mean length over the timed
  steps) / its time, against the 8 TB/s of HBM3E (``frac``) and against the rate at which this GPU
  delivers memory to a kernel that only reads (``frac_measured``; ``measured`` holds that yardstick);
* ``step_function``: the same decode step driven directly (no scheduler): what the scheduler costs;
* ``prefill``: one 2048-token prompt in one step (tokens/s and ms as the mean of three timed runs, ``ms_best`` the
  fastest of them, flops, ``frac`` of the dense matrix-core peak of the dtype, ``frac_measured`` of the rate this
  repository's own large matrix product reaches);
* ``points``: decode tokens/s at batch 1 and batch 64 through the engine; ``points_detail`` gives each
  point's ms per step, bytes per step and fractions.

``--all`` adds the secondary workloads as ``extra`` (``--extra 14b,32b,fp32`` picks among them): Qwen2.5-14B sizes
served through the scheduler (32 requests, prompts 128-4096, 128 new tokens, 512 tokens a step); Qwen2.5-32B sizes
through the engine: one request whose 16384-token prompt the scheduler prefills in portions of 2048 tokens and that
then decodes 512 tokens greedily (``decode_32b_b1_ctx16384``, with the time of its prefill phase), and 16 requests
with 4096-token prompts (``decode_32b_b16_ctx4096``), each with the bare step function on synthetic caches as a
second figure (``step_function``), and the prefill of 16384 tokens as steps of the step function alone; and the same
32B sizes in true 32-bit, all 64 layers (``fp32_32b``: decode at batch 1 through the engine, prefill of 2048 tokens).
``--workload serve`` prints the serving run alone as a line of its own.

``--workload migurax [--size s|m]`` prints a line of its own for the Migurax design (post-norm layers with a matrix-memory
recurrence or attention over a cached latent, dense or routed feed-forwards) at layer sizes that resemble a real model's,
with random weights: prefill of ``--prefill-tokens`` tokens in one step and decode steps at ``--batch`` on ``--context``-token
caches (replayed graphs), beside a Qwen2 model of the same width, layer count and dense feed-forward width; and, under
``kernels``, every kernel that is the design's own alone at those sizes beside the like kernel of the Qwen2 path, each with
the bytes it must move or the operations it must do and the fraction of the GPU's rate that this makes.

``--workload nebutar [--size s|m]`` does the same for the Nebutar design (copies of the residual joined by hyper-connections; attention
with soft-capped scores in chunks beside a gated delta rule; gated experts, some of them the identity), beside the Migurax model of
the same width and layer count (the closest one the framework has: a recurrent state per request and routed experts), and its own
kernels beside the like kernels of the Migurax and Qwen2 paths.

``--workload fotovik [--size s|m]`` does the same for the Fotovik design (a norm before and after every sublayer; attention with a window,
pooled blocks before it and a sink; causal attention with normed queries and keys beside linear attention with fixed decays; a gated
delta rule; dense feed-forwards), beside the Nebutar model of the same width and layer count (the closest one the framework has: two
mixers side by side, a delta rule, a span of layers, the same attention kernels), and its own kernels beside their like.

``--workload bafulorn [--size s|m]`` does the same for the Bafulorn design (a norm before and after every sublayer with weights around zero;
attention over a cached latent in a window with a gate; grouped-query attention whose values are its keys, in a window that keeps the
first tokens; a selective state-space recurrence; gated dense feed-forwards and experts routed by sigmoid scores with a shared expert),
beside the Migurax model of the same width and layer count (the closest one the framework has: latent attention, a recurrent state per
request, routed experts), and the kernels it added or changed beside their like.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}

QWEN25_7B = dict(
    architectures=["Qwen2ForCausalLM"], vocab_size=152064, hidden_size=3584, num_hidden_layers=28,
    num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944, max_position_embeddings=4096,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, use_sliding_window=False,
)
SHAPES = {
    "7b": ("Qwen2.5-7B", QWEN25_7B),
    "14b": ("Qwen2.5-14B", dict(QWEN25_7B, hidden_size=5120, num_hidden_layers=48, num_attention_heads=40,
                                 num_key_value_heads=8, intermediate_size=13824, rms_norm_eps=1e-5,
                                 max_position_embeddings=8192)),
    "32b": ("Qwen2.5-32B", dict(QWEN25_7B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=40,
                                 num_key_value_heads=8, intermediate_size=27648, rms_norm_eps=1e-5,
                                 max_position_embeddings=32768)),
}
CONTEXT = 2048
NEW_TOKENS = 256
PAGE = 16
PREFILL_BUDGET = 8192        # tokens a step of the engine may hold: four 2048-token prompts are prefilled at a time


def parse_args(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=224, help="timed decode steps")
    p.add_argument("--warmup", type=int, default=8, help="untimed decode steps before them")
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--shape", choices=list(SHAPES), default="7b", help="layer sizes")
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    p.add_argument("--context", type=int, default=CONTEXT, help="prompt tokens of each request in the decode runs")
    p.add_argument("--new-tokens", type=int, default=None, help="tokens each request may generate (decode: 256, serve: 128)")
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--workload", choices=["decode", "serve", "migurax", "nebutar", "fotovik", "bafulorn"], default="decode")
    p.add_argument("--size", choices=["s", "m"], default="s", help="migurax, nebutar, fotovik, bafulorn: layer sizes (s: width 2048, m: width 4096)")
    p.add_argument("--requests", type=int, default=32)
    p.add_argument("--prompt-min", type=int, default=128)
    p.add_argument("--prompt-max", type=int, default=4096)
    p.add_argument("--portion", type=int, default=512, help="serve: token budget of a step")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points, the prefill and the yardsticks")
    p.add_argument("--only", choices=["decode", "step", "prefill"], default=None,
                   help="run one part only (for profiling): the engine's decode steps at --batch, the bare step function's, "
                        "or the prefill")
    p.add_argument("--all", action="store_true", help="add the secondary workloads (14B served, 32B prefill and decode, 32B in 32-bit)")
    p.add_argument("--extra", default=None, help="which secondary workloads, comma-separated: 14b, 32b, fp32 (implies --all)")
    return p.parse_args(argv)


def say(msg: str) -> None:
    """A line of progress on standard error (standard output carries the one JSON line)."""
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def build(shape: str, layers: int, dtype: str):
    import torch
    say(f"building {SHAPES[shape][0]} sizes, {layers} layers, {dtype}, random weights")
    from torchlet_amd.engine.loading import build_model
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import RandomTensors

    d = dict(SHAPES[shape][1], num_hidden_layers=layers)
    cfg = config_class(d["architectures"][0]).from_dict(d)
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    # every tensor drawn on the GPU as the model takes it: no second copy of the weights stands by
    # (the 32B sizes in 32-bit are 131 GB of the 288)
    model = build_model(cfg, dtype, tensors=RandomTensors(cfg, seed=2, dtype=store, device="cuda"))
    torch.cuda.empty_cache()
    return cfg, model


def decode_bytes(cfg, model, batch: int, context: float) -> float:
    """Bytes one decode step must read: every weight once (of the embedding only ``batch`` rows)
    and the keys and values of the live requests, ``context`` tokens each."""
    esize = 2 if str(model.dtype).endswith("bfloat16") else 4
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    per_layer = qkv * h + qkv + cfg.num_attention_heads * cfg.head_dim * h + 3 * h * i + 2 * h
    weights = (cfg.num_hidden_layers * per_layer + h + v * h + batch * h) * esize
    kv = batch * context * cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * cfg.head_dim * esize
    return weights + kv


def prefill_flops(cfg, tokens: int) -> float:
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    linear = cfg.num_hidden_layers * (qkv * h + cfg.num_attention_heads * cfg.head_dim * h + 3 * h * i)
    attn = cfg.num_hidden_layers * 2 * cfg.num_attention_heads * cfg.head_dim * tokens * tokens   # causal: half of 4*T^2
    return 2.0 * tokens * linear + attn + 2.0 * v * h


def random_prompts(vocab: int, count: int, length: int, seed: int = 0):
    import torch
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(count)]


def engine_decode(cfg, model, batch: int, steps: int, warmup: int, context: int, new_tokens: int, budget: int = PREFILL_BUDGET) -> dict:
    """``batch`` requests with ``context``-token random prompts through the whole engine: the prompts are
    prefilled by the scheduler (portions under its token budget ``budget``), then every step decodes one token for
    each request.  The graphs of the decode steps are captured before the requests arrive; ``warmup`` decode steps
    are left untimed, ``steps`` are timed.  No stop token; nobody may finish before the timed steps are over."""
    import torch
    from torchlet_amd.engine.config import EngineConfig
    from torchlet_amd.engine.loading import make_engine
    from torchlet_amd.engine.request import Request

    say(f"engine: {batch} requests, {context}-token prompts, {warmup} + {steps} decode steps")
    pages = batch * (-(-(context + new_tokens) // PAGE)) + 1
    engine = make_engine(model, EngineConfig(page_size=PAGE, num_pages=pages, max_slots=batch, max_tokens_per_step=max(budget, batch),
                                             use_graphs=True, lookahead=True, seed=0))
    captured = engine.runner.warm_up(widths=[batch], max_len=context + new_tokens)     # ahead of need, as the Python entry point does
    reqs = [Request(prompt_tokens=p, max_new_tokens=new_tokens, temperature=0.0, stop_token_ids=frozenset())
            for p in random_prompts(cfg.vocab_size, batch, context)]
    engine.add_requests(reqs)
    finished = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    prefill_steps = engine.steps
    while any(not r.output_tokens for r in reqs):          # the prefill phase (with decode tokens of those already through)
        finished += engine.step()
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    prefill_steps = engine.steps - prefill_steps
    ahead = max(len(r.output_tokens) for r in reqs)
    if ahead + warmup + steps >= new_tokens:
        raise SystemExit(f"bench.py: {warmup} + {steps} decode steps after a prefill phase in which a request already generated "
                         f"{ahead} tokens do not fit {new_tokens} new tokens; lower --steps or raise --new-tokens")
    for _ in range(warmup):
        finished += engine.step()
    torch.cuda.synchronize()
    before = [len(r.output_tokens) for r in reqs]
    ctx0 = sum(r.computed_tokens for r in reqs) / batch
    t0 = time.perf_counter()
    for _ in range(steps):
        finished += engine.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.computed_tokens for r in reqs) / batch
    generated = sum(len(r.output_tokens) - b for r, b in zip(reqs, before))
    assert not finished and generated == batch * steps, (len(finished), generated)
    replays, ahead_steps = engine.runner.graph_replays, engine.steps_ahead
    engine.shutdown()
    del engine
    torch.cuda.empty_cache()
    ms = dt * 1e3 / steps
    mean_ctx = (ctx0 + ctx1) / 2.0 + 0.5      # keys a request's token attends to (its own included), averaged over the timed steps
    nbytes = decode_bytes(cfg, model, batch, mean_ctx)
    return {"batch": batch, "steps": steps, "ms_per_step": round(ms, 4), "tokens_per_s": round(batch * 1e3 / ms, 2),
            "mean_context": round(mean_ctx, 1), "bytes_per_step": int(nbytes), "graph_replays": replays, "steps_ahead": ahead_steps,
            "graphs_captured_ahead": captured, "prefill_phase_ms": round(prefill_s * 1e3, 2), "prefill_phase_steps": prefill_steps,
            "prefill_phase_tokens": batch * context}


def fill_context(runner, req_ids, context: int):
    """Give every request ``context`` cached tokens with random keys and values."""
    cache = runner.cache
    for r in req_ids:
        cache.add_request(r)
        if not cache.reserve(r, context):
            raise RuntimeError("cache pool too small for the benchmark")
        cache.commit(r, context)
    for g in cache.groups:
        for plane in g.tensors:
            plane.normal_(0.0, 0.5)


def step_function_decode(cfg, model, batch: int, steps: int, warmup: int, context: int) -> dict:
    """The decode step without the scheduler: the step function and the sampler driven directly, each step
    taking its tokens on the GPU from the sampling of the one before, on caches filled with random keys and
    values of ``context`` tokens (the time of a decode step does not depend on their values)."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    from torchlet_amd.sampling.sampler import Sampler

    say(f"step function: {batch} requests on {context}-token caches, {warmup} + {steps} decode steps")
    pages = batch * (-(-(context + steps + warmup + 2) // PAGE)) + 1
    runner = make_runner(model, page_size=PAGE, num_pages=pages, max_requests=batch, use_graphs=True)
    ids = [f"b{i}" for i in range(batch)]
    fill_context(runner, ids, context)
    sampler = Sampler(0)
    zeros = [0.0] * batch
    logits = runner.step([StepEntry(r, [1 + i], [0]) for i, r in enumerate(ids)])
    drawn = sampler.launch(logits, zeros, zeros, zeros)
    entries = [StepEntry(r, [0], [0]) for r in ids]
    generated = []

    def step():
        nonlocal drawn
        logits = runner.step(entries, device_tokens=(drawn.device, None))
        following = sampler.launch(logits, zeros, zeros, zeros)
        generated.append(drawn.tokens())
        drawn = following

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    assert len(generated) == warmup + steps and all(len(t) == batch for t in generated)
    del runner
    torch.cuda.empty_cache()
    mean_ctx = context + 1 + warmup + steps / 2.0
    return {"batch": batch, "steps": steps, "ms_per_step": round(ms, 4), "tokens_per_s": round(batch * 1e3 / ms, 2),
            "mean_context": round(mean_ctx, 1), "bytes_per_step": int(decode_bytes(cfg, model, batch, mean_ctx))}


def time_prefill(model, tokens: int, repeats: int = 3, context: int = 0):
    """(mean, best) ms of one step that brings ``tokens`` prompt tokens (after ``context`` tokens fed in 2048-token
    steps) over ``repeats`` runs after one that warms up."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner

    say(f"prefill: {tokens} tokens on {context} cached, {repeats} runs")
    runner = make_runner(model, page_size=PAGE, num_pages=-(-(context + tokens) // PAGE) + 2, max_requests=1)
    prompt = random_prompts(model.spec.vocab_size, 1, context + tokens)[0]
    times = []
    for i in range(repeats + 1):
        for a in range(0, context, 2048):
            runner.step([StepEntry("p", prompt[a:min(a + 2048, context)], [])])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("p", prompt[context:], [tokens - 1])])
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        runner.release("p")
        if i:                      # the first run warms up
            times.append(dt)
    del runner
    torch.cuda.empty_cache()
    return sum(times) / len(times), min(times)


def _best_ms(launch, rounds: int = 5, calls: int = 10) -> float:
    """ms of one call of ``launch``: ``calls`` of them back to back between two events (so that the host's
    part in a launch does not count), best of ``rounds`` after a warm-up round."""
    import torch
    best = float("inf")
    for i in range(rounds + 1):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(calls):
            launch()
        end.record()
        torch.cuda.synchronize()
        if i:
            best = min(best, start.elapsed_time(end) / calls)
    return best


def measure_stream_read_gbs() -> float:
    """GB/s at which a kernel that only reads gets 2 GiB from memory (far more than the caches hold)."""
    import torch
    from torchlet_amd.kernels import ops
    data = torch.empty(2 << 30, dtype=torch.uint8, device="cuda")
    data.random_(0, 255)
    ms = _best_ms(lambda: ops.stream_read(data))
    del data
    torch.cuda.empty_cache()
    return (2 << 30) / (ms * 1e-3) / 1e9


def measure_gemm_tflops(dtype) -> float:
    """TFLOP/s of this repository's own matrix product at 8192 x 8192 x 8192 (float32: 4096 cubed)."""
    import torch
    from torchlet_amd.kernels import ops
    n = 8192 if dtype == torch.bfloat16 else 4096
    x = torch.randn((n, n), device="cuda").to(dtype)
    w = torch.randn((n, n), device="cuda").to(dtype)
    out = torch.empty((n, n), dtype=dtype, device="cuda")
    ms = _best_ms(lambda: ops.linear(x, w, None, out), rounds=3, calls=4)
    del x, w, out
    torch.cuda.empty_cache()
    return 2.0 * n ** 3 / (ms * 1e-3) / 1e12


def serve(cfg, model, args) -> dict:
    """Requests through the whole engine: prompts of seeded random lengths, all arriving at
    once, cut into portions under the step's token budget beside the decode tokens of the
    requests that are further on; every request generates ``--new-tokens`` (no stop ids)."""
    import torch
    from torchlet_amd.engine.config import EngineConfig
    from torchlet_amd.engine.loading import make_engine
    from torchlet_amd.engine.request import Request

    g = torch.Generator().manual_seed(1)
    lengths = torch.randint(args.prompt_min, args.prompt_max + 1, (args.requests,), generator=g).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lengths]
    new_tokens = args.serve_new_tokens
    pages = sum(-(-(n + new_tokens) // PAGE) for n in lengths) + 1
    engine = make_engine(model, EngineConfig(page_size=PAGE, num_pages=pages, max_slots=args.requests, max_tokens_per_step=args.portion,
                                             dtype=args.dtype, use_graphs=True, seed=0))

    def run():
        say(f"serving {len(prompts)} requests, {sum(lengths)} prompt tokens, {new_tokens} new tokens each")
        engine.add_requests([Request(prompt_tokens=list(p), max_new_tokens=new_tokens) for p in prompts])
        steps0 = engine.steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = engine.run_until_done()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(done) == len(prompts) and all(len(r.output_tokens) == new_tokens for r in done)
        return dt, engine.steps - steps0

    run()                                   # warms up kernels and captures the decode graphs
    dt, steps = run()
    generated = args.requests * new_tokens
    del engine
    torch.cuda.empty_cache()
    return {
        "metric": f"served tokens/s, {SHAPES[args.shape][0]} shape, {args.requests} requests, prompts {args.prompt_min}-{args.prompt_max}, "
                  f"{new_tokens} new tokens each, at most {args.portion} tokens a step, one MI355X",
        "value": round((sum(lengths) + generated) / dt, 1), "unit": "tokens/s (prompt + generated)",
        "generated_tokens_per_s": round(generated / dt, 1), "prompt_tokens": sum(lengths), "generated_tokens": generated,
        "seconds": round(dt, 3), "engine_steps": steps, "ms_per_step": round(dt * 1e3 / steps, 3),
        "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "layers": cfg.num_hidden_layers,
        "data": "synthetic: seeded random weights, prompt lengths and token ids",
    }


def _with_roofline(r: dict) -> dict:
    gbs = r["bytes_per_step"] / (r["ms_per_step"] * 1e-3) / 1e9
    return dict(r, achieved_gbs=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 4))


def secondary_14b(args) -> dict:
    """14B sizes, all 48 layers, served: 32 requests, prompts 128-4096, 128 new tokens, 512 tokens a step."""
    import torch
    cfg, model = build("14b", SHAPES["14b"][1]["num_hidden_layers"], args.dtype)
    a = argparse.Namespace(**vars(args))
    a.shape, a.requests, a.prompt_min, a.prompt_max, a.serve_new_tokens, a.portion = "14b", 32, 128, 4096, 128, 512
    s = serve(cfg, model, a)
    del model
    torch.cuda.empty_cache()
    return {"serve_14b": {k: s[k] for k in ("value", "unit", "generated_tokens_per_s", "prompt_tokens", "generated_tokens", "seconds",
                                            "engine_steps", "ms_per_step", "layers")}}


def secondary_32b(args) -> dict:
    """32B sizes, all 64 layers, through the engine: one request with a 16384-token prompt (prefilled by the
    scheduler in portions of 2048 tokens) that decodes 512 tokens greedily, and 16 requests with 4096-token
    prompts; beside each the bare step function on synthetic caches, and the long prefill as steps of the step
    function alone."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    out = {}
    cfg, model = build("32b", SHAPES["32b"][1]["num_hidden_layers"], args.dtype)
    tokens = 16384
    runner = make_runner(model, page_size=PAGE, num_pages=-(-tokens // PAGE) + 2, max_requests=1)
    prompt = random_prompts(cfg.vocab_size, 1, tokens)[0]
    times = []
    for rep in range(3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for a0 in range(0, tokens, 2048):
            runner.step([StepEntry("p", prompt[a0:a0 + 2048], [2047] if a0 + 2048 == tokens else [])])
        torch.cuda.synchronize()
        total = time.perf_counter() - t0
        runner.release("p")
        if rep:
            times.append(total)
    del runner
    torch.cuda.empty_cache()
    mean, best = sum(times) / len(times), min(times)
    flops = sum(prefill_flops_step(cfg, 2048, a0) for a0 in range(0, tokens, 2048))
    out["prefill_32b_16384"] = {"tokens": tokens, "steps_of": 2048, "ms": round(mean * 1e3, 2), "ms_best": round(best * 1e3, 2), "runs": len(times),
                                "value": round(tokens / mean, 1), "flops": flops,
                                "frac": round(flops / mean / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12), 4), "layers": cfg.num_hidden_layers}
    # (name, requests, prompt tokens, new tokens, timed decode steps, token budget of a step)
    for name, batch, context, new_tokens, steps, budget in (("decode_32b_b1_ctx16384", 1, 16384, 512, 480, 2048),
                                                           ("decode_32b_b16_ctx4096", 16, 4096, 128, 96, 8192)):
        r = _with_roofline(engine_decode(cfg, model, batch, steps, 8, context, new_tokens, budget=budget))
        r["prefill_phase_flops"] = batch * sum(prefill_flops_step(cfg, min(2048, context - a0), a0) for a0 in range(0, context, 2048))
        r["prefill_phase_tokens_per_s"] = round(r["prefill_phase_tokens"] / (r["prefill_phase_ms"] * 1e-3), 1)
        r["step_function"] = _with_roofline(step_function_decode(cfg, model, batch, 32, 4, context))
        r["layers"], r["new_tokens"], r["token_budget"] = cfg.num_hidden_layers, new_tokens, budget
        out[name] = r
    del model
    torch.cuda.empty_cache()
    return out


def secondary_fp32_32b(args) -> dict:
    """32B sizes in true 32-bit, all 64 layers (131 GB of weights): decode at batch 1 through the engine after a
    2048-token prompt, and the prefill of 2048 tokens as one step."""
    import torch
    cfg, model = build("32b", SHAPES["32b"][1]["num_hidden_layers"], "float32")
    r = _with_roofline(engine_decode(cfg, model, 1, 32, 4, 2048, 64, budget=2048))
    pms, pbest = time_prefill(model, 2048, repeats=2)
    flops = prefill_flops(cfg, 2048)
    out = {"dtype": "fp32", "layers": cfg.num_hidden_layers, "weight_bytes": int(decode_bytes(cfg, model, 1, 0)),
           "decode_b1": r,
           "prefill": {"value": round(2048 * 1e3 / pms, 1), "tokens": 2048, "ms": round(pms, 2), "ms_best": round(pbest, 2), "runs": 2,
                       "flops": flops, "frac": round(flops / (pms * 1e-3) / (MFMA_PEAK_TFLOPS["float32"] * 1e12), 4)}}
    del model
    torch.cuda.empty_cache()
    return {"fp32_32b": out}


def secondary(args) -> dict:
    """The secondary workloads, each at its full layer count."""
    which = [w.strip() for w in (args.extra or "14b,32b,fp32").split(",") if w.strip()]
    parts = {"14b": secondary_14b, "32b": secondary_32b, "fp32": secondary_fp32_32b}
    unknown = [w for w in which if w not in parts]
    if unknown:
        raise SystemExit(f"bench.py: --extra knows 14b, 32b and fp32, not {', '.join(unknown)}")
    out = {}
    for w in which:
        out.update(parts[w](args))
    return out


def prefill_flops_step(cfg, tokens: int, context: int) -> float:
    """Flops of a step of ``tokens`` prompt tokens on top of ``context`` cached ones (no logits)."""
    h, i = cfg.hidden_size, cfg.intermediate_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    linear = cfg.num_hidden_layers * (qkv * h + cfg.num_attention_heads * cfg.head_dim * h + 3 * h * i)
    keys = tokens * context + tokens * tokens / 2.0
    attn = cfg.num_hidden_layers * 4 * cfg.num_attention_heads * cfg.head_dim * keys
    return 2.0 * tokens * linear + attn


# ---------------------------------------------------------------------------------------------- the Migurax design

def _latent_layer(heads, dim, rot, vdim, rank, q_rank, mlp):
    return dict(type="latent_attention", mlp=mlp, mixer=dict(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, kv_rank=rank, q_rank=q_rank,
                                                             scale=(dim + rot) ** -0.5, rot=dict(base=10000.0, dims=rot)))


def migurax_sizes(size: str) -> tuple[dict, dict]:
    """A Migurax configuration of four layers (recurrence + dense, latent attention + routed twice, recurrence + routed) and the
    Qwen2 configuration of the same width, layer count, vocabulary and dense feed-forward width."""
    width, heads, ff, experts, eff, top, q_rank, mheads = dict(s=(2048, 16, 8192, 16, 1024, 2, 768, 4), m=(4096, 32, 16384, 32, 2048, 4, 1536, 8))[size]
    moe = dict(kind="moe", expert=dict(ff=eff), router=dict(experts=experts, top=top))
    rec = dict(heads=mheads, dim=256, vdim=512, gate_cap=12.0)
    layers = [dict(type="mlstm", mixer=rec, mlp=dict(kind="dense", ff=ff)), _latent_layer(heads, 128, 64, 128, 512, q_rank, moe),
              _latent_layer(heads, 128, 64, 128, 512, q_rank, moe), dict(type="mlstm", mixer=rec, mlp=moe)]
    ours = dict(architecture="Migurax", vocab=32000, width=width, postln_alpha=1.0, norm=dict(eps=1e-5), layers=layers, max_positions=8192)
    like = dict(QWEN25_7B, vocab_size=32000, hidden_size=width, num_hidden_layers=4, num_attention_heads=heads, num_key_value_heads=heads // 4,
                intermediate_size=ff * 2 // 3 // 256 * 256, max_position_embeddings=8192)      # three matrices of 2/3 the width: as many weights as two
    return ours, like


def _build_from(d: dict, dtype: str):
    import torch
    from torchlet_amd.engine.loading import build_model
    from torchlet_amd.registry import architecture_of, config_class
    from torchlet_amd.weights.random_init import RandomTensors
    cfg = config_class(architecture_of(d)).from_dict(d)
    model = build_model(cfg, dtype, tensors=RandomTensors(cfg, seed=2, dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32, device="cuda"))
    torch.cuda.empty_cache()
    return cfg, model


def _decode_ms(model, batch: int, steps: int, warmup: int, context: int) -> float:
    """ms of a decode step of the bare step function (replayed graphs, tokens taken on the GPU from the sampling of the step
    before) on caches of ``context`` tokens with random contents."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    from torchlet_amd.sampling.sampler import Sampler
    runner = make_runner(model, page_size=PAGE, num_pages=batch * (-(-(context + steps + warmup + 2) // PAGE)) + 1, max_requests=batch, use_graphs=True)
    ids = [f"b{i}" for i in range(batch)]
    fill_context(runner, ids, context)
    sampler, zeros = Sampler(0), [0.0] * batch
    drawn = sampler.launch(runner.step([StepEntry(r, [1 + i], [0]) for i, r in enumerate(ids)]), zeros, zeros, zeros)
    entries = [StepEntry(r, [0], [0]) for r in ids]

    def step():
        nonlocal drawn
        drawn = sampler.launch(runner.step(entries, device_tokens=(drawn.device, None)), zeros, zeros, zeros)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    assert runner.graph_replays >= steps or not runner.use_graphs
    del runner
    torch.cuda.empty_cache()
    return ms


def _weight_bytes(model) -> int:
    """Bytes of every tensor a model's parts hold on the GPU (what a decode step reads at most of them)."""
    import torch
    seen, total = set(), 0
    for part in list(model.parts()) + [model]:
        for v in vars(part).values():
            if isinstance(v, torch.Tensor) and v.is_cuda and v.data_ptr() not in seen:
                seen.add(v.data_ptr())
                total += v.numel() * v.element_size()
    return total


def migurax_kernels(ours: dict, like: dict, batch: int, context: int, tokens: int) -> list[dict]:
    """Each kernel that is the design's own, alone, at the sizes of ``ours``, in a decode step of ``batch`` requests on ``context``
    cached tokens and in a prompt of ``tokens`` tokens, beside the like kernel of the Qwen2 path at the sizes of ``like``.  ``frac``:
    bytes that must move / time against 8 TB/s, or operations / time against the matrix cores' bfloat16 rate (against the 32-bit
    vector rate for the recurrence, which the design wants in 32-bit)."""
    import torch
    from torchlet_amd.kernels import ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, kind, launch, nbytes=0.0, flops=0.0, peak=MFMA_PEAK_TFLOPS["bfloat16"]):
        ms = _best_ms(launch, rounds=3, calls=5)
        row = {"kernel": name, "like": kind, "ms": round(ms, 4)}
        if nbytes:
            row.update(bytes=int(nbytes), frac=round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), bound="hbm")
        else:
            row.update(flops=flops, frac=round(flops / (ms * 1e-3) / (peak * 1e12), 4), bound="flops")
        rows.append(row)
        say(f"  {name}: {ms:.4f} ms, {row['frac']} of its bound")

    def tables(n_req, total):
        blocks = -(-total // PAGE)
        table = (torch.arange(n_req * blocks, dtype=torch.int32, device=dev) + 1).view(n_req, blocks)
        return table, n_req * blocks + 1

    rec = ours["layers"][0]["mixer"]
    lat = ours["layers"][1]["mixer"]
    moe = ours["layers"][1]["mlp"]
    width = ours["width"]
    # ---- the recurrence: a decode step reads and writes every state once; a prompt does 4 operations per state element and token
    h, d, v = rec["heads"], rec["dim"], rec["vdim"]
    for name, T, reqs in (("mlstm_scan decode", batch, batch), (f"mlstm_scan prompt {tokens}", tokens, 1)):
        qkv = torch.randn(T, 2 * h * d + 2 * h * v, device=dev).to(bf)
        gates = torch.randn(T, 2 * h, device=dev)
        state = torch.zeros(reqs + 1, h, d * v + d + 1, device=dev)
        out = torch.empty(T, h * v, device=dev)
        slots = torch.arange(reqs, dtype=torch.int32, device=dev)
        indptr = (torch.arange(reqs + 1, dtype=torch.int32, device=dev) * (T // reqs))
        launch = lambda: ops.mlstm_scan(qkv, h * d, 2 * h * d, gates, state, slots, indptr, out, h, d, v, 12.0, d ** -0.5, 1e-6)
        if reqs > 1:
            add(name, "paged_attention decode", launch, nbytes=2.0 * reqs * h * d * v * 4)
        else:
            add(name, "paged_attention_prompt", launch, flops=4.0 * T * h * d * v, peak=MFMA_PEAK_TFLOPS["float32"])
    # ---- the latent attention: a decode step reads every cached row once; a prompt's scores and sums
    H, R, rot = lat["heads"], lat["kv_rank"], lat["rot_dim"]
    D = R + rot
    sink = torch.zeros(H, device=dev)
    for name, T, reqs, ctx in (("latent_attention decode", batch, batch, context), (f"latent_attention prompt {tokens}", tokens, 1, 0)):
        total = ctx + T // reqs
        table, pages = tables(reqs, total)
        plane = (torch.randn(pages, 1, PAGE, D, device=dev) * 0.3).to(bf)
        q = (torch.randn(T, H * D, device=dev) * 0.3).to(bf)
        out = torch.empty(T, H * R, dtype=bf, device=dev)
        ctx_lens = torch.full((reqs,), ctx, dtype=torch.int32, device=dev)
        tq = ops.latent_tile_tokens(H, ops.LATENT_MFMA_ROWS if ops.latent_attention_mfma_fits(bf, H, R, rot) else ops.LATENT_ATTENTION_ROWS)
        if reqs > 1:
            launch = lambda: ops.latent_attention(q, out, plane, table, None, ctx_lens, None, None, T, tq, H, R, rot, PAGE, 0.07, sink,
                                                  max(1, min(ops.compute_units() // max(1, T * -(-H // 16)), total // 64, 64)), max_new_tokens=1)
            add(name, "paged_attention decode", launch, nbytes=float(reqs) * total * D * 2)
        else:
            tiles = -(-T // tq)
            tile_req = torch.zeros(tiles, dtype=torch.int32, device=dev)
            tile_tok0 = torch.arange(tiles, dtype=torch.int32, device=dev) * tq
            indptr = torch.tensor([0, T], dtype=torch.int32, device=dev)
            launch = lambda: ops.latent_attention(q, out, plane, table, indptr, ctx_lens, tile_req, tile_tok0, tiles, tq, H, R, rot, PAGE, 0.07, sink, 1)
            add(name, "paged_attention_prompt", launch, flops=float(H) * (2 * D + 2 * R) * T * T / 2)
    # ---- the products over heads (query onto the latent, values from the latent) and over experts
    for name, T in (("heads_linear decode", batch), (f"heads_linear prompt {tokens}", tokens)):
        x = torch.randn(T, H * (lat["dim"] + rot), device=dev).to(bf)
        w = torch.randn(H, R, lat["dim"], device=dev).to(bf)
        out = torch.empty(T, H * D, dtype=bf, device=dev)
        launch = lambda: ops.heads_linear(x, lat["dim"] + rot, w, out, D)
        if T == batch:
            add(name, "linear (few rows)", launch, nbytes=float(w.numel()) * 2)
        else:
            add(name, "linear (many rows)", launch, flops=2.0 * T * H * R * lat["dim"])
    E, top, ff = moe["router"]["experts"], moe["router"]["top"], moe["expert"]["ff"]
    for name, T in (("experts_linear decode", batch), (f"experts_linear prompt {tokens}", tokens)):
        x = torch.randn(T, width, device=dev).to(bf)
        w_up = (torch.randn(E, ff, width, device=dev) * 0.02).to(bf)
        logits = torch.randn(T, E, device=dev)
        weights, offsets, slot_token, pair_slot = ops.route(logits, top)
        z = torch.empty(T * top, ff, dtype=bf, device=dev)
        launch = lambda: ops.experts_linear(x, slot_token, w_up, offsets, z, "relu2")
        if T == batch:
            add(name, "linear (few rows)", launch, nbytes=float(min(E, T * top)) * ff * width * 2)
        else:
            add(name, "linear (many rows)", launch, flops=2.0 * T * top * ff * width)
    # ---- the like kernels of the Qwen2 path at the like sizes
    qh, kvh, hd = like["num_attention_heads"], like["num_key_value_heads"], 128
    table, pages = tables(batch, context + 1)
    k_plane = (torch.randn(pages, kvh, PAGE, hd, device=dev) * 0.3).to(bf)
    v_plane = (torch.randn(pages, kvh, hd, PAGE, device=dev) * 0.3).to(bf)
    q = (torch.randn(batch, qh * hd, device=dev) * 0.3).to(bf)
    out = torch.empty(batch, qh * hd, dtype=bf, device=dev)
    ctx_lens = torch.full((batch,), context, dtype=torch.int32, device=dev)
    add("paged_attention decode (Qwen2 path)", "", lambda: ops.paged_attention(q, out, k_plane, v_plane, table, None, ctx_lens, None, None, batch, ops.attention_tile_tokens(qh, kvh), qh, kvh, hd, PAGE,
                                                                              0, hd ** -0.5, 8, waves=8), nbytes=2.0 * batch * (context + 1) * kvh * hd * 2)
    table, pages = tables(1, tokens)
    k_plane = (torch.randn(pages, kvh, PAGE, hd, device=dev) * 0.3).to(bf)
    v_plane = (torch.randn(pages, kvh, hd, PAGE, device=dev) * 0.3).to(bf)
    q = (torch.randn(tokens, qh * hd, device=dev) * 0.3).to(bf)
    out = torch.empty(tokens, qh * hd, dtype=bf, device=dev)
    tq = ops.prompt_attention_tile_tokens(qh, kvh)
    tiles = -(-tokens // tq)
    tile_req = torch.zeros(tiles, dtype=torch.int32, device=dev)
    tile_tok0 = torch.arange(tiles, dtype=torch.int32, device=dev) * tq
    indptr = torch.tensor([0, tokens], dtype=torch.int32, device=dev)
    zero = torch.zeros(1, dtype=torch.int32, device=dev)
    add(f"paged_attention_prompt {tokens} (Qwen2 path)", "", lambda: ops.paged_attention_prompt(q, out, k_plane, v_plane, table, indptr, zero, tile_req, tile_tok0, tiles, tq,
                                                                                                qh, kvh, hd, PAGE, 0, hd ** -0.5, max_total_len=tokens),
        flops=float(qh) * 4 * hd * tokens * tokens / 2)
    inter = like["intermediate_size"]
    for name, T in (("linear decode (Qwen2 path, down projection)", batch), (f"linear prompt {tokens} (Qwen2 path, down projection)", tokens)):
        x = torch.randn(T, inter, device=dev).to(bf)
        w = (torch.randn(width, inter, device=dev) * 0.02).to(bf)
        out = torch.empty(T, width, dtype=bf, device=dev)
        launch = lambda: ops.linear(x, w, None, out)
        if T == batch:
            add(name, "", launch, nbytes=float(w.numel()) * 2)
        else:
            add(name, "", launch, flops=2.0 * T * width * inter)
    return rows


def migurax(args) -> dict:
    import torch
    ours, like = migurax_sizes(args.size)
    out = {"metric": f"Migurax design, size {args.size} (width {ours['width']}, 4 layers), prefill of {args.prefill_tokens} tokens and decode at batch "
                     f"{args.batch} on {args.context}-token caches, beside Qwen2 sizes of equal width, one MI355X",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
           "data": "synthetic: seeded random weights, token ids and cache contents", "config": {"migurax": ours, "qwen2": like}}
    for key, d in (("migurax", ours), ("qwen2", like)):
        say(f"building the {key} model")
        cfg, model = _build_from(d, args.dtype)
        pms, pbest = time_prefill(model, args.prefill_tokens)
        dms = _decode_ms(model, args.batch, min(args.steps, 64), args.warmup, args.context)
        out[key] = {"weight_bytes": _weight_bytes(model),
                    "prefill": {"tokens": args.prefill_tokens, "ms": round(pms, 3), "ms_best": round(pbest, 3), "tokens_per_s": round(args.prefill_tokens * 1e3 / pms, 1)},
                    "decode": {"batch": args.batch, "context": args.context, "ms_per_step": round(dms, 4), "tokens_per_s": round(args.batch * 1e3 / dms, 1)}}
        say(f"{key}: {out[key]}")
        del model
        torch.cuda.empty_cache()
    out["value"] = out["migurax"]["decode"]["tokens_per_s"]
    if args.dtype == "bfloat16" and not args.no_points:
        out["kernels"] = migurax_kernels(ours, like, args.batch, args.context, args.prefill_tokens)
    return out


# ---------------------------------------------------------------------------------------------- the Nebutar design

def nebutar_sizes(size: str) -> dict:
    """A Nebutar configuration of four layers (the middle two form a span that runs once) at the width of the Migurax sizes: attention
    heads of 128 + 128 in chunks of 1024, a delta rule with heads of 128 x 128 behind convolutions of four taps, gated experts."""
    width, heads, experts, eff, top, streams = dict(s=(2048, 16, 16, 1024, 2, 4), m=(4096, 32, 32, 2048, 4, 4))[size]
    left = dict(heads=heads, kv_heads=heads // 4, dim=128, vdim=128, scale=128 ** -0.5, softcap=30.0, mask=dict(size=1024))
    right = dict(heads=heads, kv_heads=heads // 2, dim=128, vdim=128, conv=4)
    layer = dict(type="parallel", mixer=dict(left=left, right=right, left_scale=0.7, right_scale=0.7),
                 mlp=dict(kind="moe", expert=dict(ff=eff), router=dict(experts=experts, identity=2, top=top)))
    return dict(architecture="Nebutar", vocab=32000, width=width, max_positions=8192, norm=dict(eps=1e-5), embedding=dict(scale=1.0),
                streams=streams, loop=dict(start=1, stop=3, times=1), layers=[layer] * 4)


def nebutar_kernels(ours: dict, like: dict, batch: int, context: int, tokens: int) -> list[dict]:
    """Each kernel that is the design's own, alone, at the sizes of ``ours``, in a decode step of ``batch`` requests on ``context`` cached
    tokens and in a prompt of ``tokens`` tokens, beside the like kernel of the Migurax or Qwen2 path.  ``frac``: bytes that must move /
    time against 8 TB/s, or operations / time against the matrix cores' bfloat16 rate (against the 32-bit rate for the recurrences,
    which the designs want in 32-bit)."""
    import torch
    from torchlet_amd.kernels import ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, kind, launch, nbytes=0.0, flops=0.0, peak=MFMA_PEAK_TFLOPS["bfloat16"]):
        ms = _best_ms(launch, rounds=3, calls=5)
        row = {"kernel": name, "like": kind, "ms": round(ms, 4)}
        if nbytes:
            row.update(bytes=int(nbytes), frac=round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), bound="hbm")
        else:
            row.update(flops=flops, frac=round(flops / (ms * 1e-3) / (peak * 1e12), 4), bound="flops")
        rows.append(row)
        say(f"  {name}: {ms:.4f} ms, {row['frac']} of its bound")

    def tables(n_req, total):
        blocks = -(-total // PAGE)
        table = (torch.arange(n_req * blocks, dtype=torch.int32, device=dev) + 1).view(n_req, blocks)
        return table, n_req * blocks + 1

    mixer, moe, width, S = ours["layers"][0]["mixer"], ours["layers"][0]["mlp"], ours["width"], ours["streams"]
    left, right = mixer["left"], mixer["right"]
    # ---- the delta rule beside the matrix-memory recurrence: a decode step reads and writes every state once; a prompt does 6 operations
    #      per state element and token (two sums over the rows and the update), the matrix memory 4
    h, g, d, v = right["heads"], right["kv_heads"], right["dim"], right["vdim"]
    C = 2 * g * d + h * v
    for name, T, reqs in (("delta_scan decode", batch, batch), (f"delta_scan prompt {tokens}", tokens, 1)):
        qkv = torch.randn(T, C, device=dev) * 0.1
        gates = torch.rand(T, 2 * h, device=dev) * 0.5 + 0.5
        state = torch.zeros(reqs + 1, h * d * v, device=dev)
        out = torch.empty(T, h * v, device=dev)
        slots = torch.arange(reqs, dtype=torch.int32, device=dev)
        indptr = (torch.arange(reqs + 1, dtype=torch.int32, device=dev) * (T // reqs))
        launch = lambda: ops.delta_scan(qkv, gates, state, slots, indptr, out, h, g, d, v, max_new_tokens=T // reqs)
        if reqs > 1:
            add(name, "mlstm_scan decode", launch, nbytes=2.0 * reqs * h * d * v * 4)
        else:
            add(name, f"mlstm_scan prompt {tokens}", launch, flops=6.0 * T * h * d * v, peak=MFMA_PEAK_TFLOPS["float32"])
    rec = like["layers"][0]["mixer"]
    mh, md, mv = rec["heads"], rec["dim"], rec["vdim"]
    for name, T, reqs in (("mlstm_scan decode", batch, batch), (f"mlstm_scan prompt {tokens}", tokens, 1)):
        qkv = torch.randn(T, 2 * mh * md + 2 * mh * mv, device=dev).to(bf)
        gates = torch.randn(T, 2 * mh, device=dev)
        state = torch.zeros(reqs + 1, mh, md * mv + md + 1, device=dev)
        out = torch.empty(T, mh * mv, device=dev)
        slots = torch.arange(reqs, dtype=torch.int32, device=dev)
        indptr = (torch.arange(reqs + 1, dtype=torch.int32, device=dev) * (T // reqs))
        launch = lambda: ops.mlstm_scan(qkv, mh * md, 2 * mh * md, gates, state, slots, indptr, out, mh, md, mv, 12.0, md ** -0.5, 1e-6)
        if reqs > 1:
            add(name + " (Migurax path)", "", launch, nbytes=2.0 * reqs * mh * md * mv * 4)
        else:
            add(name + " (Migurax path)", "", launch, flops=4.0 * T * mh * md * mv, peak=MFMA_PEAK_TFLOPS["float32"])
    # ---- what the delta rule reads: convolutions, silu, unit vectors, gates (reads the projections once, writes 32-bit numbers once)
    for name, T, reqs in (("delta_prepare decode", batch, batch), (f"delta_prepare prompt {tokens}", tokens, 1)):
        proj = torch.randn(T, C + h * v, device=dev).to(bf)
        conv_w = torch.randn(C, right["conv"], device=dev)
        gates = torch.randn(T, 2 * h, device=dev)
        a_log, dt_bias = torch.zeros(h, device=dev), torch.zeros(h, device=dev)
        state = torch.zeros(reqs + 1, (right["conv"] - 1) * C, device=dev)
        slots = torch.arange(reqs, dtype=torch.int32, device=dev)
        indptr = (torch.arange(reqs + 1, dtype=torch.int32, device=dev) * (T // reqs))
        token_req = torch.arange(T, dtype=torch.int32, device=dev) // (T // reqs)
        out = torch.empty(T, C, device=dev)
        launch = lambda: ops.delta_prepare(proj[:, :C], conv_w, gates, a_log, dt_bias, state, 0, slots, indptr, token_req, out, h, g, d, v, right["conv"], d ** -0.5, 1e-6)
        add(name, "rope_cache_write", launch, nbytes=float(T) * C * (2 + 4) + 2.0 * reqs * (right["conv"] - 1) * C * 4)
    # ---- attention with cap and chunks beside the Qwen2 path's attention: a decode step reads the cached keys and values it may see
    #      once; a prompt's scores and sums (only inside the chunks)
    H, G, dk, dv, chunk = left["heads"], left["kv_heads"], left["dim"], left["vdim"], left["mask"]["size"]
    for name, T, reqs, ctx in (("local_attention decode", batch, batch, context - 1), (f"local_attention prompt {tokens}", tokens, 1, 0)):
        total = ctx + T // reqs
        table, pages = tables(reqs, total)
        k_plane = (torch.randn(pages, G, PAGE, dk, device=dev) * 0.3).to(bf)
        v_plane = (torch.randn(pages, G, dv, PAGE, device=dev) * 0.3).to(bf)
        q = (torch.randn(T, H * dk, device=dev) * 0.3).to(bf)
        out = torch.empty(T, H * dv, dtype=bf, device=dev)
        token_req = torch.arange(T, dtype=torch.int32, device=dev) // (T // reqs)
        positions = (torch.arange(T, dtype=torch.int32, device=dev) % (T // reqs)) + ctx
        if reqs == 1:
            n_tiles = -(-T // ops.LOCAL_ATTENTION_TILE_TOKENS)
            tiles = (torch.tensor([0, T], dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev),
                     torch.zeros(n_tiles, dtype=torch.int32, device=dev), torch.arange(n_tiles, dtype=torch.int32, device=dev) * ops.LOCAL_ATTENTION_TILE_TOKENS, n_tiles)
        else:           # one token per request: a tile per request, no tile list
            tiles = (torch.arange(reqs + 1, dtype=torch.int32, device=dev), torch.full((reqs,), ctx, dtype=torch.int32, device=dev), None, None, reqs)
        launch = lambda: ops.local_attention(q, out, k_plane, v_plane, table, token_req, positions, H, G, dk, dv, PAGE, left["scale"], left["softcap"], chunk, 0, 0.7,
                                             tiles=tiles)
        if reqs > 1:
            seen = ctx % chunk + 1                      # keys of the chunk the decoded token lies in
            add(name, "paged_attention decode", launch, nbytes=float(reqs) * seen * G * (dk + dv) * 2)
        else:
            pairs = sum(p % chunk + 1 for p in range(T))
            add(name, f"paged_attention_prompt {tokens}", launch, flops=2.0 * H * (dk + dv) * pairs)
    qh, kvh, hd = H, G, 128
    table, pages = tables(batch, context + 1)
    k_plane = (torch.randn(pages, kvh, PAGE, hd, device=dev) * 0.3).to(bf)
    v_plane = (torch.randn(pages, kvh, hd, PAGE, device=dev) * 0.3).to(bf)
    q = (torch.randn(batch, qh * hd, device=dev) * 0.3).to(bf)
    out = torch.empty(batch, qh * hd, dtype=bf, device=dev)
    ctx_lens = torch.full((batch,), context, dtype=torch.int32, device=dev)
    add("paged_attention decode (Qwen2 path)", "", lambda: ops.paged_attention(q, out, k_plane, v_plane, table, None, ctx_lens, None, None, batch, ops.attention_tile_tokens(qh, kvh), qh, kvh, hd, PAGE,
                                                                              0, hd ** -0.5, 8, waves=8), nbytes=2.0 * batch * (context + 1) * kvh * hd * 2)
    table, pages = tables(1, tokens)
    k_plane = (torch.randn(pages, kvh, PAGE, hd, device=dev) * 0.3).to(bf)
    v_plane = (torch.randn(pages, kvh, hd, PAGE, device=dev) * 0.3).to(bf)
    q = (torch.randn(tokens, qh * hd, device=dev) * 0.3).to(bf)
    out = torch.empty(tokens, qh * hd, dtype=bf, device=dev)
    tq = ops.prompt_attention_tile_tokens(qh, kvh)
    tiles = -(-tokens // tq)
    tile_req = torch.zeros(tiles, dtype=torch.int32, device=dev)
    tile_tok0 = torch.arange(tiles, dtype=torch.int32, device=dev) * tq
    indptr = torch.tensor([0, tokens], dtype=torch.int32, device=dev)
    zero = torch.zeros(1, dtype=torch.int32, device=dev)
    add(f"paged_attention_prompt {tokens} (Qwen2 path)", "", lambda: ops.paged_attention_prompt(q, out, k_plane, v_plane, table, indptr, zero, tile_req, tile_tok0, tiles, tq,
                                                                                                qh, kvh, hd, PAGE, 0, hd ** -0.5, max_total_len=tokens),
        flops=float(qh) * 4 * hd * tokens * tokens / 2)
    # ---- the norm over the copies of the residual beside the plain residual's norm: reads and writes every copy once
    for name, T in (("streams_norm decode", batch), (f"streams_norm prompt {tokens}", tokens)):
        x = torch.randn(S, T, width, device=dev)
        pen = torch.randn(T, width, device=dev).to(bf)
        fold = (torch.eye(S, device=dev), torch.ones(S, device=dev))
        read = torch.ones(S, device=dev)
        w, b = torch.ones(width, device=dev), torch.zeros(width, device=dev)
        out = torch.empty(T, width, dtype=bf, device=dev)
        add(name, "add_rmsnorm", lambda: ops.streams_norm(x, pen, fold, read, "layernorm", w, b, 1e-5, out), nbytes=float(T) * width * (8 * S + 4))
        res = torch.randn(T, width, device=dev)
        wb = torch.ones(width, dtype=bf, device=dev)
        add(name.replace("streams_norm", "add_rmsnorm") + " (Qwen2 path)", "", lambda: ops.add_rmsnorm(res, pen, wb, 1e-5, out), nbytes=float(T) * width * 12)
    # ---- the gated experts' first product (gate and up in pairs of columns) beside the Migurax path's (one matrix, squared relu)
    E, top, ff = moe["router"]["experts"], moe["router"]["top"], moe["expert"]["ff"]
    for name, T in (("experts_linear gated decode", batch), (f"experts_linear gated prompt {tokens}", tokens)):
        x = torch.randn(T, width, device=dev).to(bf)
        w_up = (torch.randn(E, 2 * ff, width, device=dev) * 0.02).to(bf)
        logits = torch.randn(T, E + moe["router"]["identity"], device=dev)
        weights, offsets, slot_token, pair_slot = ops.route(logits, top, "all", None)
        z = torch.empty(T * top, ff, dtype=bf, device=dev)
        real = int(offsets[E])
        launch = lambda: ops.experts_linear(x, slot_token, w_up, offsets, z, "silu_pairs")
        if T == batch:
            add(name, "experts_linear decode", launch, nbytes=float(min(E, real)) * 2 * ff * width * 2)
        else:
            add(name, f"experts_linear prompt {tokens}", launch, flops=2.0 * real * 2 * ff * width)
        w_one = (torch.randn(E, ff, width, device=dev) * 0.02).to(bf)
        weights, offsets1, slot_token1, pair_slot = ops.route(torch.randn(T, E, device=dev), top)
        launch = lambda: ops.experts_linear(x, slot_token1, w_one, offsets1, z, "relu2")
        if T == batch:
            add(name.replace(" gated", "") + " (Migurax path)", "", launch, nbytes=float(min(E, T * top)) * ff * width * 2)
        else:
            add(name.replace(" gated", "") + " (Migurax path)", "", launch, flops=2.0 * T * top * ff * width)
    return rows


def nebutar(args) -> dict:
    import torch
    ours = nebutar_sizes(args.size)
    like, _ = migurax_sizes(args.size)
    out = {"metric": f"Nebutar design, size {args.size} (width {ours['width']}, 4 layers), prefill of {args.prefill_tokens} tokens and decode at batch "
                     f"{args.batch} on {args.context}-token caches, beside the Migurax design at equal width and layer count, one MI355X",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
           "data": "synthetic: seeded random weights, token ids and cache contents", "config": {"nebutar": ours, "migurax": like}}
    for key, d in (("nebutar", ours), ("migurax", like)):
        say(f"building the {key} model")
        cfg, model = _build_from(d, args.dtype)
        pms, pbest = time_prefill(model, args.prefill_tokens)
        dms = _decode_ms(model, args.batch, min(args.steps, 64), args.warmup, args.context)
        out[key] = {"weight_bytes": _weight_bytes(model),
                    "prefill": {"tokens": args.prefill_tokens, "ms": round(pms, 3), "ms_best": round(pbest, 3), "tokens_per_s": round(args.prefill_tokens * 1e3 / pms, 1)},
                    "decode": {"batch": args.batch, "context": args.context, "ms_per_step": round(dms, 4), "tokens_per_s": round(args.batch * 1e3 / dms, 1)}}
        say(f"{key}: {out[key]}")
        del model
        torch.cuda.empty_cache()
    out["value"] = out["nebutar"]["decode"]["tokens_per_s"]
    if args.dtype == "bfloat16" and not args.no_points:
        out["kernels"] = nebutar_kernels(ours, like, args.batch, args.context, args.prefill_tokens)
    return out

# ---------------------------------------------------------------------------------------------- the Fotovik design

def fotovik_sizes(size: str) -> dict:
    """A Fotovik configuration of four layers (the middle two form a span that runs once) at the width of the other designs' sizes: causal
    attention with heads of 128 + 128 beside linear attention with heads of 128 x 128; attention in a window of 1024 with blocks of 64 before
    it; a delta rule with heads of 128 x 128 behind convolutions of four taps; dense feed-forwards of four times the width."""
    width, heads = dict(s=(2048, 16), m=(4096, 32))[size]
    rot = dict(dims=64, base=1000000.0)
    left = dict(heads=heads, kv_heads=heads // 4, dim=128, vdim=128, scale=128 ** -0.5, rot=dict(rot, scaling=dict(factor=2.0)))
    right = dict(heads=heads, dim=128, vdim=128, decay=[1.0 - 2.0 ** -(3 + 5 * i / max(1, heads - 1)) for i in range(heads)])
    windowed = dict(heads=heads, kv_heads=heads // 4, dim=128, vdim=128, scale=128 ** -0.5, rot=rot, mask=dict(size=1024, pool=64))
    delta = dict(heads=heads, kv_heads=heads // 2, dim=128, vdim=128, conv=4)
    mlp = dict(kind="dense", ff=4 * width)
    return dict(architecture="Fotovik", vocab=32000, width=width, max_positions=8192, norm=dict(eps=1e-5),
                embedding=dict(scale=1.0, bigram=dict(buckets=65521, mul_prev=36313, mul_cur=27191)), loop=dict(start=1, stop=3, times=1),
                layers=[dict(type="parallel", mixer=dict(left=left, right=right), mlp=mlp), dict(type="attention", mixer=windowed, mlp=mlp),
                        dict(type="delta", mixer=delta, mlp=mlp), dict(type="attention", mixer=windowed, mlp=mlp)])


def fotovik_kernels(ours: dict, like: dict, batch: int, context: int, tokens: int) -> list[dict]:
    """Each kernel that is the design's own, alone, at the sizes of ``ours``, in a decode step of ``batch`` requests on ``context`` cached
    tokens and in a prompt of ``tokens`` tokens, beside the like kernel of the Nebutar or Qwen2 path.  ``frac``: bytes that must move / time
    against 8 TB/s, or operations / time against the matrix cores' bfloat16 rate (against the 32-bit rate for the recurrences)."""
    import torch
    from torchlet_amd.kernels import ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, kind, launch, nbytes=0.0, flops=0.0, peak=MFMA_PEAK_TFLOPS["bfloat16"]):
        ms = _best_ms(launch, rounds=3, calls=5)
        row = {"kernel": name, "like": kind, "ms": round(ms, 4)}
        if nbytes:
            row.update(bytes=int(nbytes), frac=round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), bound="hbm")
        else:
            row.update(flops=flops, frac=round(flops / (ms * 1e-3) / (peak * 1e12), 4), bound="flops")
        rows.append(row)
        say(f"  {name}: {ms:.4f} ms, {row['frac']} of its bound")

    def tables(n_req, total, span=PAGE):
        blocks = -(-total // span)
        table = (torch.arange(n_req * blocks, dtype=torch.int32, device=dev) + 1).view(n_req, blocks)
        return table, n_req * blocks + 1

    width = ours["width"]
    par, att, delta = ours["layers"][0]["mixer"], ours["layers"][1]["mixer"], ours["layers"][2]["mixer"]
    # ---- linear attention with fixed decays beside the delta rule (the same kernel without the correction): a decode step reads and writes
    #      every state once; a prompt does 4 operations per state element and token (the update and one sum over the rows), the delta rule 6
    lin = par["right"]
    h, d, v = lin["heads"], lin["dim"], lin["vdim"]
    dh, dg, dd, dv_ = delta["heads"], delta["kv_heads"], delta["dim"], delta["vdim"]
    for name, T, reqs in (("decay_scan decode", batch, batch), (f"decay_scan prompt {tokens}", tokens, 1)):
        qkv = torch.randn(T, 2 * h * d + h * v, device=dev) * 0.1
        decay = torch.tensor(lin["decay"], device=dev)
        state = torch.zeros(reqs + 1, h * d * v, device=dev)
        out = torch.empty(T, h * v, device=dev)
        slots = torch.arange(reqs, dtype=torch.int32, device=dev)
        indptr = (torch.arange(reqs + 1, dtype=torch.int32, device=dev) * (T // reqs))
        launch = lambda: ops.decay_scan(qkv, decay, state, slots, indptr, out, h, d, v, max_new_tokens=T // reqs)
        if reqs > 1:
            add(name, "delta_scan decode", launch, nbytes=2.0 * reqs * h * d * v * 4)
        else:
            add(name, f"delta_scan prompt {tokens}", launch, flops=4.0 * T * h * d * v, peak=MFMA_PEAK_TFLOPS["float32"])
        qkv2 = torch.randn(T, 2 * dg * dd + dh * dv_, device=dev) * 0.1
        gates = torch.rand(T, 2 * dh, device=dev) * 0.5 + 0.5
        state2 = torch.zeros(reqs + 1, dh * dd * dv_, device=dev)
        out2 = torch.empty(T, dh * dv_, device=dev)
        launch = lambda: ops.delta_scan(qkv2, gates, state2, slots, indptr, out2, dh, dg, dd, dv_, max_new_tokens=T // reqs)
        if reqs > 1:
            add(name.replace("decay_scan", "delta_scan") + " (the design's own delta layers, and the Nebutar path)", "", launch, nbytes=2.0 * reqs * dh * dd * dv_ * 4)
        else:
            add(name.replace("decay_scan", "delta_scan") + " (the design's own delta layers, and the Nebutar path)", "", launch,
                flops=6.0 * T * dh * dd * dv_, peak=MFMA_PEAK_TFLOPS["float32"])
    # ---- attention in a window with pooled blocks and a sink, and causal attention, beside the Nebutar path's attention in chunks (the
    #      same kernels): a decode step reads the keys and values it may see once; a prompt's scores and sums
    nb = like["layers"][0]["mixer"]["left"]
    for label, m, window, pool, chunk, cap, sink_on in (("window 1024, blocks of 64, sink", att, att["mask"]["size"], att["mask"]["pool"], 0, 0.0, True),
                                                        ("causal", par["left"], 0, 0, 0, 0.0, False),
                                                        ("chunks of 1024, capped (Nebutar path)", nb, 0, 0, nb["mask"]["size"], nb["softcap"], False)):
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for T, reqs, ctx in ((batch, batch, context - 1), (tokens, 1, 0)):
            total = ctx + T // reqs
            table, pages = tables(reqs, total)
            k_plane = (torch.randn(pages, G, PAGE, dk, device=dev) * 0.3).to(bf)
            v_plane = (torch.randn(pages, G, dv, PAGE, device=dev) * 0.3).to(bf)
            pooled = None
            if pool:
                ptable, ppages = tables(reqs, total, PAGE * pool)
                ptable = torch.nn.functional.pad(ptable, (0, table.shape[1] - ptable.shape[1])).contiguous()
                pooled = ((torch.randn(ppages, G, PAGE, dk, device=dev) * 0.3).to(bf), (torch.randn(ppages, G, dv, PAGE, device=dev) * 0.3).to(bf), ptable, pool)
            sink = torch.zeros(H, device=dev) if sink_on else None
            q = (torch.randn(T, H * dk, device=dev) * 0.3).to(bf)
            out = torch.empty(T, H * dv, dtype=bf, device=dev)
            token_req = torch.arange(T, dtype=torch.int32, device=dev) // (T // reqs)
            positions = (torch.arange(T, dtype=torch.int32, device=dev) % (T // reqs)) + ctx
            if reqs == 1:
                n_tiles = -(-T // ops.LOCAL_ATTENTION_TILE_TOKENS)
                tiles = (torch.tensor([0, T], dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev),
                         torch.zeros(n_tiles, dtype=torch.int32, device=dev), torch.arange(n_tiles, dtype=torch.int32, device=dev) * ops.LOCAL_ATTENTION_TILE_TOKENS, n_tiles)
            else:
                tiles = (torch.arange(reqs + 1, dtype=torch.int32, device=dev), torch.full((reqs,), ctx, dtype=torch.int32, device=dev), None, None, reqs)
            launch = lambda: ops.local_attention(q, out, k_plane, v_plane, table, token_req, positions, H, G, dk, dv, PAGE, m["scale"], cap, chunk, window, 1.0,
                                                 tiles=tiles, sink=sink, pooled=pooled)

            def seen(p):        # keys (tokens and pooled rows) that a query at position p reads
                lo = max(p // chunk * chunk if chunk else 0, p - window + 1 if window else 0)
                return p - lo + 1 + (max(0, p - window + 1) // pool if pool else 0)
            if reqs > 1:
                add(f"local_attention decode, {label}", "local_attention decode, chunks", launch, nbytes=float(reqs) * seen(ctx) * G * (dk + dv) * 2)
            else:
                add(f"local_attention prompt {tokens}, {label}", f"local_attention prompt {tokens}, chunks", launch,
                    flops=2.0 * H * (dk + dv) * sum(seen(p) for p in range(T)))
    # ---- the norm that norms what it adds beside the plain residual's norm: reads the residual and the branch output, writes residual and row
    for name, T in (("sandwich_norm decode", batch), (f"sandwich_norm prompt {tokens}", tokens)):
        res = torch.randn(T, width, device=dev)
        pen = torch.randn(T, width, device=dev).to(bf)
        one = torch.ones(1, device=dev)
        out = torch.empty(T, width, dtype=bf, device=dev)
        add(name, "add_rmsnorm", lambda: ops.sandwich_norm(res, pen, one, 1e-5, None, one, 1e-5, out), nbytes=float(T) * width * 12)
        wb = torch.ones(width, dtype=bf, device=dev)
        add(name.replace("sandwich_norm", "add_rmsnorm") + " (Qwen2 path)", "", lambda: ops.add_rmsnorm(res, pen, wb, 1e-5, out), nbytes=float(T) * width * 12)
    # ---- norm per head and rotation in place, the pooled rows of a prompt, the sum of the two normed branches, the embedding with its bigram row
    H, G, dk = par["left"]["heads"], par["left"]["kv_heads"], par["left"]["dim"]
    T = tokens
    x = torch.randn(T, (H + 2 * G) * dk, device=dev).to(bf)
    wq = torch.ones(dk, device=dev)
    positions = torch.arange(T, dtype=torch.int32, device=dev)
    inv = torch.rand(32, device=dev)
    add(f"head_norm_rotate prompt {tokens}", "rope_cache_write", lambda: ops.head_norm_rotate(x[:, : (H + G) * dk], H, G, dk, wq, wq, 1e-5, positions, inv, 64, True),
        nbytes=float(T) * (H + G) * dk * 4)
    G, dk, dv, pool = att["kv_heads"], att["dim"], att["vdim"], att["mask"]["pool"]
    table, pages = tables(1, T)
    ptable, ppages = tables(1, T, PAGE * pool)
    k_plane, v_plane = torch.randn(pages, G, PAGE, dk, device=dev).to(bf), torch.randn(pages, G, dv, PAGE, device=dev).to(bf)
    pk, pv = torch.zeros(ppages, G, PAGE, dk, dtype=bf, device=dev), torch.zeros(ppages, G, dv, PAGE, dtype=bf, device=dev)
    indptr, zero = torch.tensor([0, T], dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev)
    add(f"pool_blocks prompt {tokens}", "kv_cache_write", lambda: ops.pool_blocks(k_plane, v_plane, table, pk, pv, ptable, indptr, zero, T // pool + 1, PAGE, pool),
        nbytes=float(T) * G * (dk + dv) * 2)
    kk, vv = torch.randn(T, G * dk, device=dev).to(bf), torch.randn(T, G * dv, device=dev).to(bf)
    add(f"kv_cache_write prompt {tokens} (Nebutar path)", "", lambda: ops.kv_cache_write(kk, vv, torch.zeros(T, dtype=torch.int32, device=dev), positions, table, k_plane, v_plane, PAGE),
        nbytes=float(T) * G * (dk + dv) * 4)
    outs = torch.randn(2, T, width, device=dev).to(bf)
    w2 = torch.ones(2, width, device=dev)
    y = torch.empty(T, width, dtype=bf, device=dev)
    add(f"normed_sum prompt {tokens}", "add_rmsnorm", lambda: ops.normed_sum(outs, w2, 1e-5, y), nbytes=float(T) * width * 6)
    big = ours["embedding"]["bigram"]
    emb, bigram = torch.randn(ours["vocab"], width, device=dev).to(bf), torch.randn(big["buckets"] + 1, width, device=dev).to(bf)
    ids = torch.randint(0, ours["vocab"], (T,), dtype=torch.int32, device=dev)
    res2 = torch.empty(T, width, device=dev)
    last = torch.zeros(2, 1, dtype=torch.int32, device=dev)
    token_req = torch.zeros(T, dtype=torch.int32, device=dev)
    add(f"bigram_embedding prompt {tokens}", "embedding", lambda: ops.bigram_embedding(ids, emb, res2, 1.0, bigram, big["buckets"], big["mul_prev"], big["mul_cur"],
                                                                                     token_req, indptr, positions, zero, last), nbytes=float(T) * width * 8)
    add(f"embedding prompt {tokens} (Qwen2 path)", "", lambda: ops.embedding(ids, emb, res2, 1.0), nbytes=float(T) * width * 6)
    return rows


def fotovik(args) -> dict:
    import torch
    ours = fotovik_sizes(args.size)
    like = nebutar_sizes(args.size)
    out = {"metric": f"Fotovik design, size {args.size} (width {ours['width']}, 4 layers), prefill of {args.prefill_tokens} tokens and decode at batch "
                     f"{args.batch} on {args.context}-token caches, beside the Nebutar design at equal width and layer count, one MI355X",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
           "data": "synthetic: seeded random weights, token ids and cache contents", "config": {"fotovik": ours, "nebutar": like}}
    for key, d in (("fotovik", ours), ("nebutar", like)):
        say(f"building the {key} model")
        cfg, model = _build_from(d, args.dtype)
        pms, pbest = time_prefill(model, args.prefill_tokens)
        dms = _decode_ms(model, args.batch, min(args.steps, 64), args.warmup, args.context)
        out[key] = {"weight_bytes": _weight_bytes(model),
                    "prefill": {"tokens": args.prefill_tokens, "ms": round(pms, 3), "ms_best": round(pbest, 3), "tokens_per_s": round(args.prefill_tokens * 1e3 / pms, 1)},
                    "decode": {"batch": args.batch, "context": args.context, "ms_per_step": round(dms, 4), "tokens_per_s": round(args.batch * 1e3 / dms, 1)}}
        say(f"{key}: {out[key]}")
        del model
        torch.cuda.empty_cache()
    out["value"] = out["fotovik"]["decode"]["tokens_per_s"]
    if args.dtype == "bfloat16" and not args.no_points:
        out["kernels"] = fotovik_kernels(ours, like, args.batch, args.context, args.prefill_tokens)
    return out


# ---------------------------------------------------------------------------------------------- the Bafulorn design

def bafulorn_sizes(size: str) -> dict:
    """A Bafulorn configuration of four layers at the width of the other designs' sizes: attention over a latent of 512 numbers with heads
    of 128 in a window of 1024 with a gate, with experts; grouped-query attention with heads of 128 whose values are its keys, half a head
    rotated with scaled frequencies, in a window of 1024 that keeps the first four tokens, with a gated dense feed-forward; a selective
    state-space recurrence with heads of 64 over twice the width, states of 128 numbers, a convolution of four taps, with experts; and the
    latent attention once more with a dense feed-forward."""
    width, heads, ff, experts, eff, top = dict(s=(2048, 16, 5632, 16, 1024, 2), m=(4096, 32, 11264, 32, 2048, 4))[size]
    latent = dict(heads=heads, dim=128, vdim=128, kv_rank=512, scale=128 ** -0.5, mask=dict(size=1024))
    attention = dict(heads=heads, kv_heads=heads // 4, dim=128, vdim=128, scale=128 ** -0.5, mask=dict(size=1024, keep_first=4),
                     rot=dict(dims=64, base=500000.0, scaling=dict(factor=8.0, low=1.0, high=4.0, original=8192)))
    mamba = dict(heads=2 * width // 64, vdim=64, state=128, groups=1, conv=4, norm_groups=1)
    moe = dict(kind="moe", expert=dict(ff=eff), router=dict(experts=experts, top=top, scale=2.0), shared=dict(ff=eff))
    dense = dict(kind="dense", ff=ff)
    return dict(architecture="Bafulorn", vocab=32000, width=width, max_positions=8192, norm=dict(eps=1e-6), residual_mult=0.25,
                layers=[dict(type="latent_attention", mixer=latent, mlp=moe), dict(type="attention", mixer=attention, mlp=dense),
                        dict(type="mamba2", mixer=mamba, mlp=moe), dict(type="latent_attention", mixer=latent, mlp=dense)])


def bafulorn_kernels(ours: dict, like: dict, batch: int, context: int, tokens: int) -> list[dict]:
    """Each kernel that the design added or changed, alone, at the sizes of ``ours``, in a decode step of ``batch`` requests on ``context`` cached
    tokens and in a prompt of ``tokens`` tokens, beside the like kernel of the closest path the framework had.  ``frac``: bytes that must
    move / time against 8 TB/s, or operations / time against the matrix cores' bfloat16 rate (against the 32-bit rate for the recurrence)."""
    import torch
    from torchlet_amd.kernels import ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, kind, launch, nbytes=0.0, flops=0.0, peak=MFMA_PEAK_TFLOPS["bfloat16"]):
        ms = _best_ms(launch, rounds=3, calls=5)
        row = {"kernel": name, "like": kind, "ms": round(ms, 4)}
        if nbytes:
            row.update(bytes=int(nbytes), frac=round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), bound="hbm")
        else:
            row.update(flops=flops, frac=round(flops / (ms * 1e-3) / (peak * 1e12), 4), bound="flops")
        rows.append(row)
        say(f"  {name}: {ms:.4f} ms, {row['frac']} of its bound")

    def tables(n_req, total):
        blocks = -(-total // PAGE)
        table = (torch.arange(n_req * blocks, dtype=torch.int32, device=dev) + 1).view(n_req, blocks)
        return table, n_req * blocks + 1

    width = ours["width"]
    lat, att, ssm = ours["layers"][0]["mixer"], ours["layers"][1]["mixer"], ours["layers"][2]["mixer"]
    moe = ours["layers"][0]["mlp"]
    # ---- the selective recurrence beside the delta rule (the same kernel with its correction): a decode step reads and writes every
    #      state once; a prompt does 4 operations per state element and token (the update and one sum over the rows), the delta rule 6
    h, p_, n_, g_ = ssm["heads"], ssm["vdim"], ssm["state"], ssm["groups"]
    inner, gn = h * p_, g_ * n_
    for name, T, reqs in (("selective_scan decode", batch, batch), (f"selective_scan prompt {tokens}", tokens, 1)):
        cbx = torch.randn(T, 2 * gn + inner, device=dev) * 0.1
        gates = torch.rand(T, 2 * h, device=dev) * 0.5 + 0.5
        skip = torch.ones(h, device=dev)
        state = torch.zeros(reqs + 1, h * n_ * p_ + 3 * (inner + 2 * gn), device=dev)
        out = torch.empty(T, inner, device=dev)
        slots = torch.arange(reqs, dtype=torch.int32, device=dev)
        indptr = (torch.arange(reqs + 1, dtype=torch.int32, device=dev) * (T // reqs))
        launch = lambda: ops.selective_scan(cbx, gates, skip, state, slots, indptr, out, h, g_, n_, p_, max_new_tokens=T // reqs)
        dh, dg, dd, dv_ = h, max(1, h // 2), n_, p_              # a delta rule with states of the same size
        qkv2 = torch.randn(T, 2 * dg * dd + dh * dv_, device=dev) * 0.1
        out2 = torch.empty(T, dh * dv_, device=dev)
        launch2 = lambda: ops.delta_scan(qkv2, gates, state, slots, indptr, out2, dh, dg, dd, dv_, max_new_tokens=T // reqs)
        if reqs > 1:
            add(name, "delta_scan decode", launch, nbytes=2.0 * reqs * h * n_ * p_ * 4)
            add("delta_scan decode (states of the same size)", "", launch2, nbytes=2.0 * reqs * h * n_ * p_ * 4)
        else:
            add(name, f"delta_scan prompt {tokens}", launch, flops=4.0 * T * h * n_ * p_, peak=MFMA_PEAK_TFLOPS["float32"])
            add(f"delta_scan prompt {tokens} (states of the same size)", "", launch2, flops=6.0 * T * h * n_ * p_, peak=MFMA_PEAK_TFLOPS["float32"])
    # ---- what the recurrence reads (convolution with its bias, silu, step sizes and decays) beside the delta rule's: the projection read, the
    #      32-bit channels written
    T = tokens
    C = inner + 2 * gn
    proj = (torch.randn(T, 2 * inner + 2 * gn + h, device=dev) * 0.3).to(bf)
    conv_w, conv_b = torch.randn(C, 4, device=dev) * 0.3, torch.zeros(C, device=dev)
    gates, cbx = torch.empty(T, 2 * h, device=dev), torch.empty(T, C, device=dev)
    a_log, dt_bias = torch.zeros(h, device=dev), torch.zeros(h, device=dev)
    state = torch.zeros(2, h * n_ * p_ + 3 * C, device=dev)
    one_req = (torch.zeros(1, dtype=torch.int32, device=dev), torch.tensor([0, T], dtype=torch.int32, device=dev), torch.zeros(T, dtype=torch.int32, device=dev))
    add(f"selective_prepare prompt {tokens}", "delta_prepare", lambda: ops.selective_prepare(proj, inner, conv_w, conv_b, gates, a_log, dt_bias, state, h * n_ * p_, *one_req,
                                                                                              cbx, h, inner, gn, 4), nbytes=float(T) * C * 6)
    dgates, dqkv = torch.randn(T, 2 * h, device=dev), torch.empty(T, C, device=dev)         # a delta rule with as many channels: 2 kv_heads x state + heads x vdim
    if gn % n_ == 0 and n_ <= 256 and p_ <= 256:
        add(f"delta_prepare prompt {tokens} (as many channels)", "", lambda: ops.delta_prepare(proj, conv_w, dgates, a_log, dt_bias, state, h * n_ * p_, *one_req, dqkv, h, g_, n_, p_, 4,
                                                                                             1.0, 1e-6), nbytes=float(T) * C * 6)
    y, z = torch.randn(T, inner, device=dev), (torch.randn(T, inner, device=dev)).to(bf)
    wn, outn = torch.ones(inner, device=dev), torch.empty(T, inner, dtype=bf, device=dev)
    add(f"gated_head_norm prompt {tokens}, gate before the norm, one group", "gated_head_norm", lambda: ops.gated_head_norm(y, z, wn, 1e-6, outn, 1, inner, gate="silu", gate_first=True),
        nbytes=float(T) * inner * 8)
    add(f"gated_head_norm prompt {tokens}, per head of {p_} (delta rule's)", "", lambda: ops.gated_head_norm(y, z, wn, 1e-6, outn, h, p_, gate="silu"), nbytes=float(T) * inner * 8)
    # ---- attention over the cached latent in a window with a gate, beside the causal one with a sink (the Migurax path): a decode step reads the
    #      rows it may see once; a prompt's scores and sums over the latent
    H, rank = lat["heads"], lat["kv_rank"]
    for label, window, gated, sink_on in ((f"window {lat['mask']['size']}, gate", lat["mask"]["size"], True, False), ("causal, sink (Migurax path)", 0, False, True)):
        for T, reqs, ctx in ((batch, batch, context - 1), (tokens, 1, 0)):
            total = ctx + T // reqs
            table, pages = tables(reqs, total)
            plane = (torch.randn(pages, 1, PAGE, rank, device=dev) * 0.3).to(bf)
            q = (torch.randn(T, H * rank, device=dev) * 0.1).to(bf)
            out = torch.empty(T, H * rank, dtype=bf, device=dev)
            gate = (torch.randn(T, H, device=dev)).to(bf) if gated else None
            sink = torch.zeros(H, device=dev) if sink_on else None
            tq = ops.latent_tile_tokens(H, ops.LATENT_MFMA_ROWS)
            keys = min(total, window + T // reqs - 1) if window else total
            if reqs == 1:
                n_tiles = -(-T // tq)
                args = (torch.tensor([0, T], dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(n_tiles, dtype=torch.int32, device=dev),
                        torch.arange(n_tiles, dtype=torch.int32, device=dev) * tq, n_tiles)
                splits = 1
            else:
                args = (None, torch.full((reqs,), ctx, dtype=torch.int32, device=dev), None, None, reqs)
                splits = max(1, min(256 // reqs, keys // 64, 64))
            launch = lambda: ops.latent_attention(q, out, plane, table, *args, tq, H, rank, 0, PAGE, 0.09, sink, splits, max_new_tokens=T // reqs, window=window, gate=gate)
            seen = lambda p: min(p + 1, window) if window else p + 1
            if reqs > 1:
                add(f"latent_attention decode, {label}", "latent_attention decode, causal", launch, nbytes=float(reqs) * seen(ctx) * rank * 2)
            else:
                add(f"latent_attention prompt {tokens}, {label}", f"latent_attention prompt {tokens}, causal", launch, flops=4.0 * H * rank * sum(seen(p) for p in range(T)))
    # ---- attention in a window that keeps the first tokens, beside the plain window (the same kernels): a decode step reads the keys and values
    #      it may see once; a prompt's scores and sums
    H, G, dk = att["heads"], att["kv_heads"], att["dim"]
    for label, keep in ((f"window {att['mask']['size']}, {att['mask']['keep_first']} kept", att["mask"]["keep_first"]), ("plain window", 0)):
        window = att["mask"]["size"]
        for T, reqs, ctx in ((batch, batch, context - 1), (tokens, 1, 0)):
            total = ctx + T // reqs
            table, pages = tables(reqs, total)
            k_plane = (torch.randn(pages, G, PAGE, dk, device=dev) * 0.3).to(bf)
            v_plane = (torch.randn(pages, G, dk, PAGE, device=dev) * 0.3).to(bf)
            q = (torch.randn(T, H * dk, device=dev) * 0.3).to(bf)
            out = torch.empty(T, H * dk, dtype=bf, device=dev)
            token_req = torch.arange(T, dtype=torch.int32, device=dev) // (T // reqs)
            positions = (torch.arange(T, dtype=torch.int32, device=dev) % (T // reqs)) + ctx
            if reqs == 1:
                n_tiles = -(-T // ops.LOCAL_ATTENTION_TILE_TOKENS)
                tiles = (torch.tensor([0, T], dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev),
                         torch.zeros(n_tiles, dtype=torch.int32, device=dev), torch.arange(n_tiles, dtype=torch.int32, device=dev) * ops.LOCAL_ATTENTION_TILE_TOKENS, n_tiles)
            else:
                tiles = (torch.arange(reqs + 1, dtype=torch.int32, device=dev), torch.full((reqs,), ctx, dtype=torch.int32, device=dev), None, None, reqs)
            launch = lambda: ops.local_attention(q, out, k_plane, v_plane, table, token_req, positions, H, G, dk, dk, PAGE, att["scale"], 0.0, 0, window, 1.0,
                                                 tiles=tiles, keep_first=keep)
            seen = lambda p: min(p + 1, window) + min(keep, max(0, p - window + 1))
            if reqs > 1:
                add(f"local_attention decode, {label}", "local_attention decode, plain window", launch, nbytes=float(reqs) * seen(ctx) * G * 2 * dk * 2)
            else:
                add(f"local_attention prompt {tokens}, {label}", f"local_attention prompt {tokens}, plain window", launch, flops=4.0 * H * dk * sum(seen(p) for p in range(T)))
    # ---- the rotation with the keys copied as they come, beside the rotation alone; the norm with a weight vector beside the plain residual's
    #      norm; the embedding with its norm beside the embedding; the sigmoid router beside the softmax one
    T = tokens
    x = torch.randn(T, (H + G) * dk, device=dev).to(bf)
    raw = torch.empty(T, G * dk, dtype=bf, device=dev)
    positions = torch.arange(T, dtype=torch.int32, device=dev)
    inv = torch.rand(att["rot"]["dims"] // 2, device=dev)
    add(f"head_norm_rotate prompt {tokens}, keys copied", "head_norm_rotate", lambda: ops.head_norm_rotate(x, H, G, dk, None, None, 0.0, positions, inv, att["rot"]["dims"], True, raw_b=raw),
        nbytes=float(T) * ((H + G) * dk * 4 + G * dk * 2))
    add(f"head_norm_rotate prompt {tokens} (Fotovik path)", "", lambda: ops.head_norm_rotate(x, H, G, dk, None, None, 0.0, positions, inv, att["rot"]["dims"], True),
        nbytes=float(T) * (H + G) * dk * 4)
    for name, T in (("sandwich_norm decode, weight vectors", batch), (f"sandwich_norm prompt {tokens}, weight vectors", tokens)):
        res = torch.randn(T, width, device=dev)
        pen = torch.randn(T, width, device=dev).to(bf)
        wv = torch.ones(width, device=dev)
        out = torch.empty(T, width, dtype=bf, device=dev)
        add(name, "add_rmsnorm", lambda: ops.sandwich_norm(res, pen, wv, 1e-6, None, wv, 1e-6, out), nbytes=float(T) * width * 12)
        wb = torch.ones(width, dtype=bf, device=dev)
        add(name.split(",")[0].replace("sandwich_norm", "add_rmsnorm") + " (Qwen2 path)", "", lambda: ops.add_rmsnorm(res, pen, wb, 1e-5, out), nbytes=float(T) * width * 12)
    T = tokens
    emb = torch.randn(ours["vocab"], width, device=dev).to(bf)
    ids = torch.randint(0, ours["vocab"], (T,), dtype=torch.int32, device=dev)
    res2, wv = torch.empty(T, width, device=dev), torch.ones(width, device=dev)
    add(f"embedding_norm prompt {tokens}", "embedding", lambda: ops.embedding_norm(ids, emb, res2, 1.0, wv, 1e-6), nbytes=float(T) * width * 6)
    add(f"embedding prompt {tokens} (Qwen2 path)", "", lambda: ops.embedding(ids, emb, res2, 1.0), nbytes=float(T) * width * 6)
    E, top = moe["router"]["experts"], moe["router"]["top"]
    logits, corr = torch.randn(T, E, device=dev), torch.zeros(E, device=dev)
    add(f"route prompt {tokens}, sigmoid scores", "route", lambda: ops.route(logits, top, "sigmoid", corr, 2.0, 1e-20), nbytes=float(T) * (E * 4 + top * 16))
    add(f"route prompt {tokens}, softmax over all (Nebutar path)", "", lambda: ops.route(logits, top, "all", corr), nbytes=float(T) * (E * 4 + top * 16))
    # ---- the gated feed-forward's first product with relu in its epilogue beside silu (the Qwen2 path's kernel)
    ff = ours["layers"][1]["mlp"]["ff"]
    gate_up = ops.interleave_gate_up((torch.randn(ff, width, device=dev) * 0.02).to(bf), (torch.randn(ff, width, device=dev) * 0.02).to(bf))
    for T in (batch, tokens):
        xx = torch.randn(T, width, device=dev).to(bf)
        zz = torch.empty(T, ff, dtype=bf, device=dev)
        kind = "decode" if T == batch else f"prompt {tokens}"
        if T == batch:
            add(f"linear_swiglu {kind}, relu", "linear_swiglu", lambda: ops.linear_swiglu(xx, gate_up, zz, "relu"), nbytes=2.0 * ff * width * 2)
            add(f"linear_swiglu {kind}, silu (Qwen2 path)", "", lambda: ops.linear_swiglu(xx, gate_up, zz, "silu"), nbytes=2.0 * ff * width * 2)
        else:
            add(f"linear_swiglu {kind}, relu", "linear_swiglu", lambda: ops.linear_swiglu(xx, gate_up, zz, "relu"), flops=4.0 * T * ff * width)
            add(f"linear_swiglu {kind}, silu (Qwen2 path)", "", lambda: ops.linear_swiglu(xx, gate_up, zz, "silu"), flops=4.0 * T * ff * width)
    return rows


def bafulorn(args) -> dict:
    import torch
    ours = bafulorn_sizes(args.size)
    like = migurax_sizes(args.size)[0]
    out = {"metric": f"Bafulorn design, size {args.size} (width {ours['width']}, 4 layers), prefill of {args.prefill_tokens} tokens and decode at batch "
                     f"{args.batch} on {args.context}-token caches, beside the Migurax design at equal width and layer count, one MI355X",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
           "data": "synthetic: seeded random weights, token ids and cache contents", "config": {"bafulorn": ours, "migurax": like}}
    for key, d in (("bafulorn", ours), ("migurax", like)):
        say(f"building the {key} model")
        cfg, model = _build_from(d, args.dtype)
        pms, pbest = time_prefill(model, args.prefill_tokens)
        dms = _decode_ms(model, args.batch, min(args.steps, 64), args.warmup, args.context)
        out[key] = {"weight_bytes": _weight_bytes(model),
                    "prefill": {"tokens": args.prefill_tokens, "ms": round(pms, 3), "ms_best": round(pbest, 3), "tokens_per_s": round(args.prefill_tokens * 1e3 / pms, 1)},
                    "decode": {"batch": args.batch, "context": args.context, "ms_per_step": round(dms, 4), "tokens_per_s": round(args.batch * 1e3 / dms, 1)}}
        say(f"{key}: {out[key]}")
        del model
        torch.cuda.empty_cache()
    out["value"] = out["bafulorn"]["decode"]["tokens_per_s"]
    if args.dtype == "bfloat16" and not args.no_points:
        out["kernels"] = bafulorn_kernels(ours, like, args.batch, args.context, args.prefill_tokens)
    return out


def main(argv=None) -> int:
    args = parse_args(argv)
    args.serve_new_tokens = args.new_tokens or 128
    args.new_tokens = args.new_tokens or NEW_TOKENS
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not built (this engine runs on a single MI355X)")
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X; no GPU is visible", file=sys.stderr)
        return 1
    if args.workload == "migurax":
        print(json.dumps(migurax(args)))
        return 0
    if args.workload == "nebutar":
        print(json.dumps(nebutar(args)))
        return 0
    if args.workload == "fotovik":
        print(json.dumps(fotovik(args)))
        return 0
    if args.workload == "bafulorn":
        print(json.dumps(bafulorn(args)))
        return 0
    name, sizes = SHAPES[args.shape]
    full_layers = sizes["num_hidden_layers"]
    layers = args.layers if args.layers is not None else full_layers
    cfg, model = build(args.shape, layers, args.dtype)
    ptokens = args.prefill_tokens
    peak_tflops = MFMA_PEAK_TFLOPS[args.dtype]

    def prefill_point(gemm_tflops=None):
        pms, pbest = time_prefill(model, ptokens)
        flops = prefill_flops(cfg, ptokens)
        point = {"value": round(ptokens * 1e3 / pms, 1), "tokens": ptokens, "ms": round(pms, 3), "ms_best": round(pbest, 3), "runs": 3,
                 "flops": flops, "frac": round(flops / (pms * 1e-3) / (peak_tflops * 1e12), 4)}
        if gemm_tflops:
            point["frac_measured"] = round(flops / (pms * 1e-3) / (gemm_tflops * 1e12), 4)
        return point

    if args.workload == "serve":
        print(json.dumps(serve(cfg, model, args)))
        return 0
    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_point(), "layers": layers}))
        return 0
    if args.only == "step":
        print(json.dumps({"step_function": step_function_decode(cfg, model, args.batch, min(args.steps, 64), args.warmup, args.context),
                          "layers": layers}))
        return 0
    if args.only == "decode":
        args.no_points = True
    head = engine_decode(cfg, model, args.batch, args.steps, args.warmup, args.context, args.new_tokens)
    ms = head["ms_per_step"]
    achieved = head["bytes_per_step"] / (ms * 1e-3) / 1e9
    result = {
        "metric": f"decode tokens/s, {name} shape, batch {args.batch}, {args.context}-token prompts, {args.new_tokens} new tokens, "
                  f"through the engine, one MI355X",
        "value": head["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": f"synthetic: seeded random weights and token ids; {args.context}-token random prompts prefilled by the engine, "
                f"greedy decoding with no stop token",
        "config": {
            "model": f"{name} shape (Qwen2ForCausalLM)", "layers": layers, "layers_full_model": full_layers,
            "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "new_tokens": args.new_tokens,
            "context_limit": cfg.max_position_embeddings, "page_size": PAGE, "prefill_tokens": ptokens,
            "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "bytes_per_step": head["bytes_per_step"],
                     "mean_context": head["mean_context"]},
        "engine": {"graph_replays": head["graph_replays"], "steps_ahead": head["steps_ahead"]},
    }
    if not args.no_points:
        stream_gbs = measure_stream_read_gbs()
        gemm_tflops = measure_gemm_tflops(model.dtype)
        result["measured"] = {"stream_read_gbs": round(stream_gbs, 1), "gemm_tflops": round(gemm_tflops, 1),
                              "how": "a kernel of this repository that only reads 2 GiB; its own 8192-cubed matrix product"}
        result["roofline"]["frac_measured"] = round(achieved / stream_gbs, 4)
        bare = step_function_decode(cfg, model, args.batch, 64, args.warmup, args.context)
        result["step_function"] = bare
        result["prefill"] = prefill_point(gemm_tflops)
        points, detail = {}, {}
        for b in (1, 64):
            r = engine_decode(cfg, model, b, max(8, args.steps // 2), max(2, args.warmup // 2), args.context, args.new_tokens)
            gbs = r["bytes_per_step"] / (r["ms_per_step"] * 1e-3) / 1e9
            points[f"decode_b{b}"] = r["tokens_per_s"]
            detail[f"decode_b{b}"] = {"ms_per_step": r["ms_per_step"], "steps": r["steps"], "bytes_per_step": r["bytes_per_step"],
                                      "mean_context": r["mean_context"], "achieved_gbs": round(gbs, 1),
                                      "frac": round(gbs / HBM_PEAK_GBS, 4), "frac_measured": round(gbs / stream_gbs, 4)}
        result["points"] = points
        result["points_detail"] = detail
    if args.all or args.extra:
        del model
        torch.cuda.empty_cache()
        result["extra"] = secondary(args)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
