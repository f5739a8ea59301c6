"""The Fotovik design through the framework's host side on the CPU: configuration, tensor names, run order, the cache plan with pages
at two rates, the step function under every way of cutting requests, the stream after every layer run, greedy generation through
scheduler and sampler, the trace replay and the command line, with the HIP entry points replaced by the stand-ins of
``emulated_ops.py``.  The kernels are tested on the GPU (``-m gpu``)."""
import json

import numpy as np
import pytest
import torch

import plain_fotovik
import scenarios
import tiny_fotovik
from torchlet_amd.cache.manager import CacheManager
from torchlet_amd.config import ConfigError, FotovikConfig
from torchlet_amd.engine.batch import StepEntry
from torchlet_amd.engine.engine import Engine
from torchlet_amd.engine.loading import load_model, make_runner
from torchlet_amd.engine.request import Request
from torchlet_amd.parts.base import PagedNeed
from torchlet_amd.registry import load_config

TOL = dict(atol=5e-4, rtol=2e-4)       # 32-bit stand-ins against a 64-bit evaluation, logits of order ten


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("fotovik")
    return {name: tiny_fotovik.write(name, root) for name in tiny_fotovik.CONFIGS}


def _weights(name):
    return {k: v.double() for k, v in tiny_fotovik.tensors_for(name).items()}


def test_configuration_expands_to_parts_names_and_run_order(folders):
    cfg = load_config(folders["A"])
    assert isinstance(cfg, FotovikConfig)
    spec = cfg.to_spec()
    assert [(e.layer, e.add_embedding) for e in spec.order] == [(0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert [(b.kind, b.mixer.kind, b.ffn.kind if b.ffn is not None else None) for b in spec.layers] == \
        [("sandwich_residual", "parallel", "dense_ff"), ("sandwich_residual", "capped_attention", None), ("sandwich_residual", "gated_delta", "dense_ff"),
         ("sandwich_residual", "capped_attention", "dense_ff")]
    left, right = (s for _, s, _ in spec.layers[0].mixer.branches)
    assert (left.kind, left.qk_norm, left.sink, left.window, left.pool, left.position.kind, left.position.dims, left.position.factor) == \
        ("capped_attention", True, False, None, None, "rope_halves", 6, 1.5)
    assert (right.kind, right.decay, right.norm_eps) == ("decayed_linear", (0.5, 0.9, 0.99), 1e-5)
    assert spec.layers[0].mixer.normed and [s for _, _, s in spec.layers[0].mixer.branches] == [0.5, 0.5]
    att = spec.layers[1].mixer
    assert (att.sink, att.qk_norm, att.window, att.pool, att.position.kind, att.scale) == (True, False, 9, 4, "rope_pairs", 0.3)
    assert (spec.layers[2].mixer.conv, spec.layers[2].mixer.unit_eps, spec.layers[2].ffn.activation, spec.layers[2].ffn.bias) == (3, 1e-6, "gelu", False)
    assert (spec.bigram.buckets, spec.bigram.mul_prev, spec.bigram.mul_cur, spec.embed_scale, spec.tie_head) == (31, 7, 3, 2.0, False)
    from torchlet_amd.models.decoder import DecoderModel
    names = {n for n, s in DecoderModel(spec, torch.float32, "cpu").weight_specs().items() if not s.optional}
    assert names == set(tiny_fotovik.tensors_for("A"))
    assert {"embed", "bigram", "head", "final.norm", "l0.norm1", "l0.norm1b", "l0.norm2b", "l0.mix.left.q.norm", "l0.mix.left.out", "l0.mix.right.out",
            "l0.mix.right.norm", "l1.mix.sink", "l2.mix.q.conv", "l2.mix.A_log", "l2.mix.dt_bias", "l2.mix.norm", "l2.mlp.up", "l3.mlp.down"} <= names
    assert "l1.norm2" not in names and "l1.mlp.up" not in names and "l0.mix.left.sink" not in names
    assert json.loads(json.dumps(cfg.to_dict()))["loop"] == dict(start=1, stop=3, times=3)
    plain = load_config(folders["C"]).to_spec()             # no bigram table, no loop
    assert plain.bigram is None and [e.layer for e in plain.order] == [0, 1, 2, 3] and not any(e.add_embedding for e in plain.order)
    assert plain.layers[0].mixer.position is None and plain.layers[2].mixer.branches[0][1].position.factor == 1.0
    base = tiny_fotovik.CONFIGS["A"]
    layer = base["layers"][1]
    for bad in (dict(layers=[]), dict(layers=[dict(layer, type="other")]), dict(norm={}), dict(loop=dict(start=2, stop=1, times=1)),
                dict(layers=[dict(layer, mixer=dict(layer["mixer"], heads=5))]),
                dict(layers=[dict(layer, mixer=dict(layer["mixer"], rot=dict(dims=10, base=10.0)))]),
                dict(layers=[dict(layer, mixer=dict(layer["mixer"], mask=dict(size=0, pool=2)))]),
                dict(layers=[dict(layer, mlp=dict(kind="moe", ff=8))]),
                dict(embedding=dict(scale=1.0, bigram=dict(buckets=0, mul_prev=1, mul_cur=1)))):
        with pytest.raises(ConfigError):
            FotovikConfig.from_dict({**base, **bad})


def test_cache_plan_pages_at_two_rates_states_and_the_token_before(cpu_ops, folders):
    _, model = load_model(folders["A"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=40, max_requests=3)
    cache = runner.cache
    # runs: parallel, (attention, delta) x 3, attention: the looped attention's three passes share a group of token pages (kept for the
    # longer of window and block) and a group of pooled rows, one row per block
    got = [(g.need.plane_shapes, g.need.window, g.need.stride, len(g.runs)) for g in cache.groups]
    assert got == [(((2, 10), (2, 6)), None, 1, 1), (((3, 8), (3, 4)), 9, 1, 3), (((3, 8), (3, 4)), None, 4, 3),
                   (((1, 6), (1, 12)), 7, 1, 1), (((1, 6), (1, 12)), None, 7, 1)]
    assert [g.span for g in cache.groups] == [4, 4, 16, 4, 28]
    assert cache.capacity()[2] == -(-39 // 4) + 3 and cache.capacity()[4] == -(-39 // 7) + 3
    assert len(runner.caches) == 9 and runner.caches[8].state.dtype == torch.int32 and tuple(runner.caches[8].state.shape) == (4, 1)
    states = [c.state for c in runner.caches[:8]]
    assert [None if s is None else tuple(s.shape) for s in states] == \
        [(4, 3 * 5 * 7), None, (4, 4 * 5 * 7 + 2 * (20 + 28)), None, (4, 4 * 5 * 7 + 2 * (20 + 28)), None, (4, 4 * 5 * 7 + 2 * (20 + 28)), None]
    assert runner.caches[1].more[0][0] == 2 and runner.caches[3].planes[0].data_ptr() != runner.caches[1].planes[0].data_ptr()
    # a slot that is used again starts from zero; the token before is kept per slot
    runner.step([StepEntry("a", [1, 2, 3], [])])
    slot = cache.slot("a")
    assert int(runner.caches[8].state[slot, 0]) == 3 and float(states[0][slot].abs().max()) > 0
    runner.release("a")
    runner.step([StepEntry("b", [4], [])])
    assert cache.slot("b") == slot
    fresh = make_runner(model, page_size=4, num_pages=40, max_requests=3)
    fresh.step([StepEntry("b", [4], [])])
    for s, f in zip(states, fresh.caches):
        if s is not None:
            assert torch.equal(s[slot], f.state[fresh.cache.slot("b")])


def test_pages_of_pooled_rows_and_of_tokens_behind_window_and_block():
    tokens = PagedNeed(num_heads=1, head_dim=4, window=10, planes=((1, 4), (1, 6)))
    pooled = PagedNeed(num_heads=1, head_dim=4, planes=((1, 4), (1, 6)), stride=3)
    cache = CacheManager([((tokens, pooled), None, None)], page_size=4, num_pages=20, max_requests=2)
    assert cache.capacity() == [19, -(-19 // 3) + 2] and cache.layer_cache(0).more[0][0] == 1
    cache.add_request("a")
    assert cache.pages_missing("a", 9) == [3, 1]                # a pooled page spans 12 positions
    assert cache.reserve("a", 9)
    cache.commit("a", 9)
    assert cache.pages_missing("a", 12) == [0, 0] and cache.pages_missing("a", 13) == [1, 1]
    for n in range(10, 80):                                     # token by token: the window's pages and one more; pooled rows for good
        assert cache.reserve("a", n)
        cache.commit("a", n)
        cache.check()
        assert 19 - cache.free_pages()[0] <= 10 // 4 + 2 and cache.capacity()[1] - cache.free_pages()[1] == -(-n // 12)
    assert [bool(p) for p in cache.groups[1].tables["a"]] == [True] * 7
    cache.release("a")
    cache.check()
    assert cache.free_pages() == cache.capacity()


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "tail_singles", "portions", "mixed"])
def test_step_function_equals_plain_under_every_split(cpu_ops, folders, name, mode):
    lengths = [37, 5, 50, 1, 18, 33] if name != "B" else [75, 1, 27]
    seqs, refs = tiny_fotovik.sequences(name, _weights(name), lengths)
    steps = scenarios.number(getattr(scenarios, mode)(seqs) if mode != "tail_singles" else scenarios.tail_singles(seqs, tail=9))
    page = tiny_fotovik.PAGE_SIZES[name]
    _, model = load_model(folders[name], "float32", device="cpu")
    runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps, unit=page) // page) + 1, max_requests=4)
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.numpy()
        for r in s["end"]:
            runner.release(r)
        runner.cache.check()
    scenarios.check(steps, out, refs, TOL, f"{name}/{mode}")
    assert runner.cache.live_requests() == [] and runner.cache.free_pages() == runner.cache.capacity()


@pytest.mark.parametrize("seed", range(4))
def test_configurations_drawn_at_random(cpu_ops, tmp_path, seed):
    """Layers of any kind in any order and any span of them run again, through the host side: portions and mixed batches against plain."""
    import random
    rnd = random.Random(700 + seed)
    conf = tiny_fotovik.random_config(rnd, big=False)
    page = rnd.choice([4, 8, 16])
    folder = tiny_fotovik.write(f"random{seed}", tmp_path, config=conf, seed=seed)
    w = {k: v.double() for k, v in tiny_fotovik.tensors_for("", 1.0, conf, seed).items()}
    seqs, refs = tiny_fotovik.sequences("", w, [rnd.randint(1, 60) for _ in range(4)], seed=seed, config=conf)
    _, model = load_model(folder, "float32", device="cpu")
    for mode in ("portions", "mixed"):
        steps = scenarios.number(getattr(scenarios, mode)(seqs))
        runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps, unit=page) // page) + 1, max_requests=4)
        out = {}
        for s in steps:
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
            if logits is not None:
                out[s["step"]] = logits.numpy()
            for r in s["end"]:
                runner.release(r)
            runner.cache.check()
        scenarios.check(steps, out, refs, TOL, f"{conf}/{mode}")
        assert runner.cache.free_pages() == runner.cache.capacity()


def test_stream_after_every_layer_run_against_plain(cpu_ops, folders):
    """The residual after every run of a layer (a looped layer counts each time; the embedding that enters again counts with the run
    it comes before)."""
    ids = [5, 17, 3, 60, 2, 2, 41, 9, 30, 11, 90, 4, 4, 8]
    _, want = plain_fotovik.forward(tiny_fotovik.CONFIGS["A"], _weights("A"), ids)
    _, model = load_model(folders["A"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=12, max_requests=1)
    seen = []
    import emulated_ops

    def settled(stream):            # what the next norm would see: the pending output normed and added
        x = stream.residual.clone()
        emulated_ops.sandwich_norm(x, stream.pending, stream.post[0], stream.post[1], None, torch.ones(1), 1e-5, torch.empty_like(x))
        return x

    for block in model.blocks:
        inner = block.forward
        block.forward = lambda stream, ctx, cache, inner=inner: (lambda s: (seen.append(settled(s)), s)[1])(inner(stream, ctx, cache))
    runner.step([StepEntry("a", ids, [len(ids) - 1])])
    assert len(seen) == 8
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, atol=5e-5, rtol=1e-5)


def _greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain_fotovik.forward(cfg, w, ids)[0][-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_through_scheduler_and_sampler(cpu_ops, folders):
    """Prompts in portions of at most 12 tokens beside decode tokens, five requests over three slots (slots and pages are used again),
    steps enqueued ahead of their tokens (the token before comes from the GPU's own copy), against the plain loop."""
    w = _weights("B")
    cfg = tiny_fotovik.CONFIGS["B"]
    g = torch.Generator().manual_seed(11)
    prompts = [torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for n in (5, 17, 45, 1, 9)]
    _, model = load_model(folders["B"], "float32", device="cpu")
    engine = Engine(make_runner(model, page_size=16, num_pages=14, max_requests=3), max_tokens_per_step=12)
    reqs = [Request(prompt_tokens=p, seed=i, max_new_tokens=6) for i, p in enumerate(prompts)]
    for r in reqs:
        engine.add_request(r)
    engine.run_until_done()
    for r, p in zip(reqs, prompts):
        assert r.output_tokens == _greedy(cfg, w, p, 6)
    assert engine.runner.cache.live_requests() == [] and len({tuple(r.output_tokens) for r in reqs}) > 1


def test_trace_replay_reads_the_architecture_from_the_folder(cpu_ops, folders, tmp_path, monkeypatch):
    from torchlet_amd.engine import loading, trace
    monkeypatch.setattr(loading, "require_gpu", lambda: torch.device("cpu"))
    seqs, refs = tiny_fotovik.sequences("A", _weights("A"), [13, 6, 40])
    steps = scenarios.number(scenarios.mixed(seqs, seed=1))
    args = trace.parse_args(["--model", str(folders["A"]), "--dtype", "float32", "--out", str(tmp_path / "out"),
                             "--max-tokens", str(scenarios.max_tokens_needed(steps)), "--page-size", "4"])
    import io
    said = io.StringIO()
    assert trace.run(args, [json.dumps(s) for s in steps], out=said) == 0
    assert said.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    out = {s["step"]: np.fromfile(tmp_path / "out" / f"{s['step']}.f32", dtype="<f4").reshape(-1, 97) for s in steps
           if any(e["want"] for e in s["entries"])}
    scenarios.check(steps, out, refs, TOL, "trace replay")


def test_command_line_writes_a_random_folder_of_the_architecture(cpu_ops, tmp_path):
    from safetensors import safe_open
    from torchlet_amd.llm import main
    from torchlet_amd.models.decoder import DecoderModel
    src = tmp_path / "config.json"
    src.write_text(json.dumps(tiny_fotovik.CONFIGS["A"]))
    assert main(["init", "--config", str(src), "--seed", "3", "--out", str(tmp_path / "out")]) == 0
    cfg = load_config(tmp_path / "out")
    assert isinstance(cfg, FotovikConfig) and cfg.layers == tiny_fotovik.CONFIGS["A"]["layers"]
    with safe_open(str(tmp_path / "out" / "model.safetensors"), framework="pt") as f:
        stored = set(f.keys())
        g = f.get_tensor("l0.norm1")
    assert stored == {n for n, s in DecoderModel(cfg.to_spec(), torch.float32, "cpu").weight_specs().items() if not s.optional}
    assert g.dim() == 0
    _, model = load_model(tmp_path / "out", "float32", device="cpu")
    logits = make_runner(model, page_size=4, num_pages=8, max_requests=1).step([StepEntry("a", [1, 2, 3, 4, 5], [4])])
    assert logits.shape == (1, 97) and bool(torch.isfinite(logits).all())
