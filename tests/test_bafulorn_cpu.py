"""The Bafulorn design through the framework's host side on the CPU: configuration, tensor names, the cache plan with windows, kept first
tokens and states, the pages of kept tokens beside a window, the step function under every way of cutting requests, the stream after
every layer, greedy generation through scheduler and sampler, the trace replay and the command line, with the HIP entry points replaced
by the stand-ins of ``emulated_ops.py``.  The kernels are tested on the GPU (``-m gpu``)."""
import json

import numpy as np
import pytest
import torch

import plain_bafulorn
import scenarios
import tiny_bafulorn
from torchlet_amd.cache.manager import CacheManager
from torchlet_amd.config import BafulornConfig, ConfigError
from torchlet_amd.engine.batch import StepEntry
from torchlet_amd.engine.engine import Engine
from torchlet_amd.engine.loading import load_model, make_runner
from torchlet_amd.engine.request import Request
from torchlet_amd.parts.base import PagedNeed
from torchlet_amd.registry import load_config

TOL = dict(atol=3e-4, rtol=2e-4)       # 32-bit stand-ins against a 64-bit evaluation, logits of order one to four


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("bafulorn")
    return {name: tiny_bafulorn.write(name, root) for name in tiny_bafulorn.CONFIGS}


def _weights(name):
    return {k: v.double() for k, v in tiny_bafulorn.tensors_for(name).items()}


def _run(runner, steps):
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.numpy()
        for r in s["end"]:
            runner.release(r)
        runner.cache.check()
    return out


def test_configuration_expands_to_parts_and_names(folders):
    cfg = load_config(folders["A"])
    assert isinstance(cfg, BafulornConfig)
    spec = cfg.to_spec()
    assert [(b.kind, b.mixer.kind, b.ffn.kind if b.ffn is not None else None) for b in spec.layers] == \
        [("sandwich_residual", "capped_attention", "routed_experts"), ("sandwich_residual", "selective_state", None),
         ("sandwich_residual", "latent_attention", "swiglu"), ("sandwich_residual", "capped_attention", "swiglu"),
         ("sandwich_residual", "selective_state", "routed_experts")]
    att = spec.layers[0].mixer
    assert (att.window, att.keep_first, att.values_are_keys, att.qk_bias, att.o_bias, att.sink, att.pool, att.scale) == (7, 3, True, True, True, False, None, 0.35)
    assert (att.position.kind, att.position.dims, att.position.base, att.position.bands) == ("rope_halves", 6, 40.0, (4.0, 1.0, 3.0, 24.0))
    assert spec.layers[3].mixer.position.bands is None
    lat = spec.layers[2].mixer
    assert (lat.q_rank, lat.rot_dim, lat.window, lat.gate, lat.sink, lat.position, lat.kv_rank) == (0, 0, 9, True, False, None, 12)
    ssm = spec.layers[1].mixer
    assert (ssm.heads, ssm.vdim, ssm.state, ssm.groups, ssm.conv, ssm.norm_groups, ssm.norm_eps) == (4, 6, 5, 2, 3, 2, 1e-5)
    moe = spec.layers[0].ffn
    assert (moe.scores, moe.choice_bias, moe.gated, moe.activation, moe.router_bias, moe.weight_scale, moe.top, moe.shared.intermediate, moe.shared.activation) == \
        ("sigmoid", True, True, "silu", False, 1.7, 2, 20, "silu")
    assert spec.layers[4].ffn.shared is None and spec.layers[2].ffn.activation == "relu"
    assert (spec.layers[0].mixer_norm.offset, spec.layers[0].mixer_norm.gain, spec.layers[0].mixer_post_norm.gain, spec.embed_norm.kind) == (1.0, 1.0, 0.4, "offset_rmsnorm")
    from torchlet_amd.models.decoder import DecoderModel
    names = {n for n, s in DecoderModel(spec, torch.float32, "cpu").weight_specs().items() if not s.optional}
    assert names == set(tiny_bafulorn.tensors_for("A"))
    assert {"embed", "embed.norm", "head", "final.norm", "l0.norm1b", "l0.mix.q.b", "l0.mix.k.b", "l0.mix.o.b", "l0.mlp.correction", "l0.mlp.shared.gate",
            "l0.mlp.e4.down", "l1.mix.in", "l1.mix.conv.b", "l1.mix.A_log", "l1.mix.D", "l1.mix.norm", "l2.mix.dkv.norm", "l2.mix.g", "l2.mlp.gate"} <= names
    assert "l0.mix.v" not in names and "l1.norm2" not in names and "l4.mlp.shared.up" not in names and "l2.mix.sink" not in names
    plain = load_config(folders["C"]).to_spec()             # no masks, no rotation
    assert plain.layers[1].mixer.window is None and plain.layers[3].mixer.window is None and plain.layers[3].mixer.position.dims == 6
    assert plain.layers[2].mixer.position is None and plain.layers[2].mixer.keep_first == 2
    base = tiny_bafulorn.CONFIGS["A"]
    att_layer, ssm_layer, lat_layer = base["layers"][0], base["layers"][1], base["layers"][2]
    for bad in (dict(layers=[]), dict(layers=[dict(att_layer, type="other")]), dict(norm={}), dict(residual_mult="much"),
                dict(layers=[dict(att_layer, mixer=dict(att_layer["mixer"], heads=5))]),
                dict(layers=[dict(att_layer, mixer=dict(att_layer["mixer"], vdim=12))]),
                dict(layers=[dict(att_layer, mixer=dict(att_layer["mixer"], rot=dict(dims=12, base=10.0)))]),
                dict(layers=[dict(att_layer, mixer=dict(att_layer["mixer"], rot=dict(dims=6, base=10.0, scaling=dict(factor=2.0))))]),
                dict(layers=[dict(att_layer, mixer=dict(att_layer["mixer"], mask=dict(size=0)))]),
                dict(layers=[dict(lat_layer, mixer=dict(lat_layer["mixer"], mask=dict(size=4, keep_first=2)))]),
                dict(layers=[dict(ssm_layer, mixer=dict(ssm_layer["mixer"], groups=3))]),
                dict(layers=[dict(ssm_layer, mixer=dict(ssm_layer["mixer"], norm_groups=5))]),
                dict(layers=[dict(att_layer, mlp=dict(kind="moe", expert=dict(ff=8), router=dict(experts=2, top=3)))]),
                dict(layers=[dict(att_layer, mlp=dict(kind="other"))])):
        with pytest.raises(ConfigError):
            BafulornConfig.from_dict({**base, **bad})


def test_cache_plan_windows_kept_tokens_and_states(cpu_ops, folders):
    _, model = load_model(folders["A"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=40, max_requests=3)
    cache = runner.cache
    got = [(g.need.plane_shapes, g.need.window, g.need.keep_first, len(g.runs)) for g in cache.groups]
    assert got == [(((3, 10), (3, 10)), 7, 3, 1), (((1, 12),), 9, 0, 1), (((1, 8), (1, 8)), 5, 6, 1)]
    states = [c.state if c is not None else None for c in runner.caches]
    assert [None if s is None else tuple(s.shape) for s in states] == [None, (4, 4 * 5 * 6 + 2 * (24 + 20)), None, None, (4, 3 * 9 * 7 + 3 * (21 + 18))]
    # a slot that is used again starts from zero
    runner.step([StepEntry("a", [1, 2, 3], [])])
    slot = cache.slot("a")
    assert float(states[1][slot].abs().max()) > 0
    runner.release("a")
    runner.step([StepEntry("b", [4], [])])
    assert cache.slot("b") == slot
    fresh = make_runner(model, page_size=4, num_pages=40, max_requests=3)
    fresh.step([StepEntry("b", [4], [])])
    for s, f in zip(states, fresh.caches):
        if s is not None:
            assert torch.equal(s[slot], f.state[fresh.cache.slot("b")])


@pytest.mark.parametrize("keep", [0, 1, 4, 6, 13])
def test_pages_of_kept_first_tokens_stay_and_the_windows_go_back(keep):
    need = PagedNeed(num_heads=1, head_dim=4, window=10, keep_first=keep)
    cache = CacheManager([(need, None, None)], page_size=4, num_pages=30, max_requests=2, max_step_tokens=5)
    kept = -(-keep // 4)
    assert cache.capacity() == [min(29, 2 * ((10 + 5 - 2) // 4 + 2 + kept))]
    cache.add_request("a")
    assert cache.reserve("a", 3)
    cache.commit("a", 3)
    n = 3
    for step in [1, 1, 5, 2, 1, 1, 1, 4, 5, 5, 1, 3] * 4:       # portions and single tokens: the window's pages and the kept ones, no more
        n += step
        assert cache.reserve("a", n)
        table = list(cache.groups[0].tables["a"])
        first = max(0, n - step - 10 + 1) // 4                  # the first block the step's first query reads inside its window
        assert all(table[b] for b in range(min(kept, len(table)))) and all(table[b] for b in range(first, -(-n // 4)))
        cache.commit("a", n)
        cache.check()
        table = list(cache.groups[0].tables["a"])
        held = [b for b, p in enumerate(table) if p]
        assert held == sorted(set(range(min(kept, len(table)))) | set(range(max(0, n - 10 + 1) // 4, -(-n // 4))))
        assert len(held) <= cache.pages_for(n)[0]
    cache.add_request("b")                                      # a second request takes pages that the first gave back
    assert cache.reserve("b", 9)
    cache.commit("b", 9)
    cache.check()
    cache.release("a")
    cache.release("b")
    cache.check()
    assert cache.free_pages() == cache.capacity()


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "tail_singles", "portions", "mixed"])
def test_step_function_equals_plain_under_every_split(cpu_ops, folders, name, mode):
    lengths = [37, 5, 50, 1, 18, 33] if name != "B" else [75, 1, 27]
    seqs, refs = tiny_bafulorn.sequences(name, _weights(name), lengths)
    steps = scenarios.number(getattr(scenarios, mode)(seqs) if mode != "tail_singles" else scenarios.tail_singles(seqs, tail=9))
    page = tiny_bafulorn.PAGE_SIZES[name]
    _, model = load_model(folders[name], "float32", device="cpu")
    runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps, unit=page) // page) + 1, max_requests=4)
    scenarios.check(steps, _run(runner, steps), refs, TOL, f"{name}/{mode}")
    assert runner.cache.live_requests() == [] and runner.cache.free_pages() == runner.cache.capacity()


@pytest.mark.parametrize("seed", range(4))
def test_configurations_drawn_at_random(cpu_ops, tmp_path, seed):
    """Layers of any kind in any order, through the host side: portions and mixed batches against plain."""
    import random
    rnd = random.Random(900 + seed)
    conf = tiny_bafulorn.random_config(rnd, big=False)
    page = rnd.choice([4, 8, 16])
    folder = tiny_bafulorn.write(f"random{seed}", tmp_path, config=conf, seed=seed)
    w = {k: v.double() for k, v in tiny_bafulorn.tensors_for("", 1.0, conf, seed).items()}
    seqs, refs = tiny_bafulorn.sequences("", w, [rnd.randint(1, 60) for _ in range(4)], seed=seed, config=conf, min_gap=1e-3)
    _, model = load_model(folder, "float32", device="cpu")
    for mode in ("portions", "mixed"):
        steps = scenarios.number(getattr(scenarios, mode)(seqs))
        runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps, unit=page) // page) + 1, max_requests=4)
        scenarios.check(steps, _run(runner, steps), refs, TOL, f"{conf}/{mode}")
        assert runner.cache.free_pages() == runner.cache.capacity()


def test_stream_after_every_layer_against_plain(cpu_ops, folders):
    ids = [5, 17, 3, 60, 2, 2, 41, 9, 30, 11, 90, 4, 4, 8]
    _, want = plain_bafulorn.forward(tiny_bafulorn.CONFIGS["A"], _weights("A"), ids)
    _, model = load_model(folders["A"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=12, max_requests=1)
    seen = []
    import emulated_ops

    def settled(stream):            # what the next norm would see: the pending output normed, scaled and added
        x = stream.residual.clone()
        emulated_ops.sandwich_norm(x, stream.pending, stream.post[0], stream.post[1], None, torch.ones(1), 1e-5, torch.empty_like(x))
        return x

    for block in model.blocks:
        inner = block.forward
        block.forward = lambda stream, ctx, cache, inner=inner: (lambda s: (seen.append(settled(s)), s)[1])(inner(stream, ctx, cache))
    runner.step([StepEntry("a", ids, [len(ids) - 1])])
    assert len(seen) == 5
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, atol=5e-5, rtol=1e-5)


def _greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain_bafulorn.forward(cfg, w, ids)[0][-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_through_scheduler_and_sampler(cpu_ops, folders):
    """Prompts in portions of at most 12 tokens beside decode tokens, five requests over three slots (slots and pages are used again),
    steps enqueued ahead of their tokens, against the plain loop."""
    w = _weights("B")
    cfg = tiny_bafulorn.CONFIGS["B"]
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
    seqs, refs = tiny_bafulorn.sequences("A", _weights("A"), [13, 6, 40])
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
    src.write_text(json.dumps(tiny_bafulorn.CONFIGS["A"]))
    assert main(["init", "--config", str(src), "--seed", "3", "--out", str(tmp_path / "out")]) == 0
    cfg = load_config(tmp_path / "out")
    assert isinstance(cfg, BafulornConfig) and cfg.layers == tiny_bafulorn.CONFIGS["A"]["layers"]
    with safe_open(str(tmp_path / "out" / "model.safetensors"), framework="pt") as f:
        stored = set(f.keys())
    assert stored == {n for n, s in DecoderModel(cfg.to_spec(), torch.float32, "cpu").weight_specs().items() if not s.optional}
    _, model = load_model(tmp_path / "out", "float32", device="cpu")
    logits = make_runner(model, page_size=4, num_pages=8, max_requests=1).step([StepEntry("a", [1, 2, 3, 4, 5], [4])])
    assert logits.shape == (1, 97) and bool(torch.isfinite(logits).all())
