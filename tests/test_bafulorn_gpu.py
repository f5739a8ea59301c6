"""The Bafulorn design on the GPU through the framework's step function, cache manager, scheduler and entry point, against the plain
implementation: every way of cutting requests in both dtypes, the residual after every layer, long decoding from the first token over
many windows, slots and pages used again (the pages of the kept first tokens held, the window's given back), decode steps replayed as
graphs, a kept token far back that must show in the logits and the token after the kept ones that must not, configurations drawn at
random, and greedy generation."""
import pytest
import torch

import plain_bafulorn
import scenarios
import tiny_bafulorn

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
FP32_TOL = dict(atol=3e-4, rtol=3e-4)        # logits of order one to four; sums in another order than the 64-bit evaluation


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("bafulorn")
    return {name: tiny_bafulorn.write(name, root) for name in tiny_bafulorn.CONFIGS}


_weights_cache: dict = {}


def _weights(name, sharpen=1.0):
    key = (name, sharpen)
    if key not in _weights_cache:
        _weights_cache[key] = {k: v.double() for k, v in tiny_bafulorn.tensors_for(name, sharpen).items()}
    return _weights_cache[key]


def _rounded(t):
    return t.to(torch.bfloat16).double()


def _bf16_bound(conf, w, seqs, refs):
    """Three times what rounding to bfloat16 every tensor that separate kernels hand to each other does to the logits in a 64-bit evaluation."""
    return dict(atol=3 * max(float((plain_bafulorn.forward(conf, w, t, stored=_rounded)[0] - refs[r]).abs().max()) for r, t in seqs.items()), rtol=0.0)


def _tolerance(dtype, name, seqs, refs, sharpen=1.0):
    return FP32_TOL if dtype == "float32" else _bf16_bound(tiny_bafulorn.CONFIGS[name], _weights(name, sharpen), seqs, refs)


def _runner(folder, name, dtype, pages, slots=4, graphs=False):
    from torchlet_amd.engine.loading import load_model, make_runner
    _, model = load_model(folder, dtype)
    return make_runner(model, page_size=tiny_bafulorn.PAGE_SIZES[name], num_pages=pages, max_requests=slots, use_graphs=graphs)


def _replay(runner, steps):
    from torchlet_amd.engine.batch import StepEntry
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.cpu().numpy()
        for r in s["end"]:
            runner.release(r)
        runner.cache.check()
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_way_of_cutting_requests_equals_plain(folders, name, dtype):
    """Whole requests; most of a request and its last tokens one by one; portions of changing size down to two tokens; up to four live
    requests with portions beside single tokens, in a pool that holds no more than the live ones need, so pages and slots are used
    again.  The requests are several windows long."""
    lengths = [37, 5, 70, 1, 18, 33] if name != "B" else [90, 1, 47, 130]
    seqs, refs = tiny_bafulorn.sequences(name, _weights(name), lengths)
    tol = _tolerance(dtype, name, seqs, refs)
    page = tiny_bafulorn.PAGE_SIZES[name]
    for mode in ("whole", "tail_singles", "portions", "mixed"):
        steps = scenarios.number(getattr(scenarios, mode)(seqs) if mode != "tail_singles" else scenarios.tail_singles(seqs, tail=9))
        runner = _runner(folders[name], name, dtype, pages=-(-scenarios.max_tokens_needed(steps, unit=page) // page) + 1)
        scenarios.check(steps, _replay(runner, steps), refs, tol, f"{name}/{mode}/{dtype}")
        assert runner.cache.live_requests() == [] and runner.cache.free_pages() == runner.cache.capacity()


def test_stream_after_every_layer(folders):
    """The residual after every layer, in 32-bit (what the next norm's kernel sees once the pending output has been normed, scaled and
    added): layer by layer against the plain implementation."""
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.kernels import ops
    name = "A"
    ids = [5, 17, 3, 60, 2, 2, 41, 9, 30, 11, 90, 7, 7, 45, 1, 96]
    _, want = plain_bafulorn.forward(tiny_bafulorn.CONFIGS[name], _weights(name), ids)
    runner = _runner(folders[name], name, "float32", pages=12, slots=1)
    seen = []

    def settled(stream):
        x = stream.residual.clone()
        ops.sandwich_norm(x, stream.pending, stream.post[0], stream.post[1], None, torch.ones(1, device=x.device), 1e-5, torch.empty_like(x))
        return x.cpu()

    for block in runner.model.blocks:
        inner = block.forward
        block.forward = lambda stream, ctx, cache, inner=inner: (lambda s: (seen.append(settled(s)), s)[1])(inner(stream, ctx, cache))
    runner.step([StepEntry("a", ids, [len(ids) - 1])])
    assert len(seen) == len(want)
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, atol=1e-4, rtol=2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_from_the_first_token_and_slots_used_again(folders, dtype):
    """300 tokens one by one from an empty cache (a dozen windows; the window's pages go back, the pages of the kept first tokens stay)
    equal the plain implementation; the same request once more in the slot and the pages that the first one gave back, after another
    request has used them, gives the same logits bit for bit; and so does the whole request in one step, within the bound."""
    from torchlet_amd.engine.batch import StepEntry
    name = "B"
    seqs, refs = tiny_bafulorn.sequences(name, _weights(name), [300], seed=40)
    tol = _tolerance(dtype, name, seqs, refs)
    ids = seqs["r0"]
    runner = _runner(folders[name], name, dtype, pages=-(-300 // 16) + 1, slots=1)
    groups = runner.cache.groups
    assert all(g.need.window is not None for g in groups) and any(g.need.keep_first for g in groups)

    def one_by_one(req):
        rows = []
        for t in ids:
            rows.append(runner.step([StepEntry(req, [t], [0])]).cpu())
            for i, g in enumerate(groups):      # a window's pages and the kept tokens' pages, and no more
                held = runner.cache.capacity()[i] - runner.cache.free_pages()[i]
                assert held <= (g.need.window + 14) // 16 + 1 + -(-g.need.keep_first // 16), (i, held)
        runner.release(req)
        return torch.cat(rows)

    first = one_by_one("a")
    torch.testing.assert_close(first.double(), refs["r0"], **tol)
    runner.step([StepEntry("other", ids[50:150], [])])          # leaves its own state, tails and rows in the slot and the pages
    runner.release("other")
    assert torch.equal(one_by_one("b"), first)
    whole = runner.step([StepEntry("c", ids, list(range(300)))]).cpu()
    torch.testing.assert_close(whole.double(), refs["r0"], **tol)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_steps_replayed_as_graphs(folders, dtype):
    """Three requests of unequal lengths decode together from static buffers under a recorded graph (padding rows use the state row and
    the page that belong to no request): replays give what eager steps give."""
    from torchlet_amd.engine.batch import StepEntry
    name = "B"
    seqs, refs = tiny_bafulorn.sequences(name, _weights(name), [80, 9, 53], seed=7)
    got = {}
    for graphs in (False, True):
        runner = _runner(folders[name], name, dtype, pages=20, slots=3, graphs=graphs)
        assert runner.use_graphs == graphs
        rows = {r: [] for r in seqs}
        for r, t in seqs.items():
            rows[r].append(runner.step([StepEntry(r, t[:5], list(range(5)))]).cpu())
        for i in range(5, 80):
            live = [r for r, t in seqs.items() if i < len(t)]
            out = runner.step([StepEntry(r, [seqs[r][i]], [0]) for r in live]).cpu()
            for j, r in enumerate(live):
                rows[r].append(out[j: j + 1])
        got[graphs] = {r: torch.cat(v) for r, v in rows.items()}
        if graphs:
            assert runner.graph_replays > 30
    tol = _tolerance(dtype, name, seqs, refs)
    for r in seqs:
        torch.testing.assert_close(got[True][r].double(), refs[r], **tol)
        torch.testing.assert_close(got[True][r], got[False][r], atol=tol["atol"] / 2, rtol=0.0)


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Layers of any kind in any order, sizes of the matrix-core kernels (even seeds) or small odd ones: whole requests, portions and
    mixed batches in both dtypes against the plain implementation, every pool full at the end."""
    import random
    from torchlet_amd.engine.loading import load_model, make_runner
    rnd = random.Random(700 + seed)
    conf = tiny_bafulorn.random_config(rnd, big=seed % 2 == 0)
    page = 16 if seed % 2 == 0 else rnd.choice([4, 8, 16])
    folder = tiny_bafulorn.write(f"random{seed}", tmp_path, config=conf, seed=seed)
    w = {k: v.double() for k, v in tiny_bafulorn.tensors_for("", 1.0, conf, seed).items()}
    seqs, refs = tiny_bafulorn.sequences("", w, [rnd.randint(1, 120) for _ in range(4)], seed=seed, config=conf, min_gap=0.02)
    for dtype in DTYPES:
        tol = dict(atol=8e-4, rtol=3e-4) if dtype == "float32" else _bf16_bound(conf, w, seqs, refs)
        _, model = load_model(folder, dtype)
        for mode in ("whole", "portions", "mixed"):
            steps = scenarios.number(getattr(scenarios, mode)(seqs))
            runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps, unit=page) // page) + 1, max_requests=4)
            scenarios.check(steps, _replay(runner, steps), refs, tol, f"{conf}/{mode}/{dtype}")
            assert runner.cache.live_requests() == [] and runner.cache.free_pages() == runner.cache.capacity()


MIDDLE = dict(architecture="Bafulorn", vocab=1000, width=256, norm=dict(eps=1e-6), residual_mult=0.35, layers=[
    dict(type="latent_attention", mixer=dict(heads=8, dim=96, vdim=48, kv_rank=256, scale=0.1, mask=dict(size=100)),
         mlp=dict(kind="moe", expert=dict(ff=128), router=dict(experts=8, top=2, scale=2.0), shared=dict(ff=192))),
    dict(type="attention", mixer=dict(heads=8, kv_heads=2, dim=128, vdim=128, scale=0.09, mask=dict(size=70, keep_first=9),
                                      rot=dict(dims=64, base=100000.0, scaling=dict(factor=8.0, low=1.0, high=4.0, original=256))),
         mlp=dict(kind="dense", ff=640)),
    dict(type="mamba2", mixer=dict(heads=16, vdim=32, state=64, groups=2, conv=4, norm_groups=4), mlp=dict(kind="dense", ff=512)),
    dict(type="attention", mixer=dict(heads=6, kv_heads=6, dim=96, vdim=96, scale=0.1, mask=dict(size=33, keep_first=2), rot=dict(dims=96, base=10000.0)),
         mlp=dict(kind="moe", expert=dict(ff=96), router=dict(experts=5, top=3, scale=1.5))),
    dict(type="mamba2", mixer=dict(heads=6, vdim=64, state=128, groups=1, conv=3, norm_groups=1), mlp=None),
    dict(type="latent_attention", mixer=dict(heads=20, dim=32, vdim=64, kv_rank=128, scale=0.18, mask=dict(size=40)), mlp=dict(kind="dense", ff=384)),
])


@pytest.mark.parametrize("dtype", DTYPES)
def test_sizes_between_the_tiny_ones_and_a_real_model(tmp_path, dtype):
    """Widths and heads at which the products run on their tile kernels and the attentions in whole tiles: whole requests, portions and
    mixed batches against the plain implementation."""
    from torchlet_amd.engine.loading import load_model, make_runner
    folder = tiny_bafulorn.write("middle", tmp_path, config=MIDDLE, seed=51)
    w = {k: v.double() for k, v in tiny_bafulorn.tensors_for("middle", 1.0, MIDDLE, 51).items()}
    seqs, refs = tiny_bafulorn.sequences("", w, [230, 3, 121, 64], seed=3, config=MIDDLE, min_gap=0.02)
    tol = dict(atol=8e-4, rtol=3e-4) if dtype == "float32" else _bf16_bound(MIDDLE, w, seqs, refs)
    _, model = load_model(folder, dtype)
    for mode in ("whole", "portions", "mixed"):
        steps = scenarios.number(getattr(scenarios, mode)(seqs))
        runner = make_runner(model, page_size=16, num_pages=-(-scenarios.max_tokens_needed(steps, unit=16) // 16) + 1, max_requests=4)
        scenarios.check(steps, _replay(runner, steps), refs, tol, f"middle/{mode}/{dtype}")
        assert runner.cache.live_requests() == [] and runner.cache.free_pages() == runner.cache.capacity()


SHARP = dict(architecture="Bafulorn", vocab=80, width=64, norm=dict(eps=1e-5), residual_mult=0.5, layers=[
    dict(type="attention", mixer=dict(heads=4, kv_heads=1, dim=32, vdim=32, scale=0.3, rot=dict(dims=8, base=10000.0), mask=dict(size=32, keep_first=5)),
         mlp=dict(kind="dense", ff=64)),
    dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=32, vdim=32, scale=0.3, rot=dict(dims=16, base=500.0), mask=dict(size=20, keep_first=3)),
         mlp=dict(kind="dense", ff=64)),
])


@pytest.mark.parametrize("dtype", DTYPES)
def test_context_behind_the_window_reaches_the_logits_through_kept_tokens_only(tmp_path, dtype):
    """Two attention layers and nothing recurrent, attention sharpened.  Changing one of the kept first tokens of a 200-token request moves
    the last logits, and the 32-bit engine's logits move as the plain ones do, in a whole prompt and with the last token decoded alone
    after two portions.  Changing the token right after the kept ones, which by then lies far behind both windows, moves nothing at all."""
    from torchlet_amd.engine.batch import StepEntry
    sharpen = 3.0
    folder = tiny_bafulorn.write("sharp", tmp_path, sharpen=sharpen, config=SHARP, seed=31)
    w = {k: v.double() for k, v in tiny_bafulorn.tensors_for("sharp", sharpen, SHARP, 31).items()}
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, SHARP["vocab"], (200,), generator=g).tolist()
    ref = plain_bafulorn.forward(SHARP, w, ids)[0]
    tol = FP32_TOL if dtype == "float32" else dict(atol=3 * float((plain_bafulorn.forward(SHARP, w, ids, stored=_rounded)[0] - ref).abs().max()), rtol=0.0)
    from torchlet_amd.engine.loading import load_model, make_runner
    _, model = load_model(folder, dtype)
    runner = make_runner(model, page_size=16, num_pages=15, max_requests=2)

    def engine_last(tokens, cut):
        if cut:
            runner.step([StepEntry("d", tokens[:150], [])])
            runner.step([StepEntry("d", tokens[150:199], [])])
            out = runner.step([StepEntry("d", tokens[199:], [0])]).cpu()
        else:
            out = runner.step([StepEntry("d", tokens, [199])]).cpu()
        runner.release("d")
        return out[0].double()

    base = {cut: engine_last(ids, cut) for cut in (False, True)}
    torch.testing.assert_close(base[True], ref[199], **tol)
    torch.testing.assert_close(base[False], ref[199], **tol)
    for at in (0, 2, 4):            # kept by both layers, by both, by the first layer alone
        changed = ids[:at] + [(ids[at] + 1) % SHARP["vocab"]] + ids[at + 1:]
        other = plain_bafulorn.forward(SHARP, w, changed)[0][-1]
        move = other - ref[-1]
        assert float(move.abs().max()) > 10 * FP32_TOL["atol"], at
        for cut in (False, True):
            got = engine_last(changed, cut)
            torch.testing.assert_close(got, other, **tol)
            if dtype == "float32":
                assert float((got - base[cut] - move).abs().max()) < 0.05 * float(move.abs().max()) + FP32_TOL["atol"], (at, cut)
    changed = ids[:5] + [(ids[5] + 1) % SHARP["vocab"]] + ids[6:]          # the first token that no layer keeps
    assert float((plain_bafulorn.forward(SHARP, w, changed)[0][-1] - ref[-1]).abs().max()) == 0.0
    for cut in (False, True):
        assert torch.equal(engine_last(changed, cut), base[cut])


def _greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain_bafulorn.forward(cfg, w, ids)[0][-1].argmax()))
    return ids[len(prompt):]


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(folders, dtype):
    """``LLM(folder).generate``: the registry picks the architecture from config.json, the scheduler cuts the prompts into portions of at
    most 16 tokens beside decode tokens, four requests share three slots, decode steps run as graphs with steps enqueued ahead."""
    from torchlet_amd import LLM
    name = "B"
    cfg, w = tiny_bafulorn.CONFIGS[name], _weights(name)
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for n in (5, 60, 1, 23)]
    llm = LLM(str(folders[name]), max_decode_slots=3, kv_block_size=16, max_num_blocks=24, dtype=dtype, max_num_batched_tokens=16,
              max_model_len=128)
    outs = llm.generate(prompts, max_new_tokens=7)
    assert [len(o) for o in outs] == [7] * 4 and len({tuple(o) for o in outs}) > 1
    for p, o in zip(prompts, outs):
        if dtype == "float32":
            assert o == _greedy(cfg, w, p, 7)
        else:                                   # a reduced-precision engine may pick another token among near-ties
            ids = list(p)
            for tok in o:
                logits = plain_bafulorn.forward(cfg, w, ids)[0][-1]
                assert float(logits.max() - logits[tok]) <= 0.15
                ids.append(tok)
    assert llm.runner.cache.live_requests() == []
