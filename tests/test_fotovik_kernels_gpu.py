"""Each kernel of the Fotovik design's mechanisms alone, against the plain functions of ``plain_fotovik.py`` in 64-bit, at sizes that
are no multiples of the kernels' tiles: the embedding with its bigram rows and the token before a portion, the norm that norms what it
adds, the norm per head with both rotations, the attention with a window, pooled blocks and a sink (every position a query, portions
that cut blocks, pages in scrambled order with NaN wherever nothing was written, keys at the edges made to carry the weight), the
linear attention with fixed decays (portions against single steps to the bit), the sum of normed branches, the exact gelu."""
import math

import pytest
import torch

import plain_fotovik as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype, loose=1.0):
    return dict(atol=2e-5 * loose, rtol=2e-5 * loose) if dtype == torch.float32 else dict(atol=2e-2 * loose, rtol=2e-2 * loose)


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device="cuda")


# ------------------------------------------------------------------ embedding

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("copies", [0, 2])
def test_embedding_with_bigram_rows_and_the_token_before_a_portion(dtype, copies):
    """Three requests: a whole one, one continued (the token before its first comes from its slot) and a single first token; then a second
    step that continues two of them, and a new request in a slot that another one used."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    V, H, n, a, b = 50, 70, 13, 1_000_003, 77
    table, big = torch.randn(V, H, generator=g).to(dtype), torch.randn(n + 1, H, generator=g).to(dtype)
    seqs = [torch.randint(0, V, (k,), generator=g).tolist() for k in (9, 12, 5)]
    want = [plain.embedding(dict(embedding=dict(scale=3.0, bigram=dict(buckets=n, mul_prev=a, mul_cur=b))), dict(embed=table, bigram=big), torch.tensor(s))
            for s in seqs]
    last = torch.full((5, 1), -7, dtype=torch.int32, device="cuda")         # (what a used slot may hold)
    last[2, 0] = seqs[1][3]

    def step(parts, slots):
        ids = [t for s, lo, hi in parts for t in seqs[s][lo:hi]]
        lens = [hi - lo for _, lo, hi in parts]
        indptr = [0] + torch.tensor(lens).cumsum(0).tolist()
        token_req = [r for r, k in enumerate(lens) for _ in range(k)]
        positions = [p for _, lo, hi in parts for p in range(lo, hi)]
        out = torch.full((copies, len(ids), H) if copies else (len(ids), H), float("nan"), device="cuda")
        ops.bigram_embedding(_i32(ids), table.cuda(), out, 3.0, big.cuda(), n, a, b, _i32(token_req), _i32(indptr), _i32(positions), _i32(slots), last)
        ref = torch.cat([want[s][lo:hi] for s, lo, hi in parts])
        torch.testing.assert_close(out.cpu().double(), ref.expand(out.shape) if copies else ref, atol=1e-5, rtol=1e-6)

    step([(0, 0, 9), (1, 4, 10), (2, 0, 1)], [0, 2, 4])
    assert last[:, 0].tolist() == [seqs[0][8], -7, seqs[1][9], -7, seqs[2][0]]
    step([(2, 1, 5), (1, 10, 12)], [4, 2])
    step([(0, 0, 3)], [2])                                  # a first token never reads its slot


# ------------------------------------------------------------------ norms

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("parts, scalar", [(0, True), (3, True), (0, False)])
def test_norm_of_the_branch_output_addition_and_norm_of_the_sum(dtype, parts, scalar):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    T, H, eps, peps = 6, 150, 1e-5, 3e-4
    x = torch.randn(T, H, generator=g) * 3
    extra = torch.randn(T, H, generator=g)
    pen = torch.randn(parts, T, H, generator=g) if parts else (torch.randn(T, H, generator=g) * 4).to(dtype)
    p = pen.double().sum(0) if parts else pen.double()
    w = torch.tensor([1.3]) if scalar else 1 + 0.1 * torch.randn(H, generator=g)
    pw = torch.tensor([0.7]) if scalar else 1 + 0.1 * torch.randn(H, generator=g)
    normed = plain.rms(p, peps) * pw.double()
    for use_extra, use_post in ((False, True), (True, True), (True, False), (False, False)):
        new = x.double() + (extra.double() if use_extra else 0) + (normed if use_post else p)
        xs = x.cuda()
        out = torch.empty(T, H, dtype=dtype, device="cuda")
        ops.sandwich_norm(xs, pen.cuda(), pw.cuda() if use_post else None, peps, extra.cuda() if use_extra else None, w.cuda(), eps, out)
        torch.testing.assert_close(xs.cpu().double(), new, atol=2e-5, rtol=1e-5)            # the stream stays 32-bit in both engines
        torch.testing.assert_close(out.cpu().double(), plain.rms(new, eps) * w.double(), **_tol(dtype, 3))
        rows = torch.tensor([4, 0, 4], dtype=torch.int32)
        xs = x.cuda()
        few = torch.empty(3, H, dtype=dtype, device="cuda")
        ops.sandwich_norm(xs, pen.cuda(), pw.cuda() if use_post else None, peps, extra.cuda() if use_extra else None, w.cuda(), eps, few, rows.cuda(), gain=2.0)
        assert torch.equal(xs.cpu(), x)                                                      # chosen rows: nothing is written back
        torch.testing.assert_close(few.cpu().double(), 2.0 * (plain.rms(new, eps) * w.double())[rows.long()], **_tol(dtype, 3))
    xs = x.cuda()
    out = torch.empty(T, H, dtype=dtype, device="cuda")
    ops.sandwich_norm(xs, None, None, 0.0, None, w.cuda(), eps, out)                        # a first norm with nothing pending
    assert torch.equal(xs.cpu(), x)
    torch.testing.assert_close(out.cpu().double(), plain.rms(x.double(), eps) * w.double(), **_tol(dtype, 3))


@pytest.mark.parametrize("dtype", DTYPES)
def test_sum_of_normed_branches(dtype):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    B, T, H, eps = 3, 5, 90, 1e-4
    x = (torch.randn(B, T, H, generator=g) * torch.tensor([1.0, 20.0, 0.05])[:, None, None]).to(dtype)
    w = torch.randn(B, H, generator=g)
    out = torch.empty(T, H, dtype=dtype, device="cuda")
    ops.normed_sum(x.cuda(), w.cuda(), eps, out)
    want = (plain.rms(x.double(), eps) * w.double()[:, None, :]).sum(0)
    torch.testing.assert_close(out.cpu().double(), want, **_tol(dtype, 3))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim, dims, halves, normed", [(10, 6, True, True), (8, 8, False, False), (128, 64, True, True), (70, 2, False, True), (16, 0, False, True)])
def test_norm_per_head_and_rotation_in_place(dtype, dim, dims, halves, normed):
    """Queries and keys side by side in rows that are longer than both (the values follow): positions far out, both layouts, a rotation
    over fewer dimensions than the head has, scaled frequencies; what follows the keys stays as it was."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    T, H, G, eps = 7, 5, 2, 1e-5
    x = torch.randn(T, (H + G) * dim + 9, generator=g).to(dtype)
    wq, wk = 1 + 0.3 * torch.randn(dim, generator=g), 1 + 0.3 * torch.randn(dim, generator=g)
    positions = torch.tensor([0, 1, 2, 95, 96, 4000, 30000])
    rot = dict(dims=dims, base=5000.0, scaling=dict(factor=2.5)) if dims else None
    xs = x.cuda()
    inv = None
    if dims:
        i = torch.arange(dims // 2, dtype=torch.float64)
        inv = (5000.0 ** (-2.0 * i / dims) / 2.5).float().cuda()
    ops.head_norm_rotate(xs[:, : (H + G) * dim], H, G, dim, wq.cuda() if normed else None, wk.cuda() if normed else None, eps,
                         positions.int().cuda(), inv, dims, halves)
    assert torch.equal(xs[:, (H + G) * dim:].cpu(), x[:, (H + G) * dim:])
    v = x.double()[:, : (H + G) * dim].view(T, H + G, dim)
    if normed:
        v = torch.cat((plain.rms(v[:, :H], eps) * wq.double(), plain.rms(v[:, H:], eps) * wk.double()), 1)
    want = torch.empty_like(v)
    for t in range(T):          # the plain rotation counts positions from 0: put every token at its own
        full = torch.zeros(int(positions[t]) + 1, H + G, dim, dtype=torch.float64)
        full[-1] = v[t]
        want[t] = plain.rotate(full, rot, "halves" if halves else "pairs")[-1]
    # angles are 32-bit in the engine: at position p an angle is off by up to p * 2^-24 of itself
    loose = 1 + float(positions.max()) * 2 ** -24 / 2e-5 * 4 if dtype == torch.float32 else 2
    torch.testing.assert_close(xs[:, : (H + G) * dim].cpu().double().view(T, H + G, dim), want, **_tol(dtype, loose))


# ------------------------------------------------------------------ attention

def _tables(lengths, page, g, span=None):
    """Block tables of requests of the given lengths over pages handed out in scrambled order (``span``: positions a page covers)."""
    span = span or page
    blocks = [-(-n // span) for n in lengths]
    pages = sum(blocks) + 1
    order = (torch.randperm(pages - 1, generator=g) + 1).tolist()
    table = torch.zeros(len(lengths), max(blocks + [1]) + 1, dtype=torch.int32)
    for r, b in enumerate(blocks):
        for i in range(b):
            table[r, i] = order.pop()
    return table, pages


def _attend(dtype, H, G, dim, vdim, page, window, pool, sink, lengths, cuts, g, q=None, k=None, v=None, mfma=None):
    """Keys and values of requests of ``lengths`` go to scrambled pages in steps (``cuts[r]``: where request r's tokens are cut into
    steps), blocks are pooled as their last tokens arrive, and every token of every step is a query.  Returns the attention's output
    per request, ``[n, H * vdim]``, by the general kernel and (where built) by the matrix-core kernel."""
    from torchlet_amd.kernels import ops
    R = len(lengths)
    q = q or [torch.randn(n, H * dim, generator=g) for n in lengths]
    k = k or [torch.randn(n, G * dim, generator=g) for n in lengths]
    v = v or [torch.randn(n, G * vdim, generator=g) for n in lengths]
    table, pages = _tables(lengths, page, g)
    ptable, ppages = _tables(lengths, page, g, span=page * pool) if pool else (None, 0)
    width = max(table.shape[1], ptable.shape[1] if pool else 0)
    table = torch.nn.functional.pad(table, (0, width - table.shape[1])).cuda()
    nan = float("nan")
    kp = torch.full((pages, G, page, dim), nan, dtype=dtype, device="cuda")
    vp = torch.full((pages, G, vdim, page), nan, dtype=dtype, device="cuda")
    pooled = None
    if pool:
        ptable = torch.nn.functional.pad(ptable, (0, width - ptable.shape[1])).cuda()
        pkp = torch.full((ppages, G, page, dim), nan, dtype=dtype, device="cuda")
        pvp = torch.full((ppages, G, vdim, page), nan, dtype=dtype, device="cuda")
        pooled = (pkp, pvp, ptable, pool)
    outs = {False: [torch.zeros(n, H * vdim) for n in lengths], True: [torch.zeros(n, H * vdim) for n in lengths]}
    fits = ops.local_attention_mfma_fits(dtype, dim, vdim, page) if mfma is None else mfma
    steps = max(len(c) for c in cuts) + 1
    for s in range(steps):
        spans = [((([0] + c + [n])[s], ([0] + c + [n])[s + 1]) if s < len(c) + 1 else (n, n)) for c, n in zip(cuts, lengths)]
        live = [r for r in range(R) if spans[r][1] > spans[r][0]]
        if not live:
            continue
        lens = [spans[r][1] - spans[r][0] for r in live]
        indptr = [0] + torch.tensor(lens).cumsum(0).tolist()
        token_req = _i32([i for i, n in enumerate(lens) for _ in range(n)])
        positions = _i32([p for r in live for p in range(*spans[r])])
        ctx = _i32([spans[r][0] for r in live])
        qs = torch.cat([q[r][spans[r][0]: spans[r][1]] for r in live]).to(dtype).cuda()
        ks = torch.cat([k[r][spans[r][0]: spans[r][1]] for r in live]).to(dtype).cuda()
        vs = torch.cat([v[r][spans[r][0]: spans[r][1]] for r in live]).to(dtype).cuda()
        tab = table[live].contiguous()
        ops.kv_cache_write(ks, vs, token_req, positions, tab, kp, vp, page)
        step_pooled = None
        if pool:
            step_pooled = (pkp, pvp, ptable[live].contiguous(), pool)
            ops.pool_blocks(kp, vp, tab, pkp, pvp, step_pooled[2], _i32(indptr), ctx, max(lens) // pool + 1, page, pool)
        for use_mfma in ((False, True) if fits else (False,)):
            out = torch.full((qs.shape[0], H * vdim), nan, dtype=dtype, device="cuda")
            tiles = None
            if use_mfma:
                tile_req = [i for i, n in enumerate(lens) for _ in range(-(-n // 16))]
                tile_tok0 = [16 * j for n in lens for j in range(-(-n // 16))]
                tiles = (_i32(indptr), ctx, _i32(tile_req), _i32(tile_tok0), len(tile_req))
            ops.local_attention(qs, out, kp, vp, tab, token_req, positions, H, G, dim, vdim, page, 0.3, 0.0, 0, window, 1.0, tiles=tiles,
                                sink=sink.cuda() if sink is not None else None, pooled=step_pooled)
            for i, r in enumerate(live):
                outs[use_mfma][r][spans[r][0]: spans[r][1]] = out[indptr[i]: indptr[i + 1]].float().cpu()
    return q, k, v, outs, fits


def _plain_attention(q, k, v, H, G, dim, vdim, window, pool, sink, dtype):
    n = q.shape[0]
    rounded = lambda t: t.to(dtype).double()
    qq, kk, vv = rounded(q).view(n, H, dim), rounded(k).view(n, G, dim), rounded(v).view(n, G, vdim)
    mask = (window, pool) if window else None
    return torch.cat([plain.attention_head(qq[:, h], kk[:, h // (H // G)], vv[:, h // (H // G)], 0.3, mask,
                                           sink.double()[h] if sink is not None else None) for h in range(H)], -1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dim, vdim, page, window, pool, with_sink", [
    (6, 3, 10, 6, 4, 9, 4, True),         # general kernel only; a window that is no multiple of block or page
    (4, 1, 32, 16, 8, 20, 6, True),       # sizes of the matrix-core kernel
    (2, 2, 64, 64, 16, 33, 12, False),    # pooled blocks without a sink
    (4, 2, 32, 32, 16, 5, 7, True),       # a block longer than the window
    (2, 1, 32, 16, 8, 3, 1, True),        # blocks of one token: every token is read, as itself or as its own block
    (3, 1, 16, 32, 8, 1, 2, True),        # a window of one token
    (4, 4, 32, 64, 8, 0, 0, True),        # causal, with a sink
    (2, 1, 128, 64, 16, 0, 0, False),     # causal and plain
])
def test_attention_with_window_pooled_blocks_and_sink(dtype, H, G, dim, vdim, page, window, pool, with_sink):
    """Every position a query: in a whole prompt, in portions that cut blocks and pages at odd places (down to two tokens) and in single
    tokens, two requests side by side; both kernels on the same pages."""
    g = torch.Generator().manual_seed(5)
    lengths = [83, 41]
    cuts = [[30, 32, 47, 48, 49, 50, 70], [2, 25, 26, 27]]
    sink = torch.randn(H, generator=g) * 2 if with_sink else None
    q, k, v, outs, fits = _attend(dtype, H, G, dim, vdim, page, window, pool, sink, lengths, cuts, g)
    assert fits == (dtype == torch.bfloat16 and dim % 32 == 0 and vdim % 16 == 0)
    for r, n in enumerate(lengths):
        want = _plain_attention(q[r], k[r], v[r], H, G, dim, vdim, window, pool, sink, dtype)
        if dtype == torch.bfloat16 and pool:        # the pooled rows are rounded once more when they are stored
            pass
        for use_mfma in ((False, True) if fits else (False,)):
            torch.testing.assert_close(outs[use_mfma][r].double(), want, **_tol(dtype, 2 if dtype == torch.float32 else 1.5))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True])
def test_keys_at_the_edges_carry_the_weight_or_none(dtype, decoded):
    """One query; among hundreds of keys one is made to match it.  Put at the first position of the window, at the last position of the
    newest pooled block, in the middle of the oldest pooled block far back, it must come through (whole, or as its share of a block's
    mean); put just outside the window in a block that is not whole yet, it must not show at all."""
    H, G, dim, vdim, page, window, pool = 2, 1, 32, 16, 8, 24, 6
    n = 302
    last = n - 1
    first_in_window = last - window + 1                   # 278
    blocks = (last - window + 1) // pool                  # 46 blocks are seen: positions 0 .. 275; 276 and 277 are read by nobody
    g = torch.Generator().manual_seed(6)
    base_q, base_k = torch.randn(n, H * dim, generator=g) * 0.3, torch.randn(n, G * dim, generator=g) * 0.3
    base_v = torch.randn(n, G * vdim, generator=g)
    direction = torch.randn(dim, generator=g)
    direction = direction / direction.norm() * 12.0
    cuts = [[150, 290] + list(range(291, n))] if decoded else [[]]
    for place, seen, share in ((first_in_window, True, 1.0), (blocks * pool - 1, True, 1 / pool), (3, True, 1 / pool),
                               (first_in_window - 1, False, 0.0)):
        q, k, v = base_q.clone(), base_k.clone(), base_v.clone()
        q[last] = direction.repeat(H)
        k[place] = direction * (1.0 if share == 1.0 else pool)          # a pooled key keeps a sixth of it
        v[place] = 50.0
        _, _, _, outs, fits = _attend(dtype, H, G, dim, vdim, page, window, pool, None, [n], cuts, g, q=[q], k=[k], v=[v])
        want = _plain_attention(q, k, v, H, G, dim, vdim, window, pool, None, dtype)[last]
        assert (float(want.abs().min()) > 30 * share) if seen else (float(want.abs().max()) < 5)
        for use_mfma in ((False, True) if fits else (False,)):
            torch.testing.assert_close(outs[use_mfma][0][last].double(), want, **_tol(dtype, 3))
    # a sink large enough to take half the weight
    sink = torch.tensor([4.0, -30.0])
    q, k, v, outs, fits = _attend(dtype, H, G, dim, vdim, page, window, pool, sink, [40], [[39]] if decoded else [[]], g)
    with_sink = _plain_attention(q[0], k[0], v[0], H, G, dim, vdim, window, pool, sink, dtype)
    without = _plain_attention(q[0], k[0], v[0], H, G, dim, vdim, window, pool, None, dtype)
    assert float((with_sink - without)[:, :vdim].abs().max()) > 0.2 and float((with_sink - without)[:, vdim:].abs().max()) < 1e-6
    for use_mfma in ((False, True) if fits else (False,)):
        torch.testing.assert_close(outs[use_mfma][0].double(), with_sink, **_tol(dtype, 2))


# ------------------------------------------------------------------ linear attention with fixed decays

@pytest.mark.parametrize("H, dim, vdim", [(3, 5, 7), (2, 32, 48), (1, 130, 20), (6, 64, 64)])
def test_decayed_linear_attention_against_plain_and_portions_to_the_bit(H, dim, vdim):
    """Two requests whole against the plain recurrence; then token by token and in uneven portions beside another request, in slots
    that held other states before: the same bits, outputs and states left behind."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(7)
    lengths = [37, 21]
    C = 2 * H * dim + H * vdim
    decay = torch.tensor([1.0, 0.5, 0.97, 0.9, 0.999, 0.0][:H])
    raw = [torch.randn(n, C + 5, generator=g) for n in lengths]
    stride = H * dim * vdim + 11

    def run(cuts, slots):
        state = torch.randn(6, stride, generator=g).cuda()
        for s in slots:
            state[s].zero_()
        outs = [torch.zeros(n, H * vdim) for n in lengths]
        for s in range(max(len(c) for c in cuts) + 1):
            spans = [((([0] + c + [n])[s], ([0] + c + [n])[s + 1]) if s < len(c) + 1 else (n, n)) for c, n in zip(cuts, lengths)]
            live = [r for r in range(2) if spans[r][1] > spans[r][0]]
            if not live:
                continue
            lens = [spans[r][1] - spans[r][0] for r in live]
            indptr = [0] + torch.tensor(lens).cumsum(0).tolist()
            x = torch.cat([raw[r][spans[r][0]: spans[r][1]] for r in live]).cuda()
            qkv = torch.empty(x.shape[0], C, device="cuda")
            ops.silu_float(x[:, :C], qkv)
            out = torch.full((x.shape[0], H * vdim), float("nan"), device="cuda")
            ops.decay_scan(qkv, decay.cuda(), state, _i32([slots[r] for r in live]), _i32(indptr), out, H, dim, vdim, max_new_tokens=max(lens))
            for i, r in enumerate(live):
                outs[r][spans[r][0]: spans[r][1]] = out[indptr[i]: indptr[i + 1]].cpu()
        return outs, [state[s, : H * dim * vdim].cpu() for s in slots]

    whole, left = run([[], []], [4, 1])
    for r, n in enumerate(lengths):
        x = plain.silu(raw[r][:, :C].double())
        q, k, v = x[:, : H * dim].view(n, H, dim), x[:, H * dim: 2 * H * dim].view(n, H, dim), x[:, 2 * H * dim:].view(n, H, vdim)
        want = torch.cat([plain.lightning(q[:, h], k[:, h], v[:, h], float(decay[h])) for h in range(H)], -1)
        torch.testing.assert_close(whole[r].double(), want, atol=1e-4 * float(want.abs().max()), rtol=1e-5)
    for cuts, slots in (([list(range(1, 37)), list(range(1, 21))], [0, 3]), ([[2, 19, 20, 36], [5, 7]], [2, 5])):
        outs, states = run(cuts, slots)
        for r in range(2):
            assert torch.equal(outs[r], whole[r]) and torch.equal(states[r], left[r])


@pytest.mark.parametrize("dtype", DTYPES)
def test_exact_gelu(dtype):
    from torchlet_amd.kernels import ops
    x = torch.linspace(-6, 6, 1001).to(dtype)
    y = x.clone().cuda()
    ops.load(["experts"])
    ops.activation(y, "gelu")
    want = 0.5 * x.double() * (1 + torch.erf(x.double() / math.sqrt(2)))
    torch.testing.assert_close(y.cpu().double(), want, **_tol(dtype))
    tanh_form = 0.5 * x.double() * (1 + torch.tanh(math.sqrt(2 / math.pi) * (x.double() + 0.044715 * x.double() ** 3)))
    if dtype == torch.float32:          # the two forms differ by more than the bound: the exact one is what runs
        assert float((tanh_form - want).abs().max()) > 1e-4 and float((y.cpu().double() - want).abs().max()) < 1e-5
