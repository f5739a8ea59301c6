"""Each mechanism of the Bafulorn design alone, against the plain functions of ``plain_bafulorn.py`` in 64-bit, at sizes that are no
multiples of the kernels' tiles: the normed embedding, the norm with a weight around zero, frequencies scaled by wavelength and the
rotation that also copies the keys as they come, the attention with a window and kept first tokens (every position a query, portions
down to two tokens, pages in scrambled order with NaN wherever nothing was written, keys at the edges made to carry the weight), the
latent attention with a window and a gate, the selective recurrence behind its convolution (portions against single steps to the bit,
slots used again), the gate before a norm in groups, the sigmoid router with a correction, the experts' sum with a shared expert, the
gated feed-forward with relu in its fused and unfused forms."""
import pytest
import torch

import plain_bafulorn as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype, loose=1.0):
    return dict(atol=2e-5 * loose, rtol=2e-5 * loose) if dtype == torch.float32 else dict(atol=2e-2 * loose, rtol=2e-2 * loose)


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device="cuda")


def _tables(lengths, page, g):
    """Block tables of requests of the given lengths over pages handed out in scrambled order."""
    blocks = [-(-n // page) for n in lengths]
    pages = sum(blocks) + 1
    order = (torch.randperm(pages - 1, generator=g) + 1).tolist()
    table = torch.zeros(len(lengths), max(blocks + [1]) + 1, dtype=torch.int32)
    for r, b in enumerate(blocks):
        for i in range(b):
            table[r, i] = order.pop()
    return table, pages


def _steps(lengths, cuts):
    """The steps of requests cut at ``cuts[r]``: per step the live requests with their spans of positions."""
    edges = [[0] + c + [n] for c, n in zip(cuts, lengths)]
    for s in range(max(len(e) for e in edges) - 1):
        spans = {r: (e[s], e[s + 1]) for r, e in enumerate(edges) if s + 1 < len(e) and e[s + 1] > e[s]}
        if spans:
            yield spans


# ------------------------------------------------------------------ embedding and norms

@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_rows_normed_on_their_way_into_the_stream(dtype):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    V, H, eps = 50, 70, 1e-5
    table = (torch.randn(V, H, generator=g) * 3).to(dtype)
    w = torch.randn(H, generator=g) * 0.3
    ids = torch.randint(0, V, (11,), generator=g)
    out = torch.full((11, H), float("nan"), device="cuda")
    ops.embedding_norm(_i32(ids.tolist()), table.cuda(), out, 1.0, (1.0 + w).cuda(), eps)
    torch.testing.assert_close(out.cpu().double(), plain.offset_rms_norm(table.double()[ids], w.double(), eps), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_with_a_weight_stored_around_zero_and_a_factor_on_the_branch(dtype):
    """The part folds ``1 + w`` and the branch's factor into one vector at load; a block's norm after a sublayer rides on the stream and the
    next norm's kernel norms the output, adds it and norms the sum."""
    from torchlet_amd.config.base import OffsetRMSNormSpec
    from torchlet_amd.parts import NORMS, Stream
    g = torch.Generator().manual_seed(2)
    T, H, eps, m = 6, 150, 1e-5, 0.3
    pre = NORMS.build(OffsetRMSNormSpec(dim=H, eps=eps, weight_name=""), dtype, torch.device("cuda"))
    post = NORMS.build(OffsetRMSNormSpec(dim=H, eps=eps, gain=m, weight_name=""), dtype, torch.device("cuda"))
    w_pre, w_post = torch.randn(H, generator=g) * 0.3, torch.randn(H, generator=g) * 0.3
    pre.load_weights({"": w_pre.to(torch.bfloat16)})
    post.load_weights({"": w_post.to(torch.bfloat16)})
    w_pre, w_post = w_pre.to(torch.bfloat16).double(), w_post.to(torch.bfloat16).double()
    x = torch.randn(T, H, generator=g) * 3
    y = (torch.randn(T, H, generator=g) * 7).to(dtype)
    stream = Stream(x.cuda(), y.cuda())
    stream.post = (post.weight, post.eps)
    h = pre.forward(stream)
    new = x.double() + m * plain.offset_rms_norm(y.double(), w_post, eps)
    torch.testing.assert_close(stream.residual.cpu().double(), new, atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(h.cpu().double(), plain.offset_rms_norm(new, w_pre, eps), **_tol(dtype, 3))
    assert stream.pending is None and stream.post is None


def test_frequencies_scaled_by_wavelength():
    """All three bands: kept, divided, blended; against the plain list."""
    from torchlet_amd.config.base import HalfRotarySpec
    from torchlet_amd.parts import POSITION_ENCODINGS
    for dims, base, bands in ((16, 40.0, (4.0, 1.0, 3.0, 24)), (64, 300000.0, (6.0, 1.0, 4.0, 4096)), (6, 10.0, None), (32, 1e4, (2.0, 0.5, 3.0, 7))):
        enc = POSITION_ENCODINGS.build(HalfRotarySpec(dims=dims, base=base, bands=bands), torch.float32, torch.device("cuda"))
        scaling = dict(zip(("factor", "low", "high", "original"), bands)) if bands else None
        want = torch.tensor(plain.scaled_frequencies(dims, base, scaling), dtype=torch.float64)
        torch.testing.assert_close(enc.inv_freq.cpu().double(), want, atol=0.0, rtol=1e-7)
        if bands:
            plain_f = torch.tensor(plain.scaled_frequencies(dims, base, None), dtype=torch.float64)
            ratio = want / plain_f
            assert (ratio <= 1.0 + 1e-12).all() and (ratio >= 1.0 / bands[0] - 1e-12).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim, dims", [(10, 6), (96, 96), (128, 32), (8, 0)])
def test_rotation_over_part_of_a_head_with_the_keys_copied_as_they_come(dtype, dim, dims):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    T, H, G = 7, 5, 2
    x = torch.randn(T, (H + G) * dim + 9, generator=g).to(dtype)
    positions = torch.tensor([0, 1, 2, 95, 96, 4000, 30000])
    freqs = plain.scaled_frequencies(dims, 5000.0, dict(factor=8.0, low=1.0, high=4.0, original=64)) if dims else []
    inv = torch.tensor(freqs, dtype=torch.float32).cuda() if dims else None
    xs = x.cuda()
    raw = torch.full((T, G * dim), float("nan"), dtype=dtype, device="cuda")
    ops.head_norm_rotate(xs[:, : (H + G) * dim], H, G, dim, None, None, 0.0, _i32(positions.tolist()), inv, dims, True, raw_b=raw)
    assert torch.equal(raw.cpu(), x[:, H * dim: (H + G) * dim]) and torch.equal(xs[:, (H + G) * dim:].cpu(), x[:, (H + G) * dim:])
    v = x[:, : (H + G) * dim].double().view(T, H + G, dim)
    want = plain.rotate_halves(v, positions, [float(f) for f in torch.tensor(freqs, dtype=torch.float32)])
    loose = 1 + float(positions.max()) * 2 ** -24 / 2e-5 * 4 if dtype == torch.float32 else 2
    torch.testing.assert_close(xs[:, : (H + G) * dim].cpu().double().view(T, H + G, dim), want, **_tol(dtype, loose))


# ------------------------------------------------------------------ attention with a window and kept first tokens

def _attend(dtype, H, G, dim, page, window, keep, lengths, cuts, g, q=None, k=None, scale=0.3):
    """Keys (and the values, which are other tensors here so that a swap would show) go to scrambled pages in steps, every token of every
    step is a query.  Returns the outputs per request by the general kernel and (where built) by the matrix-core kernel."""
    from torchlet_amd.kernels import ops
    q = q or [torch.randn(n, H * dim, generator=g) for n in lengths]
    k = k or [torch.randn(n, G * dim, generator=g) for n in lengths]
    v = [torch.randn(n, G * dim, generator=g) for n in lengths]
    table, pages = _tables(lengths, page, g)
    table = table.cuda()
    nan = float("nan")
    kp = torch.full((pages, G, page, dim), nan, dtype=dtype, device="cuda")
    vp = torch.full((pages, G, dim, page), nan, dtype=dtype, device="cuda")
    fits = ops.local_attention_mfma_fits(dtype, dim, dim, page)
    outs = {m: [torch.zeros(n, H * dim) for n in lengths] for m in (False, True)}
    for spans in _steps(lengths, cuts):
        live = list(spans)
        lens = [spans[r][1] - spans[r][0] for r in live]
        indptr = [0] + torch.tensor(lens).cumsum(0).tolist()
        token_req = _i32([i for i, n in enumerate(lens) for _ in range(n)])
        positions = _i32([p for r in live for p in range(*spans[r])])
        ctx = _i32([spans[r][0] for r in live])
        cat = lambda xs: torch.cat([xs[r][spans[r][0]: spans[r][1]] for r in live]).to(dtype).cuda()
        tab = table[live].contiguous()
        ops.kv_cache_write(cat(k), cat(v), token_req, positions, tab, kp, vp, page)
        # what a window has left behind may be gone: pages wholly before every later query's window and beyond the kept tokens go to
        # the sentinel, as the cache manager does it
        for i, r in enumerate(live):
            if window:
                first_live = max(0, spans[r][0] - window + 1) // page
                kept = -(-keep // page)
                tab[i, kept: max(kept, first_live)] = 0
        for use_mfma in ((False, True) if fits else (False,)):
            out = torch.full((int(indptr[-1]), H * dim), nan, dtype=dtype, device="cuda")
            tiles = None
            if use_mfma:
                tile_req = [i for i, n in enumerate(lens) for _ in range(-(-n // 16))]
                tile_tok0 = [16 * j for n in lens for j in range(-(-n // 16))]
                tiles = (_i32(indptr), ctx, _i32(tile_req), _i32(tile_tok0), len(tile_req))
            ops.local_attention(cat(q), out, kp, vp, tab, token_req, positions, H, G, dim, dim, page, scale, 0.0, 0, window, 1.0, tiles=tiles,
                                keep_first=keep)
            for i, r in enumerate(live):
                outs[use_mfma][r][spans[r][0]: spans[r][1]] = out[indptr[i]: indptr[i + 1]].float().cpu()
    return q, k, v, outs, fits


def _plain_attention(q, k, v, H, G, dim, window, keep, dtype, scale=0.3):
    n = q.shape[0]
    rounded = lambda t: t.to(dtype).double()
    qq, kk, vv = rounded(q).view(n, H, dim), rounded(k).view(n, G, dim), rounded(v).view(n, G, dim)
    mask = plain.mask_matrix(n, window or None, keep)
    return torch.cat([plain.softmax_attention(qq[:, h], kk[:, h // (H // G)], vv[:, h // (H // G)], scale, mask) for h in range(H)], -1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dim, page, window, keep", [
    (6, 3, 10, 4, 9, 3),          # general kernel only; nothing is a multiple of anything
    (4, 1, 32, 8, 20, 6),         # sizes of the matrix-core kernel
    (4, 2, 96, 16, 44, 5),        # kept tokens inside one page
    (2, 2, 64, 16, 33, 37),       # more kept tokens than the window holds, over three pages
    (2, 1, 32, 8, 1, 2),          # a window of one token
    (3, 1, 16, 8, 5, 0),          # a window that keeps nothing
    (4, 4, 32, 8, 0, 0),          # causal
])
def test_attention_with_window_and_kept_first_tokens(dtype, H, G, dim, page, window, keep):
    """Every position a query: in a whole prompt, in portions that cut pages and windows at odd places (down to two tokens) and in single
    tokens, two requests side by side, the pages behind the window gone; both kernels on the same pages."""
    g = torch.Generator().manual_seed(5)
    lengths = [83, 41]
    cuts = [[30, 32, 47, 48, 49, 50, 70], [2, 25, 26, 27]]
    q, k, v, outs, fits = _attend(dtype, H, G, dim, page, window, keep, lengths, cuts, g)
    assert fits == (dtype == torch.bfloat16 and dim % 32 == 0)
    for r in range(len(lengths)):
        want = _plain_attention(q[r], k[r], v[r], H, G, dim, window, keep, dtype)
        for use_mfma in ((False, True) if fits else (False,)):
            torch.testing.assert_close(outs[use_mfma][r].double(), want, **_tol(dtype, 2 if dtype == torch.float32 else 1.5))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True])
def test_keys_at_the_edges_carry_the_weight_or_none(dtype, decoded):
    """One query at the end of 302 tokens; among the keys one is made to match it.  At the first position of the window, at the last kept
    position, at position 0 far back and at a page's border inside the window it must come through whole; just outside the window, and at
    the first position that is not kept, it must not show at all."""
    H, G, dim, page, window, keep = 2, 1, 32, 8, 24, 11
    n = 302
    last = n - 1
    g = torch.Generator().manual_seed(6)
    base_q, base_k = torch.randn(n, H * dim, generator=g) * 0.2, torch.randn(n, G * dim, generator=g) * 0.2
    seen = {"first of the window": last - window + 1, "last kept": keep - 1, "far back": 0, "page border": 296}
    unseen = {"just outside the window": last - window, "first not kept": keep}
    for what, at in {**seen, **unseen}.items():
        q, k = base_q.clone(), base_k.clone()
        q[last] = torch.randn(H * dim, generator=g)
        k[at] = q[last, :dim] * 3.0             # the key matches the first head's query
        cuts = [[n - 1]] if decoded else [[150, 290]]
        _, _, v, outs, fits = _attend(dtype, H, G, dim, page, window, keep, [n], cuts, g, q=[q], k=[k], scale=1.0)
        want = _plain_attention(q, k, v[0], H, G, dim, window, keep, dtype, scale=1.0)[last]
        value = v[0][at].to(dtype).double()
        for use_mfma in ((False, True) if fits else (False,)):
            got = outs[use_mfma][0][last].double()
            torch.testing.assert_close(got, want, **_tol(dtype, 2))
            near = float((got[:dim] - value).abs().max())
            assert (near < 0.05) == (what in seen), (what, use_mfma, near)


# ------------------------------------------------------------------ latent attention with a window and a gate

def _latent_attend(dtype, H, rank, page, window, lengths, cuts, g, scale=0.2, q=None, c=None, gated=True):
    from torchlet_amd.kernels import ops
    q = q or [torch.randn(n, H * rank, generator=g) for n in lengths]         # queries already against the latent
    c = c or [torch.randn(n, rank, generator=g) for n in lengths]             # the cached rows
    gate = [torch.randn(n, H, generator=g) * 2 for n in lengths]
    table, pages = _tables(lengths, page, g)
    table = table.cuda()
    plane = torch.full((pages, 1, page, rank), float("nan"), dtype=dtype, device="cuda")
    fits = ops.latent_attention_mfma_fits(dtype, H, rank, 0)
    outs = {m: [torch.zeros(n, H * rank) for n in lengths] for m in (False, True)}
    for spans in _steps(lengths, cuts):
        live = list(spans)
        lens = [spans[r][1] - spans[r][0] for r in live]
        indptr = [0] + torch.tensor(lens).cumsum(0).tolist()
        ctx = _i32([spans[r][0] for r in live])
        cat = lambda xs: torch.cat([xs[r][spans[r][0]: spans[r][1]] for r in live]).to(dtype).cuda()
        tab = table[live].contiguous()
        for i, r in enumerate(live):            # the cache write, by hand: the rows are cached as they are
            for p in range(*spans[r]):
                plane[int(tab[i, p // page]), 0, p % page] = c[r][p].to(dtype).cuda()
            if window:
                tab[i, : max(0, spans[r][0] - window + 1) // page] = 0
        for use_mfma in ((False, True) if fits else (False,)):
            tq = ops.latent_tile_tokens(H, ops.LATENT_MFMA_ROWS if use_mfma else ops.LATENT_ATTENTION_ROWS)
            tile_req = [i for i, n in enumerate(lens) for _ in range(-(-n // tq))]
            tile_tok0 = [tq * j for n in lens for j in range(-(-n // tq))]
            for splits in (1, 3):
                out = torch.full((int(indptr[-1]), H * rank), float("nan"), dtype=dtype, device="cuda")
                ops.latent_attention(cat(q), out, plane, tab, _i32(indptr), ctx, _i32(tile_req), _i32(tile_tok0), len(tile_req), tq, H, rank, 0,
                                     page, scale, None, splits, general=not use_mfma, max_new_tokens=max(lens), window=window,
                                     gate=cat(gate) if gated else None)
                for i, r in enumerate(live):
                    got = out[indptr[i]: indptr[i + 1]].float().cpu()
                    if splits == 1:
                        outs[use_mfma][r][spans[r][0]: spans[r][1]] = got
                    else:
                        torch.testing.assert_close(got, outs[use_mfma][r][spans[r][0]: spans[r][1]], **_tol(dtype, 2))
    return q, c, gate, outs, fits


def _plain_latent(q, c, gate, H, rank, window, dtype, scale=0.2, gated=True):
    n = q.shape[0]
    rounded = lambda t: t.to(dtype).double()
    qq, cc = rounded(q).view(n, H, rank), rounded(c)
    mask = plain.mask_matrix(n, window or None, 0)
    heads = [plain.softmax_attention(qq[:, h], cc, cc, scale, mask) * (torch.sigmoid(rounded(gate)[:, h: h + 1]) if gated else 1.0) for h in range(H)]
    return torch.cat(heads, -1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, rank, page, window", [(3, 12, 4, 9), (8, 192, 16, 40), (4, 64, 16, 33), (20, 64, 8, 1), (2, 64, 16, 0), (5, 24, 8, 96)])
def test_latent_attention_with_a_window_and_a_gate(dtype, H, rank, page, window):
    """Every position a query, whole, in portions down to two tokens and in single tokens, two requests side by side over scrambled pages,
    the pages behind the window gone, the keys dealt to one work-group and to three; both kernels on the same pages."""
    g = torch.Generator().manual_seed(7)
    lengths = [83, 41]
    cuts = [[30, 32, 47, 48, 49, 50, 70], [2, 25, 26, 27]]
    q, c, gate, outs, fits = _latent_attend(dtype, H, rank, page, window, lengths, cuts, g)
    for r in range(len(lengths)):
        want = _plain_latent(q[r], c[r], gate[r], H, rank, window, dtype)
        for use_mfma in ((False, True) if fits else (False,)):
            torch.testing.assert_close(outs[use_mfma][r].double(), want, **_tol(dtype, 2 if dtype == torch.float32 else 1.5))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decoded", [False, True])
def test_latent_rows_at_the_window_edge_carry_the_weight_or_none(dtype, decoded):
    """One query at the end of 300 tokens (in a portion, or decoded alone) whose first head matches one cached row: at the first position of
    the window and at a page border inside it the row comes through whole; just outside the window, and far back, it does not show at all."""
    H, rank, page, window, n = 2, 64, 16, 40, 300
    last = n - 1
    g = torch.Generator().manual_seed(8)
    for what, at, shows in (("first of the window", last - window + 1, True), ("just outside the window", last - window, False),
                            ("page border inside", 288, True), ("far back", 0, False)):
        q, c = torch.randn(n, H * rank, generator=g) * 0.2, torch.randn(n, rank, generator=g) * 0.2
        c[at] = torch.randn(rank, generator=g)
        q[last, :rank] = c[at] * 3.0
        _, _, _, outs, fits = _latent_attend(dtype, H, rank, page, window, [n], [[n - 1]] if decoded else [[150, 290]], g, scale=1.0, q=[q], c=[c], gated=False)
        want = _plain_latent(q, c, None, H, rank, window, dtype, scale=1.0, gated=False)[last]
        for use_mfma in ((False, True) if fits else (False,)):
            got = outs[use_mfma][0][last].double()
            torch.testing.assert_close(got, want, **_tol(dtype, 2))
            near = float((got[:rank] - c[at].to(dtype).double()).abs().max())
            assert (near < 0.05) == shows, (what, use_mfma, near)


# ------------------------------------------------------------------ the selective recurrence

def _selective(dtype, heads, vdim, state, groups, taps, lengths, cuts, g, slots, st, weights=None):
    """The mixer's middle (convolution, step sizes, recurrence) over requests cut into steps; returns y per request and the weights."""
    from torchlet_amd.kernels import ops
    inner, gn = heads * vdim, groups * state
    C = inner + 2 * gn
    if weights is None:
        weights = dict(conv=torch.randn(C, taps, generator=g) * 0.5, conv_b=torch.randn(C, generator=g) * 0.3, a_log=torch.log(torch.rand(heads, generator=g) + 0.05),
                       dt_bias=torch.randn(heads, generator=g), D=torch.randn(heads, generator=g),
                       proj=[torch.randn(n, 7 + C + heads + 5, generator=g) for n in lengths])
    w = weights
    dev = {k: v.cuda() for k, v in w.items() if k != "proj"}
    ys = [torch.zeros(n, inner) for n in lengths]
    for spans in _steps(lengths, cuts):
        live = list(spans)
        lens = [spans[r][1] - spans[r][0] for r in live]
        indptr = _i32([0] + torch.tensor(lens).cumsum(0).tolist())
        token_req = _i32([i for i, n in enumerate(lens) for _ in range(n)])
        proj = torch.cat([w["proj"][r][spans[r][0]: spans[r][1]] for r in live]).to(dtype).cuda()
        T = proj.shape[0]
        gates = torch.full((T, 2 * heads), float("nan"), device="cuda")
        cbx = torch.full((T, C), float("nan"), device="cuda")
        sl = _i32([slots[r] for r in live])
        ops.selective_prepare(proj, 7, dev["conv"], dev["conv_b"], gates, dev["a_log"], dev["dt_bias"], st, heads * state * vdim, sl, indptr, token_req,
                              cbx, heads, inner, gn, taps)
        y = torch.full((T, inner), float("nan"), device="cuda")
        ops.selective_scan(cbx, gates, dev["D"], st, sl, indptr, y, heads, groups, state, vdim, max_new_tokens=max(lens))
        at = 0
        for r, n in zip(live, lens):
            ys[r][spans[r][0]: spans[r][1]] = y[at: at + n].cpu()
            at += n
    return ys, weights


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, vdim, state, groups, taps", [(4, 6, 5, 2, 3), (6, 40, 56, 2, 4), (2, 8, 4, 2, 1), (3, 20, 130, 1, 8), (4, 64, 128, 1, 4)])
def test_selective_recurrence_against_plain_and_portions_to_the_bit(dtype, heads, vdim, state, groups, taps):
    """Whole requests against the plain convolution and recurrence; the same requests in uneven portions (shorter than the taps) and token by
    token, beside each other, in slots that another request has used, give the same bits."""
    g = torch.Generator().manual_seed(9)
    lengths = [37, 12]
    inner, gn = heads * vdim, groups * state
    C = inner + 2 * gn
    width = heads * state * vdim + (taps - 1) * C
    st = torch.zeros(4, width, device="cuda")
    whole, w = _selective(dtype, heads, vdim, state, groups, taps, lengths, [[], []], g, slots=[1, 3], st=st)
    for r, n in enumerate(lengths):
        p = w["proj"][r].to(dtype).double()[:, 7:]
        xbc = plain.silu(plain.causal_convolution(p[:, :C], w["conv"].double(), w["conv_b"].double()))
        dt = torch.nn.functional.softplus(p[:, C: C + heads] + w["dt_bias"].double(), threshold=1e9)
        want = plain.selective_recurrence(xbc[:, :inner].reshape(n, heads, vdim), xbc[:, inner: inner + gn].reshape(n, groups, state),
                                          xbc[:, inner + gn:].reshape(n, groups, state), dt, w["a_log"].double(), w["D"].double(), heads, groups)
        torch.testing.assert_close(whole[r].double(), want.reshape(n, inner), atol=5e-4, rtol=2e-4)
    left = st.clone()
    for cuts in ([[2, 3, 10, 11, 30], [1, 9]], [list(range(1, 37)), list(range(1, 12))]):
        st2 = torch.randn(4, width, device="cuda")       # what other requests left in the slots
        st2[[0, 2]] = 0.0                                # a slot is zero when it is handed out
        again, _ = _selective(dtype, heads, vdim, state, groups, taps, lengths, cuts, g, slots=[2, 0], st=st2, weights=w)
        for r in range(2):
            assert torch.equal(again[r], whole[r]), (cuts, r)
        assert torch.equal(st2[2], left[1]) and torch.equal(st2[0], left[3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inner, groups", [(24, 2), (320, 2), (30, 1), (64, 8), (1300, 2), (4096, 1)])
def test_gate_before_a_norm_in_groups(dtype, inner, groups):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(10)
    T, eps = 5, 1e-5
    y, z = torch.randn(T, inner, generator=g) * 3, (torch.randn(T, inner + 6, generator=g) * 2).to(dtype)
    w = 1 + 0.3 * torch.randn(inner, generator=g)
    out = torch.full((T, inner), float("nan"), dtype=dtype, device="cuda")
    ops.gated_head_norm(y.cuda(), z.cuda()[:, :inner], w.cuda(), eps, out, groups, inner // groups, gate="silu", gate_first=True)
    u = (y.double() * plain.silu(z.double()[:, :inner])).view(T, groups, inner // groups)
    want = (u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)).reshape(T, inner) * w.double()
    torch.testing.assert_close(out.cpu().double(), want, **_tol(dtype, 3))


# ------------------------------------------------------------------ routed experts and gated feed-forwards

def test_sigmoid_router_with_a_correction_that_changes_the_choice_only():
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(11)
    T, E, top, scale = 40, 7, 3, 1.75
    logits = torch.randn(T, E, generator=g) * 2
    logits[0] = torch.tensor([0.3, 1.0, 1.0, -2.0, 1.0, 0.0, 1.0])               # ties: the lower index wins
    correction = torch.tensor([0.0, -0.5, 0.4, 0.0, 0.1, 0.9, -0.2])
    w = {"router": torch.eye(E, dtype=torch.float64), "correction": correction.double()}
    chosen, weights = plain.sigmoid_router(logits.double(), w, dict(top=top, scale=scale))
    plain_choice, _ = plain.sigmoid_router(logits.double(), {**w, "correction": torch.zeros(E, dtype=torch.float64)}, dict(top=top, scale=scale))
    assert (chosen != plain_choice).any()
    got_w, offsets, slot_token, pair_slot = ops.route(logits.cuda(), top, "sigmoid", correction.cuda(), scale, 1e-20)
    torch.testing.assert_close(got_w.cpu().double(), weights, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(got_w.sum(-1).cpu(), torch.full((T,), scale), atol=1e-5, rtol=1e-5)
    offsets, slot_token, pair_slot = offsets.cpu(), slot_token.cpu(), pair_slot.cpu()
    for t in range(T):
        for j in range(top):
            slot = int(pair_slot[t * top + j])
            e = int(chosen[t, j])
            assert int(offsets[e]) <= slot < int(offsets[e + 1]) and int(slot_token[slot]) == t


@pytest.mark.parametrize("dtype", DTYPES)
def test_weighted_sum_of_the_experts_with_a_shared_expert_added(dtype):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(12)
    T, top, W = 9, 3, 50
    y = torch.randn(T * top, W, generator=g).to(dtype)
    shared = torch.randn(T, W, generator=g).to(dtype)
    weights = torch.rand(T, top, generator=g)
    pair_slot = torch.randperm(T * top, generator=g).to(torch.int32)
    out = torch.full((T, W), float("nan"), dtype=dtype, device="cuda")
    ops.combine(y.cuda(), pair_slot.cuda(), weights.cuda(), out, addend=shared.cuda())
    want = (y.double()[pair_slot.long()].view(T, top, W) * weights.double()[:, :, None]).sum(1) + shared.double()
    torch.testing.assert_close(out.cpu().double(), want, **_tol(dtype, 3))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["relu", "silu"])
@pytest.mark.parametrize("T", [1, 7, 40, 300])
def test_gated_feed_forward_fused_and_unfused(dtype, act, T):
    """The part at a width and an inner size that are no multiples of the tiles (and, in bfloat16, with the gate applied to the product's
    sums inside its kernel at every number of rows: the few-rows kernel and the tile kernels)."""
    from torchlet_amd.config.base import SwiGLUSpec
    from torchlet_amd.parts import FEED_FORWARDS
    g = torch.Generator().manual_seed(13)
    for H, I in ((72, 100), (128, 320)):
        ff = FEED_FORWARDS.build(SwiGLUSpec(hidden=H, intermediate=I, activation=act, gate_name="gate", up_name="up", down_name="down"), dtype, torch.device("cuda"))
        w = {"gate": torch.randn(I, H, generator=g) / H ** 0.5, "up": torch.randn(I, H, generator=g) / H ** 0.5, "down": torch.randn(H, I, generator=g) / I ** 0.5}
        ff.load_weights({k: v.to(torch.bfloat16) for k, v in w.items()})
        x = torch.randn(T, H, generator=g).to(dtype)
        out = ff.forward(x.cuda(), None, whole=True)
        wd = {k: v.to(torch.bfloat16).double() for k, v in w.items()}
        want = plain.gated_ff(x.double(), wd, "", torch.relu if act == "relu" else plain.silu)
        torch.testing.assert_close(out.cpu().double(), want, **_tol(dtype, 5 if dtype == torch.float32 else 2))
