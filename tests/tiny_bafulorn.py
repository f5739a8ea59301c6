"""Tiny random-weight folders of the Bafulorn design for the tests: sizes chosen so that what could coincide does not (query/key size
against value size against latent, heads against key heads against groups, rotated dimensions against the head, window against kept
tokens against page), every kind of layer in several orders, layers without a feed-forward, routers that pick one, some or all experts
with and without a shared expert, windows of one token, kept tokens that span pages, no mask at all, convolutions of one tap and of
several, at sizes that the matrix-core kernels take and at sizes they leave to the general ones."""
import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def _latent(heads, dim, vdim, kv_rank, scale, window=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, kv_rank=kv_rank, scale=scale)
    if window is not None:
        m["mask"] = dict(size=window)
    return m


def _attention(heads, kv_heads, dim, scale, rot=None, window=None, keep_first=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale)
    if rot is not None:
        m["rot"] = rot
    if window is not None:
        m["mask"] = dict(size=window) if keep_first is None else dict(size=window, keep_first=keep_first)
    return m


def _rot(dims, base, scaling=None):
    r = dict(dims=dims, base=base)
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def _mamba(heads, vdim, state, groups, conv, norm_groups):
    return dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=norm_groups)


def _dense(ff):
    return dict(kind="dense", ff=ff)


def _moe(ff, experts, top, scale=None, shared=None):
    m = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
    if scale is not None:
        m["router"]["scale"] = scale
    if shared is not None:
        m["shared"] = dict(ff=shared)
    return m


CONFIGS = {
    # nothing coincides and nothing is a multiple of a tile; pages of 4; a window of 9 on the latent, a window of 7 that keeps 3 tokens and
    # one of 5 that keeps 6 (more than its window, more than a page); frequencies in all three bands of the scaling; a layer without a
    # feed-forward
    "A": dict(architecture="Bafulorn", vocab=97, width=40, norm=dict(eps=1e-5), residual_mult=0.4, layers=[
        dict(type="attention", mixer=_attention(6, 3, 10, 0.35, rot=_rot(6, 40.0, (4.0, 1.0, 3.0, 24)), window=7, keep_first=3), mlp=_moe(12, 5, 2, 1.7, 20)),
        dict(type="mamba2", mixer=_mamba(4, 6, 5, 2, 3, 2), mlp=None),
        dict(type="latent_attention", mixer=_latent(3, 6, 10, 12, 0.3, window=9), mlp=_dense(24)),
        dict(type="attention", mixer=_attention(2, 1, 8, 0.4, rot=_rot(8, 900.0), window=5, keep_first=6), mlp=_dense(20)),
        dict(type="mamba2", mixer=_mamba(3, 7, 9, 1, 4, 1), mlp=_moe(8, 4, 3, 0.8)),
    ]),
    # sizes of the matrix-core kernels, pages of 16; windows that are no multiples of the page; kept tokens that span two pages
    "B": dict(architecture="Bafulorn", vocab=80, width=64, norm=dict(eps=3e-6), residual_mult=0.25, layers=[
        dict(type="latent_attention", mixer=_latent(4, 32, 48, 64, 0.18, window=40), mlp=_moe(32, 6, 3, 2.2, 32)),
        dict(type="attention", mixer=_attention(4, 2, 64, 0.12, rot=_rot(32, 50000.0, (8.0, 1.0, 4.0, 512)), window=24, keep_first=20), mlp=_dense(96)),
        dict(type="mamba2", mixer=_mamba(4, 32, 32, 2, 4, 2), mlp=_dense(64)),
        dict(type="latent_attention", mixer=_latent(2, 64, 32, 128, 0.125, window=21), mlp=None),
    ]),
    # what another model may make equal or one: no mask on one latent attention and on one attention, one head, a window of one token,
    # kept tokens without any beyond the window's start, no rotation, rotation over the whole head without scaling, a convolution of one
    # tap, one group and as many groups as heads, a router that picks one expert and one that picks all, a factor of one on the branches
    "C": dict(architecture="Bafulorn", vocab=53, width=36, norm=dict(eps=2e-5), residual_mult=1.0, layers=[
        dict(type="mamba2", mixer=_mamba(2, 8, 4, 2, 1, 1), mlp=_moe(10, 3, 1)),
        dict(type="latent_attention", mixer=_latent(1, 16, 16, 16, 0.25), mlp=_dense(36)),
        dict(type="attention", mixer=_attention(1, 1, 12, 0.3, window=1, keep_first=2), mlp=_moe(6, 2, 2, 1.0, 9)),
        dict(type="attention", mixer=_attention(3, 3, 6, 0.45, rot=_rot(6, 50.0)), mlp=None),
        dict(type="latent_attention", mixer=_latent(5, 4, 2, 6, 0.5, window=1), mlp=_dense(18)),
    ]),
}
SEEDS = {"A": 33, "B": 34, "C": 36}
PAGE_SIZES = {"A": 4, "B": 16, "C": 8}


def tensors_for(name: str, sharpen: float = 1.0, config: dict | None = None, seed: int | None = None) -> dict[str, torch.Tensor]:
    """bfloat16 tensors of configuration ``name`` (or of ``config``): the framework's random draw, then matrices scaled up to give
    activations of order one, and norm weights, biases, gates and skips away from the trivial ones.  ``sharpen`` multiplies the query
    projections.  Clear choices of experts: every token's embedding carries three of a few fixed directions of the stream with weights 1,
    0.7 and 0.4, and expert e's router row looks along direction e (the stream keeps most of the normed embedding from layer to layer), so
    that no choice hangs on the last bits of a score, where a reduced-precision engine would be free to choose otherwise; what the
    sublayers write into the stream is kept off those directions (their output matrices' columns have them taken out)."""
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import random_tensors
    conf = config or CONFIGS[name]
    seed = SEEDS[name] if seed is None else seed
    cfg = config_class("Bafulorn").from_dict(conf)
    g = torch.Generator().manual_seed(seed + 100)
    width, vocab = conf["width"], conf["vocab"]
    routed = {n: layer["mlp"]["router"]["experts"] for n, layer in enumerate(conf["layers"]) if layer.get("mlp") and layer["mlp"]["kind"] == "moe"}
    basis = torch.linalg.qr(torch.randn(width, max(1, min(width, sum(routed.values()))), generator=g)).Q.T * width ** 0.5
    directions, code, at = {}, torch.zeros(vocab, width), 0
    for n, experts in routed.items():
        directions[n] = basis[[(at + e) % basis.shape[0] for e in range(experts)]]
        at += experts
        for t in range(vocab):
            a = (t + n) % experts
            b = (a + 1 + (t // experts) % max(experts - 1, 1)) % experts
            rest = [e for e in range(experts) if e not in (a, b)]
            picks = [a, b] + ([rest[(t // 7) % len(rest)]] if rest else [])
            for weight, e in zip((1.0, 0.7, 0.4), dict.fromkeys(picks)):
                code[t] += weight * directions[n][e]
    drawn = random_tensors(cfg, seed, torch.float32)
    # the norms of the stream first (their weights are stored around zero): what looks along a direction, or must stay off it, allows for them
    norms = {k: (torch.randn(v.shape, generator=g) * 0.3).to(torch.bfloat16).float() for k, v in drawn.items()
             if k.rsplit(".", 1)[-1] in ("norm1", "norm2", "norm1b", "norm2b") or k in ("embed.norm", "final.norm")}
    out = {}
    for k, v in drawn.items():
        leaf, layer = k.rsplit(".", 1)[-1], k.split(".")[0]
        if k in norms:
            out[k] = norms[k].to(torch.bfloat16)
            continue
        if v.dim() == 2 and k != "embed" and leaf != "conv":
            v = v * (50.0 / v.shape[1] ** 0.5)                  # N(0, 1 / fan_in)
        if k == "embed":
            v = v * 12.0 + 1.5 * code / (1.0 + norms["embed.norm"])
        if routed and ((leaf in ("o", "down") and v.dim() == 2) or k.endswith(".o.b")):
            # the sublayers' outputs stay off the routers' directions, after the norm that follows them has weighed them
            seen = basis * (1.0 + norms[f"{layer}.norm1b" if ".mix." in k else f"{layer}.norm2b"])
            v = v - seen.T @ torch.linalg.solve(seen @ seen.T, seen @ v)
        if leaf == "router":
            v = v * 0.02 + directions[int(layer[1:])] * (5.0 / width) / (1.0 + norms[f"{layer}.norm2"])
        if leaf == "correction":
            v = torch.randn(v.shape, generator=g) * 0.01
        if leaf == "q" and ".mix." in k:
            v = v * sharpen
        if leaf == "conv":
            v = v * 2.0 + (torch.arange(v.shape[1]) == v.shape[1] - 1).float() * 0.5
        if leaf == "b" or leaf == "dt_bias":                    # biases of projections and convolutions, the step sizes' bias
            v = torch.randn(v.shape, generator=g) * 0.4
            if k.endswith(".o.b") and routed:
                seen = basis * (1.0 + norms[f"{layer}.norm1b"])
                v = v - seen.T @ torch.linalg.solve(seen @ seen.T, seen @ v)
        if k.endswith((".mix.norm", ".dkv.norm")):
            v = 1.0 + (v - 1.0) * 8.0
        out[k] = v.to(torch.bfloat16)
    return out


def write(name: str, root: Path, dtype=torch.bfloat16, sharpen: float = 1.0, config: dict | None = None, seed: int | None = None) -> Path:
    folder = Path(root) / f"bafulorn_{name}"
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config or CONFIGS[name], indent=1))
    save_file({k: v.to(dtype).contiguous() for k, v in tensors_for(name, sharpen, config, seed).items()}, str(folder / "model.safetensors"))
    return folder


def sequences(name: str, weights, lengths, seed: int = 0, config: dict | None = None, min_gap: float = 0.03):
    """Token sequences of the given lengths for which no token's choice of experts hangs on less than ``min_gap`` in a choice score, with the
    plain logits of each."""
    import plain_bafulorn
    cfg = config or CONFIGS[name]
    for s in range(seed, seed + 30):
        g = torch.Generator().manual_seed(s)
        seqs = {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}
        gaps: list[float] = []
        refs = {r: plain_bafulorn.forward(cfg, weights, t, gaps=gaps)[0] for r, t in seqs.items()}
        if not gaps or min(gaps) > min_gap:
            return seqs, refs
    raise AssertionError(f"no seed gives every token a clear choice of experts (last smallest margin {min(gaps):.4f})")


def random_config(rnd, big: bool) -> dict:
    """A configuration drawn at random: one to five layers of any kind in any order, sizes of the matrix-core kernels (``big``) or small odd
    ones, windows and kept tokens from none up, with or without rotation, scaling, feed-forwards and shared experts."""
    layers = []
    for _ in range(rnd.randint(1, 5)):
        kind = rnd.choice(["latent_attention", "attention", "mamba2"])
        window = rnd.choice([None, 1, 3, 7, 16, 33, 50])
        if kind == "latent_attention":
            mixer = _latent(rnd.choice([1, 2, 4, 5]), rnd.choice([32, 64] if big else [4, 6, 10]), rnd.choice([16, 32, 80] if big else [3, 8, 12]),
                            rnd.choice([64, 128] if big else [5, 12, 24]), rnd.choice([0.1, 0.25]), window)
        elif kind == "attention":
            dim = rnd.choice([32, 64, 96, 128] if big else [4, 6, 10, 24])
            kv_heads = rnd.choice([1, 2, 3])
            rot = None
            if rnd.random() < 0.85:
                scaling = rnd.choice([None, (8.0, 1.0, 4.0, 64), (2.0, 0.5, 3.0, 1000), (16.0, 1.0, 2.0, 8)])
                rot = _rot(rnd.choice([d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim]), rnd.choice([100.0, 10000.0, 1e6]), scaling)
            mixer = _attention(kv_heads * rnd.choice([1, 2, 4]), kv_heads, dim, rnd.choice([0.1, 0.25, dim ** -0.5]), rot, window,
                               rnd.choice([None, 0, 1, 4, 19]) if window is not None else None)
        else:
            groups = rnd.choice([1, 2])
            heads = groups * rnd.choice([1, 2, 3])
            vdim = rnd.choice([32, 48] if big else [3, 8, 9])
            mixer = _mamba(heads, vdim, rnd.choice([32, 64] if big else [5, 8, 17]), groups, rnd.choice([1, 2, 3, 4]),
                           rnd.choice([n for n in (1, 2, 3, heads) if (heads * vdim) % n == 0]))
        roll = rnd.random()
        if roll < 0.15:
            mlp = None
        elif roll < 0.55:
            mlp = _dense(rnd.choice([16, 48, 72]))
        else:
            experts = rnd.choice([2, 4, 7])
            mlp = _moe(rnd.choice([8, 24, 32]), experts, rnd.choice([1, 2, 3, experts]) if experts > 2 else rnd.choice([1, 2]),
                       rnd.choice([None, 1.0, 2.2]), rnd.choice([None, 16, 40]))
        layers.append(dict(type=kind, mixer=mixer, mlp=mlp))
    return dict(architecture="Bafulorn", vocab=rnd.choice([31, 90, 300]), width=rnd.choice([64, 128] if big else [24, 40, 56]),
                norm=dict(eps=rnd.choice([1e-5, 1e-6, 3e-4])), residual_mult=rnd.choice([1.0, 0.3, 0.55]), layers=layers)
