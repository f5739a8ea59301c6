"""Tiny random-weight folders of the Fotovik design for the tests: sizes chosen so that what could coincide does not (query/key size
against value size, rotated dimensions against the head, heads of the two branches, key heads against heads, window against block
against page), with and without a span of layers that runs more than once, with convolutions of one tap and of several, with and
without a bigram table, a layer without a feed-forward, attention with a window of one token, blocks of one token and blocks longer
than the window, at sizes that the matrix-core kernels take and at sizes they leave to the general ones."""
import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def _attention(heads, kv_heads, dim, vdim, scale, rot=None, mask=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot is not None:
        m["rot"] = rot
    if mask is not None:
        m["mask"] = mask
    return m


def _rot(dims, base, factor=None):
    r = dict(dims=dims, base=base)
    if factor is not None:
        r["scaling"] = dict(factor=factor)
    return r


def _linear(heads, dim, vdim, decay):
    return dict(heads=heads, dim=dim, vdim=vdim, decay=decay)


def _delta(heads, kv_heads, dim, vdim, conv):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)


def _dense(ff):
    return dict(kind="dense", ff=ff) if ff else None


CONFIGS = {
    # nothing coincides and nothing is a multiple of a tile; layers 1 and 2 run three times; a layer without a feed-forward; a window
    # of 9 with blocks of 4 over pages of 4 tokens and a window of 5 with blocks of 7 (a block longer than its window)
    "A": dict(architecture="Fotovik", vocab=97, width=40, norm=dict(eps=1e-5), embedding=dict(scale=2.0, bigram=dict(buckets=31, mul_prev=7, mul_cur=3)),
              loop=dict(start=1, stop=3, times=3), layers=[
        dict(type="parallel", mixer=dict(left=_attention(4, 2, 10, 6, 0.4, rot=_rot(6, 5000.0, 1.5)), right=_linear(3, 5, 7, [0.5, 0.9, 0.99])), mlp=_dense(24)),
        dict(type="attention", mixer=_attention(6, 3, 8, 4, 0.3, rot=_rot(8, 100.0), mask=dict(size=9, pool=4)), mlp=None),
        dict(type="delta", mixer=_delta(4, 2, 5, 7, 3), mlp=_dense(12)),
        dict(type="attention", mixer=_attention(2, 1, 6, 12, 0.5, rot=_rot(4, 3000.0), mask=dict(size=5, pool=7)), mlp=_dense(20)),
    ]),
    # sizes of the matrix-core kernels, pages of 16; the window is no multiple of block or page; two layers looped twice
    "B": dict(architecture="Fotovik", vocab=80, width=64, norm=dict(eps=3e-6), embedding=dict(scale=4.0, bigram=dict(buckets=57, mul_prev=11, mul_cur=5)),
              loop=dict(start=0, stop=2, times=2), layers=[
        dict(type="attention", mixer=_attention(8, 2, 32, 64, 0.18, rot=_rot(16, 20000.0), mask=dict(size=40, pool=12)), mlp=_dense(96)),
        dict(type="parallel", mixer=dict(left=_attention(4, 4, 64, 32, 0.12, rot=_rot(64, 10000.0, 4.0)), right=_linear(2, 32, 48, [0.8, 0.97])), mlp=_dense(64)),
        dict(type="delta", mixer=_delta(4, 1, 32, 32, 4), mlp=_dense(64)),
    ]),
    # what another model may make equal or one: no bigram table, no loop, one head, blocks of one token, a window of one token, a
    # convolution of one tap, no rotation on one attention, rotation without scaling over the whole head on the other, a decay of one
    "C": dict(architecture="Fotovik", vocab=53, width=36, norm=dict(eps=2e-5), embedding=dict(scale=1.0), layers=[
        dict(type="attention", mixer=_attention(1, 1, 16, 16, 0.25, mask=dict(size=3, pool=1)), mlp=_dense(36)),
        dict(type="delta", mixer=_delta(1, 1, 20, 6, 1), mlp=None),
        dict(type="parallel", mixer=dict(left=_attention(3, 1, 12, 12, 0.3, rot=_rot(12, 400.0)), right=_linear(1, 9, 9, [1.0])), mlp=_dense(30)),
        dict(type="attention", mixer=_attention(2, 2, 6, 10, 0.45, rot=_rot(2, 50.0), mask=dict(size=1, pool=2)), mlp=_dense(18)),
    ]),
}
SEEDS = {"A": 23, "B": 24, "C": 26}
PAGE_SIZES = {"A": 4, "B": 16, "C": 8}


def tensors_for(name: str, sharpen: float = 1.0, config: dict | None = None, seed: int | None = None) -> dict[str, torch.Tensor]:
    """bfloat16 tensors of configuration ``name`` (or of ``config``): the framework's random draw, then matrices scaled up to give
    activations of order one, sinks and norm weights away from the trivial ones.  ``sharpen`` multiplies the attentions' query projections."""
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import random_tensors
    conf = config or CONFIGS[name]
    seed = SEEDS[name] if seed is None else seed
    cfg = config_class("Fotovik").from_dict(conf)
    g = torch.Generator().manual_seed(seed + 100)
    out = {}
    for k, v in random_tensors(cfg, seed, torch.float32).items():
        if v.dim() == 2 and k not in ("embed", "bigram") and not k.endswith(".conv"):
            v = v * (50.0 / v.shape[1] ** 0.5)                  # N(0, 1 / fan_in)
        if k == "embed":
            v = v * 15.0
        if k == "bigram":
            v = v * 25.0
        if k.endswith(".q") and ".right" not in k and v.shape[1] == conf["width"] and "mix" in k:
            kind = conf["layers"][int(k.split(".")[0][1:])]["type"]
            if kind != "delta":
                v = v * sharpen
        if k.endswith(".sink"):
            v = torch.randn(v.shape, generator=g) * 1.5
        if k.endswith(".conv"):
            v = v * 2.0 + (torch.arange(v.shape[1]) == v.shape[1] - 1).float() * 0.5
        if k.endswith(".dt_bias"):
            v = torch.randn(v.shape, generator=g) * 0.7
        if k.endswith((".q.norm", ".k.norm", ".left.out", ".right.out", ".right.norm", ".mix.norm")):
            v = 1.0 + (v - 1.0) * 8.0
        if v.dim() == 0:                                        # the layers' norms: one number each
            v = 0.5 + torch.rand((), generator=g)
        out[k] = v.to(torch.bfloat16)
    return out


def write(name: str, root: Path, dtype=torch.bfloat16, sharpen: float = 1.0, config: dict | None = None, seed: int | None = None) -> Path:
    folder = Path(root) / f"fotovik_{name}"
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config or CONFIGS[name], indent=1))
    save_file({k: v.to(dtype).contiguous() for k, v in tensors_for(name, sharpen, config, seed).items()}, str(folder / "model.safetensors"))
    return folder


def sequences(name: str, weights, lengths, seed: int = 0, config: dict | None = None):
    """Token sequences of the given lengths with the plain logits of each."""
    import plain_fotovik
    cfg = config or CONFIGS[name]
    g = torch.Generator().manual_seed(seed)
    seqs = {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}
    return seqs, {r: plain_fotovik.forward(cfg, weights, t)[0] for r, t in seqs.items()}


def _random_attention(rnd, big, with_mask):
    if big:
        dim, vdim = rnd.choice([32, 64, 96, 128]), rnd.choice([16, 32, 64, 128])
    else:
        dim, vdim = rnd.choice([4, 6, 10, 24]), rnd.choice([3, 8, 12])
    kv_heads = rnd.choice([1, 2, 3])
    m = _attention(kv_heads * rnd.choice([1, 2, 4]), kv_heads, dim, vdim, rnd.choice([0.1, 0.25, dim ** -0.5]))
    if rnd.random() < 0.85:
        m["rot"] = _rot(rnd.choice([d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim]), rnd.choice([100.0, 10000.0, 1e6]),
                        rnd.choice([None, 1.0, 2.0, 8.0]))
    if with_mask:
        m["mask"] = dict(size=rnd.choice([1, 3, 7, 16, 33, 50]), pool=rnd.choice([1, 2, 5, 8, 13, 16]))
    return m


def random_config(rnd, big: bool) -> dict:
    """A configuration drawn at random: one to five layers of any kind in any order, any span of them run one to three times, sizes of
    the matrix-core kernels (``big``) or small odd ones, windows and blocks from one token up, with or without bigram table,
    rotation, scaling and feed-forwards."""
    layers = []
    for _ in range(rnd.randint(1, 5)):
        kind = rnd.choice(["attention", "delta", "parallel"])
        if kind == "attention":
            mixer = _random_attention(rnd, big, True)
        elif kind == "delta":
            kv_heads = rnd.choice([1, 2])
            mixer = _delta(kv_heads * rnd.choice([1, 2]), kv_heads, rnd.choice([32, 64] if big else [5, 8, 17]), rnd.choice([32, 48] if big else [3, 9]),
                           rnd.choice([1, 2, 3, 4]))
        else:
            heads = rnd.choice([1, 2, 5])
            mixer = dict(left=_random_attention(rnd, big, False),
                         right=_linear(heads, rnd.choice([32, 64] if big else [4, 9]), rnd.choice([16, 32] if big else [5, 6]),
                                       [rnd.choice([1.0, 0.999, 0.9, 0.5]) for _ in range(heads)]))
        layers.append(dict(type=kind, mixer=mixer, mlp=_dense(rnd.choice([16, 48, 72])) if rnd.random() < 0.8 else None))
    conf = dict(architecture="Fotovik", vocab=rnd.choice([31, 90, 300]), width=rnd.choice([64, 128] if big else [24, 40, 56]),
                norm=dict(eps=rnd.choice([1e-5, 1e-6, 3e-4])), embedding=dict(scale=rnd.choice([1.0, 3.0, 0.5])), layers=layers)
    if rnd.random() < 0.8:
        conf["embedding"]["bigram"] = dict(buckets=rnd.choice([7, 101, 1021]), mul_prev=rnd.choice([1, 127, 99991]), mul_cur=rnd.choice([1, 17, 77773]))
    if rnd.random() < 0.7:
        start = rnd.randint(0, len(layers) - 1)
        conf["loop"] = dict(start=start, stop=rnd.randint(start + 1, len(layers)), times=rnd.randint(1, 3))
    return conf
