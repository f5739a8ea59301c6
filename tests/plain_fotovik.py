"""A plain, slow implementation of the Fotovik design: whole sequences, no cache, 64-bit, one function per mechanism.

It shares nothing with the package.  ``forward(config, weights, tokens)`` returns the logits of every position and the residual
stream after every layer run.  ``weights`` maps tensor names to tensors (any float type; integer tables stay integer).

The design, in this file's notation.  ``rms(x) = x / sqrt(mean(x^2) + eps)``.  A layer is ``x += g1b rms(mixer(g1 rms(x)))`` and then
``x += g2b rms(ff(g2 rms(x)))`` with one number ``g`` per norm.  The embedding is ``scale * E[t_i] + B[(a t_{i-1} + b t_i) mod n]``
(``B[n]`` for the first token).  Layers ``start .. stop - 1`` run ``times`` times in a row; before every pass but the first the
embedding's output is added to ``x``.
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def embedding(config, w, tokens):
    e = config["embedding"]
    x = w["embed"].to(F64)[tokens] * float(e["scale"])
    big = e.get("bigram")
    if big:
        n = int(big["buckets"])
        rows = [n] + [(int(tokens[i - 1]) * int(big["mul_prev"]) + int(tokens[i]) * int(big["mul_cur"])) % n for i in range(1, len(tokens))]
        x = x + w["bigram"].to(F64)[torch.tensor(rows)]
    return x


def turn(u, v, angle):
    c, s = torch.cos(angle), torch.sin(angle)
    return u * c - v * s, v * c + u * s


def rotate(x, rot, layout):
    """``x [T, heads, dim]``; the first ``rot.dims`` entries of every head are turned; ``layout``: ``pairs`` (2i with 2i + 1) or
    ``halves`` (i with i + dims / 2)."""
    if not rot:
        return x
    T, dims = x.shape[0], int(rot["dims"])
    i = torch.arange(dims // 2, dtype=F64)
    f = float(rot["base"]) ** (-2.0 * i / dims) / float((rot.get("scaling") or {}).get("factor", 1.0))
    angle = torch.arange(T, dtype=F64)[:, None, None] * f[None, None, :]
    out = x.clone()
    if layout == "pairs":
        a, b = turn(x[..., 0:dims:2], x[..., 1:dims:2], angle)
        out[..., 0:dims:2], out[..., 1:dims:2] = a, b
    else:
        a, b = turn(x[..., : dims // 2], x[..., dims // 2: dims], angle)
        out[..., : dims // 2], out[..., dims // 2: dims] = a, b
    return out


def visible(i, size, pool):
    """What position ``i`` sees under a window of ``size`` tokens with pooled blocks of ``pool``: ``(tokens, blocks)``."""
    tokens = [j for j in range(i + 1) if i - j < size]
    blocks = [b for b in range(i // pool + 1) if b * pool + pool - 1 <= i - size] if pool else []
    return tokens, blocks


def attention_head(q, k, v, scale, mask=None, sink=None):
    """One query head: ``q [T, dim]``, ``k [T, dim]``, ``v [T, vdim]``.  ``mask``: ``None`` (causal) or ``(size, pool)``.  ``sink``: a
    number whose exponential joins the denominator."""
    T = q.shape[0]
    out = torch.zeros((T, v.shape[1]), dtype=F64)
    for i in range(T):
        if mask is None:
            keys, vals = k[: i + 1], v[: i + 1]
        else:
            tokens, blocks = visible(i, mask[0], mask[1])
            P = mask[1]
            keys = torch.cat([k[tokens]] + [k[b * P: b * P + P].mean(0, keepdim=True) for b in blocks])
            vals = torch.cat([v[tokens]] + [v[b * P: b * P + P].mean(0, keepdim=True) for b in blocks])
        s = keys @ q[i] * scale
        top = s.max() if sink is None else torch.maximum(s.max(), sink)
        e = torch.exp(s - top)
        den = e.sum() + (torch.exp(sink - top) if sink is not None else 0.0)
        out[i] = (e / den) @ vals
    return out


def attention(m, w, prefix, h, eps, layout, cached=lambda x: x, stored=lambda x: x):
    """Grouped-query attention.  ``cached``: the rounding of what a cache would hold (keys after norm and rotation, values); ``stored``: of
    what separate kernels hand to each other (the projections, the rotated queries, the heads' outputs)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = stored(h @ w[prefix + "q"].to(F64).T).view(T, H, D)
    k = stored(h @ w[prefix + "k"].to(F64).T).view(T, G, D)
    v = stored(h @ w[prefix + "v"].to(F64).T).view(T, G, V)
    if prefix + "q.norm" in w:
        q = rms(q, eps) * w[prefix + "q.norm"].to(F64)
        k = rms(k, eps) * w[prefix + "k.norm"].to(F64)
    q, k = stored(rotate(q, m.get("rot"), layout)), rotate(k, m.get("rot"), layout)
    k, v = cached(k), cached(v)
    mask = (int(m["mask"]["size"]), int(m["mask"].get("pool", 0))) if m.get("mask") else None
    outs = []
    for i in range(H):
        g = i // (H // G)
        sink = w[prefix + "sink"].to(F64)[i] if prefix + "sink" in w else None
        outs.append(attention_head(q[:, i], k[:, g], v[:, g], float(m["scale"]), mask, sink))
    return stored(torch.cat(outs, -1)) @ w[prefix + "o"].to(F64).T


def short_conv(x, taps):
    """``x [T, C]``, ``taps [C, K]``: ``y_t = sum_j taps[:, K - 1 - j] x_{t - j}``, zeros before the start."""
    T, K = x.shape[0], taps.shape[1]
    padded = torch.cat((torch.zeros((K - 1, x.shape[1]), dtype=F64), x))
    return sum(padded[j: j + T] * taps[:, j] for j in range(K))


def silu(x):
    return x * torch.sigmoid(x)


def delta_rule(q, k, v, beta, g):
    """One head: ``q, k [T, dim]``, ``v [T, vdim]``, ``beta, g [T]``."""
    S = torch.zeros((q.shape[1], v.shape[1]), dtype=F64)
    out = torch.zeros_like(v)
    for t in range(q.shape[0]):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def delta_mixer(m, w, prefix, h, eps, stored=lambda x: x):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    proj = {n: silu(short_conv(stored(h @ w[prefix + n].to(F64).T), w[prefix + n + ".conv"].to(F64))) for n in "qkv"}
    q, k, v = proj["q"].view(T, G, D), proj["k"].view(T, G, D), proj["v"].view(T, H, V)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[prefix + "b"].to(F64).T)
    g = torch.exp(-torch.exp(w[prefix + "A_log"].to(F64)) * torch.nn.functional.softplus(h @ w[prefix + "a"].to(F64).T + w[prefix + "dt_bias"].to(F64)))
    gate = silu(stored(h @ w[prefix + "g"].to(F64).T)).view(T, H, V)
    outs = []
    for i in range(H):
        j = i // (H // G)
        o = delta_rule(q[:, j], k[:, j], v[:, i], beta[:, i], g[:, i])
        outs.append(rms(o, eps) * w[prefix + "norm"].to(F64) * gate[:, i])
    return stored(torch.cat(outs, -1)) @ w[prefix + "o"].to(F64).T


def lightning(q, k, v, decay):
    """One head of the decayed linear attention: ``S_t = decay S_{t-1} + k_t v_t^T``, ``o_t = S_t^T q_t``."""
    S = torch.zeros((q.shape[1], v.shape[1]), dtype=F64)
    out = torch.zeros_like(v)
    for t in range(q.shape[0]):
        S = decay * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def lightning_mixer(m, w, prefix, h, eps, stored=lambda x: x):
    T, H, D, V = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = silu(stored(h @ w[prefix + "q"].to(F64).T)).view(T, H, D)
    k = silu(stored(h @ w[prefix + "k"].to(F64).T)).view(T, H, D)
    v = silu(stored(h @ w[prefix + "v"].to(F64).T)).view(T, H, V)
    o = torch.cat([lightning(q[:, i], k[:, i], v[:, i], float(m["decay"][i])) for i in range(H)], -1)
    o = rms(o, eps) * w[prefix + "norm"].to(F64) * torch.sigmoid(stored(h @ w[prefix + "g"].to(F64).T))
    return stored(o) @ w[prefix + "o"].to(F64).T


def parallel_mixer(m, w, prefix, h, eps, cached=lambda x: x, stored=lambda x: x):
    left = stored(attention(m["left"], w, prefix + "left.", h, eps, "halves", cached, stored))
    right = stored(lightning_mixer(m["right"], w, prefix + "right.", h, eps, stored))
    return 0.5 * (rms(left, eps) * w[prefix + "left.out"].to(F64) + rms(right, eps) * w[prefix + "right.out"].to(F64))


def dense_ff(w, prefix, h, stored=lambda x: x):
    z = stored(h @ w[prefix + "up"].to(F64).T)
    return stored(0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))) @ w[prefix + "down"].to(F64).T


def mixer(layer, w, prefix, h, eps, cached=lambda x: x, stored=lambda x: x):
    kind = layer["type"]
    if kind == "attention":
        return attention(layer["mixer"], w, prefix, h, eps, "pairs", cached, stored)
    if kind == "delta":
        return delta_mixer(layer["mixer"], w, prefix, h, eps, stored)
    if kind == "parallel":
        return parallel_mixer(layer["mixer"], w, prefix, h, eps, cached, stored)
    raise ValueError(kind)


def run_order(config):
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for p in range(times):
        order += [(i, p > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(config, w, tokens, cached=lambda x: x, stored=lambda x: x):
    """``(logits [T, vocab], residual after every layer run [runs, T, width])``, 64-bit.  ``stored``: a rounding of what the sublayers read
    and hand back (to see what an engine that keeps those in fewer bits may differ by); ``cached``: the same for cached keys and values."""
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x0 = embedding(config, w, tokens)
    x = x0.clone()
    after = []
    for i, again in run_order(config):
        layer, name = config["layers"][i], f"l{i}."
        if again:
            x = x + x0
        y = stored(mixer(layer, w, name + "mix.", stored(rms(x, eps) * w[name + "norm1"].to(F64)), eps, cached, stored))
        x = x + rms(y, eps) * w[name + "norm1b"].to(F64)
        if layer.get("mlp"):
            y = stored(dense_ff(w, name + "mlp.", stored(rms(x, eps) * w[name + "norm2"].to(F64)), stored))
            x = x + rms(y, eps) * w[name + "norm2b"].to(F64)
        after.append(x.clone())
    logits = stored(rms(x, eps) * w["final.norm"].to(F64)) @ w["head"].to(F64).T
    return logits, torch.stack(after)
