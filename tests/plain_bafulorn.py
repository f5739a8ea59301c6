"""A plain, slow implementation of the Bafulorn decoder: whole sequences, no cache, one function per mechanism, in the dtype of the
tensors it is given (the tests hand it 64-bit copies of the weights).  It shares nothing with the package.

The design: token embedding, normed; layers ``x <- x + m * post1(mixer(pre1(x)))``, ``x <- x + m * post2(ff(pre2(x)))`` with
root-mean-square norms whose weight is stored around zero; three mixers (attention over a cached latent inside a window with a gate per
head; grouped-query attention whose values are its unrotated keys, with a partial rotation, scaled frequencies and a window that also
keeps the first tokens; a selective state-space recurrence behind a short convolution); feed-forwards that are dense and gated (relu) or
routed over gated experts (silu) by a sigmoid router with a shared expert; a final norm and a head.

``forward(config, tensors, tokens, stored=None, gaps=None)`` returns ``(logits [T, vocab], the stream after every layer)``.  ``stored``: a
function applied to every tensor that separate kernels hand to each other in the engine (the yardstick of the bfloat16 engine's
rounding).  ``gaps``: a list that receives every router's margin of choice, token by token.
"""
from __future__ import annotations

import math

import torch


def _same(x):
    return x


def offset_rms_norm(x, w, eps, offset=1.0):
    """``x / sqrt(mean(x^2) + eps) * (offset + w)`` over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (offset + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------------------------------- masks

def window_sees(i: int, j: int, size: int | None, keep_first: int = 0) -> bool:
    """Whether the query at position ``i`` reads the key at ``j``: never a later one; inside a window the last ``size`` positions, itself
    included, and the first ``keep_first`` positions of the sequence whatever their distance."""
    if j > i:
        return False
    if size is None:
        return True
    return i - j < size or j < keep_first


def mask_matrix(T: int, size: int | None, keep_first: int = 0, dtype=torch.float64):
    m = torch.full((T, T), float("-inf"), dtype=dtype)
    for i in range(T):
        for j in range(T):
            if window_sees(i, j, size, keep_first):
                m[i, j] = 0.0
    return m


# ------------------------------------------------------------------------------------------------- rotation

def scaled_frequencies(dims: int, base: float, scaling: dict | None):
    """``f_i = base ** (-2i / dims)``, ``i < dims / 2``; with ``scaling`` (``factor``, ``low``, ``high``, ``original``): a frequency whose
    wavelength ``2 pi / f`` is shorter than ``original / high`` stays, one whose wavelength is longer than ``original / low`` is divided by
    ``factor``, and between the two the divided and the plain frequency are blended by ``s = (original / wavelength - low) / (high - low)``."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate_halves(x, positions, freqs):
    """``x [T, heads, dim]``: of the first ``2 len(freqs)`` numbers of every head, number ``i`` and number ``i + len(freqs)`` turn by
    ``position * freqs[i]``; the rest passes."""
    half = len(freqs)
    if half == 0:
        return x
    f = torch.tensor(freqs, dtype=x.dtype)
    a = positions.to(x.dtype)[:, None, None] * f[None, None, :]
    u, v, rest = x[..., :half], x[..., half: 2 * half], x[..., 2 * half:]
    return torch.cat((u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), rest), dim=-1)


# ------------------------------------------------------------------------------------------------- mixers

def softmax_attention(q, k, v, scale, mask):
    """``q [T, dim]``, ``k [T, dim]``, ``v [T, vdim]`` of one head; ``mask [T, T]`` of zeros and minus infinity."""
    s = (q @ k.T) * scale + mask
    return torch.softmax(s, dim=-1) @ v


def latent_attention_mixer(h, w, m, eps, stored=_same):
    """Attention over one latent per token: ``q = W_q h``; ``c = rms(W_dkv h) * w_norm`` (a plain weight); per head ``k = W_uk c`` and ``v =
    W_uv c``; a window without kept tokens; head ``n``'s output times ``sigmoid(W_g h)[n]``; ``W_o``."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = stored(h @ w["q"].T).view(T, H, d)
    c = h @ w["dkv"].T
    c = stored(c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * w["dkv.norm"])
    k = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, dv)
    gate = torch.sigmoid(stored(h @ w["g"].T))
    mask = mask_matrix(T, (m.get("mask") or {}).get("size"), 0, h.dtype)
    heads = [softmax_attention(q[:, n], k[:, n], v[:, n], m["scale"], mask) * gate[:, n: n + 1] for n in range(H)]
    return stored(torch.cat(heads, dim=-1)) @ w["o"].T


def attention_mixer(h, w, m, stored=_same):
    """Grouped-query attention whose values are the keys as projected: ``q = W_q h + b_q``, ``k = W_k h + b_k``, ``v = k``; q and k (not v)
    turn over the first ``rot.dims`` numbers of a head; a window that keeps the first tokens; ``W_o (.) + b_o``."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = stored(h @ w["q"].T + w["q.b"]).view(T, H, d)
    k = stored(h @ w["k"].T + w["k.b"]).view(T, G, d)
    v = k
    rot = m.get("rot")
    if rot:
        freqs = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        pos = torch.arange(T)
        q, k = stored(rotate_halves(q, pos, freqs)), stored(rotate_halves(k, pos, freqs))
    mk = m.get("mask") or {}
    mask = mask_matrix(T, mk.get("size"), mk.get("keep_first", 0), h.dtype)
    heads = [softmax_attention(q[:, n], k[:, n // (H // G)], v[:, n // (H // G)], m["scale"], mask) for n in range(H)]
    return stored(torch.cat(heads, dim=-1)) @ w["o"].T + w["o.b"]


def causal_convolution(x, taps, bias):
    """``x [T, channels]``, ``taps [channels, n]`` (the last column is the current token's), zeros before the start."""
    T, n = x.shape[0], taps.shape[1]
    padded = torch.cat((torch.zeros((n - 1, x.shape[1]), dtype=x.dtype), x), dim=0)
    out = torch.zeros_like(x)
    for j in range(n):
        out = out + padded[j: j + T] * taps[:, j]
    return out + bias


def selective_recurrence(x, B, C, dt, a_log, D, heads, groups):
    """``x [T, heads, vdim]``, ``B`` and ``C [T, groups, N]``, ``dt [T, heads]`` (after softplus): per head ``S <- exp(-exp(a_log) dt) S + dt B
    x^T`` (``S [N, vdim]``, zero at the start) and ``y = S^T C + D x``."""
    T, _, P = x.shape
    N = B.shape[-1]
    y = torch.zeros_like(x)
    for n in range(heads):
        g = n // (heads // groups)
        S = torch.zeros((N, P), dtype=x.dtype)
        for t in range(T):
            S = torch.exp(-torch.exp(a_log[n]) * dt[t, n]) * S + dt[t, n] * torch.outer(B[t, g], x[t, n])
            y[t, n] = S.T @ C[t, g] + D[n] * x[t, n]
    return y


def mamba2_mixer(h, w, m, eps, stored=_same):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = stored(h @ w["in"].T)
    z, xBC, dt = proj[:, :inner], proj[:, inner: 2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xBC = silu(causal_convolution(xBC, w["conv"], w["conv.b"]))
    x, B, C = xBC[:, :inner].reshape(T, H, P), xBC[:, inner: inner + G * N].reshape(T, G, N), xBC[:, inner + G * N:].reshape(T, G, N)
    dt = torch.nn.functional.softplus(dt + w["dt_bias"], threshold=1e9)
    y = selective_recurrence(x, B, C, dt, w["A_log"], w["D"], H, G).reshape(T, inner)
    y = y * silu(z)
    parts = m["norm_groups"]
    y = y.view(T, parts, inner // parts)
    y = (y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)).reshape(T, inner) * w["norm"]
    return stored(y) @ w["o"].T


# ------------------------------------------------------------------------------------------------- feed-forwards

def gated_ff(h, w, prefix, act, stored=_same):
    return stored(act(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def sigmoid_router(h, w, router: dict, gaps=None):
    """Scores ``s = sigmoid(W_r h)``; the ``top`` largest of ``s + correction`` are chosen (the lower index wins a tie); their weights are
    ``s / (sum of the chosen s + 1e-20) * scale``.  Returns ``(chosen [T, top], weights [T, top])``.  ``gaps``: a list that receives, per
    token, by how much the last chosen expert's choice score leads the best one left out."""
    s = torch.sigmoid(h @ w["router"].T)
    choice = s + w["correction"]
    ranked = torch.sort(choice, dim=-1, descending=True, stable=True)
    chosen = ranked.indices[:, : router["top"]]
    if gaps is not None and router["top"] < choice.shape[1]:
        gaps.extend((ranked.values[:, router["top"] - 1] - ranked.values[:, router["top"]]).tolist())
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20) * router["scale"]


def routed_ff(h, w, mlp, stored=_same, gaps=None):
    chosen, weights = sigmoid_router(h, w, {"scale": 1.0, **mlp["router"]}, gaps)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(chosen.shape[1]):
            e = int(chosen[t, j])
            out[t] = out[t] + weights[t, j] * stored(gated_ff(h[t: t + 1], w, f"e{e}.", silu, stored))[0]
    if mlp.get("shared"):
        out = out + stored(gated_ff(h, w, "shared.", silu, stored))
    return out


# ------------------------------------------------------------------------------------------------- the model

def under(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(config, tensors, tokens, stored=_same, gaps=None):
    eps, m = float(config["norm"]["eps"]), float(config.get("residual_mult", 1.0))
    x = offset_rms_norm(tensors["embed"][torch.as_tensor(tokens)], tensors["embed.norm"], eps)
    after = []
    for i, layer in enumerate(config["layers"]):
        w = under(tensors, f"l{i}.")
        h = stored(offset_rms_norm(x, w["norm1"], eps))
        mix = under(w, "mix.")
        if layer["type"] == "latent_attention":
            y = latent_attention_mixer(h, mix, layer["mixer"], eps, stored)
        elif layer["type"] == "attention":
            y = attention_mixer(h, mix, layer["mixer"], stored)
        elif layer["type"] == "mamba2":
            y = mamba2_mixer(h, mix, layer["mixer"], eps, stored)
        else:
            raise ValueError(layer["type"])
        x = x + m * offset_rms_norm(stored(y), w["norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = stored(offset_rms_norm(x, w["norm2"], eps))
            ff = under(w, "mlp.")
            y = gated_ff(h, ff, "", torch.relu, stored) if mlp["kind"] == "dense" else routed_ff(h, ff, mlp, stored, gaps)
            x = x + m * offset_rms_norm(stored(y), w["norm2b"], eps)
        after.append(x.clone())
    h = stored(offset_rms_norm(x, tensors["final.norm"], eps))
    return h @ tensors["head"].T, torch.stack(after)
