"""CPU stand-ins for the HIP entry points, for tests only.

The product has no CPU path.  These functions have the signatures and the semantics of
``torchlet_amd.kernels.ops`` (same operands, same in-place outputs, same block-table and
tile conventions) so that the engine's host logic -- cache manager, step function,
scheduler, trace replay -- can be exercised on a machine without a GPU by patching them
over the real module (see the ``cpu_ops`` fixture).  GPU tests never use this file.
"""
import math

import torch

ATTENTION_ROWS = 16


def attention_tile_tokens(num_heads, num_kv_heads):
    group = num_heads // num_kv_heads
    return max(1, ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def load(names):
    pass


def embedding(token_ids, table, out, scale=1.0, positions=None, pos_table=None):
    x = table.float()[token_ids.long()] * scale
    if pos_table is not None:
        x = x + pos_table.float()[positions.long()]
    out.copy_(x if out.dim() == 2 else x[None].expand_as(out))


MAX_STREAMS = 8


def streams_norm(x, pending, fold, read, kind, weight, bias, eps, out, rows=None, gain=1.0):
    S = x.shape[0]
    new = x
    if pending is not None:
        p = pending.sum(0) if pending.dim() == 3 else pending.float()
        if fold is None:
            new = x + p[None]
        else:
            mix, gate = fold
            new = torch.einsum("st,snw->tnw", mix, x) + gate[:, None, None] * p[None]
    if rows is None:
        x.copy_(new)
    else:
        new = new[:, rows.long()]
    u = new.sum(0) if read is None else torch.einsum("s,snw->nw", read, new)
    if kind == "layernorm":
        mu = u.mean(-1, keepdim=True)
        y = (u - mu) / torch.sqrt((u - mu).pow(2).mean(-1, keepdim=True) + eps) * weight.float() * gain + bias.float() * gain
    else:
        y = u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * gain * weight.float()
    out.copy_(y.to(out.dtype))


def add_rmsnorm(residual, pending, weight, eps, out, rows=None, gain=1.0):
    if pending is not None and pending.dim() == 3:
        pending = pending.sum(0)
    if rows is None:
        if pending is not None:
            residual += pending.float()
        r = residual
    else:
        idx = rows.long()
        r = residual[idx] + (pending[idx].float() if pending is not None else 0)
    y = r * (torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps) * gain) * weight.float()
    out.copy_(y.to(out.dtype))


def linear(x, weight, bias, out, general=False):
    y = x.float() @ weight.float().T
    if bias is not None:
        y = y + bias.float()
    out.copy_(y.to(out.dtype))


def linear_rope_cache_write(*args, **kwargs):
    return False          # not fused here: the caller runs the product and the rotation one after the other


def rope_cache_write(qkv, q_heads, kv_heads, head_dim, rot_heads, positions, inv_freq,
                     token_req=None, block_table=None, k_plane=None, v_plane=None, page_size=0, pairs=False, parts=None, bias=None):
    T = qkv.shape[0]
    if parts is not None:
        total = parts.sum(0) + (bias.float() if bias is not None else 0.0)
        qkv[:, : total.shape[1]] = total.to(qkv.dtype)
    x = qkv[:, : (q_heads + kv_heads) * head_dim].float().view(T, q_heads + kv_heads, head_dim)
    if inv_freq is not None:
        ang = positions.float()[:, None] * inv_freq[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        half = head_dim // 2
        if pairs:
            x1, x2 = x[:, :rot_heads, 0::2], x[:, :rot_heads, 1::2]
            turned = torch.stack((x1 * c - x2 * s, x2 * c + x1 * s), -1).reshape(T, rot_heads, head_dim)
        else:
            x1, x2 = x[:, :rot_heads, :half], x[:, :rot_heads, half:]
            turned = torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), -1)
        x = torch.cat((turned, x[:, rot_heads:]), 1)
        qkv[:, : (q_heads + kv_heads) * head_dim] = x.reshape(T, -1).to(qkv.dtype)
    if k_plane is not None:
        k = qkv[:, q_heads * head_dim: (q_heads + kv_heads) * head_dim].view(T, kv_heads, head_dim)
        v = qkv[:, (q_heads + kv_heads) * head_dim: (q_heads + 2 * kv_heads) * head_dim].view(T, kv_heads, head_dim)
        for t in range(T):
            p = int(positions[t])
            page = int(block_table[int(token_req[t]), p // page_size])
            k_plane[page, :, p % page_size] = k[t]
            v_plane[page, :, :, p % page_size] = v[t]


def paged_attention(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
                    tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale, splits=1, general=False, merge_tokens=None, waves=4):
    _attend(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale)


def _attend(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale):
    group = num_heads // num_kv_heads
    for tile in range(num_tiles):
        if tile_req is None:        # every request brings one token: tile i is the token of request i
            r, t0, first, n_new = tile, 0, tile, 1
        else:
            r = int(tile_req[tile]); t0 = int(tile_tok0[tile])
            first = int(req_indptr[r]); n_new = int(req_indptr[r + 1]) - first
        ctx = int(ctx_lens[r])
        for i in range(t0, min(t0 + tile_tokens, n_new)):
            pos = ctx + i
            lo = max(0, pos - window + 1) if window else 0
            keys = torch.arange(lo, pos + 1)
            pages = block_table[r, keys // page_size].long()
            k = k_plane[pages, :, keys % page_size].float()       # [n, kvh, hd]
            v = v_plane[pages, :, :, keys % page_size].float()
            qi = q[first + i].float().view(num_heads, head_dim)
            kk = k.repeat_interleave(group, dim=1)
            vv = v.repeat_interleave(group, dim=1)
            s = torch.einsum("hd,nhd->hn", qi, kk) * scale
            o = torch.einsum("hn,nhd->hd", torch.softmax(s, -1), vv)
            out[first + i] = o.reshape(-1).to(out.dtype)


def interleave_gate_up(gate, up):
    I, K = gate.shape
    blocks = -(-I // 32)
    g = torch.zeros((blocks * 32, K), dtype=gate.dtype)
    u = torch.zeros_like(g)
    g[:I] = gate
    u[:I] = up
    return torch.stack((g.view(blocks, 32, K), u.view(blocks, 32, K)), dim=1).reshape(blocks * 64, K).contiguous()


GATE_ACTIVATIONS = {"silu": 0, "relu": 1}


def _gate(g, activation):
    return torch.relu(g) if activation == "relu" else g / (1 + torch.exp(-g))


def linear_swiglu(x, gate_up, out, activation="silu"):
    I, K = out.shape[1], x.shape[1]
    w = gate_up.float().view(-1, 2, 32, K)
    g = x.float() @ w[:, 0].reshape(-1, K)[:I].T
    u = x.float() @ w[:, 1].reshape(-1, K)[:I].T
    out.copy_((_gate(g, activation) * u).to(out.dtype))


PREFILL_ATTENTION_ROWS = 64
PREFILL_ATTENTION_MAX_HEAD_DIM = 128


def prefill_attention_tile_tokens(num_heads, num_kv_heads):
    group = num_heads // num_kv_heads
    return max(1, PREFILL_ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def paged_attention_prefill(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
                            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale):
    _attend(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale)


def linear_partials_pay(M, N, K):
    return False


def linear_partials(x, weight):
    K = x.shape[1]
    half = (K // 2 // 8) * 8 or K
    a = x[:, :half].float() @ weight[:, :half].float().T
    b = x[:, half:].float() @ weight[:, half:].float().T
    return torch.stack((a, b))


def swiglu(gate_up, out, activation="silu"):
    I = gate_up.shape[1] // 2
    g, u = gate_up[:, :I].float(), gate_up[:, I:].float()
    out.copy_((_gate(g, activation) * u).to(out.dtype))


def _mix32(x):
    x = x & 0xFFFFFFFF
    x ^= x >> 16; x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15; x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def sample(logits, temperature, keys, out):
    for row in range(logits.shape[0]):
        t = float(temperature[row]) if temperature is not None else 0.0
        if t <= 0:
            out[row] = int(logits[row].argmax())
            continue
        key = int(keys[row]) & 0xFFFFFFFF
        best, besti = -math.inf, 0
        for i in range(logits.shape[1]):
            r = _mix32(_mix32(key ^ i) + 0x9E3779B9)
            u = ((r >> 8) + 0.5) / 16777216.0
            v = float(logits[row, i]) / t - math.log(-math.log(u))
            if v > best:
                best, besti = v, i
        out[row] = besti


# ---------------------------------------------------------------- norm after the sum, recurrence, latent attention, experts

def scaled_add_rmsnorm(residual, pending, alpha, weight, eps, out):
    r = alpha * residual
    if pending is not None:
        r = r + (pending.sum(0) if pending.dim() == 3 else pending.float())
    y = r / torch.sqrt(r.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    residual.copy_(y)
    if out is not None:
        out.copy_(y.to(out.dtype))


def mlstm_scan(qkv, k_off, v_off, gates, state, slots, req_indptr, out, heads, dim, vdim, cap, qscale, denom_eps):
    squash = (lambda z: cap * torch.tanh(z / cap)) if cap else (lambda z: z)
    for r in range(req_indptr.numel() - 1):
        st = state[int(slots[r])]
        S = st[:, : dim * vdim].reshape(heads, dim, vdim).clone()
        n = st[:, dim * vdim: dim * vdim + dim].clone()
        m = st[:, dim * vdim + dim].clone()
        for t in range(int(req_indptr[r]), int(req_indptr[r + 1])):
            q = qkv[t, : heads * dim].float().view(heads, dim) * qscale
            k = qkv[t, k_off: k_off + heads * dim].float().view(heads, dim)
            v = qkv[t, v_off: v_off + heads * vdim].float().view(heads, vdim)
            i = squash(gates[t, :heads])
            f = torch.nn.functional.logsigmoid(squash(gates[t, heads:]))
            m_new = torch.maximum(f + m, i)
            keep, take = torch.exp(f + m - m_new), torch.exp(i - m_new)
            S = keep[:, None, None] * S + take[:, None, None] * k[:, :, None] * v[:, None, :]
            n = keep[:, None] * n + take[:, None] * k
            m = m_new
            den = torch.maximum((n * q).sum(-1).abs(), torch.exp(-m)) + denom_eps
            out[t] = (torch.einsum("hdv,hd->hv", S, q) / den[:, None]).reshape(-1)
        st[:, : dim * vdim] = S.reshape(heads, -1)
        st[:, dim * vdim: dim * vdim + dim] = n
        st[:, dim * vdim + dim] = m


def gated_head_norm(o, gate_values, weight, eps, out, heads, vdim, gate="sigmoid", gain=1.0, gate_first=False):
    T = o.shape[0]
    g = gate_values.float()
    g = torch.sigmoid(g) if gate == "sigmoid" else g * torch.sigmoid(g)
    x = o.view(T, heads, vdim)
    if gate_first:
        x = x * g.reshape(T, heads, vdim)
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.float().view(-1, vdim)
    out.copy_((y.reshape(T, -1) * (1.0 if gate_first else g) * gain).to(out.dtype))


def selective_prepare(proj, x_off, conv_w, conv_b, gates, a_log, dt_bias, state, tail_off, slots, req_indptr, token_req, qkv, heads, inner, gn, taps):
    C = inner + 2 * gn
    for r in range(req_indptr.numel() - 1):
        lo, hi = int(req_indptr[r]), int(req_indptr[r + 1])
        if hi <= lo:
            continue
        st = state[int(slots[r])]
        tail = st[tail_off: tail_off + (taps - 1) * C].view(taps - 1, C)
        x = torch.cat((tail, proj[lo:hi, x_off: x_off + C].float()), 0)
        y = sum(x[j: j + hi - lo] * conv_w[:, j] for j in range(taps)) + conv_b
        y = y * torch.sigmoid(y)
        qkv[lo:hi] = torch.cat((y[:, inner + gn:], y[:, inner: inner + gn], y[:, :inner]), dim=1)          # C, B, x
        if taps > 1:
            tail.copy_(x[-(taps - 1):])
    dt = torch.nn.functional.softplus(proj[:, x_off + C: x_off + C + heads].float() + dt_bias)
    gates[:, :heads] = dt
    gates[:, heads:] = torch.exp(-torch.exp(a_log) * dt)


def selective_scan(qkv, gates, skip, state, slots, req_indptr, out, heads, groups, dim, vdim, max_new_tokens=None):
    of = torch.arange(heads) // (heads // groups)
    for r in range(req_indptr.numel() - 1):
        st = state[int(slots[r])]
        S = st[: heads * dim * vdim].view(heads, vdim, dim).transpose(1, 2).clone()
        for t in range(int(req_indptr[r]), int(req_indptr[r + 1])):
            q = qkv[t, : groups * dim].view(groups, dim)[of]
            k = qkv[t, groups * dim: 2 * groups * dim].view(groups, dim)[of]
            v = qkv[t, 2 * groups * dim:].view(heads, vdim)
            S = S * gates[t, heads:, None, None] + k[:, :, None] * (gates[t, :heads, None] * v)[:, None, :]
            out[t] = (torch.einsum("hde,hd->he", S, q) + skip[:, None] * v).reshape(-1)
        st[: heads * dim * vdim] = S.transpose(1, 2).reshape(-1)


def embedding_norm(token_ids, table, out, scale, weight, eps):
    x = table.float()[token_ids.long()] * scale
    out.copy_(x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight)


DELTA_MAX_TAPS = 8
DELTA_MAX_DIM = 256
LOCAL_ATTENTION_MAX_DIM = 256


def delta_prepare(proj, conv_w, gates, a_log, dt_bias, state, tail_off, slots, req_indptr, token_req, qkv, heads, kv_heads, dim, vdim,
                  taps, qscale, unit_eps):
    C = 2 * kv_heads * dim + heads * vdim
    for r in range(req_indptr.numel() - 1):
        lo, hi = int(req_indptr[r]), int(req_indptr[r + 1])
        if hi <= lo:
            continue
        st = state[int(slots[r])]
        tail = st[tail_off: tail_off + (taps - 1) * C].view(taps - 1, C)
        x = torch.cat((tail, proj[lo:hi, :C].float()), 0)                    # the inputs from taps - 1 tokens before the step on
        y = sum(x[j: j + hi - lo] * conv_w[:, j] for j in range(taps))
        y = y * torch.sigmoid(y)
        qk = y[:, : 2 * kv_heads * dim].view(hi - lo, 2 * kv_heads, dim)
        qk = qk / torch.sqrt(qk.pow(2).sum(-1, keepdim=True) + unit_eps)
        qk[:, :kv_heads] *= qscale
        qkv[lo:hi, : 2 * kv_heads * dim] = qk.reshape(hi - lo, -1)
        qkv[lo:hi, 2 * kv_heads * dim:] = y[:, 2 * kv_heads * dim:]
        if taps > 1:
            tail.copy_(x[-(taps - 1):])
    beta = torch.sigmoid(gates[:, :heads])
    decay = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(gates[:, heads:] + dt_bias))
    gates[:, :heads] = beta
    gates[:, heads:] = decay


def delta_scan(qkv, gates, state, slots, req_indptr, out, heads, kv_heads, dim, vdim, max_new_tokens=None):
    of = torch.arange(heads) // (heads // kv_heads)
    for r in range(req_indptr.numel() - 1):
        st = state[int(slots[r])]
        S = st[: heads * dim * vdim].view(heads, vdim, dim).transpose(1, 2).clone()          # a head's state lies column by column
        for t in range(int(req_indptr[r]), int(req_indptr[r + 1])):
            q = qkv[t, : kv_heads * dim].view(kv_heads, dim)[of]
            k = qkv[t, kv_heads * dim: 2 * kv_heads * dim].view(kv_heads, dim)[of]
            v = qkv[t, 2 * kv_heads * dim:].view(heads, vdim)
            S = S * gates[t, heads:, None, None]
            u = gates[t, :heads, None] * (v - torch.einsum("hde,hd->he", S, k))
            S = S + k[:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hde,hd->he", S, q).reshape(-1)
        st[: heads * dim * vdim] = S.transpose(1, 2).reshape(-1)


def kv_cache_write(k, v, token_req, positions, block_table, k_plane, v_plane, page_size):
    kv_heads, dim, vdim = k_plane.shape[1], k_plane.shape[3], v_plane.shape[2]
    for t in range(k.shape[0]):
        p = int(positions[t])
        page = int(block_table[int(token_req[t]), p // page_size])
        if page:
            k_plane[page, :, p % page_size] = k[t].view(kv_heads, dim)
            v_plane[page, :, :, p % page_size] = v[t].view(kv_heads, vdim)


LOCAL_ATTENTION_TILE_TOKENS = 16


def local_attention_mfma_fits(dtype, dim, vdim, page_size):
    return False


def local_attention(q, out, k_plane, v_plane, block_table, token_req, positions, heads, kv_heads, dim, vdim, page_size, scale,
                    softcap=0.0, chunk=0, window=0, gain=1.0, tiles=None, sink=None, pooled=None, keep_first=0):
    group = heads // kv_heads
    for t in range(q.shape[0]):
        p, r = int(positions[t]), int(token_req[t])
        lo = 0
        if chunk:
            lo = max(lo, p // chunk * chunk)
        if window:
            lo = max(lo, p - window + 1)
        keys = torch.cat((torch.arange(0, min(keep_first, lo)), torch.arange(lo, p + 1)))
        pages = block_table[r, keys // page_size].long()
        k = k_plane[pages, :, keys % page_size].float().repeat_interleave(group, dim=1)      # [n, heads, dim]
        v = v_plane[pages, :, :, keys % page_size].float().repeat_interleave(group, dim=1)
        if pooled is not None:
            pk_plane, pv_plane, pool_table, pool = pooled
            rows = torch.arange(max(0, p - window + 1) // pool)
            ppages = pool_table[r, rows // page_size].long()
            k = torch.cat((pk_plane[ppages, :, rows % page_size].float().repeat_interleave(group, dim=1), k))
            v = torch.cat((pv_plane[ppages, :, :, rows % page_size].float().repeat_interleave(group, dim=1), v))
        s = torch.einsum("hd,nhd->hn", q[t].float().view(heads, dim), k) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        if sink is not None:
            w = torch.softmax(torch.cat((s, sink.float()[:, None]), -1), -1)[:, :-1]
        else:
            w = torch.softmax(s, -1)
        out[t] = (torch.einsum("hn,nhd->hd", w, v).reshape(-1) * gain).to(out.dtype)


def pool_blocks(k_plane, v_plane, block_table, pk_plane, pv_plane, pool_table, req_indptr, ctx_lens, most_blocks, page_size, pool):
    for r in range(req_indptr.numel() - 1):
        ctx, n = int(ctx_lens[r]), int(req_indptr[r + 1]) - int(req_indptr[r])
        assert (ctx + n) // pool - ctx // pool <= most_blocks
        for b in range(ctx // pool, (ctx + n) // pool):
            ppage = int(pool_table[r, b // page_size])
            if not ppage:
                continue
            keys = torch.arange(b * pool, b * pool + pool)
            pages = block_table[r, keys // page_size].long()
            pk_plane[ppage, :, b % page_size] = k_plane[pages, :, keys % page_size].float().mean(0).to(pk_plane.dtype)
            pv_plane[ppage, :, :, b % page_size] = v_plane[pages, :, :, keys % page_size].float().mean(0).to(pv_plane.dtype)


def head_norm_rotate(x, heads_a, heads_b, dim, norm_a, norm_b, eps, positions, inv_freq, dims, halves, raw_b=None):
    T = x.shape[0]
    if raw_b is not None:
        raw_b.copy_(x[:, heads_a * dim:])
    v = x.float().reshape(T, heads_a + heads_b, dim).clone()
    if norm_a is not None or norm_b is not None:
        w = torch.cat([(norm_a if norm_a is not None else torch.ones(dim)).float().expand(heads_a, dim),
                       (norm_b if norm_b is not None else torch.ones(dim)).float().expand(heads_b, dim)])
        v = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w
    if inv_freq is not None:
        ang = positions.float()[:, None, None] * inv_freq.float()[None, None, :]
        c, sn = ang.cos(), ang.sin()
        if halves:
            a, b = v[..., : dims // 2].clone(), v[..., dims // 2: dims].clone()
            v[..., : dims // 2], v[..., dims // 2: dims] = a * c - b * sn, b * c + a * sn
        else:
            a, b = v[..., 0:dims:2].clone(), v[..., 1:dims:2].clone()
            v[..., 0:dims:2], v[..., 1:dims:2] = a * c - b * sn, b * c + a * sn
    x.copy_(v.reshape(T, -1).to(x.dtype))


def decay_scan(qkv, decay, state, slots, req_indptr, out, heads, dim, vdim, max_new_tokens=None):
    for r in range(req_indptr.numel() - 1):
        st = state[int(slots[r])]
        S = st[: heads * dim * vdim].view(heads, vdim, dim).transpose(1, 2).clone()
        for t in range(int(req_indptr[r]), int(req_indptr[r + 1])):
            q = qkv[t, : heads * dim].view(heads, dim)
            k = qkv[t, heads * dim: 2 * heads * dim].view(heads, dim)
            v = qkv[t, 2 * heads * dim:].view(heads, vdim)
            S = S * decay[:, None, None] + k[:, :, None] * v[:, None, :]
            out[t] = torch.einsum("hde,hd->he", S, q).reshape(-1)
        st[: heads * dim * vdim] = S.transpose(1, 2).reshape(-1)


def silu_float(x, out):
    v = x.float()
    out.copy_(v * torch.sigmoid(v))


def bigram_embedding(token_ids, table, out, scale, bigram, buckets, mul_prev, mul_cur, token_req, req_indptr, positions, slots, last_token):
    rows = []
    for t in range(token_ids.numel()):
        r = int(token_req[t])
        if int(positions[t]) == 0:
            rows.append(buckets)
        else:
            prev = int(token_ids[t - 1]) if t > int(req_indptr[r]) else int(last_token[int(slots[r]), 0])
            rows.append((prev * mul_prev + int(token_ids[t]) * mul_cur) % buckets)
    x = table.float()[token_ids.long()] * scale + bigram.float()[torch.tensor(rows, dtype=torch.long)]
    out.copy_(x if out.dim() == 2 else x[None].expand_as(out))
    for r in range(req_indptr.numel() - 1):
        if int(req_indptr[r + 1]) > int(req_indptr[r]):
            last_token[int(slots[r]), 0] = int(token_ids[int(req_indptr[r + 1]) - 1])


def sandwich_norm(residual, pending, post_weight, post_eps, extra, weight, eps, out, rows=None, gain=1.0):
    y = None
    if pending is not None:
        y = pending.sum(0) if pending.dim() == 3 else pending.float()
        if post_weight is not None:
            y = y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + post_eps) * post_weight.float()
    r = residual if rows is None else residual[rows.long()]
    add = None
    if extra is not None:
        add = extra if rows is None else extra[rows.long()]
    if y is not None:
        y = y if rows is None else y[rows.long()]
        add = y if add is None else add + y
    if add is not None:
        if rows is None:
            residual += add
            r = residual
        else:
            r = r + add
    out.copy_((r / torch.sqrt(r.pow(2).mean(-1, keepdim=True) + eps) * gain * weight.float()).to(out.dtype))


def normed_sum(x, weights, eps, out):
    v = x.float()
    out.copy_((v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * weights[:, None, :]).sum(0).to(out.dtype))


LATENT_ATTENTION_ROWS = 16
LATENT_MAX_RANK = 1024
ACTIVATIONS = {"none": 0, "relu2": 1, "silu": 2, "gelu_tanh": 3, "gelu": 4, "relu2_pairs": 17, "silu_pairs": 18, "gelu_tanh_pairs": 19, "gelu_pairs": 20}


LATENT_MFMA_ROWS = 64
LATENT_MFMA_MAX_BLOCKS = 1536


def latent_tile_tokens(heads, rows=LATENT_ATTENTION_ROWS):
    return max(1, rows // min(heads, LATENT_ATTENTION_ROWS))


def latent_attention_mfma_fits(dtype, heads, rank, rot):
    return False


def _turn(x, positions, inv_freq):
    """x [T, ..., rot]: the first 2 * len(inv_freq) entries turned in neighbouring pairs."""
    d = 2 * inv_freq.numel()
    ang = positions.float()[:, None] * inv_freq[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [d // 2]
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    u, v = x[..., 0:d:2], x[..., 1:d:2]
    y = x.clone()
    y[..., 0:d:2] = u * c - v * s
    y[..., 1:d:2] = v * c + u * s
    return y


def latent_prepare(down, q_rank, rank, rot, rot_dims, wq, wkv, eps, positions, inv_freq, cq, token_req=None, block_table=None,
                   plane=None, page_size=0, kv_off=None):
    kv_off = q_rank if kv_off is None else kv_off
    x = down.float()
    norm = lambda t, w: t / torch.sqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    if q_rank:
        cq.copy_(norm(x[:, :q_rank], wq).to(cq.dtype))
    if plane is None:
        return
    c = norm(x[:, kv_off: kv_off + rank], wkv)
    kr = _turn(x[:, kv_off + rank: kv_off + rank + rot], positions, inv_freq)
    row = torch.cat((c, kr), dim=-1).to(plane.dtype)
    for t in range(down.shape[0]):
        p = int(positions[t])
        page = int(block_table[int(token_req[t]), p // page_size])
        if page:
            plane[page, 0, p % page_size] = row[t]


def rotate_pairs(src, src_head, src_off, dst, dst_head, dst_off, positions, inv_freq, heads, rot):
    T = src.shape[0]
    x = torch.stack([src[:, h * src_head + src_off: h * src_head + src_off + rot] for h in range(heads)], dim=1).float()
    y = _turn(x, positions, inv_freq).to(dst.dtype)
    for h in range(heads):
        dst[:, h * dst_head + dst_off: h * dst_head + dst_off + rot] = y[:, h]


def latent_attention(q, out, plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles, tile_tokens, heads, rank, rot,
                     page_size, scale, sink, splits=1, general=False, max_new_tokens=None, window=0, gate=None):
    D = rank + rot
    for tile in range(num_tiles):
        if tile_req is None:
            r, t0, first, n_new = tile, 0, tile, 1
        else:
            r = int(tile_req[tile]); t0 = int(tile_tok0[tile])
            first = int(req_indptr[r]); n_new = int(req_indptr[r + 1]) - first
        ctx = int(ctx_lens[r])
        for i in range(t0, min(t0 + tile_tokens, n_new)):
            pos = ctx + i
            keys = torch.arange(max(0, pos - window + 1) if window else 0, pos + 1)
            rows = plane[block_table[r, keys // page_size].long(), 0, keys % page_size].float()     # [n, D]
            s = (q[first + i].float().view(heads, D) @ rows.T) * scale
            top = s.max(-1, keepdim=True).values
            if sink is not None:
                top = torch.maximum(top, sink[:, None])
            e = torch.exp(s - top)
            den = e.sum(-1, keepdim=True) + (torch.exp(sink[:, None] - top) if sink is not None else 0.0)
            o = (e / den) @ rows[:, :rank]
            if gate is not None:
                o = o * torch.sigmoid(gate[first + i, :heads].float())[:, None]
            out[first + i] = o.reshape(-1).to(out.dtype)


def heads_linear(x, x_head, weight, out, out_head, general=False):
    G, N, K = weight.shape
    for g in range(G):
        out[:, g * out_head: g * out_head + N] = (x[:, g * x_head: g * x_head + K].float() @ weight[g].float().T).to(out.dtype)


def _act(y, activation):
    if activation.endswith("_pairs"):
        return _act(y[:, 0::2], activation[: -len("_pairs")]) * y[:, 1::2]
    if activation == "relu2":
        return torch.clamp(y, min=0) ** 2
    if activation == "silu":
        return y * torch.sigmoid(y)
    if activation == "gelu_tanh":
        return 0.5 * y * (1 + torch.tanh(math.sqrt(2 / math.pi) * (y + 0.044715 * y ** 3)))
    if activation == "gelu":
        return 0.5 * y * (1 + torch.erf(y / math.sqrt(2.0)))
    return y


def experts_linear(x, slot_token, weight, offsets, out, activation="none", general=False):
    for e in range(weight.shape[0]):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            rows = x[slot_token[lo:hi].long()] if slot_token is not None else x[lo:hi]
            out[lo:hi] = _act(rows.float() @ weight[e].float().T, activation).to(out.dtype)


def route(logits, top, scores="chosen", choice_bias=None, weight_scale=1.0, weight_eps=0.0):
    T, E = logits.shape
    if scores == "all":
        s = torch.softmax(logits, dim=-1)
        best = (s if choice_bias is None else s + choice_bias).topk(top, dim=-1)
        weights = s.gather(1, best.indices)
    elif scores == "sigmoid":
        s = torch.sigmoid(logits)
        best = (s if choice_bias is None else s + choice_bias).topk(top, dim=-1)
        weights = s.gather(1, best.indices)
        weights = weights / (weights.sum(-1, keepdim=True) + weight_eps)
    else:
        best = logits.topk(top, dim=-1)               # ties: not met in tests
        weights = torch.softmax(best.values, dim=-1)
    weights = weights * weight_scale
    chosen = best.indices.reshape(-1)
    order = torch.sort(chosen, stable=True).indices
    slot_token = (order // top).to(torch.int32)
    pair_slot = torch.empty(T * top, dtype=torch.int32)
    pair_slot[order] = torch.arange(T * top, dtype=torch.int32)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.bincount(chosen, minlength=E).cumsum(0)
    return weights, offsets, slot_token, pair_slot


def combine(y, pair_slot, weights, out, identity=None, addend=None):
    T, top = weights.shape
    rows = y[pair_slot.long()].float().view(T, top, -1)
    if identity is not None:
        x, offsets, experts = identity
        own = (pair_slot >= offsets[experts]).view(T, top, 1)
        rows = torch.where(own, x.float()[:, None, :], rows)
    total = (rows * weights[:, :, None]).sum(1)
    if addend is not None:
        total = total + addend.float()
    out.copy_(total.to(out.dtype))


def activation(x, kind):
    x.copy_(_act(x.float(), kind).to(x.dtype))


def compute_units():
    return 256
