"""Grouped-query attention with soft-capped scores and a mask in chunks, over a paged cache of keys and values of two sizes.

``q = W_q h`` (``heads x dim``), ``k = W_k h`` (``kv_heads x dim``), ``v = W_v h`` (``kv_heads x vdim``), no biases and no position
encoding; query head ``i`` reads key/value head ``i // (heads / kv_heads)``; ``score = q . k * scale``, then ``score <- cap *
tanh(score / cap)``; query ``p`` reads the keys ``j <= p`` with ``j // chunk == p // chunk`` (chunks are counted from position 0 of
the sequence, whatever portion a step brings) and, with a window, ``j > p - window``; an ordinary softmax in 32-bit; ``W_o`` on the
heads' values side by side.  The cache has two planes per page, keys ``[kv_heads, page, dim]`` and values, transposed, ``[kv_heads, vdim,
page]``; pages that lie wholly before the chunk of a request's next position go back to the pool.  The bfloat16 engine runs on the matrix
cores in tiles of up to 16 tokens of a request, a wave to a tile and head (where the kernel is built for the sizes: a decoded token is
a tile of one, and the fetches of its keys are what its time is made of either way); the 32-bit engine and other sizes take the kernel
that walks the keys of one token and head.

Four more mechanisms, each off unless its specification names it.  A position encoding over the first dimensions of every head (pairs or
halves), and before it a root-mean-square norm of queries and keys per head with one weight vector each: one kernel does both in place,
in 32-bit, before the keys go to their pages.  A sink: one learned number per head whose exponential joins the softmax's denominator.
Pooled blocks beside a window: every block of ``pool`` positions that lies wholly before a query's window is read as one key and one value,
the means of the block's cached keys and values.  The pooled rows are a second group of pages at one row per ``pool`` positions, written by
the step that brings a block's last token (so the tokens' own pages are kept for ``max(window, pool)`` positions and no longer).

Three more.  Kept first tokens: beside a window a query also reads the first ``keep_first`` positions of its sequence, at their own
positions; the pages that hold them are not given back with the window's.  Values that are the keys: no value projection; the values are
the keys as projected (bias added) before norm and rotation, copied by the kernel that turns the keys.  Biases on the query and key
projections and on the output projection.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import KEEP_COMPUTE, KEEP_FLOAT32, KEEP_STORED, MIXERS, POSITION_ENCODINGS, PagedNeed, StagedMixer, WeightSpec


@MIXERS.register("capped_attention")
class CappedAttention(StagedMixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.heads % spec.kv_heads:
            raise ConfigError(f"attention: {spec.heads} heads are not a multiple of {spec.kv_heads} key/value heads")
        if spec.dim > ops.LOCAL_ATTENTION_MAX_DIM or spec.vdim > ops.LOCAL_ATTENTION_MAX_DIM:
            raise ConfigError(f"attention kernels with two head sizes are built for up to {ops.LOCAL_ATTENTION_MAX_DIM} dimensions, not {spec.dim} / {spec.vdim}")
        for name in ("chunk", "window"):
            if getattr(spec, name) is not None and getattr(spec, name) < 1:
                raise ConfigError(f"attention: a {name} must hold at least one key, got {getattr(spec, name)}")
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = spec.hidden, spec.heads, spec.kv_heads, spec.dim, spec.vdim
        self.q_width, self.k_width, self.v_width = spec.heads * spec.dim, spec.kv_heads * spec.dim, spec.kv_heads * spec.vdim
        self.shared_kv = bool(spec.values_are_keys)
        if self.shared_kv and spec.vdim != spec.dim:
            raise ConfigError(f"attention: values that are the keys have the keys' size, not {spec.vdim} against {spec.dim}")
        self.in_width = self.q_width + self.k_width + (0 if self.shared_kv else self.v_width)
        self.mix_width = spec.heads * spec.vdim
        self.scale = float(spec.scale)
        self.softcap = float(spec.softcap) if spec.softcap else 0.0
        self.chunk, self.window = spec.chunk or 0, spec.window or 0
        self.tile_tokens = ops.LOCAL_ATTENTION_TILE_TOKENS       # the step context makes tiles of this many tokens ahead of the layers
        self.pool = int(spec.pool or 0)
        self.keep_first = int(spec.keep_first or 0) if self.window else 0      # (without a window every token is read anyway)
        if self.keep_first < 0 or (self.keep_first and (self.chunk or self.pool)):
            raise ConfigError("attention: kept first tokens stand beside a plain window (no chunks, no pooled blocks)")
        if self.pool and not self.window:
            raise ConfigError("attention: pooled blocks stand beside a window; without one every token is read itself")
        if self.pool and self.chunk:
            raise ConfigError("attention: pooled blocks beside a mask in chunks are not built")
        self.position = POSITION_ENCODINGS.build(spec.position, dtype, device) if spec.position is not None else None
        if self.position is not None and (not hasattr(self.position, "halves") or self.position.dims > spec.dim):
            raise ConfigError(f"attention: the encoding {spec.position.kind!r} is not one over the first dimensions of a head of {spec.dim}")
        self.qk_norm = bool(spec.qk_norm)
        self.q_norm = self.k_norm = self.sink = None

    def parts(self):
        yield self
        if self.position is not None:
            yield from self.position.parts()

    def paged_need(self):
        planes = ((self.kv_heads, self.dim), (self.kv_heads, self.vdim))
        if not self.pool:
            return PagedNeed(num_heads=self.kv_heads, head_dim=self.dim, window=self.spec.window, chunk=self.spec.chunk, planes=planes,
                             keep_first=self.keep_first)
        # a block's tokens must all be held when its last one arrives: the tokens' pages are kept for the longer of window and block
        return (PagedNeed(num_heads=self.kv_heads, head_dim=self.dim, window=max(self.window, self.pool), planes=planes),
                PagedNeed(num_heads=self.kv_heads, head_dim=self.dim, planes=planes, stride=self.pool))

    def kernel_libraries(self):
        return ["local_attention"]

    def weight_specs(self):
        specs = {"q": WeightSpec((self.q_width, self.hidden)), "k": WeightSpec((self.k_width, self.hidden))}
        if not self.shared_kv:
            specs["v"] = WeightSpec((self.v_width, self.hidden))
        specs["o"] = WeightSpec((self.hidden, self.mix_width))
        if self.spec.qk_bias:
            specs["q.b"] = WeightSpec((self.q_width,), keep=KEEP_STORED)
            specs["k.b"] = WeightSpec((self.k_width,), keep=KEEP_STORED)
        if self.spec.o_bias:
            specs["o.b"] = WeightSpec((self.hidden,), keep=KEEP_STORED)
        if self.qk_norm:
            specs["q.norm"] = WeightSpec((self.dim,), keep=KEEP_FLOAT32, init="one_plus_normal")
            specs["k.norm"] = WeightSpec((self.dim,), keep=KEEP_FLOAT32, init="one_plus_normal")
        if self.spec.sink:
            specs["sink"] = WeightSpec((self.heads,), keep=KEEP_FLOAT32)
        return specs

    def load_weights(self, tensors):
        self.w_in = self._place(torch.cat([tensors[n] for n in ("qk" if self.shared_kv else "qkv")], dim=0), KEEP_COMPUTE)
        self.w_o = self._place(tensors["o"], KEEP_COMPUTE)
        if self.spec.qk_bias:
            rest = [] if self.shared_kv else [torch.zeros(self.v_width, dtype=tensors["q.b"].dtype)]
            self.b_in = self._place(torch.cat([tensors["q.b"], tensors["k.b"]] + rest), KEEP_STORED)
        if self.spec.o_bias:
            self.b_o = self._place(tensors["o.b"], KEEP_STORED)
        if self.qk_norm:
            self.q_norm = self._place(tensors["q.norm"], KEEP_FLOAT32)
            self.k_norm = self._place(tensors["k.norm"], KEEP_FLOAT32)
        if self.spec.sink:
            self.sink = self._place(tensors["sink"], KEEP_FLOAT32)

    def mix(self, proj, h, ctx, cache, out, gain=1.0):
        # the cache hands out planes of [pages, kv_heads, page, width]; this mixer keeps the values of a page transposed
        k_plane, v_plane = cache.planes
        v_plane = v_plane.view(v_plane.shape[0], self.kv_heads, self.vdim, cache.page_size)
        table = ctx.block_tables[cache.group]
        q = proj[:, : self.q_width]
        if self.shared_kv:          # the keys as projected: the kernel that turns them copies them here first
            values = torch.empty((proj.shape[0], self.k_width), dtype=self.dtype, device=proj.device)
        else:
            values = proj[:, self.q_width + self.k_width:]
        if self.qk_norm or self.position is not None or self.shared_kv:
            # queries and keys lie side by side in the projection's rows: normed per head and turned in place, in 32-bit, with one rounding
            ops.head_norm_rotate(proj[:, : self.q_width + self.k_width], self.heads, self.kv_heads, self.dim, self.q_norm, self.k_norm,
                                 float(self.spec.qk_norm_eps), ctx.positions,
                                 self.position.inv_freq if self.position is not None else None,
                                 self.position.dims if self.position is not None else 0,
                                 bool(self.position.halves) if self.position is not None else False,
                                 raw_b=values if self.shared_kv else None)
        pooled = None
        if self.pool:
            pool_group, (pk_plane, pv_plane) = cache.more[0]
            pv_plane = pv_plane.view(pv_plane.shape[0], self.kv_heads, self.vdim, cache.page_size)
            pooled = (pk_plane, pv_plane, ctx.block_tables[pool_group], self.pool)
        if cache.writable:
            ops.kv_cache_write(proj[:, self.q_width: self.q_width + self.k_width], values,
                               ctx.token_req, ctx.positions, table, k_plane, v_plane, cache.page_size)
            if pooled is not None:      # the blocks whose last token this step brings
                ops.pool_blocks(k_plane, v_plane, table, pk_plane, pv_plane, pooled[2], ctx.req_indptr, ctx.ctx_lens,
                                ctx.max_new_tokens // self.pool + 1, cache.page_size, self.pool)
        tiles = None
        if h.is_cuda and ops.local_attention_mfma_fits(self.dtype, self.dim, self.vdim, cache.page_size) \
                and proj.stride(0) % 8 == 0 and proj.data_ptr() % 16 == 0:
            tiles = (ctx.req_indptr, ctx.ctx_lens, *ctx.tiles(ops.LOCAL_ATTENTION_TILE_TOKENS))
        ops.local_attention(q, out, k_plane, v_plane, table, ctx.token_req, ctx.positions, self.heads, self.kv_heads, self.dim, self.vdim,
                            cache.page_size, self.scale, self.softcap, self.chunk, self.window, gain, tiles=tiles, sink=self.sink, pooled=pooled,
                            keep_first=self.keep_first)
