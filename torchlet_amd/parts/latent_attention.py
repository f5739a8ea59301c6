"""Attention over a cached latent, with a sink in the softmax.

Queries come through a latent: ``c_q = rmsnorm(W_dq h) * w_dq``, ``q = W_uq c_q``, per head ``dim`` unrotated and
``rot_dim`` rotated numbers.  ``W_dkv h`` gives ``kv_rank`` numbers whose norm ``c = rmsnorm(.) * w_dkv`` is the token's
latent, and ``rot_dim`` more that are one rotated key part shared by all heads.  Per head the unrotated key is ``W_uk c``
and the value ``W_uv c``; the score of query ``t`` and key ``s <= t`` is ``(q_t . k_s + q_t^rot . k_s^rot) * scale``, the
softmax's denominator also holds ``exp(sink_head)`` (a term without key or value), and ``W_o`` follows on the heads' values.

Each of these is a field of the specification: without a query latent (``q_rank`` 0) the queries are ``W_q h``; without a rotated part
(``rot_dim`` 0) a score is ``q . k`` alone; with a window a query reads its last ``window`` keys, itself included, and pages that lie wholly
behind the window go back to the pool; with a gate head ``n``'s output is multiplied by ``sigmoid(W_g h)[n]`` (inside the attention kernel,
where the sums are divided by the softmax's denominator).

Only ``c`` and the rotated key part are cached: one page plane whose rows hold ``kv_rank + rot_dim`` numbers.  The key
up-projection is taken to the query's side, ``q_t . (W_uk c_s) = (W_uk^T q_t) . c_s``, so a head's query becomes a vector
of the cache row's shape and all heads read the same rows: the attention kernel is one dot product per key and its
weighted sum runs over the latents; the value up-projection ``W_uv`` is applied to that sum.  Prompts and decode steps
take the same path, so how a request is cut cannot change what it computes beyond the order of the sums.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import KEEP_COMPUTE, KEEP_FLOAT32, KEEP_STORED, MIXERS, POSITION_ENCODINGS, Mixer, PagedNeed, WeightSpec

_MIN_KEYS_PER_SPLIT = 64        # two steps of the matrix-core kernel


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.kv_rank > ops.LATENT_MAX_RANK:
            raise ConfigError(f"latent attention is built for latents of up to {ops.LATENT_MAX_RANK} numbers, not {spec.kv_rank}")
        self.hidden, self.heads = spec.hidden, spec.heads
        self.dim, self.rot, self.vdim, self.rank, self.q_rank = spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank, spec.q_rank
        self.row = spec.kv_rank + spec.rot_dim               # numbers of a cache row, and of a head's query against it
        self.scale = float(spec.scale)
        self.window = int(spec.window or 0)
        if spec.window is not None and spec.window < 1:
            raise ConfigError(f"latent attention: a window holds at least one key, got {spec.window}")
        if self.rot and spec.position is None:
            raise ConfigError("latent attention: a rotated part needs a position encoding")
        self.position = POSITION_ENCODINGS.build(spec.position, dtype, device) if spec.position is not None else None
        if self.position is not None and not hasattr(self.position, "inv_freq"):
            raise ConfigError("latent attention folds a rotation in pairs into its kernels; its position encoding must offer inv_freq")
        # tiles of 64 rows where the matrix-core kernel is built for these sizes, of 16 for the general kernel
        on_matrix_cores = torch.device(device).type == "cuda" and ops.latent_attention_mfma_fits(dtype, self.heads, self.rank, self.rot)
        self.tile_tokens = ops.latent_tile_tokens(self.heads, ops.LATENT_MFMA_ROWS if on_matrix_cores else ops.LATENT_ATTENTION_ROWS)
        self.general_tile_tokens = ops.latent_tile_tokens(self.heads, ops.LATENT_ATTENTION_ROWS)
        self.compute_units = ops.compute_units()
        self.w_down = self.w_dq_norm = self.w_dkv_norm = self.w_uq = self.w_uk_t = self.w_uv = self.sink = self.w_o = None
        # the columns of the fused first projection: [query latent, or the queries themselves | latent | rotated key part | gate]
        self.q_cols = self.q_rank if self.q_rank else self.heads * self.dim
        self.gate_at = self.q_cols + self.row
        self.down_cols = self.gate_at + (self.heads if spec.gate else 0)

    def paged_need(self):
        return PagedNeed(num_heads=1, head_dim=self.row, planes=((1, self.row),), window=self.spec.window)

    def kernel_libraries(self):
        return ["latent", "experts"]

    def parts(self):
        yield self
        if self.position is not None:
            yield from self.position.parts()

    def weight_specs(self):
        H, n = self.hidden, self.heads
        # (the order of declaration is the order of the random-weights mode's draws)
        specs = {}
        if self.q_rank:
            specs.update({"dq": WeightSpec((self.q_rank, H)), "dq.norm": WeightSpec((self.q_rank,), keep=KEEP_STORED, init="one_plus_normal"),
                          "uq": WeightSpec((n * (self.dim + self.rot), self.q_rank))})
        else:
            specs["q"] = WeightSpec((n * (self.dim + self.rot), H))
        specs.update({
            "dkv": WeightSpec((self.row, H)), "dkv.norm": WeightSpec((self.rank,), keep=KEEP_STORED, init="one_plus_normal"),
            "uk": WeightSpec((n * self.dim, self.rank)), "uv": WeightSpec((n * self.vdim, self.rank)),
            "o": WeightSpec((H, n * self.vdim)),
        })
        if self.spec.sink:
            specs["sink"] = WeightSpec((n,), keep=KEEP_FLOAT32)
        if self.spec.gate:
            specs["g"] = WeightSpec((n, H))
        return specs

    def load_weights(self, tensors):
        n = self.heads
        first = [tensors["dq"] if self.q_rank else tensors["q"], tensors["dkv"]] + ([tensors["g"]] if self.spec.gate else [])
        self.w_down = self._place(torch.cat(first, dim=0), KEEP_COMPUTE)    # one product reads h once
        self.w_dkv_norm = self._place(tensors["dkv.norm"], KEEP_STORED)
        if self.q_rank:
            self.w_dq_norm = self._place(tensors["dq.norm"], KEEP_STORED)
            self.w_uq = self._place(tensors["uq"], KEEP_COMPUTE)
        # per head the key up-projection transposed, [rank, dim]: it multiplies the unrotated query
        self.w_uk_t = self._place(tensors["uk"].view(n, self.dim, self.rank).transpose(1, 2).contiguous(), KEEP_COMPUTE)
        self.w_uv = self._place(tensors["uv"].view(n, self.vdim, self.rank).contiguous(), KEEP_COMPUTE)
        self.sink = self._place(tensors["sink"], KEEP_FLOAT32) if self.spec.sink else None
        self.w_o = self._place(tensors["o"], KEEP_COMPUTE)

    def _splits(self, ctx, tiles: int) -> int:
        """Work-groups that share a tile's keys: enough to give every compute unit one, no part under 64 keys."""
        groups = max(1, tiles * -(-self.heads // ops.LATENT_ATTENTION_ROWS))
        keys = ctx.max_total_len if not self.window else min(ctx.max_total_len, self.window + ctx.max_new_tokens - 1)
        return max(1, min(self.compute_units // groups, keys // _MIN_KEYS_PER_SPLIT, 64))

    def forward(self, h, ctx, cache):
        T, n = h.shape[0], self.heads
        dev = h.device
        inv_freq = self.position.inv_freq if self.position is not None else torch.zeros(0, dtype=torch.float32, device=dev)
        rot_dims = 2 * inv_freq.numel()
        plane = cache.planes[0]
        table = ctx.block_tables[cache.group]
        down = torch.empty((T, self.down_cols), dtype=self.dtype, device=dev)
        ops.linear(h, self.w_down, None, down)
        write = (ctx.token_req, table, plane, cache.page_size) if cache.writable else (None, None, None, 0)
        if self.q_rank:
            cq = torch.empty((T, self.q_rank), dtype=self.dtype, device=dev)
            ops.latent_prepare(down, self.q_rank, self.rank, self.rot, rot_dims, self.w_dq_norm, self.w_dkv_norm, float(self.spec.norm_eps),
                               ctx.positions, inv_freq, cq, *write)
            q = torch.empty((T, n * (self.dim + self.rot)), dtype=self.dtype, device=dev)
            ops.linear(cq, self.w_uq, None, q)
        else:                       # the queries are the first columns of the projection
            ops.latent_prepare(down, 0, self.rank, self.rot, rot_dims, None, self.w_dkv_norm, float(self.spec.norm_eps),
                               ctx.positions, inv_freq, None, *write, kv_off=self.q_cols)
            q = down[:, : self.q_cols]
        # the query against a cache row: [W_uk^T q_unrotated, rotated part], head by head
        qrow = torch.empty((T, n * self.row), dtype=self.dtype, device=dev)
        ops.heads_linear(q, self.dim + self.rot, self.w_uk_t, qrow, self.row)
        if self.rot:
            ops.rotate_pairs(q, self.dim + self.rot, self.dim, qrow, self.row, self.rank, ctx.positions, inv_freq, n, self.rot)
        # (sequences whose block table the matrix-core kernel cannot keep in shared memory go to the general kernel and its tiles)
        general = table.shape[1] > ops.LATENT_MFMA_MAX_BLOCKS
        tq = self.general_tile_tokens if general else self.tile_tokens
        tile_req, tile_tok0, tiles = ctx.tiles(tq)
        if ctx.decode_only and tiles == T:          # one token per request: no tile list to look up
            tile_req = tile_tok0 = None
        mixed_latent = torch.empty((T, n * self.rank), dtype=self.dtype, device=dev)
        ops.latent_attention(qrow, mixed_latent, plane, table, ctx.req_indptr, ctx.ctx_lens, tile_req, tile_tok0, tiles, tq,
                             n, self.rank, self.rot, cache.page_size, self.scale, self.sink, self._splits(ctx, tiles),
                             general=general, max_new_tokens=ctx.max_new_tokens, window=self.window,
                             gate=down[:, self.gate_at:] if self.spec.gate else None)
        values = torch.empty((T, n * self.vdim), dtype=self.dtype, device=dev)
        ops.heads_linear(mixed_latent, self.rank, self.w_uv, values, self.vdim)
        if self.dtype == torch.bfloat16 and ops.linear_partials_pay(T, self.hidden, n * self.vdim):
            return ops.linear_partials(values, self.w_o)      # few rows against a narrow matrix: the next norm adds the slabs up
        out = torch.empty((T, self.hidden), dtype=self.dtype, device=dev)
        ops.linear(values, self.w_o, None, out)
        return out
