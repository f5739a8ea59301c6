"""A decoder built from a :class:`~torchlet_amd.config.base.ModelSpec`.

embedding (times ``embed_scale``, plus the position's row of a learned table if the specification names one, plus a hashed bigram row if
it names one) -> the runs of the layer order (before a run that says so the embedding's output enters the stream again) -> final norm on the wanted rows
(times ``logit_scale``) -> LM head (plus its bias, if the specification says it has one)
(/root/reference/src/torchlet/v10_triton_paged_gqa/model/qwen2_5.py:55-87, where the factors are 1 and
there is no bias).  The class
knows nothing of any architecture: which parts a layer has, their sizes, the names of
their tensors and the order of the runs all come from the specification.
"""
from __future__ import annotations

import torch

from ..config.base import ModelSpec
from ..kernels import ops
from ..parts import BLOCKS, NORMS, StateNeed, Stream, WeightSpec
from ..parts.base import KEEP_COMPUTE, KEEP_STORED, join_name, place, under


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.blocks = [BLOCKS.build(b, dtype, self.device) for b in spec.layers]
        self.final_norm = NORMS.build(spec.final_norm, dtype, self.device)
        self.embed: torch.Tensor | None = None
        self.head: torch.Tensor | None = None
        self.head_bias: torch.Tensor | None = None
        self.position_table: torch.Tensor | None = None
        self.bigram_table: torch.Tensor | None = None
        self.keeps_embedding = any(e.add_embedding for e in spec.order)
        self.embed_norm = NORMS.build(spec.embed_norm, dtype, self.device) if spec.embed_norm is not None else None
        if self.embed_norm is not None and (not hasattr(self.embed_norm, "embed") or spec.bigram is not None or spec.position_table_name
                                            or spec.streams or self.keeps_embedding):
            raise ValueError("a norm on the embedding needs a norm that makes the normed rows itself, over one plain residual of token rows alone")
        if (spec.bigram is not None or self.keeps_embedding) and spec.streams:
            raise ValueError("a bigram embedding or an embedding that enters the stream again runs over one plain residual")
        if spec.bigram is not None and spec.position_table_name:
            raise ValueError("a bigram embedding beside a learned position table is not built")

    # ------------------------------------------------------------------ weights
    def weight_specs(self) -> dict[str, WeightSpec]:
        s = self.spec
        specs = {join_name(s.embed_name, s.weight_suffix): WeightSpec((s.vocab_size, s.hidden))}
        if s.position_table_name:
            specs[join_name(s.position_table_name, s.weight_suffix)] = WeightSpec((s.max_positions, s.hidden), keep=KEEP_STORED)
        if s.bigram is not None:
            specs[join_name(s.bigram.name, s.weight_suffix)] = WeightSpec((s.bigram.buckets + 1, s.hidden))
        for i, block in enumerate(self.blocks):
            for k, v in block.weight_specs().items():
                specs[join_name(s.layer_name(i), k)] = v
        for k, v in self.final_norm.weight_specs().items():
            specs[join_name(s.final_norm_name, k)] = v
        if self.embed_norm is not None:
            for k, v in self.embed_norm.weight_specs().items():
                specs[join_name(s.embed_norm_name, k)] = v
        # a tied head is the embedding matrix; a checkpoint may still carry a copy of it
        specs[join_name(s.head_name, s.weight_suffix)] = WeightSpec((s.vocab_size, s.hidden), optional=s.tie_head)
        if s.head_bias:
            specs[f"{s.head_name}.bias"] = WeightSpec((s.vocab_size,), keep=KEEP_STORED)
        return specs

    def load_weights(self, tensors: dict[str, torch.Tensor]) -> None:
        s = self.spec
        self.embed = place(tensors[join_name(s.embed_name, s.weight_suffix)], KEEP_COMPUTE, self.dtype, self.device)
        if s.position_table_name:
            self.position_table = place(tensors[join_name(s.position_table_name, s.weight_suffix)], KEEP_STORED, self.dtype, self.device)
        if s.bigram is not None:
            self.bigram_table = place(tensors[join_name(s.bigram.name, s.weight_suffix)], KEEP_COMPUTE, self.dtype, self.device)
        for i, block in enumerate(self.blocks):      # (`tensors` may read from disk on access: each name is touched once)
            block.load_weights(under(tensors, s.layer_name(i)))
        self.final_norm.load_weights(under(tensors, s.final_norm_name))
        if self.embed_norm is not None:      # (its name may lie below the embedding's: the tensor is asked for by its full name)
            self.embed_norm.load_weights({k: tensors[join_name(s.embed_norm_name, k)] for k in self.embed_norm.weight_specs()})
        if s.tie_head:
            self.head = self.embed
        else:
            self.head = place(tensors[join_name(s.head_name, s.weight_suffix)], KEEP_COMPUTE, self.dtype, self.device)
        if s.head_bias:
            self.head_bias = place(tensors[f"{s.head_name}.bias"], KEEP_STORED, self.dtype, self.device)

    # ------------------------------------------------------------------ cache needs
    def cache_plan(self):
        """Per run of the order: ``(paged need, state need, cache_of)``; a model whose embedding reads the token before keeps it as one
        more entry after the runs: an int32 per request."""
        plan = []
        for e in self.spec.order:
            mixer = self.blocks[e.layer].mixer
            plan.append((mixer.paged_need(), mixer.state_need(), e.cache_of))
        if self.spec.bigram is not None:
            plan.append((None, StateNeed(shape=(1,), dtype=torch.int32), None))
        return plan

    def tile_token_sizes(self) -> set[int]:
        return {p.tile_tokens for p in self.parts() if hasattr(p, "tile_tokens")}

    def parts(self):
        """Every part of the model: each block with what is inside it, and the final norm."""
        for b in self.blocks:
            yield from b.parts()
        yield from self.final_norm.parts()
        if self.embed_norm is not None:
            yield from self.embed_norm.parts()

    def graph_safe(self) -> bool:
        """Every part of every block (and the final norm) says that it runs from device-side values only,
        so a decode step can be captured once as a graph and replayed."""
        return all(getattr(p, "graph_safe", False) for p in self.parts())

    def kernel_libraries(self) -> list[str]:
        libs = ["elementwise", "gemm", "sampling"]
        for part in self.parts():
            if hasattr(part, "kernel_libraries"):
                libs += part.kernel_libraries()
        return list(dict.fromkeys(libs))

    # ------------------------------------------------------------------ the step
    def forward(self, ctx, caches) -> torch.Tensor | None:
        """Run the tokens of ``ctx`` through every run of the order; ``caches[i]`` is the
        cache view of run ``i``.  Returns float32 logits ``[wanted rows, vocab]`` (``None``
        when no row is wanted)."""
        T = ctx.num_tokens
        # the 32-bit residual, or the copies of it that blocks joined by hyper-connections keep: all start as the embedding's output
        shape = (self.spec.streams, T, self.spec.hidden) if self.spec.streams else (T, self.spec.hidden)
        if self.keeps_embedding:            # a second copy of the embedding's output, for the runs before which it enters the stream again
            shape = (2, T, self.spec.hidden)
        residual = torch.empty(shape, dtype=torch.float32, device=self.device)
        big = self.spec.bigram
        if big is not None:
            ops.bigram_embedding(ctx.token_ids, self.embed, residual, self.spec.embed_scale, self.bigram_table, big.buckets, big.mul_prev,
                                 big.mul_cur, ctx.token_req, ctx.req_indptr, ctx.positions, ctx.slots, caches[len(self.spec.order)].state)
        elif self.embed_norm is not None:
            self.embed_norm.embed(ctx.token_ids, self.embed, residual, self.spec.embed_scale)
        else:
            ops.embedding(ctx.token_ids, self.embed, residual, self.spec.embed_scale,
                          *((ctx.positions, self.position_table) if self.position_table is not None else ()))
        embedded = None
        if self.keeps_embedding:
            residual, embedded = residual[0], residual[1]
        stream = Stream(residual)
        for i, e in enumerate(self.spec.order):
            if e.add_embedding:             # the next norm adds it beside the pending branch output
                stream.extra = embedded
            stream = self.blocks[e.layer].forward(stream, ctx, caches[i])
        if ctx.want_rows is None or ctx.num_wanted == 0:
            return None
        h = self.final_norm.forward(stream, rows=ctx.want_rows, gain=self.spec.logit_scale)
        logits = torch.empty((ctx.num_wanted, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        ops.linear(h, self.head, self.head_bias, logits)
        return logits
