"""Several mixers side by side on one input: ``y = sum_i scale_i * mixer_i(h)``.

Every branch is a :class:`~torchlet_amd.parts.base.StagedMixer`.  Their input projections are stacked into one matrix, so one
product reads ``h`` once; each branch mixes its own columns of the result and writes ``scale_i`` times its ``mix_width`` numbers per
token (the factor applied in 32-bit, before the one rounding) into its own columns of one buffer; and the output projections are
stacked side by side, ``[W_o1 | W_o2 | ...]``, so one product sums the branches in its 32-bit accumulators.  The branches' caches
are one run's cache: at most one branch keeps pages and at most one a fixed-size state.

``normed``: ``y = sum_i scale_i * rms(W_o,i mixer_i(h)) * w_i`` with a weight vector ``<name>.out`` over the model width per branch.  The
output projections then stay apart (each branch's result is normed by itself); the norms and the weighted sum are one kernel, in 32-bit.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import KEEP_COMPUTE, KEEP_FLOAT32, MIXERS, Mixer, StagedMixer, WeightSpec, join_name, project_out, under


@MIXERS.register("parallel")
class ParallelMixer(Mixer):
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if not spec.branches:
            raise ConfigError("a parallel mixer needs at least one branch")
        self.names = [name for name, _, _ in spec.branches]
        self.scales = [float(scale) for _, _, scale in spec.branches]
        self.branches = [MIXERS.build(s, dtype, device) for _, s, _ in spec.branches]
        for name, b in zip(self.names, self.branches):
            if not isinstance(b, StagedMixer):
                raise ConfigError(f"branch {name!r} of a parallel mixer is a {type(b).__name__}, which is not built in stages")
        if any(getattr(b.spec, "qk_bias", False) or getattr(b.spec, "o_bias", False) for b in self.branches):
            raise ConfigError("a parallel mixer stacks its branches' projections into one product; branches with biases are not built")
        if sum(b.paged_need() is not None for b in self.branches) > 1 or sum(b.state_need() is not None for b in self.branches) > 1:
            raise ConfigError("a parallel mixer holds one run's cache: at most one branch with pages and one with a state")
        self.hidden = spec.hidden
        self.normed = bool(spec.normed)
        self.norm_eps = float(spec.norm_eps)
        self.w_in = self.w_o = None
        self.w_outs: list = []          # normed: per branch its output projection
        self.out_weights = None         # normed: [branches, hidden], each branch's weight times its scale

    @property
    def graph_safe(self):
        return all(b.graph_safe for b in self.branches)

    def paged_need(self):
        return next((n for n in (b.paged_need() for b in self.branches) if n is not None), None)

    def state_need(self):
        return next((n for n in (b.state_need() for b in self.branches) if n is not None), None)

    def parts(self):
        yield self
        for b in self.branches:
            yield from b.parts()

    def weight_specs(self):
        specs = {join_name(name, k): v for name, b in zip(self.names, self.branches) for k, v in b.weight_specs().items()}
        if self.normed:
            for name in self.names:
                specs[f"{name}.out"] = WeightSpec((self.hidden,), keep=KEEP_FLOAT32, init="one_plus_normal")
        return specs

    def load_weights(self, tensors):
        for name, b in zip(self.names, self.branches):
            b.load_weights({k: v for k, v in under(tensors, name).items() if not (self.normed and k == "out")})
        self.w_in = torch.cat([b.w_in for b in self.branches], dim=0).contiguous()
        if self.normed:
            self.w_outs = [b.w_o for b in self.branches]
            self.out_weights = self._place(torch.stack([tensors[f"{name}.out"].float() * scale for name, scale in zip(self.names, self.scales)]),
                                           KEEP_FLOAT32)
        else:
            self.w_o = torch.cat([b.w_o for b in self.branches], dim=1).contiguous()
        for b in self.branches:          # the branches' own copies are views of nothing: drop them
            b.w_in = b.w_o = None

    def forward(self, h, ctx, cache):
        T = h.shape[0]
        proj = torch.empty((T, self.w_in.shape[0]), dtype=self.dtype, device=h.device)
        ops.linear(h, self.w_in, None, proj)
        if self.normed:
            outs = torch.empty((len(self.branches), T, self.hidden), dtype=self.dtype, device=h.device)
            at_in = 0
            for i, b in enumerate(self.branches):
                mixed = torch.empty((T, b.mix_width), dtype=self.dtype, device=h.device)
                b.mix(proj[:, at_in: at_in + b.in_width], h, ctx, cache, mixed)
                ops.linear(mixed, self.w_outs[i], None, outs[i])
                at_in += b.in_width
            y = torch.empty((T, self.hidden), dtype=self.dtype, device=h.device)
            ops.normed_sum(outs, self.out_weights, self.norm_eps, y)
            return y
        mixed = torch.empty((T, self.w_o.shape[1]), dtype=self.dtype, device=h.device)
        at_in = at_out = 0
        for b, scale in zip(self.branches, self.scales):
            b.mix(proj[:, at_in: at_in + b.in_width], h, ctx, cache, mixed[:, at_out: at_out + b.mix_width], scale)
            at_in += b.in_width
            at_out += b.mix_width
        return project_out(mixed, self.w_o, self.dtype)
