"""Linear attention with one fixed decay per head (lightning attention), with a fixed-size state per request.

Per token ``q = silu(W_q h)`` and ``k = silu(W_k h)`` (``heads x dim``) and ``v = silu(W_v h)`` (``heads x vdim``), head by head; head ``i`` moves
its state ``S [dim, vdim]`` by ``S <- decay_i S + k v^T`` and gives ``o = S^T q``.  The heads' outputs side by side are divided by their root
mean square (all of them together), multiplied by a weight vector and by ``sigmoid(W_g h)``, and projected by ``W_o``.  A request's slot
holds the states of all heads in 32-bit, zero when the slot is handed out; activations of the projections, state, outputs and norm are
32-bit under every engine.  The recurrence runs in the delta rule's kernel without that rule's correction term, token by token from where
the state stands, so a portion of n tokens is n single steps by construction.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import KEEP_COMPUTE, KEEP_FLOAT32, MIXERS, StagedMixer, StateNeed, WeightSpec


@MIXERS.register("decayed_linear")
class DecayedLinearAttention(StagedMixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if len(spec.decay) != spec.heads:
            raise ConfigError(f"decayed linear attention: {len(spec.decay)} decays for {spec.heads} heads")
        if any(not 0.0 <= float(d) <= 1.0 for d in spec.decay):
            raise ConfigError("decayed linear attention: a decay lies between 0 and 1")
        if spec.dim > ops.DELTA_MAX_DIM:
            raise ConfigError(f"decayed linear attention: built for up to {ops.DELTA_MAX_DIM} query/key dimensions per head, not {spec.dim}")
        self.hidden, self.heads, self.dim, self.vdim = spec.hidden, spec.heads, spec.dim, spec.vdim
        self.qk_width, self.v_width = spec.heads * spec.dim, spec.heads * spec.vdim
        self.channels = 2 * self.qk_width + self.v_width         # q, k, v: what passes silu and enters the recurrence
        self.in_width = self.channels + self.v_width             # ... and the output gate
        self.mix_width = self.v_width
        self.decay = torch.tensor([float(d) for d in spec.decay], dtype=torch.float32, device=device)
        self.w_norm = None

    def state_need(self):
        return StateNeed(shape=(self.heads * self.dim * self.vdim,), dtype=torch.float32)

    def kernel_libraries(self):
        return ["recurrent"]

    def weight_specs(self):
        H = self.hidden
        return {"q": WeightSpec((self.qk_width, H)), "k": WeightSpec((self.qk_width, H)), "v": WeightSpec((self.v_width, H)),
                "g": WeightSpec((self.v_width, H)), "o": WeightSpec((H, self.v_width)),
                "norm": WeightSpec((self.v_width,), keep=KEEP_FLOAT32, init="one_plus_normal")}

    def load_weights(self, tensors):
        self.w_in = self._place(torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0), KEEP_COMPUTE)
        self.w_norm = self._place(tensors["norm"], KEEP_FLOAT32)
        self.w_o = self._place(tensors["o"], KEEP_COMPUTE)

    def mix(self, proj, h, ctx, cache, out, gain=1.0):
        T = h.shape[0]
        qkv = torch.empty((T, self.channels), dtype=torch.float32, device=h.device)
        ops.silu_float(proj[:, : self.channels], qkv)
        o = torch.empty((T, self.v_width), dtype=torch.float32, device=h.device)
        ops.decay_scan(qkv, self.decay, cache.state, ctx.slots, ctx.req_indptr, o, self.heads, self.dim, self.vdim,
                       max_new_tokens=ctx.max_new_tokens)
        # the heads side by side are one vector for the norm
        ops.gated_head_norm(o, proj[:, self.channels:], self.w_norm, float(self.spec.norm_eps), out, 1, self.v_width, gate="sigmoid", gain=gain)
