"""A selective state-space recurrence (Mamba-2) with a fixed-size state per request.

One projection gives per token ``[z | x | B | C | dt]``: ``inner = heads * vdim`` numbers twice, ``groups * state`` twice, ``heads``.  x, B and C
pass a causal convolution of ``conv`` taps per channel (with a bias; zeros before the start of the sequence) and silu; ``dt <- softplus(dt +
dt_bias)``.  Head ``n`` (reading B and C of group ``n // (heads / groups)``) moves its state ``S [state, vdim]``::

    S <- exp(-exp(A_log[n]) dt) S + dt B x^T;    y = S^T C + D[n] x

and the mixer's output is ``W_o (norm(y * silu(z)) * w_norm)``, the norm a root-mean-square norm over ``norm_groups`` equal parts of the
``inner`` numbers, the gate before it.  A request's slot holds the states of all heads and the last ``conv - 1`` inputs of every convolved
channel, in 32-bit, zero when the slot is handed out.  The convolution's output, step sizes, decays, the state and the gated norm are
32-bit under every engine; the projections run in the compute dtype.  The recurrence is the delta rule's kernel without that rule's
correction term, with B as its keys, C as its queries, dt as its step size and x as its values, so it runs token by token from where the
state stands and a portion of n tokens is n single steps by construction.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import KEEP_COMPUTE, KEEP_FLOAT32, MIXERS, StagedMixer, StateNeed, WeightSpec
from . import gated_delta  # noqa: F401  (the initialisation laws of decays and taps)


@MIXERS.register("selective_state")
class SelectiveState(StagedMixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.heads % spec.groups:
            raise ConfigError(f"selective state: {spec.heads} heads are not a multiple of {spec.groups} groups")
        if spec.conv < 1 or spec.conv > ops.DELTA_MAX_TAPS:
            raise ConfigError(f"selective state: convolutions of 1 to {ops.DELTA_MAX_TAPS} taps are built, not {spec.conv}")
        if spec.state > ops.DELTA_MAX_DIM:
            raise ConfigError(f"selective state: built for states of up to {ops.DELTA_MAX_DIM} numbers per channel, not {spec.state}")
        self.hidden, self.heads, self.groups, self.vdim, self.state, self.taps = spec.hidden, spec.heads, spec.groups, spec.vdim, spec.state, spec.conv
        self.inner, self.gn = spec.heads * spec.vdim, spec.groups * spec.state
        if spec.norm_groups < 1 or self.inner % spec.norm_groups:
            raise ConfigError(f"selective state: {self.inner} inner channels do not split into {spec.norm_groups} equal parts")
        self.channels = self.inner + 2 * self.gn                 # convolved channels: x, B, C
        self.in_width = 2 * self.inner + 2 * self.gn + self.heads
        self.mix_width = self.inner
        self.state_floats = spec.heads * spec.state * spec.vdim  # the heads' states; the convolution's tails follow
        self.w_conv = self.b_conv = self.a_log = self.dt_bias = self.skip = self.w_norm = None

    def state_need(self):
        return StateNeed(shape=(self.state_floats + (self.taps - 1) * self.channels,), dtype=torch.float32)

    def kernel_libraries(self):
        return ["recurrent"]

    def weight_specs(self):
        H = self.hidden
        return {
            "in": WeightSpec((self.in_width, H)),
            "conv": WeightSpec((self.channels, self.taps), keep=KEEP_FLOAT32, init="conv_taps"),
            "conv.b": WeightSpec((self.channels,), keep=KEEP_FLOAT32),
            "dt_bias": WeightSpec((self.heads,), keep=KEEP_FLOAT32),
            "A_log": WeightSpec((self.heads,), keep=KEEP_FLOAT32, init="log_decay"),
            "D": WeightSpec((self.heads,), keep=KEEP_FLOAT32, init="one_plus_normal"),
            "norm": WeightSpec((self.inner,), keep=KEEP_FLOAT32, init="one_plus_normal"),
            "o": WeightSpec((H, self.inner)),
        }

    def load_weights(self, tensors):
        self.w_in = self._place(tensors["in"], KEEP_COMPUTE)
        self.w_conv = self._place(tensors["conv"], KEEP_FLOAT32)
        self.b_conv = self._place(tensors["conv.b"], KEEP_FLOAT32)
        self.dt_bias = self._place(tensors["dt_bias"], KEEP_FLOAT32)
        self.a_log = self._place(tensors["A_log"], KEEP_FLOAT32)
        self.skip = self._place(tensors["D"], KEEP_FLOAT32)
        self.w_norm = self._place(tensors["norm"], KEEP_FLOAT32)
        self.w_o = self._place(tensors["o"], KEEP_COMPUTE)

    def mix(self, proj, h, ctx, cache, out, gain=1.0):
        T = h.shape[0]
        gates = torch.empty((T, 2 * self.heads), dtype=torch.float32, device=h.device)
        cbx = torch.empty((T, self.channels), dtype=torch.float32, device=h.device)
        # convolutions (from the slot's tails, which move on) with their bias, silu; the raw step sizes become dt and the decay
        ops.selective_prepare(proj, self.inner, self.w_conv, self.b_conv, gates, self.a_log, self.dt_bias, cache.state, self.state_floats,
                              ctx.slots, ctx.req_indptr, ctx.token_req, cbx, self.heads, self.inner, self.gn, self.taps)
        y = torch.empty((T, self.inner), dtype=torch.float32, device=h.device)
        ops.selective_scan(cbx, gates, self.skip, cache.state, ctx.slots, ctx.req_indptr, y, self.heads, self.groups, self.state, self.vdim,
                           max_new_tokens=ctx.max_new_tokens)
        # the gate comes before the norm, and the norm runs over norm_groups equal parts of the row
        ops.gated_head_norm(y, proj[:, : self.inner], self.w_norm, float(self.spec.norm_eps), out, self.spec.norm_groups,
                            self.inner // self.spec.norm_groups, gate="silu", gain=gain, gate_first=True)
