"""Feed-forward layers with an elementwise activation: a dense one with biases, and a mixture of experts.

Dense: ``W_down act(W_up h + b_up) + b_down``.  Routed: the router's logits ``z = W_r h + b_r`` leave their product in
32-bit (the operands are ``h`` as the stream's norm rounded it and the router's matrix as stored, so the products are
exact and the sums 32-bit); per token the ``top`` largest are chosen (the lower index wins a tie), their softmax (over
the chosen ones alone, in 32-bit) weighs the experts' outputs ``W_down,e act(W_up,e h)``, which are summed in the order
of the choices.  The choice, the sort of the (token, choice) pairs by expert and the products over the experts' rows all
happen on the GPU from device-side counts: nothing of a step's routing is read on the host, so decode steps can be
recorded as graphs.

The routed layer has other forms as well, each a field of its specification.  Gated experts, ``W_down,e (act(W_gate,e h) *
W_up,e h)``: the rows of gate and up are interleaved into one matrix per expert and the product's epilogue applies the gate to
each pair of neighbouring columns.  Scores over all experts: ``s = softmax(z)`` over every logit, the ``top`` largest of ``s +
correction`` are chosen (the correction enters the choice only) and the weights are the chosen ``s`` as they are.  Identity
experts: the router's last ``identity`` outputs have no tensors; a token that chooses one gets its own input times the weight.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import FEED_FORWARDS, KEEP_COMPUTE, KEEP_FLOAT32, FeedForward, WeightSpec, join_name, under


def _activation(name: str) -> str:
    if name not in ops.ACTIVATIONS:
        raise ConfigError(f"no activation {name!r}; built: {', '.join(sorted(ops.ACTIVATIONS))}")
    return name


@FEED_FORWARDS.register("dense_ff")
class DenseFF(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden, self.inter, self.act = spec.hidden, spec.intermediate, _activation(spec.activation)
        self.w_up = self.b_up = self.w_down = self.b_down = None

    def kernel_libraries(self):
        return ["experts"]

    def weight_specs(self):
        specs = {"up": WeightSpec((self.inter, self.hidden)), "down": WeightSpec((self.hidden, self.inter))}
        if self.spec.bias:
            specs["up.b"] = WeightSpec((self.inter,), keep=KEEP_FLOAT32)
            specs["down.b"] = WeightSpec((self.hidden,), keep=KEEP_FLOAT32)
        return specs

    def load_weights(self, tensors):
        self.w_up = self._place(tensors["up"], KEEP_COMPUTE)
        self.w_down = self._place(tensors["down"], KEEP_COMPUTE)
        if self.spec.bias:
            self.b_up = self._place(tensors["up.b"], KEEP_FLOAT32)
            self.b_down = self._place(tensors["down.b"], KEEP_FLOAT32)

    def forward(self, h, ctx):
        T = h.shape[0]
        z = torch.empty((T, self.inter), dtype=self.dtype, device=h.device)
        ops.linear(h, self.w_up, self.b_up, z)
        ops.activation(z, self.act)
        y = torch.empty((T, self.hidden), dtype=self.dtype, device=h.device)
        ops.linear(z, self.w_down, self.b_down, y)
        return y


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden, self.inter, self.experts, self.top = spec.hidden, spec.intermediate, spec.experts, spec.top
        self.identity = int(spec.identity)
        self.outputs = self.experts + self.identity          # of the router
        if not 0 < spec.top <= self.outputs:
            raise ConfigError(f"a router picks between 1 and all of its experts, not {spec.top} of {self.outputs}")
        if spec.scores not in ops.ROUTER_SCORES:
            raise ConfigError(f"a router's scores are the softmax over the 'chosen' logits or over 'all', or their 'sigmoid', not {spec.scores!r}")
        # one more feed-forward that every token passes, added to the weighted sum (any registered kind that returns a whole tensor)
        self.shared = FEED_FORWARDS.build(spec.shared, dtype, device) if spec.shared is not None else None
        self.act = _activation(spec.activation + "_pairs" if spec.gated else spec.activation)
        self.w_router = self.b_router = self.correction = self.w_up = self.w_down = None

    def kernel_libraries(self):
        return ["experts"]

    def parts(self):
        yield self
        if self.shared is not None:
            yield from self.shared.parts()

    def weight_specs(self):
        specs = {"router": WeightSpec((self.outputs, self.hidden))}
        if self.shared is not None:
            specs.update({join_name("shared", k): v for k, v in self.shared.weight_specs().items()})
        if self.spec.router_bias:
            specs["router.b"] = WeightSpec((self.outputs,), keep=KEEP_FLOAT32)
        if self.spec.choice_bias:
            specs["correction"] = WeightSpec((self.outputs,), keep=KEEP_FLOAT32)
        for e in range(self.experts):
            if self.spec.gated:
                specs[f"e{e}.gate"] = WeightSpec((self.inter, self.hidden))
            specs[f"e{e}.up"] = WeightSpec((self.inter, self.hidden))
            specs[f"e{e}.down"] = WeightSpec((self.hidden, self.inter))
        return specs

    def load_weights(self, tensors):
        self.w_router = self._place(tensors["router"], KEEP_COMPUTE)
        self.b_router = self._place(tensors["router.b"], KEEP_FLOAT32) if self.spec.router_bias else None
        self.correction = self._place(tensors["correction"], KEEP_FLOAT32) if self.spec.choice_bias else None
        if self.spec.gated:       # rows 2i and 2i + 1 of an expert's first matrix: row i of its gate and of its up
            up = [torch.stack((tensors[f"e{e}.gate"], tensors[f"e{e}.up"]), dim=1).reshape(2 * self.inter, self.hidden) for e in range(self.experts)]
        else:
            up = [tensors[f"e{e}.up"] for e in range(self.experts)]
        self.w_up = self._place(torch.stack(up), KEEP_COMPUTE)
        self.w_down = self._place(torch.stack([tensors[f"e{e}.down"] for e in range(self.experts)]), KEEP_COMPUTE)
        if self.shared is not None:
            self.shared.load_weights(under(tensors, "shared"))

    def forward(self, h, ctx):
        T = h.shape[0]
        logits = torch.empty((T, self.outputs), dtype=torch.float32, device=h.device)
        ops.linear(h, self.w_router, self.b_router, logits)
        weights, offsets, slot_token, pair_slot = ops.route(logits, self.top, self.spec.scores, self.correction, float(self.spec.weight_scale),
                                                            float(self.spec.weight_eps))
        z = torch.empty((T * self.top, self.inter), dtype=self.dtype, device=h.device)
        ops.experts_linear(h, slot_token, self.w_up, offsets, z, self.act)
        y = torch.empty((T * self.top, self.hidden), dtype=self.dtype, device=h.device)
        ops.experts_linear(z, None, self.w_down, offsets, y)
        out = torch.empty((T, self.hidden), dtype=self.dtype, device=h.device)
        # (slots of identity experts lie behind those of the last expert with tensors: their rows of z and y are never written or read)
        shared = None
        if self.shared is not None:
            # (a part that may leave slabs of partial sums for a norm to add up is asked for the whole product)
            shared = self.shared.forward(h, ctx, whole=True) if getattr(self.shared, "takes_whole", False) else self.shared.forward(h, ctx)
            if shared.dim() != 2:
                raise ValueError(f"a shared expert must return one [tokens, hidden] tensor; {type(self.shared).__name__} returned {tuple(shared.shape)}")
        ops.combine(y, pair_slot, weights, out, identity=(h, offsets, self.experts) if self.identity else None, addend=shared)
        return out
