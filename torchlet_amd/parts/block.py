"""Pre-norm residual block: ``x += mixer(norm1(x)); x += ffn(norm2(x))``
(/root/reference/src/torchlet/v10_triton_paged_gqa/layer/transformer_block.py:37-40).

The additions are deferred: a branch's output is left ``pending`` on the stream and the
next norm (the block's second one, the next block's first one, or the model's final one)
adds it in 32-bit while it normalises.

The other arrangement built here puts the norm after the sum: ``x <- norm1(alpha * x + mixer(x))``, then
``x <- norm2(alpha * x + ffn(x))``; the sublayers read the normed stream itself, and the sum and the norm are one
kernel that leaves the stream in 32-bit and, for the products that read it next, in the activation dtype.

A third one keeps several copies of the residual, joined by hyper-connections (:class:`HyperConnectionBlock`).

A fourth one norms a sublayer's output as well as its input (:class:`SandwichBlock`): ``x <- x + post1(mixer(norm1(x)))``, then ``x <- x +
post2(ffn(norm2(x)))``; the output is left pending with its norm's weight, and the next norm's kernel norms it, adds it and norms the sum.
"""
from __future__ import annotations

from ..config.base import ConfigError
from .base import BLOCKS, FEED_FORWARDS, KEEP_FLOAT32, MIXERS, NORMS, Block, Stream, WeightSpec, join_name, under


@BLOCKS.register("prenorm_residual")
class PreNormBlock(Block):
    graph_safe = True       # the arrangement itself; its four parts answer for themselves

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device)
        self._children = {
            spec.mixer_norm_name: self.mixer_norm,
            spec.mixer_name: self.mixer,
            spec.ffn_norm_name: self.ffn_norm,
            spec.ffn_name: self.ffn,
        }

    def parts(self):
        yield self
        for part in self._children.values():
            yield from part.parts()

    def weight_specs(self):
        return {join_name(name, k): v for name, part in self._children.items() for k, v in part.weight_specs().items()}

    def load_weights(self, tensors):
        for name, part in self._children.items():
            part.load_weights(under(tensors, name))

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        # a part that says it takes a norm that has not run yet (``takes_lazy_norm``) may get one, see LazyNorm
        h = (self.mixer_norm.lazy(stream) if getattr(self.mixer, "takes_lazy_norm", False) else None) or self.mixer_norm.forward(stream)
        stream.pending = self.mixer.forward(h, ctx, cache)
        h = (self.ffn_norm.lazy(stream) if getattr(self.ffn, "takes_lazy_norm", False) else None) or self.ffn_norm.forward(stream)
        stream.pending = self.ffn.forward(h, ctx)
        return stream


@BLOCKS.register("postnorm_residual")
class PostNormBlock(Block):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.alpha = float(spec.alpha)
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device) if spec.ffn is not None else None
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device) if spec.ffn is not None else None
        self._children = {spec.mixer_norm_name: self.mixer_norm, spec.mixer_name: self.mixer}
        if self.ffn is not None:
            self._children.update({spec.ffn_norm_name: self.ffn_norm, spec.ffn_name: self.ffn})

    parts = PreNormBlock.parts
    weight_specs = PreNormBlock.weight_specs
    load_weights = PreNormBlock.load_weights

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = stream.normed
        if h is None:                # the first block reads the embedding rows
            h = stream.residual if self.dtype == stream.residual.dtype else stream.residual.to(self.dtype)
        stream.pending = self.mixer.forward(h, ctx, cache)
        h = self.mixer_norm.renorm(stream, self.alpha)
        if self.ffn is not None:
            stream.pending = self.ffn.forward(h, ctx)
            h = self.ffn_norm.renorm(stream, self.alpha)
        stream.normed = h
        return stream


@BLOCKS.register("hyper_connections")
class HyperConnectionBlock(Block):
    """Pre-norm sublayers over ``S`` copies of the residual, ``stream.residual [S, T, hidden]`` in 32-bit.  Sublayer ``q`` reads
    ``u = sum_s in_q[s] x_s``, and its output ``y`` enters all copies at once, ``x_t <- sum_s mix_q[s, t] x_s + out_q[t] y``.  The
    entry is deferred like the plain block's addition: the output is left pending on the stream with its ``(mix, out)``, and the
    next norm's kernel (the block's second one, the next block's first one, the model's final one, which reads the sum of the
    copies) does the entry, the read and the norm in one pass over the copies."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.streams = int(spec.streams)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device) if spec.ffn is not None else None
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device) if spec.ffn is not None else None
        self._children = {spec.mixer_norm_name: self.mixer_norm, spec.mixer_name: self.mixer}
        if self.ffn is not None:
            self._children.update({spec.ffn_norm_name: self.ffn_norm, spec.ffn_name: self.ffn})
        self.connections = list(spec.connection_names[: 2 if self.ffn is not None else 1])
        self.read: list = []        # per sublayer: in [S]
        self.fold: list = []        # per sublayer: (mix [S, S] indexed from, to; out [S])

    parts = PreNormBlock.parts

    def weight_specs(self):
        S = self.streams
        specs = PreNormBlock.weight_specs(self)
        for name in self.connections:
            specs[f"{name}.in"] = WeightSpec((S,), keep=KEEP_FLOAT32, init="one_plus_normal")
            specs[f"{name}.out"] = WeightSpec((S,), keep=KEEP_FLOAT32, init="one_plus_normal")
            specs[f"{name}.mix"] = WeightSpec((S, S), keep=KEEP_FLOAT32, init="near_identity")
        return specs

    def load_weights(self, tensors):
        PreNormBlock.load_weights(self, tensors)
        self.read = [self._place(tensors[f"{name}.in"], KEEP_FLOAT32) for name in self.connections]
        self.fold = [(self._place(tensors[f"{name}.mix"], KEEP_FLOAT32), self._place(tensors[f"{name}.out"], KEEP_FLOAT32))
                     for name in self.connections]

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        if stream.residual.dim() != 3 or stream.residual.shape[0] != self.streams:
            raise ValueError(f"a block over {self.streams} copies of the residual got a stream of shape {tuple(stream.residual.shape)}")
        h = self.mixer_norm.forward(stream, read=self.read[0])
        stream.pending, stream.fold = self.mixer.forward(h, ctx, cache), self.fold[0]
        if self.ffn is not None:
            h = self.ffn_norm.forward(stream, read=self.read[1])
            stream.pending, stream.fold = self.ffn.forward(h, ctx), self.fold[1]
        return stream


@BLOCKS.register("sandwich_residual")
class SandwichBlock(Block):
    """A norm before and after each sublayer.  The norm after a sublayer is not run here: its weight and eps are left on the stream
    (``stream.post``) beside the pending output, and the next norm that folds the stream (this block's second one, the next block's first
    one, the model's final one) does ``x += pending / rms(pending) * weight`` in 32-bit inside its own kernel.  So every norm that can follow
    must be of a kind that says ``folds_post_norm``, and the norms after the sublayers must be root-mean-square norms with a plain weight."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.mixer_post = NORMS.build(spec.mixer_post_norm, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device) if spec.ffn is not None else None
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device) if spec.ffn is not None else None
        self.ffn_post = NORMS.build(spec.ffn_post_norm, dtype, device) if spec.ffn is not None else None
        self._children = {spec.mixer_norm_name: self.mixer_norm, spec.mixer_name: self.mixer, spec.mixer_post_norm_name: self.mixer_post}
        if self.ffn is not None:
            self._children.update({spec.ffn_norm_name: self.ffn_norm, spec.ffn_name: self.ffn, spec.ffn_post_norm_name: self.ffn_post})
        for norm in (self.mixer_norm, self.mixer_post, self.ffn_norm, self.ffn_post):
            if norm is not None and not getattr(norm, "folds_post_norm", False):
                raise ConfigError(f"a block with norms after its sublayers needs norms that fold a normed branch output; {type(norm).__name__} does not")

    parts = PreNormBlock.parts
    weight_specs = PreNormBlock.weight_specs
    load_weights = PreNormBlock.load_weights

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = self.mixer_norm.forward(stream)
        stream.pending, stream.post = self.mixer.forward(h, ctx, cache), (self.mixer_post.weight, self.mixer_post.eps)
        if self.ffn is not None:
            h = self.ffn_norm.forward(stream)
            stream.pending, stream.post = self.ffn.forward(h, ctx), (self.ffn_post.weight, self.ffn_post.eps)
        return stream
