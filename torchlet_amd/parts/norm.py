"""Root-mean-square norm, fused with the addition of the pending branch output.

``h = r * rsqrt(mean(r^2) + eps) * weight`` with ``r = residual + pending``; the epsilon
sits inside the root and the weight multiplies last, without a ``1 +`` offset
(/root/reference/src/torchlet/v10_triton_paged_gqa/kernel/rms_norm.py:13-19).  All of it
is computed in 32-bit; ``r`` is stored back as the new 32-bit residual.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import KEEP_FLOAT32, KEEP_STORED, NORMS, LazyNorm, Norm, Stream, WeightSpec


def _over_streams(kind: str, stream: Stream, weight, bias, eps: float, dtype, rows, gain: float, read) -> torch.Tensor:
    """The norm ``kind`` of ``sum_s read[s] x_s`` over the copies of the residual, after the pending output has entered them
    through ``stream.fold``: one kernel for the fold, the read and the norm.  A plain residual ``[T, hidden]`` is one stream."""
    x = stream.residual if stream.residual.dim() == 3 else stream.residual.unsqueeze(0)
    n = x.shape[1] if rows is None else rows.numel()
    out = torch.empty((n, x.shape[2]), dtype=dtype, device=x.device)
    ops.streams_norm(x, stream.pending, stream.fold, read, kind, weight, bias, eps, out, rows, gain)
    if rows is None:
        stream.pending = None
        stream.fold = None
    return out


def _no_post_norm(stream: Stream, kind: str) -> None:
    if stream.post is not None or stream.extra is not None:
        raise ValueError(f"a {kind} does not fold a normed branch output or a second addend into the stream; a norm that says folds_post_norm does")


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.dim = spec.dim
        self.eps = float(spec.eps)
        self.weight: torch.Tensor | None = None

    def weight_specs(self):
        return {self.spec.weight_name: WeightSpec((self.dim,), keep=KEEP_STORED, init="one_plus_normal")}

    def load_weights(self, tensors):
        self.weight = self._place(tensors[self.spec.weight_name], KEEP_STORED)

    def forward(self, stream: Stream, rows: torch.Tensor | None = None, gain: float = 1.0, read: torch.Tensor | None = None) -> torch.Tensor:
        _no_post_norm(stream, "rmsnorm")
        if stream.residual.dim() == 3:
            return _over_streams("rmsnorm", stream, self.weight, None, self.eps, self.dtype, rows, gain, read)
        n = stream.residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.dim), dtype=self.dtype, device=stream.residual.device)
        ops.add_rmsnorm(stream.residual, stream.pending, self.weight, self.eps, out, rows, gain)
        if rows is None:
            stream.pending = None
        return out

    def renorm(self, stream: Stream, alpha: float = 1.0) -> torch.Tensor:
        if self.dtype == torch.float32:              # the residual itself is what the next sublayer reads
            ops.scaled_add_rmsnorm(stream.residual, stream.pending, alpha, self.weight, self.eps, None)
            stream.pending = None
            return stream.residual
        out = torch.empty(stream.residual.shape, dtype=self.dtype, device=stream.residual.device)
        ops.scaled_add_rmsnorm(stream.residual, stream.pending, alpha, self.weight, self.eps, out)
        stream.pending = None
        return out

    def lazy(self, stream: Stream) -> LazyNorm | None:
        # one row in bfloat16: the kernels that read the norm's output can make it while their weights arrive
        if self.dtype == torch.bfloat16 and stream.residual.dim() == 2 and stream.residual.shape[0] == 1 and stream.residual.is_cuda:
            return LazyNorm(self, stream, "rmsnorm", weight=self.weight, eps=self.eps)
        return None


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """``(r - mean(r)) / sqrt(mean((r - mean(r))^2) + eps) * weight + bias`` in 32-bit, fused with the entry of the pending branch
    output into the residual (one plain residual, or several copies joined by hyper-connections)."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.dim = spec.dim
        self.eps = float(spec.eps)
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None

    def weight_specs(self):
        return {self.spec.weight_name: WeightSpec((self.dim,), keep=KEEP_FLOAT32, init="one_plus_normal"),
                self.spec.bias_name: WeightSpec((self.dim,), keep=KEEP_FLOAT32)}

    def load_weights(self, tensors):
        self.weight = self._place(tensors[self.spec.weight_name], KEEP_FLOAT32)
        self.bias = self._place(tensors[self.spec.bias_name], KEEP_FLOAT32)

    def forward(self, stream: Stream, rows: torch.Tensor | None = None, gain: float = 1.0, read: torch.Tensor | None = None) -> torch.Tensor:
        _no_post_norm(stream, "layernorm")
        return _over_streams("layernorm", stream, self.weight, self.bias, self.eps, self.dtype, rows, gain, read)


@NORMS.register("scalar_rmsnorm")
class ScalarRMSNorm(Norm):
    """``r / sqrt(mean(r^2) + eps) * g`` with one number ``g`` for all coordinates, in 32-bit.  It folds everything a stream can carry
    into the residual on the way, in the same kernel: the pending branch output, plain or, where the block left a norm on it
    (``stream.post``), divided by its own root mean square and multiplied by that norm's weight first; and a second addend
    (``stream.extra``)."""
    graph_safe = True
    folds_post_norm = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.dim = spec.dim
        self.eps = float(spec.eps)
        self.weight: torch.Tensor | None = None

    def weight_specs(self):
        return {self.spec.weight_name: WeightSpec((), keep=KEEP_FLOAT32, init="one_plus_normal")}

    def load_weights(self, tensors):
        self.weight = self._place(tensors[self.spec.weight_name].reshape(1), KEEP_FLOAT32)

    def forward(self, stream: Stream, rows: torch.Tensor | None = None, gain: float = 1.0, read: torch.Tensor | None = None) -> torch.Tensor:
        if stream.residual.dim() != 2 or stream.fold is not None:
            raise ValueError("a scalar_rmsnorm runs over one plain residual")
        n = stream.residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.dim), dtype=self.dtype, device=stream.residual.device)
        post_w, post_eps = stream.post if stream.post is not None else (None, 0.0)
        ops.sandwich_norm(stream.residual, stream.pending, post_w, post_eps, stream.extra, self.weight, self.eps, out, rows, gain)
        if rows is None:
            stream.pending = stream.post = stream.extra = None
        return out


@NORMS.register("offset_rmsnorm")
class OffsetRMSNorm(Norm):
    """``r / sqrt(mean(r^2) + eps) * (offset + w) * gain`` with a weight vector ``w`` stored around zero (``offset`` 1), in 32-bit: the
    offset and the fixed gain are folded into the vector once, at load, in 32-bit.  Like :class:`ScalarRMSNorm` it folds everything a
    stream can carry (the pending branch output, normed with the weight its block left beside it; a second addend) in the same kernel."""
    graph_safe = True
    folds_post_norm = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.dim = spec.dim
        self.eps = float(spec.eps)
        self.weight: torch.Tensor | None = None

    def weight_specs(self):
        return {self.spec.weight_name: WeightSpec((self.dim,), keep=KEEP_FLOAT32, init="normal" if self.spec.offset else "one_plus_normal")}

    def load_weights(self, tensors):
        w = (tensors[self.spec.weight_name].to(torch.float32) + float(self.spec.offset)) * float(self.spec.gain)
        self.weight = self._place(w, KEEP_FLOAT32)

    def forward(self, stream: Stream, rows: torch.Tensor | None = None, gain: float = 1.0, read: torch.Tensor | None = None) -> torch.Tensor:
        if stream.residual.dim() != 2 or stream.fold is not None:
            raise ValueError("an offset_rmsnorm runs over one plain residual")
        n = stream.residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.dim), dtype=self.dtype, device=stream.residual.device)
        post_w, post_eps = stream.post if stream.post is not None else (None, 0.0)
        ops.sandwich_norm(stream.residual, stream.pending, post_w, post_eps, stream.extra, self.weight, self.eps, out, rows, gain)
        if rows is None:
            stream.pending = stream.post = stream.extra = None
        return out

    def embed(self, token_ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
        """``out[t] = norm(table[token_ids[t]] * scale)``: the embedding's rows normed on their way into the 32-bit stream, one kernel."""
        ops.embedding_norm(token_ids, table, out, scale, self.weight, self.eps)
