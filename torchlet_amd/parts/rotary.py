"""Rotary position encoding with the split-half pairing ``(j, j + head_dim/2)``.

``inv_freq[j] = 1 / theta**(2j / head_dim)`` is computed once in 32-bit exactly as the
reference builds its table (/root/reference/src/torchlet/v10_triton_paged_gqa/layer/rope.py:29-35);
the angle of a token is ``float32(position) * inv_freq[j]`` and the rotation
``y1 = x1*cos - x2*sin, y2 = x2*cos + x1*sin`` (kernel/rope.py:28-37) is done in 32-bit
inside the kernel, so no table of ``max_positions`` rows is kept.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import POSITION_ENCODINGS, PositionEncoding


@POSITION_ENCODINGS.register("rope_split_half")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.head_dim % 2:
            raise ConfigError(f"rotary encoding needs an even head size, got {spec.head_dim}")
        self.head_dim = spec.head_dim
        self.max_positions = spec.max_positions
        j = torch.arange(0, spec.head_dim, 2, dtype=torch.float32)
        self.inv_freq = (1.0 / (float(spec.theta) ** (j / spec.head_dim))).to(device)

    def fused_inv_freq(self) -> torch.Tensor:
        """The attention mixer folds this encoding into its cache-write kernel."""
        return self.inv_freq

    def apply(self, q, k, positions):
        for x in (q, k):
            if x is None:
                continue
            T, heads, hd = x.shape
            flat = x.as_strided((T, heads * hd), (x.stride(0), 1))
            ops.rope_cache_write(flat, heads, 0, hd, heads, positions, self.inv_freq)


@POSITION_ENCODINGS.register("rope_pairs")
class PairRotaryEncoding(PositionEncoding):
    """The interleaved layout: of the first ``dims`` entries of a vector, entry ``2i`` is paired with ``2i + 1`` and the pair
    ``(u, v)`` at position ``p`` becomes ``(u cos a - v sin a, v cos a + u sin a)`` with ``a = float32(p) * f_i``,
    ``f_i = base**(-2i / dims)`` (taken in 64-bit on the host, then rounded once to 32-bit); entries beyond ``dims`` pass
    unchanged.  Mixers fold the rotation into their own kernels through :attr:`inv_freq`; :meth:`apply` turns whole heads."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.dims % 2 or spec.dims <= 0:
            raise ConfigError(f"rotary encoding in pairs needs an even, positive number of dimensions, got {spec.dims}")
        self.dims = spec.dims
        self.halves = False
        i = torch.arange(spec.dims // 2, dtype=torch.float64)
        self.inv_freq = (float(spec.base) ** (-2.0 * i / spec.dims) / float(getattr(spec, "factor", 1.0))).to(torch.float32).to(device)

    def apply(self, q, k, positions):
        for x in (q, k):
            if x is None:
                continue
            T, heads, hd = x.shape
            flat = x.as_strided((T, heads * hd), (x.stride(0), 1))
            ops.rotate_pairs(flat, hd, 0, flat, hd, 0, positions, self.inv_freq, heads, hd)


def scale_by_wavelength(freq: torch.Tensor, factor: float, low: float, high: float, original: float) -> torch.Tensor:
    """Frequencies scaled band by band (64-bit): a frequency whose wavelength ``2 pi / f`` is shorter than ``original / high`` stays, one whose
    wavelength is longer than ``original / low`` becomes ``f / factor``, and between the two ``(1 - s) f / factor + s f`` with ``s = (original /
    wavelength - low) / (high - low)``."""
    if not (factor > 0 and original > 0 and 0 < low < high):
        raise ConfigError(f"rotary encoding: scaling by wavelength wants factor > 0, original > 0 and 0 < low < high, got {(factor, low, high, original)}")
    wavelength = 2.0 * torch.pi / freq
    s = (original / wavelength - low) / (high - low)
    blended = (1.0 - s) * freq / factor + s * freq
    return torch.where(wavelength < original / high, freq, torch.where(wavelength > original / low, freq / factor, blended))


@POSITION_ENCODINGS.register("rope_halves")
class HalfRotaryEncoding(PositionEncoding):
    """The rotate-half layout over the first ``dims`` entries of a vector: entry ``i`` is paired with ``i + dims / 2`` and the pair
    ``(u, v)`` at position ``p`` becomes ``(u cos a - v sin a, v cos a + u sin a)`` with ``a = float32(p) * f_i``, ``f_i = base**(-2i / dims) /
    factor`` (taken in 64-bit on the host, then rounded once to 32-bit); entries beyond ``dims`` pass unchanged.  Mixers fold the rotation
    into their own kernels through :attr:`inv_freq`, :attr:`dims` and :attr:`halves`; :meth:`apply` turns whole heads in place."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.dims % 2 or spec.dims <= 0:
            raise ConfigError(f"rotary encoding over halves needs an even, positive number of dimensions, got {spec.dims}")
        if not float(spec.factor) > 0:
            raise ConfigError(f"rotary encoding: the scaling factor must be positive, got {spec.factor}")
        self.dims = spec.dims
        self.halves = True
        i = torch.arange(spec.dims // 2, dtype=torch.float64)
        freq = float(spec.base) ** (-2.0 * i / spec.dims) / float(spec.factor)
        if spec.bands is not None:
            freq = scale_by_wavelength(freq, *(float(b) for b in spec.bands))
        self.inv_freq = freq.to(torch.float32).to(device)

    def apply(self, q, k, positions):
        for x in (q, k):
            if x is None:
                continue
            T, heads, hd = x.shape
            flat = x.as_strided((T, heads * hd), (x.stride(0), 1))
            ops.head_norm_rotate(flat, heads, 0, hd, None, None, 0.0, positions, self.inv_freq, self.dims, True)
