"""Python face of the HIP kernels: one function per kernel entry point.

Every function takes ``torch`` tensors that already live on the GPU, checks shapes and
dtypes on the host (a kernel is never launched on operands it was not written for),
and launches on the current HIP stream.  Outputs are written into tensors the caller
allocated; nothing here allocates device memory except :func:`paged_attention`'s
split-merge scratch.  There is no CPU implementation: a missing library, or a tensor
that is not on the GPU, raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p

import torch

from . import build as _build


class KernelError(RuntimeError):
    pass


_libs: dict[str, ctypes.CDLL] = {}

_DT = {torch.float32: 0, torch.bfloat16: 1}

GATE_ACTIVATIONS = {"silu": 0, "relu": 1}      # the activation of a gated feed-forward's gate


def _lib(name: str) -> ctypes.CDLL:
    lib = _libs.get(name)
    if lib is None:
        try:
            path = _build.build(name)
        except _build.BuildError as exc:
            raise KernelError(f"kernel library {name!r} is not built and cannot be built here: {exc}") from exc
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as exc:
            raise KernelError(f"cannot load {path}: {exc}") from exc
        lib.tl_last_error.restype = ctypes.c_char_p
        _libs[name] = lib
        if name == "gemm" and torch.cuda.is_available():
            lib.tl_gemm_set_compute_units(c_int(compute_units()))
        if name == "recurrent" and torch.cuda.is_available():
            lib.tl_mlstm_set_compute_units(c_int(compute_units()))
    return lib


def load(names) -> None:
    """Build (in parallel, if needed) and load the named libraries ahead of use."""
    missing = [n for n in names if n not in _libs]
    stale = [n for n in missing if not _build.is_current(n)]
    if stale:
        _build.build_many(stale)
    for n in missing:
        _lib(n)


MEASURED_COMPUTE_UNITS = 256      # the MI355X on which the kernels' plans were fitted
_compute_units: int | None = None


def compute_units() -> int:
    """The compute units of the current GPU, read from the device once; the matrix-product library's planners are
    told the same number, and parts that deal work to the compute units (how many parts a request's keys are cut
    into) get it from here.  Without a GPU: the MI355X's 256, for which the plans were measured."""
    global _compute_units
    if _compute_units is None:
        if not torch.cuda.is_available():
            return MEASURED_COMPUTE_UNITS
        _compute_units = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
        if "gemm" in _libs:
            _libs["gemm"].tl_gemm_set_compute_units(c_int(_compute_units))
    return _compute_units


def loaded_libraries() -> list[str]:
    return sorted(str(_build.lib_path(n)) for n in _libs)


def _check(lib: ctypes.CDLL, code: int) -> None:
    if code != 0:
        raise KernelError(lib.tl_last_error().decode())


def _ptr(t: torch.Tensor | None) -> c_void_p:
    if t is None:
        return c_void_p(0)
    if not t.is_cuda:
        raise KernelError(f"kernel operand on {t.device}; the kernels run on the GPU only")
    return c_void_p(t.data_ptr())


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _dt(t: torch.Tensor, what: str) -> int:
    code = _DT.get(t.dtype)
    if code is None:
        raise KernelError(f"{what}: dtype {t.dtype} is not built (float32 and bfloat16 are)")
    return code


def _vec(t: torch.Tensor | None, n: int, what: str) -> int:
    """Check a weight/bias vector; returns 1 when it is float32, 0 for bfloat16."""
    if t is None:
        return 0
    if t.shape != (n,) or not t.is_contiguous():
        raise KernelError(f"{what}: expected a contiguous vector of {n}, got {tuple(t.shape)}")
    return 1 if _dt(t, what) == 0 else 0


def _i32(t: torch.Tensor | None, what: str, n: int | None = None) -> None:
    if t is None:
        return
    if t.dtype != torch.int32 or not t.is_contiguous() or (n is not None and t.numel() < n):
        raise KernelError(f"{what}: expected contiguous int32 of at least {n} elements, got {t.dtype} {tuple(t.shape)}")


# ----------------------------------------------------------------------------- ops

def embedding(token_ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0,
              positions: torch.Tensor | None = None, pos_table: torch.Tensor | None = None) -> None:
    """``out[t] = float(table[token_ids[t]]) * scale (+ float(pos_table[positions[t]]))``; ``out`` is the 32-bit residual ``[T, H]``, or
    ``[S, T, H]``: S copies of it."""
    T = token_ids.numel()
    V, H = table.shape
    _i32(token_ids, "embedding ids", T)
    copies = out.shape[0] if out.dim() == 3 else 1
    if out.shape[-2:] != (T, H) or out.dim() not in (2, 3) or out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous():
        raise KernelError(f"embedding: out must be contiguous float32 [{T}, {H}] or [copies, {T}, {H}], got {out.dtype} {tuple(out.shape)}")
    pos_rows = 0
    if pos_table is not None:
        _i32(positions, "embedding positions", T)
        if positions is None or pos_table.dim() != 2 or pos_table.shape[1] != H or not pos_table.is_contiguous():
            raise KernelError(f"embedding: a position table [rows, {H}] comes with the tokens' positions")
        pos_rows = pos_table.shape[0]
    lib = _lib("elementwise")
    _check(lib, lib.tl_embedding(_ptr(token_ids), _ptr(table), c_int(_dt(table, "embedding table")), _ptr(out),
                                 c_int(T), c_int(H), c_int(V), c_float(scale), _ptr(positions if pos_rows else None),
                                 _ptr(pos_table), c_int(_dt(pos_table, "position table") if pos_rows else 0), c_int(pos_rows),
                                 c_int(copies), _stream()))


def embedding_norm(token_ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float, weight: torch.Tensor, eps: float) -> None:
    """``out[t] = r / sqrt(mean(r^2) + eps) * weight`` with ``r = float(table[token_ids[t]]) * scale``: ``out`` is the 32-bit residual ``[T, H]``,
    ``weight`` float32 ``[H]``."""
    T = token_ids.numel()
    V, H = table.shape
    _i32(token_ids, "embedding ids", T)
    if out.shape != (T, H) or out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous():
        raise KernelError(f"embedding_norm: out must be contiguous float32 [{T}, {H}], got {out.dtype} {tuple(out.shape)}")
    if weight.dtype != torch.float32 or weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"embedding_norm: the norm's weight must be contiguous float32 [{H}]")
    lib = _lib("elementwise")
    _check(lib, lib.tl_embedding_norm(_ptr(token_ids), _ptr(table), c_int(_dt(table, "embedding table")), _ptr(out), c_int(T), c_int(H), c_int(V),
                                      c_float(scale), _ptr(weight), c_float(eps), _stream()))


def bigram_embedding(token_ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float, bigram: torch.Tensor, buckets: int,
                     mul_prev: int, mul_cur: int, token_req: torch.Tensor, req_indptr: torch.Tensor, positions: torch.Tensor,
                     slots: torch.Tensor, last_token: torch.Tensor) -> None:
    """``out[t] = float(table[token_ids[t]]) * scale + float(bigram[row(t)])`` with ``row(t) = (previous token * mul_prev + token * mul_cur) mod
    buckets``, or ``buckets`` for a token at position 0.  The token before a request's first token of the step is ``last_token[slot]`` (int32
    ``[slots, 1]``), where the step then leaves the request's last token.  ``out`` is the 32-bit residual ``[T, H]`` or ``[copies, T, H]``."""
    T = token_ids.numel()
    V, H = table.shape
    R = req_indptr.numel() - 1
    _i32(token_ids, "embedding ids", T)
    _i32(token_req, "token_req", T)
    _i32(positions, "positions", T)
    _i32(req_indptr, "req_indptr", R + 1)
    _i32(slots, "slots", R)
    copies = out.shape[0] if out.dim() == 3 else 1
    if out.shape[-2:] != (T, H) or out.dim() not in (2, 3) or out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous():
        raise KernelError(f"bigram_embedding: out must be contiguous float32 [{T}, {H}] or [copies, {T}, {H}], got {out.dtype} {tuple(out.shape)}")
    if bigram.shape != (buckets + 1, H) or bigram.dtype != table.dtype or not bigram.is_contiguous() or buckets <= 0:
        raise KernelError(f"bigram_embedding: the bigram table must be [{buckets + 1}, {H}] of {table.dtype}")
    if last_token.dtype != torch.int32 or not last_token.is_contiguous() or last_token.dim() != 2 or last_token.shape[1] != 1:
        raise KernelError("bigram_embedding: the requests' last tokens are int32 [slots, 1]")
    lib = _lib("elementwise")
    _check(lib, lib.tl_bigram_embedding(_ptr(token_ids), _ptr(table), _ptr(out), c_int(T), c_int(H), c_int(V), c_float(scale), _ptr(token_req),
                                        _ptr(req_indptr), c_int(R), _ptr(positions), _ptr(slots), _ptr(last_token), _ptr(bigram), c_int(buckets),
                                        ctypes.c_long(mul_prev), ctypes.c_long(mul_cur), c_int(copies), c_int(_dt(table, "embedding table")), _stream()))


def sandwich_norm(residual: torch.Tensor, pending: torch.Tensor | None, post_weight: torch.Tensor | None, post_eps: float,
                  extra: torch.Tensor | None, weight: torch.Tensor, eps: float, out: torch.Tensor, rows: torch.Tensor | None = None,
                  gain: float = 1.0) -> None:
    """``r = residual (+ extra) + (pending / sqrt(mean(pending^2) + post_eps) * post_weight, or pending as it is without a post_weight)``, written
    back to the float32 residual ``[T, H]`` unless ``rows`` selects rows; ``out = r / sqrt(mean(r^2) + eps) * weight * gain`` in its own dtype.
    ``pending``: ``[T, H]`` of ``out``'s dtype or float32 slabs ``[P, T, H]`` that are added up; ``extra``: float32 ``[T, H]``; ``weight`` and
    ``post_weight``: float32, one number or ``H`` of them."""
    T, H = residual.shape
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("sandwich_norm: the residual must be contiguous float32")
    n = T if rows is None else rows.numel()
    _i32(rows, "rows", n)
    if out.shape != (n, H) or not out.is_contiguous():
        raise KernelError(f"sandwich_norm: out must be contiguous [{n}, {H}], got {tuple(out.shape)}")
    parts = 0
    if pending is not None:
        if pending.dim() == 3:
            parts = pending.shape[0]
            if pending.dtype != torch.float32 or pending.shape[1:] != residual.shape or not pending.is_contiguous():
                raise KernelError(f"sandwich_norm: partial sums {pending.dtype} {tuple(pending.shape)} are not float32 [P, {T}, {H}]")
        elif pending.shape != residual.shape or pending.dtype != out.dtype or not pending.is_contiguous():
            raise KernelError(f"sandwich_norm: pending {pending.dtype} {tuple(pending.shape)} does not match the residual and the output's dtype")
    if extra is not None and (extra.dtype != torch.float32 or extra.shape != residual.shape or not extra.is_contiguous()):
        raise KernelError("sandwich_norm: the second addend must be contiguous float32 like the residual")
    for w, what in ((weight, "weight"), (post_weight, "post_weight")):
        if w is not None and (w.dtype != torch.float32 or not w.is_contiguous() or w.numel() not in (1, H)):
            raise KernelError(f"sandwich_norm: {what} must be float32, one number or {H}")
    lib = _lib("elementwise")
    _check(lib, lib.tl_sandwich_norm(_ptr(residual), _ptr(pending), c_int(parts), c_int(T), _ptr(post_weight if pending is not None else None),
                                     c_int(post_weight.numel() if post_weight is not None else 0), c_float(post_eps), _ptr(extra), _ptr(weight),
                                     c_int(weight.numel()), c_float(eps), c_float(gain), _ptr(out), _ptr(rows), c_int(n), c_int(H),
                                     c_int(_dt(out, "sandwich_norm")), _stream()))


def normed_sum(x: torch.Tensor, weights: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """``out[t] = sum_b x[b, t] / sqrt(mean(x[b, t]^2) + eps) * weights[b]``: ``x [B, T, H]`` and ``out [T, H]`` of one dtype, ``weights`` float32 ``[B, H]``."""
    B, T, H = x.shape
    if not x.is_contiguous() or out.shape != (T, H) or out.dtype != x.dtype or not out.is_contiguous() \
            or weights.dtype != torch.float32 or weights.shape != (B, H) or not weights.is_contiguous():
        raise KernelError("normed_sum: shapes or dtypes do not fit")
    lib = _lib("elementwise")
    _check(lib, lib.tl_normed_sum(_ptr(x), c_int(B), c_int(T), c_int(H), _ptr(weights), c_float(eps), _ptr(out), c_int(_dt(x, "normed_sum")), _stream()))


NORM_KINDS = {"rmsnorm": 0, "layernorm": 1}
MAX_STREAMS = 8


def streams_norm(x: torch.Tensor, pending: torch.Tensor | None, fold, read: torch.Tensor | None, kind: str, weight: torch.Tensor,
                 bias: torch.Tensor | None, eps: float, out: torch.Tensor, rows: torch.Tensor | None = None, gain: float = 1.0) -> None:
    """Over ``S`` copies of the residual, ``x`` float32 ``[S, T, H]``: the pending branch output ``p`` (``[T, H]`` of ``out``'s dtype, or
    float32 slabs ``[P, T, H]`` of partial sums) enters all copies at once, ``x_t <- sum_s mix[s, t] x_s + gate[t] p`` with ``fold = (mix
    [S, S], gate [S])`` float32 on the GPU (``fold=None``: ``x_t <- x_t + p``), then ``u = sum_s read[s] x_s`` (``read=None``: the sum of the
    copies) and ``out = norm(u) * gain``: ``kind`` ``rmsnorm`` (``u / sqrt(mean(u^2) + eps) * weight``) or ``layernorm`` (``(u - mean) /
    sqrt(mean((u - mean)^2) + eps) * weight + bias``).  Without ``rows`` the copies are updated in place; with ``rows`` (int32 source rows)
    only those rows are read and nothing is written back."""
    if x.dim() != 3 or x.dtype != torch.float32 or not x.is_contiguous() or not 1 <= x.shape[0] <= MAX_STREAMS:
        raise KernelError(f"streams_norm: the residual copies must be contiguous float32 [S <= {MAX_STREAMS}, T, H], got {x.dtype} {tuple(x.shape)}")
    S, T, H = x.shape
    n = T if rows is None else rows.numel()
    if out.shape != (n, H) or not out.is_contiguous():
        raise KernelError(f"streams_norm: out must be contiguous [{n}, {H}], got {tuple(out.shape)}")
    if kind not in NORM_KINDS or (kind == "layernorm") != (bias is not None):
        raise KernelError(f"streams_norm: norm {kind!r} with{'out' if bias is None else ''} a bias is not built")
    parts = 0
    if pending is not None:
        if pending.dim() == 3:
            parts = pending.shape[0]
            if pending.dtype != torch.float32 or pending.shape[1:] != (T, H) or not pending.is_contiguous():
                raise KernelError(f"streams_norm: partial sums {pending.dtype} {tuple(pending.shape)} are not float32 [P, {T}, {H}]")
        elif pending.shape != (T, H) or pending.dtype != out.dtype or not pending.is_contiguous():
            raise KernelError(f"streams_norm: pending {pending.dtype} {tuple(pending.shape)} does not match [{T}, {H}] of {out.dtype}")
    mix = gate = None
    if fold is not None:
        mix, gate = fold
        if pending is None or mix.shape != (S, S) or gate.shape != (S,) or mix.dtype != torch.float32 or gate.dtype != torch.float32 \
                or not mix.is_contiguous() or not gate.is_contiguous():
            raise KernelError(f"streams_norm: a fold is float32 (mix [{S}, {S}], gate [{S}]) and comes with a pending output")
    if read is not None and (read.shape != (S,) or read.dtype != torch.float32 or not read.is_contiguous()):
        raise KernelError(f"streams_norm: read must be contiguous float32 [{S}]")
    _i32(rows, "streams_norm rows")
    wf = _vec(weight, H, "streams_norm weight")
    bf = _vec(bias, H, "streams_norm bias")
    lib = _lib("elementwise")
    _check(lib, lib.tl_streams_norm(_ptr(x), c_int(S), c_int(T), c_int(H), _ptr(pending), c_int(parts), _ptr(mix), _ptr(gate), _ptr(read),
                                    c_int(NORM_KINDS[kind]), _ptr(weight), c_int(wf), _ptr(bias), c_int(bf), c_float(eps), c_float(gain),
                                    _ptr(out), _ptr(rows), c_int(n), c_int(_dt(out, "streams_norm")), _stream()))


def add_rmsnorm(residual: torch.Tensor, pending: torch.Tensor | None, weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: torch.Tensor | None = None, gain: float = 1.0) -> None:
    """``r = residual (+ pending)``; ``out = r * (rsqrt(mean(r^2) + eps) * gain) * weight``.

    ``pending`` is ``[T, H]`` of the activation dtype, or float32 ``[P, T, H]``: slabs of partial
    sums (from :func:`linear_partials`) that are added up here.  Without ``rows`` every row is
    processed and ``r`` is written back into ``residual``; with ``rows`` (int32 source rows) only
    those are read and ``residual`` is untouched."""
    T, H = residual.shape
    n = T if rows is None else rows.numel()
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("add_rmsnorm: the residual must be contiguous float32")
    parts = 0
    if pending is not None:
        if pending.dim() == 3:
            parts = pending.shape[0]
            if pending.dtype != torch.float32 or pending.shape[1:] != residual.shape or not pending.is_contiguous():
                raise KernelError(f"add_rmsnorm: partial sums {pending.dtype} {tuple(pending.shape)} are not float32 [P, {T}, {H}]")
        elif pending.shape != residual.shape or pending.dtype != out.dtype or not pending.is_contiguous():
            raise KernelError(f"add_rmsnorm: pending {pending.dtype} {tuple(pending.shape)} does not match residual/out")
    if out.shape != (n, H) or not out.is_contiguous():
        raise KernelError(f"add_rmsnorm: out must be contiguous [{n}, {H}], got {tuple(out.shape)}")
    _i32(rows, "add_rmsnorm rows")
    wf = _vec(weight, H, "add_rmsnorm weight")
    lib = _lib("elementwise")
    _check(lib, lib.tl_add_rmsnorm(_ptr(residual), _ptr(pending), c_int(parts), c_int(T), _ptr(weight), c_int(wf),
                                   c_float(eps), c_float(gain), _ptr(out), _ptr(rows), c_int(n), c_int(H),
                                   c_int(_dt(out, "add_rmsnorm")), _stream()))


def linear_partials_pay(M: int, N: int, K: int) -> bool:
    """Whether a bfloat16 product whose consumer can add slabs up should come from
    :func:`linear_partials` (K a multiple of 64): up to 64 rows when its 64 x 64 output tiles are
    too few to fill the GPU (from 2 rows on; one row against a matrix of more than 4096 rows); with more rows
    when the library's estimate finds a tile shape with K split 2-8 ways faster than the best
    whole product, slabs included."""
    return bool(_lib("gemm").tl_gemm_partials_pay(c_int(M), c_int(N), c_int(K)))


def linear_partials(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x @ weight.T`` as float32 slabs ``[P, M, N]`` of partial sums over P ranges of K (bfloat16
    operands, K a multiple of 8; more than 64 rows need a multiple of 64): for a product with too
    few output tiles to fill the GPU, where splitting K over work-groups does.  The slabs are
    summed by :func:`add_rmsnorm` (or by :func:`rope_cache_write`); P may be 1."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.shape[1] != K or not weight.is_contiguous() or x.stride(1) != 1:
        raise KernelError("linear_partials: bfloat16 operands and fitting shapes only")
    lib = _lib("gemm")
    out = torch.empty((lib.tl_gemm_partials_parts(c_int(M), c_int(N), c_int(K)), M, N), dtype=torch.float32, device=x.device)
    parts = c_int(0)
    _check(lib, lib.tl_gemm_partials(_ptr(x), _ptr(weight), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(x.stride(0)),
                                     ctypes.byref(parts), _stream()))
    return out[: parts.value]


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
           general: bool = False) -> None:
    """``out = x @ weight.T (+ bias)``; ``x [M, K]`` (rows may be strided), ``weight [N, K]``
    contiguous and of ``x``'s dtype, ``out [M, N]`` of that dtype or float32.  The library picks
    the kernel for the shape; ``general=True`` forces the general 32-bit-arithmetic kernel."""
    M, K = x.shape
    N, K2 = weight.shape
    if K2 != K or out.shape != (M, N):
        raise KernelError(f"linear: shapes x{tuple(x.shape)} w{tuple(weight.shape)} out{tuple(out.shape)} do not fit")
    if x.dtype != weight.dtype or x.stride(1) != 1 or out.stride(1) != 1 or not weight.is_contiguous():
        raise KernelError("linear: x and weight must share a dtype, weight contiguous, unit stride on the last axis")
    if out.dtype not in (x.dtype, torch.float32):
        raise KernelError(f"linear: out dtype {out.dtype} must be {x.dtype} or float32")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    entry = lib.tl_gemm_general if general else lib.tl_gemm
    _check(lib, entry(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N), c_int(K),
                                    c_int(x.stride(0)), c_int(out.stride(0)), c_int(_dt(x, "linear")),
                                    c_int(1 if out.dtype == torch.float32 else 0), _stream()))


def linear_f32_variant(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor, matrix_cores) -> None:
    """One named kernel of the 32-bit products (for tests and tuning): 0 / False the general tile kernel (``v_fma_f32``),
    1 / True the matrix-core tile kernel (``v_mfma_f32_32x32x2_f32``, K a multiple of 4), 2 and 3 the kernels for up to 16
    rows on multiply-adds and on the matrix cores (``v_mfma_f32_16x16x4_f32``); all multiply and add in true 32-bit."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.float32 or weight.dtype != torch.float32 or out.dtype != torch.float32 or out.shape != (M, N) \
            or weight.shape[1] != K or not weight.is_contiguous() or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("linear_f32_variant: float32 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_f32_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N), c_int(K),
                                        c_int(x.stride(0)), c_int(out.stride(0)), c_int(int(matrix_cores)), _stream()))


def linear_few_rows_variant(x, weight, bias, out, strips_per_wave: int, waves_along_k: int, rows_per_strip: int = 0) -> None:
    """One named instance of the few-rows matrix-core kernel (for tests and tuning); ``rows_per_strip``: the weight
    rows a work-group takes, up to 16 ``strips_per_wave`` (0: exactly that many)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.shape != (M, N) or not weight.is_contiguous():
        raise KernelError("linear_few_rows_variant: bfloat16 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_skinny_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N),
                                           c_int(K), c_int(x.stride(0)), c_int(out.stride(0)),
                                           c_int(1 if out.dtype == torch.float32 else 0), c_int(strips_per_wave),
                                           c_int(waves_along_k), c_int(rows_per_strip), _stream()))


def linear_many_rows_variant(x, weight, bias, out, tile_m: int, tile_n: int, slab: int = 32) -> None:
    """One named tile shape of the many-rows matrix-core kernel (for tests and tuning)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.shape != (M, N) or not weight.is_contiguous():
        raise KernelError("linear_many_rows_variant: bfloat16 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_tile_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N),
                                         c_int(K), c_int(x.stride(0)), c_int(out.stride(0)),
                                         c_int(1 if out.dtype == torch.float32 else 0), c_int(tile_m), c_int(tile_n), c_int(slab), _stream()))


DIRECT_TILES = ((64, 64), (64, 128), (64, 192), (64, 256), (64, 320), (128, 128), (128, 192), (128, 256), (256, 128), (192, 256), (256, 192), (256, 256), (256, 160))


def linear_direct_variant(x, weight, bias, out, tile_m: int, tile_n: int) -> None:
    """One named tile shape of the many-rows kernel that fetches its operands straight into
    shared memory (K a multiple of 64; for tests and tuning)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.shape != (M, N) or not weight.is_contiguous():
        raise KernelError("linear_direct_variant: bfloat16 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_direct_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N),
                                           c_int(K), c_int(x.stride(0)), c_int(out.stride(0)),
                                           c_int(1 if out.dtype == torch.float32 else 0), c_int(tile_m), c_int(tile_n), _stream()))


def linear_direct_split_variant(x, weight, tile_m: int, tile_n: int, parts: int, stages: int = 0) -> torch.Tensor:
    """One named tile shape of the direct-load kernel with K split into ``parts``: float32 slabs
    ``[parts, M, N]`` (K a multiple of 64; ``stages=4`` with 128 x 128: the four-slab instance; for
    tests and tuning)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.shape[1] != K or not weight.is_contiguous() or x.stride(1) != 1:
        raise KernelError("linear_direct_split_variant: bfloat16 operands and fitting shapes only")
    out = torch.empty((parts, M, N), dtype=torch.float32, device=x.device)
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_direct_split_variant(_ptr(x), _ptr(weight), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(x.stride(0)),
                                                 c_int(tile_m), c_int(tile_n), c_int(parts), c_int(stages), _stream()))
    return out


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The layout :func:`linear_swiglu` wants: blocks of 64 rows, 32 rows of ``gate`` then the
    32 rows of ``up`` with the same indices; the last block is padded with zero rows."""
    I, K = gate.shape
    blocks = -(-I // 32)
    g = torch.zeros((blocks * 32, K), dtype=gate.dtype, device=gate.device)
    u = torch.zeros_like(g)
    g[:I] = gate
    u[:I] = up
    return torch.stack((g.view(blocks, 32, K), u.view(blocks, 32, K)), dim=1).reshape(blocks * 64, K).contiguous()


def linear_swiglu(x: torch.Tensor, gate_up: torch.Tensor, out: torch.Tensor, activation: str = "silu") -> None:
    """``out = act(x @ gate.T) * (x @ up.T)`` on the matrix cores with the gate applied to the
    32-bit accumulators (``activation``: ``silu`` or ``relu``); ``gate_up`` from :func:`interleave_gate_up`,
    bfloat16 only, ``x [M, K]`` with K a multiple of 8."""
    M, K = x.shape
    I = out.shape[1]
    if x.dtype != torch.bfloat16 or gate_up.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("linear_swiglu: bfloat16 only")
    if gate_up.shape != (-(-I // 32) * 64, K) or out.shape[0] != M or not gate_up.is_contiguous() or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError(f"linear_swiglu: shapes x{tuple(x.shape)} w{tuple(gate_up.shape)} out{tuple(out.shape)} do not fit")
    if activation not in GATE_ACTIVATIONS:
        raise KernelError(f"linear_swiglu: the gate's activation is one of {', '.join(GATE_ACTIVATIONS)}, not {activation!r}")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_swiglu(_ptr(x), _ptr(gate_up), _ptr(out), c_int(M), c_int(I), c_int(K),
                                   c_int(x.stride(0)), c_int(out.stride(0)), c_int(GATE_ACTIVATIONS[activation]), _stream()))


def linear_swiglu_direct_variant(x: torch.Tensor, gate_up: torch.Tensor, out: torch.Tensor, tile_m: int, tile_n: int) -> None:
    """:func:`linear_swiglu` on one named tile shape of the kernel that fetches its operands straight into shared
    memory (K a multiple of 64; for tests and tuning)."""
    M, K = x.shape
    I = out.shape[1]
    if x.dtype != torch.bfloat16 or gate_up.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 \
            or gate_up.shape != (-(-I // 32) * 64, K) or out.shape[0] != M or not gate_up.is_contiguous() or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("linear_swiglu_direct_variant: bfloat16 operands and fitting shapes only")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_swiglu_direct_variant(_ptr(x), _ptr(gate_up), _ptr(out), c_int(M), c_int(I), c_int(K),
                                                  c_int(x.stride(0)), c_int(out.stride(0)), c_int(tile_m), c_int(tile_n), _stream()))


def rope_cache_write(qkv: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int, rot_heads: int,
                     positions: torch.Tensor, inv_freq: torch.Tensor | None,
                     token_req: torch.Tensor | None = None, block_table: torch.Tensor | None = None,
                     k_plane: torch.Tensor | None = None, v_plane: torch.Tensor | None = None,
                     page_size: int = 0, pairs: bool = False, parts: torch.Tensor | None = None,
                     bias: torch.Tensor | None = None) -> None:
    """Rotate the first ``rot_heads`` heads of each row of ``qkv [T, >= (q+2kv)*hd]`` in
    place by the token's position (``inv_freq`` float32 ``[hd/2]``; ``None``: no rotation;
    ``pairs``: frequency j turns the neighbours ``(2j, 2j+1)`` instead of ``(j, j+hd/2)``)
    and, when planes are given, store rotated k and raw v of every token in its page:
    ``k_plane [pages, kv_heads, page, hd]``, ``v_plane [pages, kv_heads, hd, page]`` (values
    lie transposed inside a page).  With ``parts`` (float32 ``[P, T, width]``, slabs of partial
    sums of the projection, and its ``bias``) the rows are the sums of the slabs instead of what
    ``qkv`` holds: the queries are written to ``qkv``, keys and values to their pages only."""
    T = qkv.shape[0]
    if qkv.stride(1) != 1:
        raise KernelError("rope_cache_write: qkv needs unit stride on the last axis")
    _i32(positions, "positions", T)
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2):
        raise KernelError("rope_cache_write: inv_freq must be float32 [head_dim/2]")
    bt_stride = 0
    if k_plane is not None:
        _i32(token_req, "token_req", T)
        _i32(block_table, "block_table")
        bt_stride = block_table.stride(0)
        _check_planes("rope_cache_write", k_plane, v_plane, qkv.dtype, kv_heads, page_size, head_dim)
    num_parts = part_stride = parts_ld = bf = 0
    if parts is not None:
        if parts.dtype != torch.float32 or parts.dim() != 3 or parts.shape[1] != T or not parts.is_contiguous():
            raise KernelError("rope_cache_write: parts must be contiguous float32 [P, T, width]")
        num_parts, part_stride, parts_ld = parts.shape[0], parts.stride(0), parts.shape[2]
        bf = _vec(bias, parts_ld, "projection bias")
    elif bias is not None:
        raise KernelError("rope_cache_write: a bias comes with slabs of partial sums only")
    lib = _lib("elementwise")
    _check(lib, lib.tl_rope_cache_write(_ptr(qkv), c_int(qkv.stride(0)), c_int(T), c_int(q_heads), c_int(kv_heads),
                                        c_int(head_dim), c_int(rot_heads), _ptr(positions), _ptr(inv_freq), _ptr(token_req),
                                        _ptr(block_table), c_int(bt_stride), _ptr(k_plane), _ptr(v_plane), c_int(page_size),
                                        c_int(1 if pairs else 0), c_int(_dt(qkv, "rope_cache_write")),
                                        _ptr(parts), c_int(num_parts), ctypes.c_size_t(part_stride), c_int(parts_ld),
                                        _ptr(bias), c_int(bf), _stream()))


def pair_layout_rows(num_heads: int, head_dim: int) -> torch.Tensor:
    """Row order that turns a projection into the pair layout: within every head the rows
    ``j`` and ``j + head_dim/2`` (the two that frequency ``j`` of the split-half rotary encoding
    turns) become the neighbours ``2j`` and ``2j + 1``.  Scores are sums over the head's
    dimensions, so they do not change when queries and keys are reordered alike."""
    half = head_dim // 2
    within = torch.stack((torch.arange(half), torch.arange(half) + half), dim=1).reshape(-1)
    return (torch.arange(num_heads)[:, None] * head_dim + within[None, :]).reshape(-1)


def linear_rope_cache_write(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
                            q_heads: int, kv_heads: int, head_dim: int, positions: torch.Tensor, inv_freq: torch.Tensor,
                            token_req: torch.Tensor | None = None, block_table: torch.Tensor | None = None,
                            k_plane: torch.Tensor | None = None, v_plane: torch.Tensor | None = None,
                            page_size: int = 0) -> bool:
    """The query/key/value projection of a decode step with the rotation and the cache write in
    its epilogue: ``out[:, :q_heads*hd]`` gets the rotated queries; with planes given, ``weight``
    has ``(q_heads + 2 kv_heads) * hd`` rows and rotated keys and values go to their pages.  The
    rows of the query and key heads are in the pair layout (:func:`pair_layout_rows`).  Built
    for bfloat16 and up to 16 rows; returns ``False`` without doing anything for other shapes."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or M > 16 or M == 0 or head_dim % 4:
        return False
    if x.stride(1) != 1 or out.stride(1) != 1 or not weight.is_contiguous() or weight.shape[1] != K or out.shape[0] != M:
        raise KernelError("linear_rope_cache_write: shapes or strides do not fit")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2:
        raise KernelError("linear_rope_cache_write: inv_freq must be float32 [head_dim/2]")
    _i32(positions, "positions", M)
    bt_stride = 0
    if k_plane is not None:
        _i32(token_req, "token_req", M)
        _i32(block_table, "block_table")
        bt_stride = block_table.stride(0)
        _check_planes("linear_rope_cache_write", k_plane, v_plane, x.dtype, kv_heads, page_size, head_dim)
    if N != (q_heads + (2 * kv_heads if k_plane is not None else 0)) * head_dim or out.shape[1] < q_heads * head_dim:
        raise KernelError("linear_rope_cache_write: the projection's rows do not match the heads")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    rc = lib.tl_gemm_rope(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N), c_int(K),
                          c_int(x.stride(0)), c_int(out.stride(0)), _ptr(positions), _ptr(inv_freq), _ptr(token_req),
                          _ptr(block_table), c_int(bt_stride), _ptr(k_plane), _ptr(v_plane), c_int(page_size),
                          c_int(q_heads), c_int(kv_heads), c_int(head_dim), _stream())
    if rc == 100:          # not built for this shape
        return False
    _check(lib, rc)
    return True


def _norm_args(what: str, residual: torch.Tensor, pending: torch.Tensor | None, weight: torch.Tensor, eps: float,
               residual_out: torch.Tensor):
    """The arguments that describe ``norm(residual + pending)`` of one row to a kernel that makes it itself."""
    H = residual.shape[-1]
    if residual.dtype != torch.float32 or residual_out.dtype != torch.float32 or residual.numel() != H or residual_out.numel() != H \
            or not residual.is_contiguous() or not residual_out.is_contiguous():
        raise KernelError(f"{what}: the residual and its successor must be one contiguous float32 row")
    parts = part_stride = 0
    if pending is not None:
        if pending.dim() == 3:
            if pending.dtype != torch.float32 or pending.shape[1:] != (1, H) or not pending.is_contiguous():
                raise KernelError(f"{what}: partial sums {pending.dtype} {tuple(pending.shape)} are not float32 [P, 1, {H}]")
            parts, part_stride = pending.shape[0], pending.stride(0)
        elif pending.dtype != torch.bfloat16 or pending.numel() != H or not pending.is_contiguous():
            raise KernelError(f"{what}: pending {pending.dtype} {tuple(pending.shape)} is not a bfloat16 row of {H}")
    wf = _vec(weight, H, f"{what} norm weight")
    return (_ptr(residual), _ptr(residual_out), _ptr(pending), c_int(parts), ctypes.c_long(part_stride), _ptr(weight), c_int(wf),
            c_float(eps))


def linear_rope_cache_write_normed(residual: torch.Tensor, pending: torch.Tensor | None, norm_weight: torch.Tensor, eps: float,
                                   residual_out: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None,
                                   out: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int, positions: torch.Tensor,
                                   inv_freq: torch.Tensor, token_req: torch.Tensor | None = None,
                                   block_table: torch.Tensor | None = None, k_plane: torch.Tensor | None = None,
                                   v_plane: torch.Tensor | None = None, page_size: int = 0) -> bool:
    """:func:`linear_rope_cache_write` for ONE row whose input is ``norm(residual + pending)`` (see
    :func:`add_rmsnorm`), made inside the kernel: ``residual [1, K]`` float32, ``pending`` bfloat16
    ``[1, K]``, float32 slabs ``[P, 1, K]`` or ``None``; the sum goes to ``residual_out`` (another
    tensor than ``residual``).  Returns ``False`` without doing anything for shapes it is not built for."""
    K = residual.shape[-1]
    N = weight.shape[0]
    if weight.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or residual.shape[0] != 1 or head_dim % 4:
        return False
    if out.stride(1) != 1 or not weight.is_contiguous() or weight.shape[1] != K or out.shape[0] != 1:
        raise KernelError("linear_rope_cache_write_normed: shapes or strides do not fit")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2:
        raise KernelError("linear_rope_cache_write_normed: inv_freq must be float32 [head_dim/2]")
    _i32(positions, "positions", 1)
    bt_stride = 0
    if k_plane is not None:
        _i32(token_req, "token_req", 1)
        _i32(block_table, "block_table")
        bt_stride = block_table.stride(0)
        _check_planes("linear_rope_cache_write_normed", k_plane, v_plane, torch.bfloat16, kv_heads, page_size, head_dim)
    if N != (q_heads + (2 * kv_heads if k_plane is not None else 0)) * head_dim or out.shape[1] < q_heads * head_dim:
        raise KernelError("linear_rope_cache_write_normed: the projection's rows do not match the heads")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    rc = lib.tl_gemm_rope_normed(*_norm_args("linear_rope_cache_write_normed", residual, pending, norm_weight, eps, residual_out),
                                 _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(N), c_int(K), c_int(out.stride(0)),
                                 _ptr(positions), _ptr(inv_freq), _ptr(token_req), _ptr(block_table), c_int(bt_stride),
                                 _ptr(k_plane), _ptr(v_plane), c_int(page_size), c_int(q_heads), c_int(kv_heads),
                                 c_int(head_dim), _stream())
    if rc == 100:          # not built for this shape
        return False
    _check(lib, rc)
    return True


def linear_swiglu_normed(residual: torch.Tensor, pending: torch.Tensor | None, norm_weight: torch.Tensor, eps: float,
                         residual_out: torch.Tensor, gate_up: torch.Tensor, out: torch.Tensor) -> bool:
    """:func:`linear_swiglu` for ONE row whose input is ``norm(residual + pending)``, made inside the
    kernel (see :func:`linear_rope_cache_write_normed`).  Returns ``False`` without doing anything
    for shapes it is not built for."""
    K = residual.shape[-1]
    I = out.shape[1]
    if gate_up.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or residual.shape[0] != 1:
        return False
    if gate_up.shape != (-(-I // 32) * 64, K) or out.shape[0] != 1 or not gate_up.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"linear_swiglu_normed: shapes w{tuple(gate_up.shape)} out{tuple(out.shape)} do not fit a row of {K}")
    lib = _lib("gemm")
    rc = lib.tl_gemm_swiglu_normed(*_norm_args("linear_swiglu_normed", residual, pending, norm_weight, eps, residual_out),
                                   _ptr(gate_up), _ptr(out), c_int(I), c_int(K), _stream())
    if rc == 100:
        return False
    _check(lib, rc)
    return True


def _check_planes(what, k_plane, v_plane, dtype, kv_heads, page_size, head_dim) -> None:
    for p, shape in ((k_plane, (kv_heads, page_size, head_dim)), (v_plane, (kv_heads, head_dim, page_size))):
        if p.dtype != dtype or p.dim() != 4 or tuple(p.shape[1:]) != shape or not p.is_contiguous():
            raise KernelError(f"{what}: plane {tuple(p.shape)} {p.dtype} is not [pages, {', '.join(map(str, shape))}] {dtype}")
    if k_plane.shape[0] != v_plane.shape[0]:
        raise KernelError(f"{what}: key and value planes differ in their number of pages")


ATTENTION_ROWS = 16   # rows (tokens x heads of one group) a work-group owns


def attention_library(head_dim: int) -> str:
    """The attention library that serves ``head_dim``: one is compiled per multiple of 16 and takes the seven even
    sizes below it too (its general kernel pads them inside; the matrix-core kernels are for the multiple itself)."""
    if head_dim % 2 or not 2 <= head_dim <= 256:
        raise KernelError(f"attention kernels take even head sizes from 2 to 256, not {head_dim}")
    return f"attention_hd{-(-head_dim // 16) * 16}"

SPLIT_SCRATCH_BYTES = 256 << 20     # most memory the parts of a split attention may take before they are merged


def attention_tile_tokens(num_heads: int, num_kv_heads: int) -> int:
    """New tokens of one request that share a tile, given the group size."""
    group = num_heads // num_kv_heads
    return max(1, ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def paged_attention(q: torch.Tensor, out: torch.Tensor, k_plane: torch.Tensor, v_plane: torch.Tensor,
                    block_table: torch.Tensor, req_indptr: torch.Tensor, ctx_lens: torch.Tensor,
                    tile_req: torch.Tensor, tile_tok0: torch.Tensor, num_tiles: int, tile_tokens: int,
                    num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int,
                    scale: float, splits: int = 1, general: bool = False, merge_tokens=None, waves: int = 4) -> None:
    """Causal attention of the step's tokens over their requests' cached keys.

    ``q [T, >= heads*hd]`` (row-strided view), ``out [T, heads*hd]``, ``k_plane [pages,
    kv_heads, page, hd]``, ``v_plane [pages, kv_heads, hd, page]``, ``block_table [R,
    max_blocks]`` int32; the new token ``i`` of request ``r`` sits at position
    ``ctx_lens[r] + i``.  ``window`` 0: all keys.  bfloat16 with pages of a multiple of 4
    tokens runs on the matrix cores; ``general=True`` forces the general kernel.  When the
    tiles cover only some of the step's tokens and ``splits > 1``, ``merge_tokens = (int32
    indices of those tokens, their number)`` keeps the merge of the parts to their rows.
    ``tile_req = tile_tok0 = None``: every request brings exactly one token, token ``i`` that of
    request ``i`` (a decode step); the kernel then looks nothing up before it asks for the
    request's length, block table and query.  ``waves``: 4 or 8 to a work-group of the matrix-core kernel
    (they deal a part's keys among themselves; the other kernels take no notice)."""
    T = q.shape[0]
    if waves not in (4, 8):
        raise KernelError("paged_attention: work-groups of 4 or 8 waves")
    if q.stride(1) != 1 or out.shape != (T, num_heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("paged_attention: q/out shapes or dtypes do not fit")
    _check_planes("paged_attention", k_plane, v_plane, q.dtype, num_kv_heads, page_size, head_dim)
    for name, t in (("block_table", block_table), ("ctx_lens", ctx_lens)):
        _i32(t, name)
    if tile_req is None:        # every request brings one token: tile i is the token of request i
        if tile_tok0 is not None or num_tiles != T or ctx_lens.numel() < T or block_table.shape[0] < T:
            raise KernelError("paged_attention: without a tile list every request brings exactly one token")
        req_indptr = None
    else:
        for name, t in (("req_indptr", req_indptr), ("tile_req", tile_req), ("tile_tok0", tile_tok0)):
            _i32(t, name)
        if tile_req.numel() < num_tiles or tile_tok0.numel() < num_tiles:
            raise KernelError("paged_attention: tile arrays shorter than the number of tiles")
    if merge_tokens is not None:
        _i32(merge_tokens[0], "merge_tokens", merge_tokens[1])
    part_o = part_ml = None
    # the parts are indexed by the step's tokens: a few decode tokens beside a long portion would make the
    # scratch large for nothing, so the split count gives way (fewer parts: the same result up to rounding)
    padded = -(-head_dim // 16) * 16            # the parts are as wide as the library's head size
    splits = max(1, min(splits, SPLIT_SCRATCH_BYTES // (T * num_heads * (padded + 2) * 4)))
    if splits > 1:
        part_o = torch.empty((T * num_heads * splits, padded), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * splits, 2), dtype=torch.float32, device=q.device)
    lib = _lib(attention_library(head_dim))
    _check(lib, lib.tl_paged_attention(_ptr(q), c_int(q.stride(0)), _ptr(out), _ptr(k_plane), _ptr(v_plane),
                                       _ptr(block_table), c_int(block_table.stride(0)), _ptr(req_indptr), _ptr(ctx_lens),
                                       _ptr(tile_req), _ptr(tile_tok0), c_int(num_tiles), c_int(T), c_int(tile_tokens),
                                       c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_int(page_size), c_int(window),
                                       c_float(scale), c_int(splits), _ptr(part_o), _ptr(part_ml),
                                       _ptr(merge_tokens[0]) if merge_tokens is not None else c_void_p(None),
                                       c_int(merge_tokens[1] if merge_tokens is not None else 0),
                                       c_int(_dt(q, "paged_attention")), c_int(1 if general else 0), c_int(waves), _stream()))


PREFILL_ATTENTION_ROWS = 64      # rows a work-group of the prompt-portion kernel owns
PREFILL_ATTENTION_MAX_HEAD_DIM = 128


def prefill_attention_tile_tokens(num_heads: int, num_kv_heads: int) -> int:
    group = num_heads // num_kv_heads
    return max(1, PREFILL_ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def paged_attention_prefill(q: torch.Tensor, out: torch.Tensor, k_plane: torch.Tensor, v_plane: torch.Tensor,
                            block_table: torch.Tensor, req_indptr: torch.Tensor, ctx_lens: torch.Tensor,
                            tile_req: torch.Tensor, tile_tok0: torch.Tensor, num_tiles: int, tile_tokens: int,
                            num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int,
                            scale: float) -> None:
    """The attention of :func:`paged_attention` for prompt portions: bfloat16, head sizes up
    to 128, pages of a multiple of 4 tokens; tiles of ``tile_tokens`` tokens (64 rows) whose keys
    and values pass through shared memory once per work-group.  Writes the rows of its tiles only."""
    T = q.shape[0]
    if q.dtype != torch.bfloat16 or head_dim > PREFILL_ATTENTION_MAX_HEAD_DIM or head_dim % 16 or page_size % 4:
        raise KernelError("paged_attention_prefill: bfloat16, head sizes that are multiples of 16 up to 128 and pages of a multiple of 4 tokens only")
    if q.stride(1) != 1 or out.shape != (T, num_heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("paged_attention_prefill: q/out shapes or dtypes do not fit")
    _check_planes("paged_attention_prefill", k_plane, v_plane, q.dtype, num_kv_heads, page_size, head_dim)
    for name, t in (("block_table", block_table), ("req_indptr", req_indptr), ("ctx_lens", ctx_lens),
                    ("tile_req", tile_req), ("tile_tok0", tile_tok0)):
        _i32(t, name)
    if tile_req.numel() < num_tiles or tile_tok0.numel() < num_tiles:
        raise KernelError("paged_attention_prefill: tile arrays shorter than the number of tiles")
    lib = _lib(f"attention_hd{head_dim}")
    _check(lib, lib.tl_paged_attention_prefill(_ptr(q), c_int(q.stride(0)), _ptr(out), _ptr(k_plane), _ptr(v_plane),
                                               _ptr(block_table), c_int(block_table.stride(0)), _ptr(req_indptr),
                                               _ptr(ctx_lens), _ptr(tile_req), _ptr(tile_tok0), c_int(num_tiles),
                                               c_int(tile_tokens), c_int(num_heads), c_int(num_kv_heads), c_int(page_size),
                                               c_int(window), c_float(scale), _stream()))


PROMPT_ATTENTION_ROWS = 128      # rows a work-group of the 128-row prompt kernel owns
PROMPT_ATTENTION_HEAD_DIMS = (64, 128)


PROMPT_ATTENTION_MAX_BLOCKS = 2048     # pages of a sequence whose block-table entries a work-group keeps in shared memory


def prompt_attention_fits(dtype: torch.dtype, head_dim: int, page_size: int, max_blocks: int = 0, scale: float = 1.0) -> bool:
    """Whether :func:`paged_attention_prompt` is built for this case: bfloat16, head size 64 or
    128, pages of 8, 16, 32, ... tokens, sequences of up to 2048 pages (``max_blocks``: the
    longest sequence of the step in pages), a positive factor on the scores."""
    return (dtype == torch.bfloat16 and head_dim in PROMPT_ATTENTION_HEAD_DIMS and page_size >= 8
            and page_size & (page_size - 1) == 0 and max_blocks <= PROMPT_ATTENTION_MAX_BLOCKS and scale > 0)


def prompt_attention_tile_tokens(num_heads: int, num_kv_heads: int) -> int:
    group = num_heads // num_kv_heads
    return max(1, PROMPT_ATTENTION_ROWS // min(group, PROMPT_ATTENTION_ROWS))


def paged_attention_prompt(q: torch.Tensor, out: torch.Tensor, k_plane: torch.Tensor, v_plane: torch.Tensor,
                           block_table: torch.Tensor, req_indptr: torch.Tensor, ctx_lens: torch.Tensor,
                           tile_req: torch.Tensor, tile_tok0: torch.Tensor, num_tiles: int, tile_tokens: int,
                           num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int,
                           scale: float, max_total_len: int | None = None, splits: int = 1,
                           merge_tokens: tuple[torch.Tensor, int] | None = None) -> None:
    """The attention of :func:`paged_attention` for prompt portions in tiles of 128 rows
    (``tile_tokens`` tokens times the heads of a group): bfloat16, head size 64 or 128, pages
    of a multiple of 8 tokens; keys and values go straight into shared memory once per
    work-group.  Writes the rows of its tiles only.  ``max_total_len``: the longest sequence of the
    step (cached + new tokens; default: what the block table could hold).  ``splits`` > 1 deals
    every tile's keys to that many work-groups (for few tiles against long sequences) and merges
    their parts for the tokens listed in ``merge_tokens`` (int32 indices, how many): the tokens
    of the tiles' requests."""
    T = q.shape[0]
    used_blocks = block_table.shape[1] if max_total_len is None else min(block_table.shape[1], -(-max_total_len // page_size))
    if not prompt_attention_fits(q.dtype, head_dim, page_size, used_blocks):
        raise KernelError("paged_attention_prompt: bfloat16, head size 64 or 128, pages of 8, 16, 32, ... tokens and "
                          f"sequences of up to {PROMPT_ATTENTION_MAX_BLOCKS} pages only")
    if q.stride(1) != 1 or out.shape != (T, num_heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("paged_attention_prompt: q/out shapes or dtypes do not fit")
    _check_planes("paged_attention_prompt", k_plane, v_plane, q.dtype, num_kv_heads, page_size, head_dim)
    for name, t in (("block_table", block_table), ("req_indptr", req_indptr), ("ctx_lens", ctx_lens),
                    ("tile_req", tile_req), ("tile_tok0", tile_tok0)):
        _i32(t, name)
    if tile_req.numel() < num_tiles or tile_tok0.numel() < num_tiles:
        raise KernelError("paged_attention_prompt: tile arrays shorter than the number of tiles")
    lib = _lib(f"attention_hd{head_dim}")
    part_o = part_ml = tokens = None
    count = 0
    if splits > 1:
        if merge_tokens is None or merge_tokens[1] <= 0:
            raise KernelError("paged_attention_prompt: splits > 1 need the tokens whose parts are merged")
        tokens, count = merge_tokens
        _i32(tokens, "merge_tokens")
        if tokens.numel() < count:
            raise KernelError("paged_attention_prompt: merge_tokens shorter than its count")
        splits = max(1, min(splits, SPLIT_SCRATCH_BYTES // (T * num_heads * (head_dim + 2) * 4)))
        part_o = torch.empty((T * num_heads * splits, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * splits, 2), dtype=torch.float32, device=q.device)
    _check(lib, lib.tl_paged_attention_prompt(_ptr(q), c_int(q.stride(0)), _ptr(out), _ptr(k_plane), _ptr(v_plane),
                                              _ptr(block_table), c_int(block_table.stride(0)), _ptr(req_indptr),
                                              _ptr(ctx_lens), _ptr(tile_req), _ptr(tile_tok0), c_int(num_tiles),
                                              c_int(tile_tokens), c_int(num_heads), c_int(num_kv_heads), c_int(page_size),
                                              c_int(window), c_float(scale), c_int(max(1, used_blocks)),
                                              c_int(splits), _ptr(part_o), _ptr(part_ml), _ptr(tokens), c_int(count), _stream()))


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, activation: str = "silu") -> None:
    """``out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i]``; ``activation``: ``silu`` or ``relu``."""
    T, I2 = gate_up.shape
    if I2 % 2 or out.shape != (T, I2 // 2) or out.dtype != gate_up.dtype or not out.is_contiguous() or not gate_up.is_contiguous():
        raise KernelError("swiglu: shapes or dtypes do not fit")
    if activation not in GATE_ACTIVATIONS:
        raise KernelError(f"swiglu: the gate's activation is one of {', '.join(GATE_ACTIVATIONS)}, not {activation!r}")
    lib = _lib("elementwise")
    _check(lib, lib.tl_swiglu(_ptr(gate_up), _ptr(out), c_int(T), c_int(I2 // 2), c_int(_dt(out, "swiglu")), c_int(GATE_ACTIVATIONS[activation]), _stream()))


def sample(logits: torch.Tensor, temperature: torch.Tensor | None, keys: torch.Tensor | None, out: torch.Tensor) -> None:
    """Token per row of float32 ``logits [N, V]``: arg max where ``temperature`` is 0 (or
    absent), else a Gumbel-max draw from ``softmax(logits / temperature)`` seeded by the
    row's int32 ``keys`` entry."""
    N, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 with unit stride on the last axis")
    if temperature is not None and (temperature.dtype != torch.float32 or temperature.numel() < N or not temperature.is_contiguous()):
        raise KernelError("sample: temperature must be contiguous float32 [N]")
    _i32(keys, "sample keys", N)
    _i32(out, "sample out", N)
    lib = _lib("sampling")
    scratch = torch.empty((2, N, lib.tl_sample_chunks(c_int(V))), dtype=torch.int32, device=logits.device)
    _check(lib, lib.tl_sample(_ptr(logits), c_int(N), c_int(V), c_int(logits.stride(0)), _ptr(temperature), _ptr(keys),
                              _ptr(out), _ptr(scratch), _stream()))


def stream_read(data: torch.Tensor, groups: int = 0) -> torch.Tensor:
    """Read every byte of ``data`` (contiguous, on the GPU) once with a kernel that does nothing else, and
    return the exclusive-or of its 32-bit words per work-group (int32; ``groups`` work-groups, 0: the default).  A yardstick: the time it takes is
    what this GPU needs to deliver that much memory to a kernel, whatever the kernel does with it."""
    if not data.is_contiguous() or data.data_ptr() % 16 or data.numel() * data.element_size() < 16:
        raise KernelError("stream_read: contiguous, 16-byte aligned memory of at least 16 bytes")
    lib = _lib("elementwise")
    lib.tl_stream_read.argtypes = [c_void_p, ctypes.c_size_t, c_void_p, c_int, c_void_p]
    sink = torch.empty(groups or lib.tl_stream_read_groups(), dtype=torch.int32, device=data.device)
    _check(lib, lib.tl_stream_read(_ptr(data), ctypes.c_size_t(data.numel() * data.element_size()), _ptr(sink), c_int(groups), _stream()))
    return sink


# ------------------------------------------------------------- the norm after the sum

def scaled_add_rmsnorm(residual: torch.Tensor, pending: torch.Tensor | None, alpha: float, weight: torch.Tensor, eps: float,
                       out: torch.Tensor | None) -> None:
    """``residual <- rmsnorm(alpha * residual + pending) * weight`` in place (float32 ``[T, H]``); ``out`` (optional, of the
    activation dtype) receives the rounded result.  ``pending``: ``[T, H]`` of ``out``'s dtype (float32 without ``out``),
    float32 slabs ``[P, T, H]`` of partial sums, or ``None``."""
    T, H = residual.shape
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("scaled_add_rmsnorm: the residual must be contiguous float32")
    act = out.dtype if out is not None else torch.float32
    if out is not None and (out.shape != (T, H) or not out.is_contiguous()):
        raise KernelError(f"scaled_add_rmsnorm: out must be contiguous [{T}, {H}], got {tuple(out.shape)}")
    parts = 0
    if pending is not None:
        if pending.dim() == 3:
            parts = pending.shape[0]
            if pending.dtype != torch.float32 or pending.shape[1:] != residual.shape or not pending.is_contiguous():
                raise KernelError(f"scaled_add_rmsnorm: partial sums {pending.dtype} {tuple(pending.shape)} are not float32 [P, {T}, {H}]")
        elif pending.shape != residual.shape or pending.dtype != act or not pending.is_contiguous():
            raise KernelError(f"scaled_add_rmsnorm: pending {pending.dtype} {tuple(pending.shape)} does not match the residual")
    wf = _vec(weight, H, "scaled_add_rmsnorm weight")
    lib = _lib("elementwise")
    _check(lib, lib.tl_scaled_add_rmsnorm(_ptr(residual), _ptr(pending), c_int(parts), c_int(T), c_float(alpha), _ptr(weight), c_int(wf),
                                          c_float(eps), _ptr(out), c_int(T), c_int(H), c_int(_DT[act]), _stream()))


# ------------------------------------------------------------- matrix-memory recurrence

def mlstm_scan(qkv: torch.Tensor, k_off: int, v_off: int, gates: torch.Tensor, state: torch.Tensor, slots: torch.Tensor,
               req_indptr: torch.Tensor, out: torch.Tensor, heads: int, dim: int, vdim: int, cap: float | None,
               qscale: float, denom_eps: float) -> None:
    """The matrix-memory recurrence over the step's tokens, request by request from the state its slot holds:
    ``qkv [T, >=]`` holds per token the queries at column 0 (``heads * dim``), the keys at ``k_off`` and the values at
    ``v_off`` (``heads * vdim``); ``gates`` float32 ``[T, 2 * heads]`` the raw input and forget gates (bias added);
    ``state`` float32 ``[slots, heads, dim * vdim + dim + 1]`` (S, n, m per head) is updated in place; ``out`` float32
    ``[T, heads * vdim]`` receives ``S^T q / (max(|n.q|, exp(-m)) + denom_eps)``."""
    T = qkv.shape[0]
    R = req_indptr.numel() - 1
    if qkv.stride(1) != 1 or qkv.shape[1] < max(heads * dim, k_off + heads * dim, v_off + heads * vdim):
        raise KernelError("mlstm_scan: the rows of qkv do not hold queries, keys and values at the given columns")
    if gates.dtype != torch.float32 or gates.shape != (T, 2 * heads) or not gates.is_contiguous():
        raise KernelError(f"mlstm_scan: gates must be contiguous float32 [{T}, {2 * heads}]")
    if out.dtype != torch.float32 or out.shape != (T, heads * vdim) or not out.is_contiguous():
        raise KernelError(f"mlstm_scan: out must be contiguous float32 [{T}, {heads * vdim}]")
    if state.dtype != torch.float32 or state.dim() != 3 or state.shape[1:] != (heads, dim * vdim + dim + 1) or state.stride(2) != 1 \
            or state.stride(1) != dim * vdim + dim + 1:
        raise KernelError(f"mlstm_scan: state {tuple(state.shape)} is not float32 [slots, {heads}, {dim * vdim + dim + 1}]")
    _i32(slots, "slots", R)
    _i32(req_indptr, "req_indptr", R + 1)
    lib = _lib("recurrent")
    before = torch.empty((R, heads, dim + 1), dtype=torch.float32, device=qkv.device)      # n and m as the step finds them
    _check(lib, lib.tl_mlstm_scan(_ptr(qkv), c_int(qkv.stride(0)), c_int(k_off), c_int(v_off), _ptr(gates), _ptr(state),
                                  ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(before), _ptr(req_indptr), _ptr(out), c_int(R), c_int(heads),
                                  c_int(dim), c_int(vdim), c_float(cap if cap else 0.0), c_float(qscale), c_float(denom_eps),
                                  c_int(max(1, T - R + 1)), c_int(_dt(qkv, "mlstm_scan")), _stream()))


GATES = {"sigmoid": 0, "silu": 1}


def gated_head_norm(o: torch.Tensor, gate_values: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor, heads: int, vdim: int,
                    gate: str = "sigmoid", gain: float = 1.0, gate_first: bool = False) -> None:
    """``out[t, h] = o[t, h] / sqrt(mean(o[t, h]^2) + eps) * weight[h] * gate(gate_values[t, h]) * gain`` per token and head:
    ``o`` float32 ``[T, heads * vdim]``, ``gate_values`` and ``out`` row-strided views ``[T, heads * vdim]`` of one dtype; ``weight``
    ``[heads * vdim]``, or ``[vdim]``: one vector for all heads; ``gate``: ``sigmoid`` or ``silu``.  ``gate_first``: the gate comes before the
    norm, ``out = u / sqrt(mean(u^2) + eps) * weight * gain`` with ``u = o * gate(gate_values)``; a "head" is whatever stretch of the row is
    normed together."""
    T = o.shape[0]
    if o.dtype != torch.float32 or o.shape != (T, heads * vdim) or not o.is_contiguous():
        raise KernelError("gated_head_norm: o must be contiguous float32 [T, heads * vdim]")
    if out.shape != o.shape or out.stride(1) != 1 or gate_values.dtype != out.dtype or gate_values.shape != o.shape or gate_values.stride(1) != 1:
        raise KernelError("gated_head_norm: gate and out do not fit")
    shared = weight.numel() == vdim and heads > 1
    wf = _vec(weight, vdim if shared else heads * vdim, "gated_head_norm weight")
    lib = _lib("recurrent")
    _check(lib, lib.tl_gated_head_norm(_ptr(o), _ptr(gate_values), c_int(gate_values.stride(0)), _ptr(weight), c_int(wf), c_int(1 if shared else 0),
                                       c_float(eps), _ptr(out), c_int(out.stride(0)), c_int(T), c_int(heads), c_int(vdim), c_int(GATES[gate]),
                                       c_float(gain), c_int(1 if gate_first else 0), c_int(_dt(out, "gated_head_norm")), _stream()))


# ------------------------------------------------------------- gated delta rule

DELTA_MAX_TAPS = 8
DELTA_MAX_DIM = 256


def delta_prepare(proj: torch.Tensor, conv_w: torch.Tensor, gates: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                  state: torch.Tensor, tail_off: int, slots: torch.Tensor, req_indptr: torch.Tensor, token_req: torch.Tensor,
                  qkv: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, qscale: float, unit_eps: float) -> None:
    """What the gated delta rule reads, made from the projections of the step's tokens.  ``proj [T, >= C]`` (a row-strided view) holds per
    token the raw queries (``kv_heads * dim``), keys (the same) and values (``heads * vdim``), ``C`` channels in all.  Every channel passes
    a causal convolution, ``y[t] = sum_j conv_w[c, j] x[t - (taps - 1) + j]``, whose inputs before the step's first token of a request
    come from the request's slot (``state[slot, tail_off + i * C + c]``, ``i = 0 .. taps - 2`` oldest first), then silu; queries and keys
    become unit vectors per head (``unit_eps`` under the root), queries times ``qscale``; the result goes to ``qkv`` float32 ``[T, C]``.
    ``gates`` float32 ``[T, 2 * heads]`` holds the raw ``W_b h`` and ``W_a h`` and receives ``sigmoid(.)`` and ``exp(-exp(a_log) * softplus(. +
    dt_bias))`` in their place.  Afterwards the slots' tails hold the last ``taps - 1`` inputs of every request."""
    T = proj.shape[0]
    R = req_indptr.numel() - 1
    C = 2 * kv_heads * dim + heads * vdim
    if proj.stride(1) != 1 or proj.shape[1] < C or qkv.dtype != torch.float32 or qkv.shape != (T, C) or not qkv.is_contiguous():
        raise KernelError("delta_prepare: the projections or the output do not hold the convolved channels")
    if conv_w.dtype != torch.float32 or conv_w.shape != (C, taps) or not conv_w.is_contiguous() or not 1 <= taps <= DELTA_MAX_TAPS:
        raise KernelError(f"delta_prepare: taps must be contiguous float32 [{C}, {taps}], up to {DELTA_MAX_TAPS} of them")
    if gates.dtype != torch.float32 or gates.shape != (T, 2 * heads) or not gates.is_contiguous():
        raise KernelError(f"delta_prepare: gates must be contiguous float32 [{T}, {2 * heads}]")
    for v, what in ((a_log, "a_log"), (dt_bias, "dt_bias")):
        if v.dtype != torch.float32 or v.shape != (heads,) or not v.is_contiguous():
            raise KernelError(f"delta_prepare: {what} must be contiguous float32 [{heads}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < tail_off + (taps - 1) * C:
        raise KernelError(f"delta_prepare: state {tuple(state.shape)} does not hold the convolutions' tails")
    _i32(slots, "slots", R)
    _i32(req_indptr, "req_indptr", R + 1)
    _i32(token_req, "token_req", T)
    lib = _lib("recurrent")
    _check(lib, lib.tl_delta_prepare(_ptr(proj), c_int(proj.stride(0)), _ptr(conv_w), _ptr(gates), _ptr(a_log), _ptr(dt_bias), _ptr(state),
                                     ctypes.c_long(state.stride(0)), ctypes.c_long(tail_off), _ptr(slots), _ptr(req_indptr), _ptr(token_req),
                                     _ptr(qkv), c_int(T), c_int(R), c_int(heads), c_int(kv_heads), c_int(dim), c_int(vdim), c_int(taps),
                                     c_float(qscale), c_float(unit_eps), c_int(_dt(proj, "delta_prepare")), _stream()))


def delta_scan(qkv: torch.Tensor, gates: torch.Tensor, state: torch.Tensor, slots: torch.Tensor, req_indptr: torch.Tensor, out: torch.Tensor,
               heads: int, kv_heads: int, dim: int, vdim: int, max_new_tokens: int | None = None) -> None:
    """The gated delta rule over the step's tokens, request by request from the state its slot holds: ``qkv`` float32 ``[T, C]`` as
    :func:`delta_prepare` left it (queries, keys, values), ``gates`` float32 ``[T, 2 * heads]`` (beta, decay); head ``h`` of ``state[slot]``
    (float32, ``dim x vdim`` numbers from ``h * dim * vdim`` on, column by column: ``[vdim][dim]``) moves by ``S <- g S; u = beta (v - S^T k); S <- S + k u^T`` and ``out`` float32
    ``[T, heads * vdim]`` receives ``S^T q``."""
    T = qkv.shape[0]
    R = req_indptr.numel() - 1
    C = 2 * kv_heads * dim + heads * vdim
    if qkv.dtype != torch.float32 or qkv.shape != (T, C) or not qkv.is_contiguous():
        raise KernelError(f"delta_scan: qkv must be contiguous float32 [{T}, {C}]")
    if gates.dtype != torch.float32 or gates.shape != (T, 2 * heads) or not gates.is_contiguous():
        raise KernelError(f"delta_scan: gates must be contiguous float32 [{T}, {2 * heads}]")
    if out.dtype != torch.float32 or out.shape != (T, heads * vdim) or not out.is_contiguous():
        raise KernelError(f"delta_scan: out must be contiguous float32 [{T}, {heads * vdim}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < heads * dim * vdim or dim > DELTA_MAX_DIM:
        raise KernelError(f"delta_scan: state {tuple(state.shape)} does not hold {heads} states of {dim} x {vdim} (up to {DELTA_MAX_DIM} rows)")
    _i32(slots, "slots", R)
    _i32(req_indptr, "req_indptr", R + 1)
    lib = _lib("recurrent")
    _check(lib, lib.tl_delta_scan(_ptr(qkv), _ptr(gates), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(req_indptr), _ptr(out),
                                  c_int(R), c_int(heads), c_int(kv_heads), c_int(dim), c_int(vdim),
                                  c_int(max(1, T - R + 1) if max_new_tokens is None else max_new_tokens), _stream()))


def decay_scan(qkv: torch.Tensor, decay: torch.Tensor, state: torch.Tensor, slots: torch.Tensor, req_indptr: torch.Tensor, out: torch.Tensor,
               heads: int, dim: int, vdim: int, max_new_tokens: int | None = None) -> None:
    """Linear attention with one fixed decay per head over the step's tokens, request by request from the state its slot holds: ``qkv``
    float32 ``[T, 2 * heads * dim + heads * vdim]`` (queries, keys, values, head by head), ``decay`` float32 ``[heads]``; head ``h`` of
    ``state[slot]`` (float32, laid out as :func:`delta_scan`'s) moves by ``S <- decay[h] S + k v^T`` and ``out`` float32 ``[T, heads * vdim]``
    receives ``S^T q``."""
    T = qkv.shape[0]
    R = req_indptr.numel() - 1
    C = 2 * heads * dim + heads * vdim
    if qkv.dtype != torch.float32 or qkv.shape != (T, C) or not qkv.is_contiguous():
        raise KernelError(f"decay_scan: qkv must be contiguous float32 [{T}, {C}]")
    if decay.dtype != torch.float32 or decay.shape != (heads,) or not decay.is_contiguous():
        raise KernelError(f"decay_scan: decay must be contiguous float32 [{heads}]")
    if out.dtype != torch.float32 or out.shape != (T, heads * vdim) or not out.is_contiguous():
        raise KernelError(f"decay_scan: out must be contiguous float32 [{T}, {heads * vdim}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < heads * dim * vdim or dim > DELTA_MAX_DIM:
        raise KernelError(f"decay_scan: state {tuple(state.shape)} does not hold {heads} states of {dim} x {vdim} (up to {DELTA_MAX_DIM} rows)")
    _i32(slots, "slots", R)
    _i32(req_indptr, "req_indptr", R + 1)
    lib = _lib("recurrent")
    _check(lib, lib.tl_decay_scan(_ptr(qkv), _ptr(decay), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(req_indptr), _ptr(out),
                                  c_int(R), c_int(heads), c_int(dim), c_int(vdim),
                                  c_int(max(1, T - R + 1) if max_new_tokens is None else max_new_tokens), _stream()))


def selective_prepare(proj: torch.Tensor, x_off: int, conv_w: torch.Tensor, conv_b: torch.Tensor, gates: torch.Tensor, a_log: torch.Tensor,
                      dt_bias: torch.Tensor, state: torch.Tensor, tail_off: int, slots: torch.Tensor, req_indptr: torch.Tensor,
                      token_req: torch.Tensor, qkv: torch.Tensor, heads: int, inner: int, gn: int, taps: int) -> None:
    """What a selective state-space recurrence reads, made from the projection of the step's tokens.  ``proj [T, >= x_off + channels + heads]``
    (rows may be strided) holds per token, from column ``x_off`` on, ``channels = inner + 2 * gn`` convolved channels ``[x | B | C]`` and then
    ``heads`` raw step sizes.  Every channel passes a causal convolution with a bias, ``y[t] = conv_b[c] + sum_j conv_w[c, j] x[t - (taps - 1) +
    j]``, whose inputs before the step's first token of a request come from the request's slot (``state[slot, tail_off + i * channels + c]``,
    oldest first), then silu; the result goes to ``qkv`` float32 ``[T, channels]`` in the order ``[C | B | x]``.  ``gates`` float32 ``[T, 2 *
    heads]`` receives ``dt = softplus(raw + dt_bias)`` and ``exp(-exp(a_log) * dt)``.  Afterwards the slots' tails hold the last ``taps - 1``
    inputs of every request."""
    T = proj.shape[0]
    R = req_indptr.numel() - 1
    C = inner + 2 * gn
    if proj.stride(1) != 1 or proj.shape[1] < x_off + C + heads or qkv.dtype != torch.float32 or qkv.shape != (T, C) or not qkv.is_contiguous():
        raise KernelError("selective_prepare: the projection or the output does not hold the convolved channels")
    if conv_w.dtype != torch.float32 or conv_w.shape != (C, taps) or not conv_w.is_contiguous() or not 1 <= taps <= DELTA_MAX_TAPS \
            or conv_b.dtype != torch.float32 or conv_b.shape != (C,) or not conv_b.is_contiguous():
        raise KernelError(f"selective_prepare: taps must be contiguous float32 [{C}, {taps}] (up to {DELTA_MAX_TAPS} of them) with a bias [{C}]")
    if gates.dtype != torch.float32 or gates.shape != (T, 2 * heads) or not gates.is_contiguous():
        raise KernelError(f"selective_prepare: gates must be contiguous float32 [{T}, {2 * heads}]")
    for v, what in ((a_log, "a_log"), (dt_bias, "dt_bias")):
        if v.dtype != torch.float32 or v.shape != (heads,) or not v.is_contiguous():
            raise KernelError(f"selective_prepare: {what} must be contiguous float32 [{heads}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < tail_off + (taps - 1) * C:
        raise KernelError(f"selective_prepare: state {tuple(state.shape)} does not hold the convolutions' tails")
    _i32(slots, "slots", R)
    _i32(req_indptr, "req_indptr", R + 1)
    _i32(token_req, "token_req", T)
    lib = _lib("recurrent")
    _check(lib, lib.tl_selective_prepare(_ptr(proj), c_int(proj.stride(0)), c_int(x_off), _ptr(conv_w), _ptr(conv_b), _ptr(gates), _ptr(a_log),
                                         _ptr(dt_bias), _ptr(state), ctypes.c_long(state.stride(0)), ctypes.c_long(tail_off), _ptr(slots),
                                         _ptr(req_indptr), _ptr(token_req), _ptr(qkv), c_int(T), c_int(R), c_int(heads), c_int(inner), c_int(gn),
                                         c_int(taps), c_int(_dt(proj, "selective_prepare")), _stream()))


def selective_scan(qkv: torch.Tensor, gates: torch.Tensor, skip: torch.Tensor, state: torch.Tensor, slots: torch.Tensor, req_indptr: torch.Tensor,
                   out: torch.Tensor, heads: int, groups: int, dim: int, vdim: int, max_new_tokens: int | None = None) -> None:
    """A selective state-space recurrence over the step's tokens, request by request from the state its slot holds: ``qkv`` float32 ``[T, 2 *
    groups * dim + heads * vdim]`` as :func:`selective_prepare` left it (C, B, x), ``gates`` float32 ``[T, 2 * heads]`` (dt, decay), ``skip``
    float32 ``[heads]``; head ``h`` (reading B and C of group ``h // (heads / groups)``) of ``state[slot]`` (float32, ``dim x vdim`` numbers from ``h *
    dim * vdim`` on, column by column: ``[vdim][dim]``) moves by ``S <- decay S + dt B x^T`` and ``out`` float32 ``[T, heads * vdim]`` receives
    ``S^T C + skip[h] x``."""
    T = qkv.shape[0]
    R = req_indptr.numel() - 1
    C = 2 * groups * dim + heads * vdim
    if qkv.dtype != torch.float32 or qkv.shape != (T, C) or not qkv.is_contiguous():
        raise KernelError(f"selective_scan: qkv must be contiguous float32 [{T}, {C}]")
    if gates.dtype != torch.float32 or gates.shape != (T, 2 * heads) or not gates.is_contiguous():
        raise KernelError(f"selective_scan: gates must be contiguous float32 [{T}, {2 * heads}]")
    if skip.dtype != torch.float32 or skip.shape != (heads,) or not skip.is_contiguous():
        raise KernelError(f"selective_scan: skip must be contiguous float32 [{heads}]")
    if out.dtype != torch.float32 or out.shape != (T, heads * vdim) or not out.is_contiguous():
        raise KernelError(f"selective_scan: out must be contiguous float32 [{T}, {heads * vdim}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < heads * dim * vdim or dim > DELTA_MAX_DIM or heads % groups:
        raise KernelError(f"selective_scan: state {tuple(state.shape)} does not hold {heads} states of {dim} x {vdim} (up to {DELTA_MAX_DIM} rows)")
    _i32(slots, "slots", R)
    _i32(req_indptr, "req_indptr", R + 1)
    lib = _lib("recurrent")
    _check(lib, lib.tl_selective_scan(_ptr(qkv), _ptr(gates), _ptr(skip), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(req_indptr),
                                      _ptr(out), c_int(R), c_int(heads), c_int(groups), c_int(dim), c_int(vdim),
                                      c_int(max(1, T - R + 1) if max_new_tokens is None else max_new_tokens), _stream()))


def silu_float(x: torch.Tensor, out: torch.Tensor) -> None:
    """``out = silu(float32(x))``: ``x [T, C]`` a row-strided view of either dtype, ``out`` contiguous float32 ``[T, C]``."""
    if x.dim() != 2 or x.stride(1) != 1 or out.dtype != torch.float32 or out.shape != x.shape or not out.is_contiguous():
        raise KernelError("silu_float: x must be [T, C] with unit stride along C and out contiguous float32 of the same shape")
    lib = _lib("recurrent")
    _check(lib, lib.tl_silu_float(_ptr(x), c_int(x.stride(0)), _ptr(out), c_int(x.shape[0]), c_int(x.shape[1]), c_int(_dt(x, "silu_float")), _stream()))


# ------------------------------------------------------------- attention with two head sizes, a cap and a local mask

LOCAL_ATTENTION_MAX_DIM = 256


def _check_local_planes(what, k_plane, v_plane, dtype, kv_heads, dim, vdim, page_size):
    if k_plane.dtype != dtype or v_plane.dtype != dtype or not k_plane.is_contiguous() or not v_plane.is_contiguous() \
            or k_plane.shape[1:] != (kv_heads, page_size, dim) or v_plane.shape[1:] != (kv_heads, vdim, page_size) or k_plane.shape[0] != v_plane.shape[0]:
        raise KernelError(f"{what}: cache planes {tuple(k_plane.shape)} / {tuple(v_plane.shape)} are not [pages, {kv_heads}, {page_size}, {dim}] and "
                          f"[pages, {kv_heads}, {vdim}, {page_size}] of {dtype}")


def kv_cache_write(k: torch.Tensor, v: torch.Tensor, token_req: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
                   k_plane: torch.Tensor, v_plane: torch.Tensor, page_size: int) -> None:
    """The step's keys ``k [T, kv_heads * dim]`` and values ``v [T, kv_heads * vdim]`` (row-strided views) go to their places in the pages:
    token ``t`` of request ``token_req[t]`` at position ``p`` to slot ``p % page_size`` of page ``block_table[request, p // page_size]`` of
    ``k_plane [pages, kv_heads, page_size, dim]`` and ``v_plane [pages, kv_heads, vdim, page_size]`` (the values of a page lie transposed).
    What would go to page 0 is dropped."""
    T = k.shape[0]
    kv_heads, dim, vdim = k_plane.shape[1], k_plane.shape[3], v_plane.shape[2]
    _check_local_planes("kv_cache_write", k_plane, v_plane, k.dtype, kv_heads, dim, vdim, page_size)
    if k.shape != (T, kv_heads * dim) or v.shape != (T, kv_heads * vdim) or k.stride(1) != 1 or v.stride(1) != 1 or v.dtype != k.dtype:
        raise KernelError("kv_cache_write: keys or values do not fit the planes")
    _i32(token_req, "token_req", T)
    _i32(positions, "positions", T)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("kv_cache_write: the block table must be int32 [requests, blocks]")
    lib = _lib("local_attention")
    _check(lib, lib.tl_kv_cache_write(_ptr(k), c_int(k.stride(0)), _ptr(v), c_int(v.stride(0)), c_int(T), c_int(kv_heads), c_int(dim), c_int(vdim),
                                      _ptr(token_req), _ptr(positions), _ptr(block_table), c_int(block_table.stride(0)), c_int(block_table.shape[1]),
                                      _ptr(k_plane), _ptr(v_plane), c_int(k_plane.shape[0]), c_int(page_size), c_int(_dt(k, "kv_cache_write")), _stream()))


LOCAL_ATTENTION_TILE_TOKENS = 16      # tokens of a tile of the matrix-core kernel


def local_attention_mfma_fits(dtype: torch.dtype, dim: int, vdim: int, page_size: int) -> bool:
    """Whether the matrix-core kernel of :func:`local_attention` is built for these sizes (bfloat16; key sizes 32, 64, 96, 128, 192, 256;
    value sizes 16, 32, 64, 96, 128, 192, 256; pages of a multiple of 8 tokens)."""
    return dtype == torch.bfloat16 and bool(_lib("local_attention").tl_local_attention_mfma_fits(c_int(dim), c_int(vdim), c_int(page_size)))


def local_attention(q: torch.Tensor, out: torch.Tensor, k_plane: torch.Tensor, v_plane: torch.Tensor, block_table: torch.Tensor,
                    token_req: torch.Tensor, positions: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, page_size: int,
                    scale: float, softcap: float = 0.0, chunk: int = 0, window: int = 0, gain: float = 1.0, tiles=None,
                    sink: torch.Tensor | None = None, pooled=None, keep_first: int = 0) -> None:
    """Attention of the step's queries ``q [T, heads * dim]`` over their requests' cached keys and values (which hold the step's own tokens
    already): query head ``i`` reads key/value head ``i // (heads / kv_heads)``; ``score = q . k * scale``, then (``softcap > 0``) ``softcap *
    tanh(score / softcap)``; a query at position ``p`` reads the keys ``j <= p`` with ``j // chunk == p // chunk`` (``chunk > 0``) and ``j > p -
    window`` (``window > 0``); softmax and weighted sum in 32-bit; ``out [T, heads * vdim]`` receives the result times ``gain``.  ``q`` and ``out``
    may be row-strided views.  Without ``tiles`` one work-group per token and head walks the keys (every dtype and size).  ``tiles =
    (req_indptr, ctx_lens, tile_req, tile_tok0, number of tiles)`` (tiles of up to 16 consecutive tokens of one request, as a step
    context makes them) runs the matrix-core kernel, where :func:`local_attention_mfma_fits` says it is built.  ``sink`` (float32 ``[heads]``):
    ``exp(sink[head])`` joins the softmax's denominator.  ``pooled = (pk_plane, pv_plane, pool_table, pool)`` (with a window): a query at
    ``p`` also reads the rows ``0 .. (p - window + 1) // pool - 1`` of these planes (laid out like the tokens', with a block table of their own).
    ``keep_first`` (with a window, without chunks): a query also reads the keys at the positions ``0 .. keep_first - 1``, wherever it stands."""
    T = q.shape[0]
    if keep_first < 0 or (keep_first and (window <= 0 or chunk)):
        raise KernelError("local_attention: kept first tokens stand beside a window, without chunks")
    _check_local_planes("local_attention", k_plane, v_plane, q.dtype, kv_heads, dim, vdim, page_size)
    if sink is not None and (sink.dtype != torch.float32 or sink.shape != (heads,) or not sink.is_contiguous()):
        raise KernelError(f"local_attention: the sink must be contiguous float32 [{heads}]")
    pk_plane = pv_plane = pool_table = None
    pool = 0
    if pooled is not None:
        pk_plane, pv_plane, pool_table, pool = pooled
        _check_local_planes("local_attention (pooled)", pk_plane, pv_plane, q.dtype, kv_heads, dim, vdim, page_size)
        if pool <= 0 or window <= 0 or pool_table.dtype != torch.int32 or pool_table.dim() != 2 or pool_table.stride(1) != 1 \
                or pool_table.shape[0] != block_table.shape[0]:
            raise KernelError("local_attention: pooled blocks need a window, a block size and an int32 block table [requests, blocks]")
    pool_args = (_ptr(sink), _ptr(pk_plane), _ptr(pv_plane), _ptr(pool_table), c_int(pool_table.stride(0) if pool else 0))
    if q.shape != (T, heads * dim) or out.shape != (T, heads * vdim) or q.stride(1) != 1 or out.stride(1) != 1 or out.dtype != q.dtype \
            or heads % kv_heads or max(dim, vdim) > LOCAL_ATTENTION_MAX_DIM:
        raise KernelError("local_attention: queries or output do not fit")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("local_attention: the block table must be int32 [requests, blocks]")
    lib = _lib("local_attention")
    if tiles is not None:
        req_indptr, ctx_lens, tile_req, tile_tok0, n_tiles = tiles
        if not local_attention_mfma_fits(q.dtype, dim, vdim, page_size) or q.stride(0) % 8 or q.data_ptr() % 16:
            raise KernelError("local_attention: the matrix-core kernel is not built for these operands")
        R = block_table.shape[0]
        _i32(req_indptr, "req_indptr", R + 1)
        _i32(ctx_lens, "ctx_lens", R)
        _i32(tile_req, "tile_req", n_tiles)
        _i32(tile_tok0, "tile_tok0", n_tiles)
        if tile_req is None and n_tiles > R:
            raise KernelError("local_attention: without a tile list there is one tile per request")
        _check(lib, lib.tl_local_attention_tiles(_ptr(q), c_int(q.stride(0)), _ptr(out), c_int(out.stride(0)), _ptr(k_plane), _ptr(v_plane),
                                                 c_int(k_plane.shape[0]), _ptr(block_table), c_int(block_table.stride(0)), c_int(block_table.shape[1]),
                                                 _ptr(req_indptr), _ptr(ctx_lens), _ptr(tile_req), _ptr(tile_tok0), c_int(n_tiles), c_int(heads),
                                                 c_int(kv_heads), c_int(dim), c_int(vdim), c_int(page_size), c_float(scale), c_float(softcap),
                                                 c_int(chunk), c_int(window), c_float(gain), *pool_args, c_int(pool_table.shape[1] if pool else 0),
                                                 c_int(pool), c_int(keep_first), _stream()))
        return
    _i32(token_req, "token_req", T)
    _i32(positions, "positions", T)
    _check(lib, lib.tl_local_attention(_ptr(q), c_int(q.stride(0)), _ptr(out), c_int(out.stride(0)), _ptr(k_plane), _ptr(v_plane), c_int(k_plane.shape[0]),
                                       _ptr(block_table), c_int(block_table.stride(0)), c_int(block_table.shape[1]), _ptr(token_req), _ptr(positions),
                                       c_int(T), c_int(heads), c_int(kv_heads), c_int(dim), c_int(vdim), c_int(page_size), c_float(scale),
                                       c_float(softcap), c_int(chunk), c_int(window), c_float(gain), *pool_args, c_int(pool), c_int(keep_first),
                                       c_int(_dt(q, "local_attention")), _stream()))


def pool_blocks(k_plane: torch.Tensor, v_plane: torch.Tensor, block_table: torch.Tensor, pk_plane: torch.Tensor, pv_plane: torch.Tensor,
                pool_table: torch.Tensor, req_indptr: torch.Tensor, ctx_lens: torch.Tensor, most_blocks: int, page_size: int, pool: int) -> None:
    """The pooled rows of the blocks of ``pool`` positions whose last token this step brought: for request ``r``, which held ``ctx_lens[r]``
    tokens and got ``req_indptr[r + 1] - req_indptr[r]``, the blocks ``ctx // pool .. (ctx + n) // pool - 1``; row ``b`` of ``pk_plane`` / ``pv_plane``
    (through ``pool_table``) receives the means of the cached keys and values of the positions ``b * pool .. b * pool + pool - 1`` (summed in
    32-bit, rounded once).  ``most_blocks``: an upper bound of the blocks one request completes in the step."""
    kv_heads, dim, vdim = k_plane.shape[1], k_plane.shape[3], v_plane.shape[2]
    _check_local_planes("pool_blocks", k_plane, v_plane, k_plane.dtype, kv_heads, dim, vdim, page_size)
    _check_local_planes("pool_blocks (pooled)", pk_plane, pv_plane, k_plane.dtype, kv_heads, dim, vdim, page_size)
    R = req_indptr.numel() - 1
    for t, what in ((block_table, "block table"), (pool_table, "pooled block table")):
        if t.dtype != torch.int32 or t.dim() != 2 or t.stride(1) != 1 or t.shape[0] < R:
            raise KernelError(f"pool_blocks: the {what} must be int32 [requests, blocks]")
    _i32(req_indptr, "req_indptr", R + 1)
    _i32(ctx_lens, "ctx_lens", R)
    if pool <= 0 or most_blocks < 0:
        raise KernelError("pool_blocks: a block holds at least one position")
    lib = _lib("local_attention")
    _check(lib, lib.tl_pool_blocks(_ptr(k_plane), _ptr(v_plane), c_int(k_plane.shape[0]), _ptr(block_table), c_int(block_table.stride(0)),
                                   c_int(block_table.shape[1]), _ptr(pk_plane), _ptr(pv_plane), c_int(pk_plane.shape[0]), _ptr(pool_table),
                                   c_int(pool_table.stride(0)), c_int(pool_table.shape[1]), _ptr(req_indptr), _ptr(ctx_lens), c_int(R),
                                   c_int(most_blocks), c_int(kv_heads), c_int(dim), c_int(vdim), c_int(page_size), c_int(pool),
                                   c_int(_dt(k_plane, "pool_blocks")), _stream()))


def head_norm_rotate(x: torch.Tensor, heads_a: int, heads_b: int, dim: int, norm_a: torch.Tensor | None, norm_b: torch.Tensor | None, eps: float,
                     positions: torch.Tensor | None, inv_freq: torch.Tensor | None, dims: int, halves: bool,
                     raw_b: torch.Tensor | None = None) -> None:
    """In place on ``x [T, (heads_a + heads_b) * dim]`` (a row-strided view: queries, then keys), per token and head, in 32-bit with one rounding:
    a root-mean-square norm over the head's ``dim`` numbers with the weight ``norm_a`` (the first ``heads_a`` heads) or ``norm_b`` (float32
    ``[dim]``; ``None``: no norm), then the rotation of the first ``dims`` numbers by ``float32(position) * inv_freq[i]`` (float32 ``[dims / 2]``;
    ``None``: no rotation), pairing ``2i`` with ``2i + 1`` or, ``halves``, ``i`` with ``i + dims / 2``.  ``raw_b [T, heads_b * dim]`` (of ``x``'s
    dtype, rows may be strided) receives the last ``heads_b`` heads as they come, before norm and rotation."""
    T = x.shape[0]
    heads = heads_a + heads_b
    if raw_b is not None and (raw_b.dtype != x.dtype or raw_b.shape != (T, heads_b * dim) or raw_b.stride(1) != 1):
        raise KernelError(f"head_norm_rotate: the copy of the second heads must be [T, {heads_b * dim}] of {x.dtype}")
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] != heads * dim or dim > LOCAL_ATTENTION_MAX_DIM:
        raise KernelError(f"head_norm_rotate: x {tuple(x.shape)} is not [T, {heads} heads of {dim}] (up to {LOCAL_ATTENTION_MAX_DIM} numbers a head)")
    for w in (norm_a, norm_b):
        if w is not None and (w.dtype != torch.float32 or w.shape != (dim,) or not w.is_contiguous()):
            raise KernelError(f"head_norm_rotate: a norm's weight must be contiguous float32 [{dim}]")
    if (norm_a is None) != (norm_b is None) and heads_a and heads_b:
        raise KernelError("head_norm_rotate: a norm for both kinds of heads or for neither")
    if inv_freq is not None:
        if dims <= 0 or dims % 2 or dims > dim or inv_freq.dtype != torch.float32 or inv_freq.shape != (dims // 2,) or not inv_freq.is_contiguous():
            raise KernelError(f"head_norm_rotate: a rotation over {dims} of {dim} numbers needs float32 frequencies [{dims // 2}]")
        _i32(positions, "positions", T)
        if positions is None:
            raise KernelError("head_norm_rotate: a rotation needs the tokens' positions")
    lib = _lib("local_attention")
    _check(lib, lib.tl_head_norm_rotate(_ptr(x), c_int(x.stride(0)), c_int(T), c_int(heads_a), c_int(heads_b), c_int(dim), _ptr(norm_a), _ptr(norm_b),
                                        c_float(eps), _ptr(positions if inv_freq is not None else None), _ptr(inv_freq), c_int(dims if inv_freq is not None else 0),
                                        c_int(1 if halves else 0), _ptr(raw_b), c_int(raw_b.stride(0) if raw_b is not None else 0),
                                        c_int(_dt(x, "head_norm_rotate")), _stream()))


# ------------------------------------------------------------- attention over a cached latent

LATENT_ATTENTION_ROWS = 16       # rows (tokens x heads) a work-group of the latent attention owns
LATENT_MAX_RANK = 1024


LATENT_MFMA_ROWS = 64            # rows of a tile of its matrix-core kernel
LATENT_MFMA_MAX_BLOCKS = 1536    # block-table entries of a request that its work-groups keep in shared memory


def latent_tile_tokens(heads: int, rows: int = LATENT_ATTENTION_ROWS) -> int:
    """New tokens of one request that share a tile of ``rows`` rows of the latent attention (a row: a token and one of
    up to 16 heads)."""
    return max(1, rows // min(heads, LATENT_ATTENTION_ROWS))


def latent_attention_mfma_fits(dtype: torch.dtype, heads: int, rank: int, rot: int) -> bool:
    """Whether :func:`latent_attention` runs these sizes on the matrix cores (bfloat16, cache rows of a multiple of 32 numbers up
    to 640, latents of a multiple of 64 numbers up to 512); it then takes tiles of up to 64 rows, else of up to 16."""
    return dtype == torch.bfloat16 and bool(_lib("latent").tl_latent_attention_mfma_fits(c_int(rank), c_int(rot), c_int(heads * (rank + rot))))


def latent_prepare(down: torch.Tensor, q_rank: int, rank: int, rot: int, rot_dims: int, wq: torch.Tensor | None, wkv: torch.Tensor,
                   eps: float, positions: torch.Tensor, inv_freq: torch.Tensor, cq: torch.Tensor | None, token_req: torch.Tensor | None = None,
                   block_table: torch.Tensor | None = None, plane: torch.Tensor | None = None, page_size: int = 0, kv_off: int | None = None) -> None:
    """From the fused first projection ``down [T, >= kv_off + rank + rot]``: ``cq = rmsnorm(down[:, :q_rank]) * wq`` (``q_rank`` 0: no query
    latent, ``wq`` and ``cq`` ``None``) and, with a plane ``[pages, 1, page, rank + rot]``, the token's cache row ``[rmsnorm(down[:, kv_off:kv_off +
    rank]) * wkv, the next rot numbers with the first rot_dims of them turned in pairs by the token's position]``.  ``kv_off``: the column
    where the key/value latent starts (default: right after the query latent)."""
    T = down.shape[0]
    kv_off = q_rank if kv_off is None else kv_off
    if down.stride(1) != 1 or kv_off < q_rank or down.shape[1] < kv_off + rank + rot or (q_rank == 0) != (cq is None) or (q_rank == 0) != (wq is None) \
            or (cq is not None and (cq.shape != (T, q_rank) or cq.dtype != down.dtype or not cq.is_contiguous())):
        raise KernelError("latent_prepare: shapes do not fit")
    _i32(positions, "positions", T)
    if inv_freq.dtype != torch.float32 or inv_freq.numel() != rot_dims // 2 or rot_dims % 2 or rot_dims > rot:
        raise KernelError("latent_prepare: inv_freq must be float32 [rot_dims / 2]")
    bt_stride = 0
    if plane is not None:
        _i32(token_req, "token_req", T)
        _i32(block_table, "block_table")
        bt_stride = block_table.stride(0)
        if plane.dtype != down.dtype or plane.dim() != 4 or tuple(plane.shape[1:]) != (1, page_size, rank + rot) or not plane.is_contiguous():
            raise KernelError(f"latent_prepare: plane {tuple(plane.shape)} {plane.dtype} is not [pages, 1, {page_size}, {rank + rot}] {down.dtype}")
    lib = _lib("latent")
    _check(lib, lib.tl_latent_prepare(_ptr(down), c_int(down.stride(0)), c_int(q_rank), c_int(kv_off), c_int(rank), c_int(rot), c_int(rot_dims),
                                      _ptr(wq), c_int(_vec(wq, q_rank, "query latent norm")), _ptr(wkv), c_int(_vec(wkv, rank, "latent norm")),
                                      c_float(eps), _ptr(positions), _ptr(inv_freq), _ptr(token_req), _ptr(block_table), c_int(bt_stride),
                                      _ptr(plane), c_int(page_size), _ptr(cq), c_int(T), c_int(_dt(down, "latent_prepare")), _stream()))


def rotate_pairs(src: torch.Tensor, src_head: int, src_off: int, dst: torch.Tensor, dst_head: int, dst_off: int,
                 positions: torch.Tensor, inv_freq: torch.Tensor, heads: int, rot: int) -> None:
    """Per token and head, ``rot`` numbers from ``src[t, h * src_head + src_off:]`` to ``dst[t, h * dst_head + dst_off:]``, the first
    ``2 * len(inv_freq)`` of them turned in neighbouring pairs by ``position * inv_freq``."""
    T = src.shape[0]
    rot_dims = 2 * inv_freq.numel()
    if src.dtype != dst.dtype or src.stride(1) != 1 or dst.stride(1) != 1 or dst.shape[0] != T or rot_dims > rot \
            or src.shape[1] < (heads - 1) * src_head + src_off + rot or dst.shape[1] < (heads - 1) * dst_head + dst_off + rot:
        raise KernelError("rotate_pairs: shapes do not fit")
    _i32(positions, "positions", T)
    if inv_freq.dtype != torch.float32:
        raise KernelError("rotate_pairs: inv_freq must be float32")
    lib = _lib("latent")
    _check(lib, lib.tl_rotate_pairs(_ptr(src), c_int(src.stride(0)), c_int(src_head), c_int(src_off), _ptr(dst), c_int(dst.stride(0)),
                                    c_int(dst_head), c_int(dst_off), _ptr(positions), _ptr(inv_freq), c_int(T), c_int(heads), c_int(rot),
                                    c_int(rot_dims), c_int(_dt(src, "rotate_pairs")), _stream()))


def latent_attention(q: torch.Tensor, out: torch.Tensor, plane: torch.Tensor, block_table: torch.Tensor, req_indptr: torch.Tensor | None,
                     ctx_lens: torch.Tensor, tile_req: torch.Tensor | None, tile_tok0: torch.Tensor | None, num_tiles: int,
                     tile_tokens: int, heads: int, rank: int, rot: int, page_size: int, scale: float, sink: torch.Tensor | None,
                     splits: int = 1, general: bool = False, max_new_tokens: int | None = None, window: int = 0,
                     gate: torch.Tensor | None = None) -> None:
    """Causal attention of the step's tokens over their requests' cached rows ``plane [pages, 1, page, rank + rot]``: ``q [T,
    heads * (rank + rot)]`` holds per head the query brought into the cache row's shape, a score is the dot product of the two
    times ``scale``, the softmax's denominator also holds ``exp(sink[head])`` (float32 ``[heads]``; ``None``: no sink), and ``out
    [T, heads * rank]`` receives the weighted sums of the rows' first ``rank`` numbers.  ``tile_req = tile_tok0 = None``: every
    request brings one token.  ``splits``: work-groups that share a tile's keys (merged afterwards).  bfloat16 at sizes that
    :func:`latent_attention_mfma_fits` runs on the matrix cores (``general=True`` forces the general kernel); ``max_new_tokens``:
    the most tokens a request brings in this step (default: ``tile_tokens``), by which the matrix-core kernel sizes its work-groups.
    ``window > 0``: a query reads its last ``window`` keys only, itself included.  ``gate [T, >= heads]`` (of ``q``'s dtype, rows may be
    strided): head ``n``'s output of token ``t`` is multiplied by ``sigmoid(gate[t, n])``."""
    T = q.shape[0]
    D = rank + rot
    if q.stride(1) != 1 or q.shape[1] < heads * D or out.shape != (T, heads * rank) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("latent_attention: q/out shapes or dtypes do not fit")
    if plane.dtype != q.dtype or plane.dim() != 4 or tuple(plane.shape[1:]) != (1, page_size, D) or not plane.is_contiguous():
        raise KernelError(f"latent_attention: plane {tuple(plane.shape)} {plane.dtype} is not [pages, 1, {page_size}, {D}] {q.dtype}")
    if rank > LATENT_MAX_RANK:
        raise KernelError(f"latent_attention: built for latents of up to {LATENT_MAX_RANK} numbers")
    for name, t in (("block_table", block_table), ("ctx_lens", ctx_lens)):
        _i32(t, name)
    if tile_req is None:
        if tile_tok0 is not None or num_tiles != T or ctx_lens.numel() < T or block_table.shape[0] < T:
            raise KernelError("latent_attention: without a tile list every request brings exactly one token")
        req_indptr = None
    else:
        for name, t in (("req_indptr", req_indptr), ("tile_req", tile_req), ("tile_tok0", tile_tok0)):
            _i32(t, name)
        if tile_req.numel() < num_tiles or tile_tok0.numel() < num_tiles:
            raise KernelError("latent_attention: tile arrays shorter than the number of tiles")
    if sink is not None and (sink.dtype != torch.float32 or sink.numel() != heads or not sink.is_contiguous()):
        raise KernelError("latent_attention: sink must be float32 [heads]")
    if window < 0 or (gate is not None and (gate.dtype != q.dtype or gate.dim() != 2 or gate.shape[0] != T or gate.shape[1] < heads or gate.stride(1) != 1)):
        raise KernelError("latent_attention: a window is not negative, and a gate is [T, >= heads] of the queries' dtype")
    splits = max(1, min(splits, SPLIT_SCRATCH_BYTES // (T * heads * (rank + 2) * 4)))
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty((T * heads * splits, rank), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * heads * splits, 2), dtype=torch.float32, device=q.device)
    lib = _lib("latent")
    _check(lib, lib.tl_latent_attention(_ptr(q), c_int(q.stride(0)), _ptr(out), _ptr(plane), _ptr(block_table), c_int(block_table.stride(0)),
                                        _ptr(req_indptr), _ptr(ctx_lens), _ptr(tile_req), _ptr(tile_tok0), c_int(num_tiles), c_int(T),
                                        c_int(tile_tokens), c_int(heads), c_int(rank), c_int(rot), c_int(page_size), c_float(scale),
                                        _ptr(sink), c_int(splits), _ptr(part_o), _ptr(part_ml), c_int(_dt(q, "latent_attention")),
                                        c_int(1 if general else 0), c_int(tile_tokens if max_new_tokens is None else max_new_tokens),
                                        c_int(window), _ptr(gate), c_int(gate.stride(0) if gate is not None else 0), _stream()))


# ------------------------------------------------------------- products over groups, routing

# ``*_pairs``: the product's columns come in pairs (gate, up) and the output, half as wide, is ``act(gate) * up``
ACTIVATIONS = {"none": 0, "relu2": 1, "silu": 2, "gelu_tanh": 3, "gelu": 4, "relu2_pairs": 17, "silu_pairs": 18, "gelu_tanh_pairs": 19, "gelu_pairs": 20}


def heads_linear(x: torch.Tensor, x_head: int, weight: torch.Tensor, out: torch.Tensor, out_head: int, general: bool = False) -> None:
    """Per head ``h``: ``out[:, h * out_head : h * out_head + N] = x[:, h * x_head : h * x_head + K] @ weight[h].T`` with
    ``weight [heads, N, K]``; ``x`` and ``out`` may be views with longer rows.  bfloat16 with K a multiple of 32 and 16-byte aligned
    rows runs on the matrix cores (``general=True`` forces the general kernel)."""
    G, N, K = weight.shape
    T = x.shape[0]
    if x.dtype != weight.dtype or out.dtype != x.dtype or x.stride(1) != 1 or out.stride(1) != 1 or out.shape[0] != T or not weight.is_contiguous() \
            or x.shape[1] < (G - 1) * x_head + K or out.shape[1] < (G - 1) * out_head + N:
        raise KernelError("heads_linear: shapes or dtypes do not fit")
    lib = _lib("experts")
    _check(lib, lib.tl_grouped_gemm(_ptr(x), c_int(x.stride(0)), c_int(x_head), c_void_p(0), _ptr(weight), _ptr(out), c_int(out.stride(0)),
                                    c_int(out_head), c_void_p(0), c_int(G), c_int(T), c_int(N), c_int(K), c_int(0),
                                    c_int(_dt(x, "heads_linear")), c_int(1 if general else 0), _stream()))


def experts_linear(x: torch.Tensor, slot_token: torch.Tensor | None, weight: torch.Tensor, offsets: torch.Tensor, out: torch.Tensor,
                   activation: str = "none", general: bool = False) -> None:
    """``out[slot] = act(x[row(slot)] @ weight[e].T)`` for the slots ``offsets[e] .. offsets[e + 1] - 1`` of every expert ``e``;
    ``row(slot)`` is ``slot_token[slot]`` (a token routed to the expert) or, without it, the slot itself.  ``weight [experts, N, K]``,
    ``out [slots, N]``, or ``[slots, N / 2]`` for an activation in pairs (columns ``2i`` and ``2i + 1`` of the product give ``act(.) * .``).
    Slots beyond ``offsets[experts]`` (of experts without tensors) are left alone."""
    G, N, K = weight.shape
    S = out.shape[0]
    pairs = ACTIVATIONS[activation] >= 16
    if x.dtype != weight.dtype or out.dtype != x.dtype or x.stride(1) != 1 or x.shape[1] != K or out.shape != (S, N // 2 if pairs else N) \
            or not out.is_contiguous() or not weight.is_contiguous() or (slot_token is None and x.shape[0] != S) or (pairs and N % 2):
        raise KernelError("experts_linear: shapes or dtypes do not fit")
    _i32(offsets, "offsets", G + 1)
    _i32(slot_token, "slot_token", S)
    lib = _lib("experts")
    _check(lib, lib.tl_grouped_gemm(_ptr(x), c_int(x.stride(0)), c_int(0), _ptr(slot_token), _ptr(weight), _ptr(out), c_int(out.shape[1]), c_int(0),
                                    _ptr(offsets), c_int(G), c_int(S), c_int(N), c_int(K), c_int(ACTIVATIONS[activation]),
                                    c_int(_dt(x, "experts_linear")), c_int(1 if general else 0), _stream()))


ROUTER_SCORES = {"chosen": 0, "all": 1, "sigmoid": 2}


def route(logits: torch.Tensor, top: int, scores: str = "chosen", choice_bias: torch.Tensor | None = None, weight_scale: float = 1.0,
          weight_eps: float = 0.0):
    """The router's choice for every row of float32 ``logits [T, experts]`` and the sort of the (token, choice) pairs by expert.
    ``scores="chosen"``: the ``top`` largest logits are chosen and weighed by the softmax over those alone; ``"all"``: the scores are the
    softmax over all logits, the ``top`` largest of score (+ ``choice_bias [experts]``, float32, which enters the choice only) are chosen
    and weighed by their scores as they are; ``"sigmoid"``: the scores are the logits' sigmoids, the choice goes by score (+ ``choice_bias``)
    and the weights are the chosen scores divided by their sum plus ``weight_eps``.  All weights are multiplied by ``weight_scale``.  The
    lower index wins a tie.  Returns ``(weights [T, top] float32, offsets [experts + 1],
    slot_token [T * top], pair_slot [T * top])``, all on the GPU: expert ``e`` owns the slots ``offsets[e] .. offsets[e + 1] - 1``, slot
    ``s`` reads token ``slot_token[s]``, and the output row of token ``t``'s ``j``-th choice is ``pair_slot[t * top + j]``."""
    T, E = logits.shape
    if logits.dtype != torch.float32 or not logits.is_contiguous() or not 0 < top <= min(E, 64) or E > 4096:
        raise KernelError("route: contiguous float32 logits, up to 4096 experts and up to 64 choices")
    if choice_bias is not None and (choice_bias.dtype != torch.float32 or choice_bias.shape != (E,) or not choice_bias.is_contiguous()):
        raise KernelError(f"route: the choice's bias must be contiguous float32 [{E}]")
    ints = torch.empty(T * top * 3 + E + 1, dtype=torch.int32, device=logits.device)
    chosen, slot_token, pair_slot, offsets = ints[: T * top], ints[T * top: 2 * T * top], ints[2 * T * top: 3 * T * top], ints[3 * T * top:]
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    lib = _lib("experts")
    _check(lib, lib.tl_route(_ptr(logits), c_int(T), c_int(E), c_int(top), c_int(ROUTER_SCORES[scores]), _ptr(choice_bias), _ptr(chosen), _ptr(weights),
                             _ptr(offsets), _ptr(slot_token), _ptr(pair_slot), c_float(weight_scale), c_float(weight_eps), _stream()))
    return weights, offsets, slot_token, pair_slot


def combine(y: torch.Tensor, pair_slot: torch.Tensor, weights: torch.Tensor, out: torch.Tensor, identity=None,
            addend: torch.Tensor | None = None) -> None:
    """``out[t] = sum_j weights[t, j] * y[pair_slot[t * top + j]]``, summed in 32-bit in the order of the choices.  ``identity = (x,
    offsets, experts)``: a pair whose slot is ``offsets[experts]`` or later chose an expert without tensors, and ``x[t]`` stands in for
    its row of ``y``.  ``addend [T, W]`` (a shared expert's output) is added last, in 32-bit, before the one rounding."""
    T, top = weights.shape
    W = out.shape[1]
    if y.shape != (T * top, W) or out.shape[0] != T or y.dtype != out.dtype or not y.is_contiguous() or not out.is_contiguous() \
            or weights.dtype != torch.float32 or not weights.is_contiguous():
        raise KernelError("combine: shapes or dtypes do not fit")
    _i32(pair_slot, "pair_slot", T * top)
    x = offsets = None
    experts = 0
    if identity is not None:
        x, offsets, experts = identity
        if x.shape != (T, W) or x.dtype != out.dtype or not x.is_contiguous():
            raise KernelError("combine: the input that stands in for identity experts does not fit")
        _i32(offsets, "offsets", experts + 1)
    if addend is not None and (addend.shape != (T, W) or addend.dtype != out.dtype or not addend.is_contiguous()):
        raise KernelError("combine: the addend does not fit the output")
    lib = _lib("experts")
    _check(lib, lib.tl_combine(_ptr(y), _ptr(pair_slot), _ptr(weights), _ptr(out), _ptr(x), _ptr(offsets), c_int(experts), c_int(T), c_int(top),
                               c_int(W), _ptr(addend), c_int(_dt(out, "combine")), _stream()))


def activation(x: torch.Tensor, kind: str) -> None:
    """The elementwise activation ``kind`` (``relu2``: the square of relu) on contiguous ``x``, in place."""
    if not x.is_contiguous():
        raise KernelError("activation: contiguous tensors only")
    lib = _lib("experts")
    _check(lib, lib.tl_activation(_ptr(x), ctypes.c_long(x.numel()), c_int(ACTIVATIONS[kind]), c_int(_dt(x, "activation")), _stream()))
