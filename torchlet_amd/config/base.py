"""Typed model configurations and the part specifications they expand to.

A configuration class reads an architecture's own ``config.json`` keys, checks them
and expands into a :class:`ModelSpec`: plain data that names, layer by layer, which
mixer, feed-forward, norm and position encoding to build and with which sizes, and
the order in which the layers run.  Parts are built from these specifications only;
none of them sees a configuration or knows which model it is in.
"""
from __future__ import annotations

import dataclasses
import json
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A ``config.json`` that is incomplete, inconsistent or asks for what is not built."""


# ----------------------------------------------------------------------- part specs
# ``kind`` selects the class in the matching registry of ``torchlet_amd.parts``.

@dataclass(frozen=True)
class PartSpec:
    kind: ClassVar[str] = ""


@dataclass(frozen=True)
class RMSNormSpec(PartSpec):
    """``weight_name``: the norm's one tensor below the norm's own name; empty: the tensor bears the norm's name itself."""
    kind: ClassVar[str] = "rmsnorm"
    dim: int = 0
    eps: float = 1e-6
    weight_name: str = "weight"


@dataclass(frozen=True)
class LayerNormSpec(PartSpec):
    """``(x - mean) / sqrt(mean of squared deviations + eps) * weight + bias``.  ``weight_name`` / ``bias_name``: the two tensors
    below the norm's own name; an empty ``weight_name``: the weight bears the norm's name itself."""
    kind: ClassVar[str] = "layernorm"
    dim: int = 0
    eps: float = 1e-5
    weight_name: str = "weight"
    bias_name: str = "bias"


@dataclass(frozen=True)
class ScalarRMSNormSpec(PartSpec):
    """``x / sqrt(mean(x^2) + eps) * g`` with one number ``g`` for all coordinates (a tensor without axes).  ``weight_name`` as in
    :class:`RMSNormSpec`."""
    kind: ClassVar[str] = "scalar_rmsnorm"
    dim: int = 0
    eps: float = 1e-6
    weight_name: str = "weight"


@dataclass(frozen=True)
class OffsetRMSNormSpec(PartSpec):
    """``x / sqrt(mean(x^2) + eps) * (offset + w) * gain`` with a weight vector ``w`` that is stored around zero (``offset`` 1) or as it
    multiplies (``offset`` 0); ``gain``: one more fixed factor (a branch's share of the residual sum, where the norm follows a sublayer).
    The norm folds a normed branch output and a second addend into the stream, so it may stand in blocks that norm their sublayers'
    outputs.  ``weight_name`` as in :class:`RMSNormSpec`."""
    kind: ClassVar[str] = "offset_rmsnorm"
    dim: int = 0
    eps: float = 1e-6
    offset: float = 1.0
    gain: float = 1.0
    weight_name: str = "weight"


@dataclass(frozen=True)
class RotarySpec(PartSpec):
    """Split-half rotary position encoding over the whole head."""
    kind: ClassVar[str] = "rope_split_half"
    head_dim: int = 0
    theta: float = 1_000_000.0
    max_positions: int = 0


@dataclass(frozen=True)
class AttentionSpec(PartSpec):
    """Grouped-query attention over a paged key/value cache."""
    kind: ClassVar[str] = "gqa_attention"
    hidden: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    qkv_bias: bool = True
    window: int | None = None          # None: every earlier key; W: the last W keys
    position: PartSpec | None = None   # position encoding applied to q and k
    scale: float | None = None         # factor on the scores before the softmax; None: head_dim ** -0.5


@dataclass(frozen=True)
class SwiGLUSpec(PartSpec):
    """``down(act(gate(h)) * up(h))`` without biases; ``activation``: ``silu`` or ``relu``; the three matrices' names below the part's."""
    kind: ClassVar[str] = "swiglu"
    hidden: int = 0
    intermediate: int = 0
    activation: str = "silu"
    gate_name: str = "gate_proj.weight"
    up_name: str = "up_proj.weight"
    down_name: str = "down_proj.weight"


@dataclass(frozen=True)
class PairRotarySpec(PartSpec):
    """Rotary position encoding in the interleaved layout: of the first ``dims`` entries of a vector, entry ``2i`` is
    paired with ``2i + 1`` and turned by ``position * base**(-2i / dims)``; what lies beyond ``dims`` passes unchanged."""
    kind: ClassVar[str] = "rope_pairs"
    dims: int = 0
    base: float = 10000.0
    factor: float = 1.0        # linear scaling: every frequency is divided by it


@dataclass(frozen=True)
class HalfRotarySpec(PartSpec):
    """Rotary position encoding in the rotate-half layout over the first ``dims`` entries of a vector: entry ``i`` is paired with
    ``i + dims / 2`` and turned by ``position * base**(-2i / dims) / factor``; what lies beyond ``dims`` passes unchanged."""
    kind: ClassVar[str] = "rope_halves"
    dims: int = 0
    base: float = 10000.0
    factor: float = 1.0
    # ``bands = (factor, low, high, original)``: frequencies are scaled by their wavelength ``2 pi / f`` instead of all alike: shorter
    # than ``original / high`` a frequency stays, longer than ``original / low`` it is divided by ``factor``, and between the two it is
    # ``(1 - s) f / factor + s f`` with ``s = (original / wavelength - low) / (high - low)``
    bands: tuple | None = None


@dataclass(frozen=True)
class MLSTMSpec(PartSpec):
    """Matrix-memory recurrence (the mLSTM of xLSTM): per head a ``dim x vdim`` state with exponential input gate, sigmoid
    forget gate and a running maximum that starts at ``m_start``; gate pre-activations are capped by ``gate_cap * tanh(./gate_cap)``
    (``None``: no cap); the output's denominator is ``max(|n.q|, exp(-m)) + denom_eps``; each head's output is divided by
    its root mean square (``norm_eps``), multiplied by a weight and by a sigmoid gate."""
    kind: ClassVar[str] = "mlstm"
    hidden: int = 0
    heads: int = 0
    dim: int = 0
    vdim: int = 0
    gate_cap: float | None = None
    norm_eps: float = 1e-6
    denom_eps: float = 1e-6
    query_scale: float | None = None     # None: dim ** -0.5


@dataclass(frozen=True)
class LatentAttentionSpec(PartSpec):
    """Attention whose keys and values are up-projections of one cached latent per token (``kv_rank`` numbers, normed) beside one
    rotated key part (``rot_dim`` numbers) that all heads share; queries come through a latent of ``q_rank`` numbers.  ``sink``:
    the softmax's denominator also holds ``exp`` of one learned number per head."""
    kind: ClassVar[str] = "latent_attention"
    hidden: int = 0
    heads: int = 0
    dim: int = 0            # unrotated query/key dimensions per head
    rot_dim: int = 0        # rotated ones
    vdim: int = 0
    kv_rank: int = 0
    q_rank: int = 0
    scale: float = 1.0
    norm_eps: float = 1e-6
    sink: bool = True
    position: PartSpec | None = None     # encoding of the rotated parts
    # ``q_rank`` 0: no query latent, ``q = W_q h`` (tensor ``q``).  ``rot_dim`` 0: no rotated part.  ``window``: a query reads the last
    # ``window`` positions, itself included.  ``gate``: head ``n``'s output is multiplied by ``sigmoid(W_g h)[n]`` (tensor ``g [heads, hidden]``).
    window: int | None = None
    gate: bool = False


@dataclass(frozen=True)
class CappedAttentionSpec(PartSpec):
    """Grouped-query attention over a paged cache whose keys and values differ in size (``dim`` and ``vdim`` per head), without a
    position encoding of its own: ``score = q . k * scale``, then ``score <- softcap * tanh(score / softcap)`` (``None``: no cap);
    query ``i`` reads the keys ``j <= i`` of its own chunk of ``chunk`` positions (chunks are counted from position 0; ``None``:
    no chunks) and, with ``window``, the last ``window`` of them; an ordinary softmax; an output projection without bias."""
    kind: ClassVar[str] = "capped_attention"
    hidden: int = 0
    heads: int = 0
    kv_heads: int = 0
    dim: int = 0
    vdim: int = 0
    scale: float = 1.0
    softcap: float | None = None
    chunk: int | None = None
    window: int | None = None
    # Further mechanisms, each off unless named.  ``position``: a position encoding whose ``turn`` the mixer applies to queries and keys
    # (``rope_pairs`` or ``rope_halves``, over the first dimensions of every head).  ``qk_norm``: queries and keys pass a root-mean-square norm
    # per head before the rotation, with the weights ``q.norm`` and ``k.norm`` of ``dim`` numbers each, shared by all heads (``qk_norm_eps``).
    # ``sink``: the softmax's denominator also holds ``exp`` of one learned number per head (tensor ``sink``), unscaled, without key or
    # value.  ``pool``: with a window, one key and one value (the means of the cached ones) for every block of ``pool`` positions that lies
    # wholly before the window; tokens that have left the window and whose block is not whole yet are not read at all.
    position: PartSpec | None = None
    qk_norm: bool = False
    qk_norm_eps: float = 1e-6
    sink: bool = False
    pool: int | None = None
    # ``keep_first``: beside a window, a query also reads the first ``keep_first`` positions of its sequence (at their own positions).
    # ``values_are_keys``: there is no value projection; the values are the keys as projected (bias added), before norm and rotation.
    # ``qk_bias`` / ``o_bias``: the query and key projections / the output projection have biases (``q.b``, ``k.b``, ``o.b``).
    keep_first: int = 0
    values_are_keys: bool = False
    qk_bias: bool = False
    o_bias: bool = False


@dataclass(frozen=True)
class DecayedLinearSpec(PartSpec):
    """Linear attention with one fixed decay per head (lightning attention): ``q = silu(W_q h)``, ``k = silu(W_k h)`` (``heads x dim``),
    ``v = silu(W_v h)`` (``heads x vdim``); per head ``S <- decay S + k v^T``, ``o = S^T q``; the heads side by side are divided by their
    root mean square together (``norm_eps``), multiplied by a weight vector and by ``sigmoid(W_g h)``, and projected."""
    kind: ClassVar[str] = "decayed_linear"
    hidden: int = 0
    heads: int = 0
    dim: int = 0
    vdim: int = 0
    decay: tuple = ()
    norm_eps: float = 1e-6


@dataclass(frozen=True)
class GatedDeltaSpec(PartSpec):
    """The gated delta rule: per head a ``dim x vdim`` state with ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``,
    ``g = exp(-exp(A_log) softplus(W_a h + dt_bias))`` and ``beta = sigmoid(W_b h)`` per head; queries and keys (``kv_heads`` of them,
    shared by ``heads / kv_heads`` heads each) and values pass a causal convolution of ``conv`` taps per channel and silu; queries and
    keys are made unit vectors (``unit_eps`` under the root), queries times ``query_scale`` (``None``: ``dim ** -0.5``); each head's output is
    divided by its root mean square (``norm_eps``), multiplied by one weight vector of ``vdim`` numbers and by ``silu(W_g h)``."""
    kind: ClassVar[str] = "gated_delta"
    hidden: int = 0
    heads: int = 0
    kv_heads: int = 0
    dim: int = 0
    vdim: int = 0
    conv: int = 4
    norm_eps: float = 1e-6
    unit_eps: float = 1e-6
    query_scale: float | None = None


@dataclass(frozen=True)
class SelectiveStateSpec(PartSpec):
    """A selective state-space recurrence (Mamba-2): one projection gives per token ``[z | x | B | C | dt]`` (``heads * vdim`` twice, ``groups *
    state`` twice, ``heads``); x, B and C pass a causal convolution of ``conv`` taps per channel with a bias, and silu; ``dt <- softplus(dt +
    dt_bias)``; head ``n`` (reading B and C of group ``n // (heads / groups)``) moves its state ``S [state, vdim]`` by ``S <- exp(-exp(A_log) dt) S
    + dt B x^T`` and gives ``y = S^T C + D x``; the heads side by side times ``silu(z)`` are divided by their root mean square in ``norm_groups``
    equal parts (``norm_eps``), multiplied by a weight vector, and projected."""
    kind: ClassVar[str] = "selective_state"
    hidden: int = 0
    heads: int = 0
    vdim: int = 0
    state: int = 0
    groups: int = 1
    conv: int = 4
    norm_groups: int = 1
    norm_eps: float = 1e-6


@dataclass(frozen=True)
class ParallelMixerSpec(PartSpec):
    """Several mixers side by side on the same input: ``sum_i scale_i * mixer_i(h)``.  ``branches``: ``(name, specification, scale)``
    of each; ``name`` is the branch's sub-module name in the checkpoint."""
    kind: ClassVar[str] = "parallel"
    hidden: int = 0
    branches: tuple = ()
    # ``normed``: every branch's projected output is first divided by its root mean square over the model width (``norm_eps``) and
    # multiplied by a weight vector ``<name>.out``: ``sum_i scale_i * rms(mixer_i(h)) * w_i``.
    normed: bool = False
    norm_eps: float = 1e-6


@dataclass(frozen=True)
class DenseFFSpec(PartSpec):
    """``down(act(up(h)))`` with an elementwise activation (``relu2``: the square of relu) and optional biases."""
    kind: ClassVar[str] = "dense_ff"
    hidden: int = 0
    intermediate: int = 0
    activation: str = "relu2"
    bias: bool = True


@dataclass(frozen=True)
class RoutedExpertsSpec(PartSpec):
    """``experts`` small feed-forward layers without biases, ``down(act(up(h)))`` or, ``gated``, ``down(act(gate(h)) * up(h))``; a linear
    router (in 32-bit; ``router_bias``: with a bias) scores them, the ``top`` largest scores per token are chosen and weigh the chosen
    experts' outputs.  ``scores``: ``"chosen"``: the choice goes by the logits and the weights are the softmax over the chosen ones alone;
    ``"all"``: the scores are the softmax over all logits and the weights are the chosen experts' scores as they are; ``"sigmoid"``: the
    scores are the logits' sigmoids and the weights the chosen scores divided by their sum (plus ``weight_eps``).  ``choice_bias``: a
    vector ``correction`` is added to the scores for the choice only.  ``identity``: the router has that many outputs beyond ``experts``;
    an expert chosen among those returns its input.  ``weight_scale``: a factor on the weights.  ``shared``: the specification of one more
    feed-forward (tensors below ``shared``) that runs for every token and is added to the experts' weighted sum."""
    kind: ClassVar[str] = "routed_experts"
    hidden: int = 0
    intermediate: int = 0
    experts: int = 0
    top: int = 1
    activation: str = "relu2"
    router_bias: bool = True
    gated: bool = False
    scores: str = "chosen"
    choice_bias: bool = False
    identity: int = 0
    weight_scale: float = 1.0
    weight_eps: float = 1e-20
    shared: PartSpec | None = None


@dataclass(frozen=True)
class BlockSpec(PartSpec):
    """One layer: a mixer and a feed-forward, each behind its own norm.

    The ``*_name`` fields are the checkpoint's sub-module names of the four parts.
    """
    kind: ClassVar[str] = "prenorm_residual"
    mixer: PartSpec = None            # type: ignore[assignment]
    ffn: PartSpec = None              # type: ignore[assignment]
    mixer_norm: PartSpec = None       # type: ignore[assignment]
    ffn_norm: PartSpec = None         # type: ignore[assignment]
    mixer_name: str = "self_attn"
    ffn_name: str = "mlp"
    mixer_norm_name: str = "input_layernorm"
    ffn_norm_name: str = "post_attention_layernorm"


@dataclass(frozen=True)
class PostNormBlockSpec(BlockSpec):
    """One layer with the norm after the sum: ``x <- norm1(alpha * x + mixer(x))``, then ``x <- norm2(alpha * x + ffn(x))``;
    the sublayers read ``x`` itself.  ``ffn`` (and then ``ffn_norm``) may be ``None``: the layer ends after the first step."""
    kind: ClassVar[str] = "postnorm_residual"
    alpha: float = 1.0


@dataclass(frozen=True)
class SandwichBlockSpec(BlockSpec):
    """One layer with a norm before and after each sublayer: ``x <- x + mixer_post_norm(mixer(mixer_norm(x)))``, then ``x <- x +
    ffn_post_norm(ffn(ffn_norm(x)))``.  ``ffn`` (and then its two norms) may be ``None``."""
    kind: ClassVar[str] = "sandwich_residual"
    mixer_post_norm: PartSpec = None       # type: ignore[assignment]
    ffn_post_norm: PartSpec = None         # type: ignore[assignment]
    mixer_post_norm_name: str = "norm1b"
    ffn_post_norm_name: str = "norm2b"


@dataclass(frozen=True)
class HyperBlockSpec(BlockSpec):
    """One layer over ``streams`` copies of the residual joined by hyper-connections.  Sublayer ``q`` (1: the mixer, 2: the
    feed-forward) has a read vector ``in [streams]``, a matrix ``mix [streams, streams]`` (indexed from, to) and a write vector
    ``out [streams]`` below ``connection_names[q - 1]``: ``u = sum_s in[s] x_s``, ``y = sublayer(norm(u))``, then all streams at once
    ``x_t <- sum_s mix[s, t] x_s + out[t] y``.  ``ffn`` (and then ``ffn_norm``) may be ``None``."""
    kind: ClassVar[str] = "hyper_connections"
    streams: int = 1
    connection_names: tuple = ("hc1", "hc2")


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order: which layer runs, and whose cache it uses.

    ``cache_of`` is ``None`` when this run owns a cache of its own (keyed by its place
    in the order), or the index of an earlier entry of the order whose cache this run
    reads without writing to it.
    """
    layer: int
    cache_of: int | None = None
    add_embedding: bool = False     # the embedding's output (the stream as it was before the first run) is added to the stream before this run


@dataclass(frozen=True)
class HashedBigramSpec:
    """A second embedding table ``[buckets + 1, hidden]`` under ``name`` whose row ``(previous token * mul_prev + token * mul_cur) mod
    buckets`` is added to a token's embedding; a sequence's first token takes the last row.  The previous token is part of a request's state."""
    name: str = "bigram"
    buckets: int = 0
    mul_prev: int = 0
    mul_cur: int = 0


@dataclass(frozen=True)
class ModelSpec:
    """Everything needed to build a decoder: parts, their names, and the run order."""
    vocab_size: int
    hidden: int
    layers: tuple[BlockSpec, ...]
    order: tuple[RunEntry, ...]
    final_norm: PartSpec
    tie_head: bool
    max_positions: int
    embed_name: str = "model.embed_tokens"
    layers_prefix: str = "model.layers"
    final_norm_name: str = "model.norm"
    head_name: str = "lm_head"
    embed_scale: float = 1.0       # factor on the embedding rows as they enter the residual stream
    logit_scale: float = 1.0       # factor on the logits (applied to the final norm's output, in 32-bit)
    head_bias: bool = False        # the output head has a bias vector ``<head_name>.bias``
    weight_suffix: str = "weight"  # the embedding's and the head's matrix below their names; empty: the tensor bears the name itself
    layers_format: str = ""        # the name of layer i as a format string (``"l{}"``); empty: ``<layers_prefix>.<i>``
    position_table_name: str = ""  # a learned table ``[max_positions, hidden]`` whose row of the position is added to the (scaled) embedding; empty: none
    streams: int = 0               # copies of the residual that the blocks keep (hyper-connections); 0: the one plain residual
    bigram: HashedBigramSpec | None = None   # a hashed bigram row added to every token's (scaled) embedding
    embed_norm: PartSpec | None = None       # a norm that the embedding's output passes before it becomes the stream
    embed_norm_name: str = "embed.norm"

    def layer_name(self, i: int) -> str:
        return self.layers_format.format(i) if self.layers_format else f"{self.layers_prefix}.{i}"

    def __post_init__(self):
        for i, e in enumerate(self.order):
            if not 0 <= e.layer < len(self.layers):
                raise ConfigError(f"run order entry {i} names layer {e.layer}; there are {len(self.layers)} layers")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ConfigError(f"run order entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if self.order[e.cache_of].cache_of is not None:
                    raise ConfigError(f"run order entry {i} reads the cache of entry {e.cache_of}, which owns none")


# ------------------------------------------------------------------------- configs

@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's typed configuration.

    Subclasses declare their ``config.json`` keys as dataclass fields (a field without
    a default is required), check them in :meth:`validate` and expand to parts in
    :meth:`to_spec`.
    """

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "ModelConfig":
        d = cls.normalise(dict(d))
        kwargs = {}
        missing = []
        for f in fields(cls):
            if f.name in d and d[f.name] is not None:
                kwargs[f.name] = d[f.name]
            elif f.default is dataclasses.MISSING and f.default_factory is dataclasses.MISSING:
                missing.append(f.name)
        if missing:
            raise ConfigError(f"{cls.architecture}: config.json lacks required key(s): {', '.join(missing)}")
        try:
            cfg = cls(**kwargs)
        except TypeError as exc:  # wrong python type for a field
            raise ConfigError(f"{cls.architecture}: {exc}") from exc
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "ModelConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    @classmethod
    def normalise(cls, d: dict[str, Any]) -> dict[str, Any]:
        """Hook: map alternative spellings of keys onto the fields (default: none)."""
        return d

    def validate(self) -> None:  # pragma: no cover - overridden
        pass

    def to_spec(self) -> ModelSpec:  # pragma: no cover - overridden
        raise NotImplementedError

    def to_dict(self) -> dict[str, Any]:
        """The ``config.json`` content of this configuration."""
        d = {f.name: getattr(self, f.name) for f in fields(self)}
        d["architectures"] = [self.architecture]
        return d

    def save(self, folder: str | Path) -> None:
        Path(folder).mkdir(parents=True, exist_ok=True)
        (Path(folder) / "config.json").write_text(json.dumps(self.to_dict(), indent=2) + "\n")

