"""Configuration of the Fotovik decoder: token embedding times a factor plus a hashed bigram row; layers with a norm before and after
each sublayer (root-mean-square norms with one number as weight); three kinds of mixer: ``attention`` (grouped queries, rotation in
pairs, a window with pooled blocks before it, a sink in the softmax), ``delta`` (the gated delta rule behind short convolutions) and
``parallel`` (causal attention with normed queries and keys and a rotation over halves, beside linear attention with a fixed decay per
head; the two outputs normed over the model width and averaged); a dense feed-forward with the exact gelu, or none; a span of layers
that runs several times in a row, each pass with a cache of its own, the embedding's output entering the stream again before every
pass but the first.

``config.json`` keys: ``architecture`` (``"Fotovik"``), ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``embedding.bigram`` (``buckets``,
``mul_prev``, ``mul_cur``; absent: no bigram table), ``loop`` (``start``, ``stop``, ``times``; absent: every layer once), ``max_positions``
(absent: 2**20) and ``layers``, one entry per layer: ``type``, ``mixer`` and ``mlp`` (``kind`` ``dense`` with ``ff``, or null).  Mixer keys:
attention ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot`` (``dims``, ``base``, ``scaling.factor``; absent: no rotation), ``mask`` (``size``,
``pool``; absent: causal); delta ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``; parallel ``left`` (an attention's keys) and ``right``
(``heads``, ``dim``, ``vdim``, ``decay``).  Tensor names: ``embed``, ``bigram``, ``final.norm``, ``head``, and below ``l<i>.``: ``norm1``, ``norm1b``,
``norm2``, ``norm2b``, ``mix.*``, ``mlp.up``, ``mlp.down``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, ClassVar

from .base import (CappedAttentionSpec, ConfigError, DecayedLinearSpec, DenseFFSpec, GatedDeltaSpec, HalfRotarySpec, HashedBigramSpec,
                   ModelConfig, ModelSpec, PairRotarySpec, ParallelMixerSpec, RunEntry, SandwichBlockSpec, ScalarRMSNormSpec)

ATTENTION_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
DELTA_KEYS = ("heads", "kv_heads", "dim", "vdim", "conv")
LINEAR_KEYS = ("heads", "dim", "vdim", "decay")
MIXER_TYPES = ("attention", "delta", "parallel")


def _positive_int(where: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"Fotovik: {where} must be a positive integer, got {v!r}")
    return v


def _number(where: str, v) -> float:
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"Fotovik: {where} must be a number, got {v!r}")
    return float(v)


def _keys(where: str, m, keys) -> dict:
    missing = [k for k in keys if not isinstance(m, dict) or k not in m]
    if missing:
        raise ConfigError(f"Fotovik: {where} lacks key(s): {', '.join(missing)}")
    return m


@dataclass(frozen=True)
class FotovikConfig(ModelConfig):
    architecture: ClassVar[str] = "Fotovik"

    vocab: int
    width: int
    layers: list
    norm: dict
    embedding: dict = field(default_factory=lambda: {"scale": 1.0})
    loop: dict = field(default_factory=dict)
    max_positions: int = 1 << 20
    torch_dtype: str = ""

    # ------------------------------------------------------------------ checks
    def _check_attention(self, where: str, m) -> None:
        _keys(where, m, ATTENTION_KEYS)
        for k in ("heads", "kv_heads", "dim", "vdim"):
            _positive_int(f"{where}.{k}", m[k])
        if m["heads"] % m["kv_heads"]:
            raise ConfigError(f"Fotovik: {where}: {m['heads']} heads are not a multiple of {m['kv_heads']} key/value heads")
        _number(f"{where}.scale", m["scale"])
        rot = m.get("rot")
        if rot is not None:
            _keys(f"{where}.rot", rot, ("dims", "base"))
            dims = _positive_int(f"{where}.rot.dims", rot["dims"])
            if dims % 2 or dims > m["dim"]:
                raise ConfigError(f"Fotovik: {where}.rot.dims must be even and at most dim ({m['dim']}), got {dims}")
            if not _number(f"{where}.rot.base", rot["base"]) > 0:
                raise ConfigError(f"Fotovik: {where}.rot.base must be positive")
            scaling = rot.get("scaling")
            if scaling is not None and not _number(f"{where}.rot.scaling.factor", (scaling or {}).get("factor")) > 0:
                raise ConfigError(f"Fotovik: {where}.rot.scaling.factor must be positive")
        mask = m.get("mask")
        if mask is not None:
            _positive_int(f"{where}.mask.size", mask.get("size") if isinstance(mask, dict) else None)
            if mask.get("pool") is not None:
                _positive_int(f"{where}.mask.pool", mask["pool"])

    def validate(self) -> None:
        _positive_int("vocab", self.vocab)
        _positive_int("width", self.width)
        _positive_int("max_positions", self.max_positions)
        if not isinstance(self.norm, dict) or not _number("norm.eps", self.norm.get("eps")) > 0:
            raise ConfigError("Fotovik: norm.eps must be a positive number")
        if not isinstance(self.embedding, dict):
            raise ConfigError("Fotovik: 'embedding' must be an object")
        _number("embedding.scale", self.embedding.get("scale", 1.0))
        big = self.embedding.get("bigram")
        if big is not None:
            _keys("embedding.bigram", big, ("buckets", "mul_prev", "mul_cur"))
            _positive_int("embedding.bigram.buckets", big["buckets"])
            for k in ("mul_prev", "mul_cur"):
                if not isinstance(big[k], int) or isinstance(big[k], bool) or big[k] < 0:
                    raise ConfigError(f"Fotovik: embedding.bigram.{k} must be a non-negative integer")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("Fotovik: 'layers' must be a non-empty list")
        if self.loop:
            for k in ("start", "stop", "times"):
                if not isinstance(self.loop.get(k), int) or isinstance(self.loop.get(k), bool):
                    raise ConfigError(f"Fotovik: loop.{k} must be an integer")
            if not 0 <= self.loop["start"] <= self.loop["stop"] <= len(self.layers) or self.loop["times"] < 1:
                raise ConfigError(f"Fotovik: loop {self.loop} does not fit {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind not in MIXER_TYPES:
                raise ConfigError(f"Fotovik: layer {i} has mixer type {kind!r}; built: {', '.join(MIXER_TYPES)}")
            m = layer.get("mixer")
            if kind == "attention":
                self._check_attention(f"layer {i} mixer", m)
            elif kind == "delta":
                _keys(f"layer {i} mixer", m, DELTA_KEYS)
                for k in DELTA_KEYS:
                    _positive_int(f"layer {i} mixer.{k}", m[k])
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"Fotovik: layer {i} mixer: {m['heads']} heads are not a multiple of {m['kv_heads']} query/key heads")
            else:
                _keys(f"layer {i} mixer", m, ("left", "right"))
                self._check_attention(f"layer {i} mixer.left", m["left"])
                right = _keys(f"layer {i} mixer.right", m["right"], LINEAR_KEYS)
                for k in ("heads", "dim", "vdim"):
                    _positive_int(f"layer {i} mixer.right.{k}", right[k])
                if not isinstance(right["decay"], (list, tuple)) or len(right["decay"]) != right["heads"]:
                    raise ConfigError(f"Fotovik: layer {i} mixer.right.decay must list one decay per head")
                for d in right["decay"]:
                    if not 0.0 <= _number(f"layer {i} mixer.right.decay", d) <= 1.0:
                        raise ConfigError(f"Fotovik: layer {i} mixer.right.decay: a decay lies between 0 and 1")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"Fotovik: layer {i} has mlp kind {mlp.get('kind')!r}; built: dense, or null")
                _positive_int(f"layer {i} mlp.ff", mlp.get("ff"))

    # ------------------------------------------------------------------ parts
    def _attention(self, m: dict, layout: str, qk_norm: bool, sink: bool) -> CappedAttentionSpec:
        rot, position = m.get("rot"), None
        if rot is not None:
            factor = float((rot.get("scaling") or {}).get("factor", 1.0))
            cls = PairRotarySpec if layout == "pairs" else HalfRotarySpec
            position = cls(dims=rot["dims"], base=float(rot["base"]), factor=factor)
        mask = m.get("mask") or {}
        return CappedAttentionSpec(hidden=self.width, heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], scale=float(m["scale"]),
                                   window=mask.get("size"), pool=mask.get("pool"), position=position, qk_norm=qk_norm,
                                   qk_norm_eps=float(self.norm["eps"]), sink=sink)

    def _mixer(self, layer: dict):
        m, eps = layer["mixer"], float(self.norm["eps"])
        if layer["type"] == "attention":
            return self._attention(m, "pairs", qk_norm=False, sink=True)
        if layer["type"] == "delta":
            return GatedDeltaSpec(hidden=self.width, heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], conv=m["conv"],
                                  norm_eps=eps, unit_eps=1e-6)
        right = m["right"]
        linear = DecayedLinearSpec(hidden=self.width, heads=right["heads"], dim=right["dim"], vdim=right["vdim"],
                                   decay=tuple(float(d) for d in right["decay"]), norm_eps=eps)
        return ParallelMixerSpec(hidden=self.width, normed=True, norm_eps=eps,
                                 branches=(("left", self._attention(m["left"], "halves", qk_norm=True, sink=False), 0.5), ("right", linear, 0.5)))

    def run_order(self) -> list[RunEntry]:
        n = len(self.layers)
        if not self.loop:
            return [RunEntry(layer=i) for i in range(n)]
        a, b, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        order = [RunEntry(layer=i) for i in range(a)]
        for p in range(times):          # before every pass but the first the embedding's output enters the stream again, once, ahead of the pass's first layer
            order += [RunEntry(layer=i, add_embedding=(p > 0 and i == a)) for i in range(a, b)]
        return order + [RunEntry(layer=i) for i in range(b, n)]

    def to_spec(self) -> ModelSpec:
        norm = ScalarRMSNormSpec(dim=self.width, eps=float(self.norm["eps"]), weight_name="")
        blocks = []
        for layer in self.layers:
            mlp = layer.get("mlp")
            ffn = DenseFFSpec(hidden=self.width, intermediate=mlp["ff"], activation="gelu", bias=False) if mlp is not None else None
            blocks.append(SandwichBlockSpec(mixer=self._mixer(layer), ffn=ffn, mixer_norm=norm, mixer_post_norm=norm,
                                            ffn_norm=norm if ffn is not None else None, ffn_post_norm=norm if ffn is not None else None,
                                            mixer_name="mix", ffn_name="mlp", mixer_norm_name="norm1", ffn_norm_name="norm2",
                                            mixer_post_norm_name="norm1b", ffn_post_norm_name="norm2b"))
        big = self.embedding.get("bigram")
        bigram = HashedBigramSpec(name="bigram", buckets=big["buckets"], mul_prev=big["mul_prev"], mul_cur=big["mul_cur"]) if big else None
        return ModelSpec(vocab_size=self.vocab, hidden=self.width, layers=tuple(blocks), order=tuple(self.run_order()), final_norm=norm,
                         tie_head=False, max_positions=self.max_positions, embed_name="embed", final_norm_name="final.norm", head_name="head",
                         embed_scale=float(self.embedding.get("scale", 1.0)), weight_suffix="", layers_format="l{}", bigram=bigram)

    def to_dict(self) -> dict[str, Any]:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": dict(self.norm),
             "embedding": dict(self.embedding), "layers": [dict(layer) for layer in self.layers]}
        if self.loop:
            d["loop"] = dict(self.loop)
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        if self.torch_dtype:
            d["torch_dtype"] = self.torch_dtype
        return d
