"""Configuration of the Bafulorn decoder: a normed token embedding; layers with a norm before and after each sublayer whose outputs
enter the stream times a fixed factor, ``x <- x + m * post(sublayer(pre(x)))``, every norm a root-mean-square norm whose weight vector is
stored around zero; three kinds of mixer: ``latent_attention`` (attention over one cached latent per token, without positions, inside a
window, each head's output times a sigmoid gate), ``attention`` (grouped queries with biases, the values being the keys as projected, a
rotation over the first dimensions of a head in the rotate-half layout with frequencies scaled by wavelength, a window that also keeps
the first tokens) and ``mamba2`` (a selective state-space recurrence behind a short convolution, gated and normed in groups); a
feed-forward that is dense and gated (relu), routed over gated experts (silu) by a sigmoid router with a shared expert, or absent.

``config.json`` keys: ``architecture`` (``"Bafulorn"``), ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``max_positions`` (absent: 2**20) and
``layers``, one entry per layer: ``type``, ``mixer`` and ``mlp``.  Mixer keys: latent_attention ``heads``, ``dim``, ``vdim``, ``kv_rank``, ``scale``,
``mask.size`` (absent: causal); attention ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot`` (``dims``, ``base``, ``scaling`` with ``factor``, ``low``,
``high``, ``original``; absent: no rotation / no scaling), ``mask`` (``size``, ``keep_first``; absent: causal); mamba2 ``heads``, ``vdim``, ``state``,
``groups``, ``conv``, ``norm_groups``.  ``mlp``: ``kind`` ``dense`` with ``ff``; ``kind`` ``moe`` with ``expert.ff``, ``router`` (``experts``, ``top``, ``scale``) and
``shared.ff`` (absent: no shared expert); or null.  Tensor names: ``embed``, ``embed.norm``, ``final.norm``, ``head``, and below ``l<i>.``: ``norm1``,
``norm1b``, ``norm2``, ``norm2b``, ``mix.*``, ``mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import (CappedAttentionSpec, ConfigError, HalfRotarySpec, LatentAttentionSpec, ModelConfig, ModelSpec, OffsetRMSNormSpec,
                   RoutedExpertsSpec, RunEntry, SandwichBlockSpec, SelectiveStateSpec, SwiGLUSpec)

MIXER_KEYS = {
    "latent_attention": ("heads", "dim", "vdim", "kv_rank", "scale"),
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale"),
    "mamba2": ("heads", "vdim", "state", "groups", "conv", "norm_groups"),
}
SCALING_KEYS = ("factor", "low", "high", "original")


def _positive_int(where: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"Bafulorn: {where} must be a positive integer, got {v!r}")
    return v


def _number(where: str, v) -> float:
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"Bafulorn: {where} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class BafulornConfig(ModelConfig):
    architecture: ClassVar[str] = "Bafulorn"

    vocab: int
    width: int
    layers: list
    norm: dict
    residual_mult: float = 1.0
    max_positions: int = 1 << 20
    torch_dtype: str = ""

    # ------------------------------------------------------------------ checks
    def _check_mask(self, where: str, m: dict, keep_first: bool) -> None:
        mask = m.get("mask")
        if mask is None:
            return
        if not isinstance(mask, dict):
            raise ConfigError(f"Bafulorn: {where}.mask must be an object")
        _positive_int(f"{where}.mask.size", mask.get("size"))
        kept = mask.get("keep_first", 0)
        if not isinstance(kept, int) or isinstance(kept, bool) or kept < 0 or (kept and not keep_first):
            raise ConfigError(f"Bafulorn: {where}.mask.keep_first must be a non-negative integer (and only an attention mixer keeps first tokens)")

    def _check_mixer(self, i: int, kind: str, m) -> None:
        where = f"layer {i} mixer"
        missing = [k for k in MIXER_KEYS[kind] if not isinstance(m, dict) or k not in m]
        if missing:
            raise ConfigError(f"Bafulorn: layer {i} ({kind}) lacks mixer key(s): {', '.join(missing)}")
        for k in MIXER_KEYS[kind]:
            if k == "scale":
                _number(f"{where}.scale", m[k])
            else:
                _positive_int(f"{where}.{k}", m[k])
        if kind == "latent_attention":
            self._check_mask(where, m, keep_first=False)
        elif kind == "attention":
            if m["heads"] % m["kv_heads"]:
                raise ConfigError(f"Bafulorn: {where}: {m['heads']} heads are not a multiple of {m['kv_heads']} key/value heads")
            if m["vdim"] != m["dim"]:
                raise ConfigError(f"Bafulorn: {where}: the values are the keys, so vdim ({m['vdim']}) must equal dim ({m['dim']})")
            self._check_mask(where, m, keep_first=True)
            rot = m.get("rot")
            if rot is not None:
                if not isinstance(rot, dict) or "dims" not in rot or "base" not in rot:
                    raise ConfigError(f"Bafulorn: {where}.rot needs 'dims' and 'base'")
                dims = _positive_int(f"{where}.rot.dims", rot["dims"])
                if dims % 2 or dims > m["dim"]:
                    raise ConfigError(f"Bafulorn: {where}.rot.dims must be even and at most dim ({m['dim']}), got {dims}")
                if not _number(f"{where}.rot.base", rot["base"]) > 0:
                    raise ConfigError(f"Bafulorn: {where}.rot.base must be positive")
                scaling = rot.get("scaling")
                if scaling is not None:
                    if not isinstance(scaling, dict) or any(k not in scaling for k in SCALING_KEYS):
                        raise ConfigError(f"Bafulorn: {where}.rot.scaling needs {', '.join(SCALING_KEYS)}")
                    factor, low, high, original = (_number(f"{where}.rot.scaling.{k}", scaling[k]) for k in SCALING_KEYS)
                    if not (factor > 0 and original > 0 and 0 < low < high):
                        raise ConfigError(f"Bafulorn: {where}.rot.scaling wants factor > 0, original > 0 and 0 < low < high")
        else:
            if m["heads"] % m["groups"]:
                raise ConfigError(f"Bafulorn: {where}: {m['heads']} heads are not a multiple of {m['groups']} groups")
            if (m["heads"] * m["vdim"]) % m["norm_groups"]:
                raise ConfigError(f"Bafulorn: {where}: {m['heads'] * m['vdim']} inner channels do not split into {m['norm_groups']} equal parts")

    def validate(self) -> None:
        _positive_int("vocab", self.vocab)
        _positive_int("width", self.width)
        _positive_int("max_positions", self.max_positions)
        _number("residual_mult", self.residual_mult)
        if not isinstance(self.norm, dict) or not _number("norm.eps", self.norm.get("eps")) > 0:
            raise ConfigError("Bafulorn: norm.eps must be a positive number")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("Bafulorn: 'layers' must be a non-empty list")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind not in MIXER_KEYS:
                raise ConfigError(f"Bafulorn: layer {i} has mixer type {kind!r}; built: {', '.join(sorted(MIXER_KEYS))}")
            self._check_mixer(i, kind, layer.get("mixer"))
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                raise ConfigError(f"Bafulorn: layer {i} has mlp kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r}; built: dense, moe, or null")
            if mlp["kind"] == "dense":
                _positive_int(f"layer {i} mlp.ff", mlp.get("ff"))
                continue
            _positive_int(f"layer {i} mlp.expert.ff", (mlp.get("expert") or {}).get("ff"))
            router = mlp.get("router") or {}
            experts, top = _positive_int(f"layer {i} mlp.router.experts", router.get("experts")), _positive_int(f"layer {i} mlp.router.top", router.get("top"))
            if top > experts:
                raise ConfigError(f"Bafulorn: layer {i} picks {top} of {experts} experts")
            _number(f"layer {i} mlp.router.scale", router.get("scale", 1.0))
            if mlp.get("shared") is not None:
                _positive_int(f"layer {i} mlp.shared.ff", (mlp.get("shared") or {}).get("ff"))

    # ------------------------------------------------------------------ parts
    def _mixer(self, layer: dict):
        m, eps = layer["mixer"], float(self.norm["eps"])
        mask = m.get("mask") or {}
        if layer["type"] == "latent_attention":
            return LatentAttentionSpec(hidden=self.width, heads=m["heads"], dim=m["dim"], rot_dim=0, vdim=m["vdim"], kv_rank=m["kv_rank"], q_rank=0,
                                       scale=float(m["scale"]), norm_eps=eps, sink=False, position=None, window=mask.get("size"), gate=True)
        if layer["type"] == "attention":
            rot, position = m.get("rot"), None
            if rot is not None:
                scaling = rot.get("scaling")
                bands = tuple(float(scaling[k]) for k in SCALING_KEYS) if scaling is not None else None
                position = HalfRotarySpec(dims=rot["dims"], base=float(rot["base"]), bands=bands)
            return CappedAttentionSpec(hidden=self.width, heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], scale=float(m["scale"]),
                                       window=mask.get("size"), keep_first=int(mask.get("keep_first", 0)) if mask else 0, position=position,
                                       values_are_keys=True, qk_bias=True, o_bias=True)
        return SelectiveStateSpec(hidden=self.width, heads=m["heads"], vdim=m["vdim"], state=m["state"], groups=m["groups"], conv=m["conv"],
                                  norm_groups=m["norm_groups"], norm_eps=eps)

    def _gated(self, ff: int, activation: str) -> SwiGLUSpec:
        return SwiGLUSpec(hidden=self.width, intermediate=ff, activation=activation, gate_name="gate", up_name="up", down_name="down")

    def _ffn(self, layer: dict):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        if mlp["kind"] == "dense":
            return self._gated(mlp["ff"], "relu")
        router, shared = mlp["router"], mlp.get("shared")
        return RoutedExpertsSpec(hidden=self.width, intermediate=mlp["expert"]["ff"], experts=router["experts"], top=router["top"], activation="silu",
                                 router_bias=False, gated=True, scores="sigmoid", choice_bias=True, weight_scale=float(router.get("scale", 1.0)),
                                 weight_eps=1e-20, shared=self._gated(shared["ff"], "silu") if shared is not None else None)

    def to_spec(self) -> ModelSpec:
        eps, mult = float(self.norm["eps"]), float(self.residual_mult)
        pre = OffsetRMSNormSpec(dim=self.width, eps=eps, offset=1.0, weight_name="")
        post = OffsetRMSNormSpec(dim=self.width, eps=eps, offset=1.0, gain=mult, weight_name="")      # the branch's factor rides on its norm's weight
        blocks = []
        for layer in self.layers:
            ffn = self._ffn(layer)
            blocks.append(SandwichBlockSpec(mixer=self._mixer(layer), ffn=ffn, mixer_norm=pre, mixer_post_norm=post,
                                            ffn_norm=pre if ffn is not None else None, ffn_post_norm=post if ffn is not None else None,
                                            mixer_name="mix", ffn_name="mlp", mixer_norm_name="norm1", ffn_norm_name="norm2",
                                            mixer_post_norm_name="norm1b", ffn_post_norm_name="norm2b"))
        return ModelSpec(vocab_size=self.vocab, hidden=self.width, layers=tuple(blocks), order=tuple(RunEntry(layer=i) for i in range(len(blocks))),
                         final_norm=pre, tie_head=False, max_positions=self.max_positions, embed_name="embed", final_norm_name="final.norm",
                         head_name="head", weight_suffix="", layers_format="l{}", embed_norm=pre, embed_norm_name="embed.norm")

    def to_dict(self) -> dict[str, Any]:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": dict(self.norm),
             "residual_mult": self.residual_mult, "layers": [dict(layer) for layer in self.layers]}
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        if self.torch_dtype:
            d["torch_dtype"] = self.torch_dtype
        return d
