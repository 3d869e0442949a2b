"""Typed configuration of the Tirurax decoder, read from config.json keys.

A Tirurax model is a list of layers, each with a mixer of its own kind and sizes and an
optional feed-forward; each sublayer reads the residual stream itself and its output is
RMS-normed before it is added.  config.json:

    architecture   "Tirurax"
    vocab, width   sizes of the table and of the stream
    norm.eps       eps of every RMS norm of the layers
    layers[i]      type     "delta" | "attention"
                   mixer    delta:     heads, kv_heads, dim, vdim, conv (taps)
                            attention: heads, kv_heads, dim, vdim, scale, mask.size
                   mlp      null, or {kind: "dense", ff}

Mixers: `delta` is the gated delta rule (`parts.delta.GatedDelta`); `attention` is
grouped-query attention without rotation, with biased projections, one RMS norm over the
whole query and key projections, a distance term of slope 2^(-8 (h + 1) / heads), chunked
visibility and a sink in the softmax (`parts.attention.Attention` with those options).
The feed-forward is down(relu(up x)^2).  Checkpoint names: `embed`, `l<i>.norm1`,
`l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`, `head`.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .specs import (AttentionSpec, DenseMLPSpec, GatedDeltaSpec, LayerSpec, ModelSpec, NormSpec,
                    PositionSpec, default_schedule)

ARCHITECTURE = "Tirurax"
# constants the design fixes
DISTANCE_SLOPE_RANGE = 8.0     # slope of head h: 2^(-8 (h + 1) / heads)
UNIT_EPS = 1e-6                # q, k of the delta rule: x / sqrt(sum(x^2) + 1e-6)
MAX_POSITIONS = 1 << 30        # no table of positions: a sequence is as long as the cache allows


class TiruraxConfigError(ValueError):
    pass


def _int(source: Mapping[str, Any], key: str, where: str, least: int = 1) -> int:
    if key not in source:
        raise TiruraxConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or int(value) != value \
            or value < least or value > 2**31 - 1:
        raise TiruraxConfigError(f"config.json: {where}.{key} must be an integer of at least "
                                 f"{least}, got {value!r}")
    return int(value)


def _number(source: Mapping[str, Any], key: str, where: str) -> float:
    if key not in source:
        raise TiruraxConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) \
            or value <= 0:
        raise TiruraxConfigError(f"config.json: {where}.{key} must be a positive number, "
                                 f"got {value!r}")
    return float(value)


def _known_keys(source: Mapping[str, Any], known, where: str) -> None:
    """Options this decoder does not implement are refused, never ignored."""
    extra = sorted(set(source) - set(known))
    if extra:
        raise TiruraxConfigError(f"config.json: {where} has keys this decoder does not know: {extra}")


@dataclass(frozen=True)
class TiruraxDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    type = "delta"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "kv_heads", "dim", "vdim", "conv"), where)
        mixer = cls(heads=_int(source, "heads", where), kv_heads=_int(source, "kv_heads", where),
                    dim=_int(source, "dim", where), vdim=_int(source, "vdim", where),
                    conv=_int(source, "conv", where))
        if mixer.heads % mixer.kv_heads:
            raise TiruraxConfigError(f"config.json: {where}.heads must be a multiple of kv_heads")
        return mixer

    def to_dict(self):
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads,
                "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class TiruraxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: Optional[int]        # mask.size; None: every earlier position is visible

    type = "attention"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "kv_heads", "dim", "vdim", "scale", "mask"), where)
        mask = source.get("mask")
        chunk = None
        if mask is not None:
            if not isinstance(mask, dict):
                raise TiruraxConfigError(f"config.json: {where}.mask must be an object")
            _known_keys(mask, ("size",), where + ".mask")
            chunk = _int(mask, "size", where + ".mask")
        mixer = cls(heads=_int(source, "heads", where), kv_heads=_int(source, "kv_heads", where),
                    dim=_int(source, "dim", where), vdim=_int(source, "vdim", where),
                    scale=_number(source, "scale", where), chunk=chunk)
        if mixer.heads % mixer.kv_heads:
            raise TiruraxConfigError(f"config.json: {where}.heads must be a multiple of kv_heads")
        return mixer

    def to_dict(self):
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "scale": self.scale, "vdim": self.vdim}
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        return out


MIXERS = {"delta": TiruraxDelta, "attention": TiruraxAttention}


@dataclass(frozen=True)
class TiruraxLayer:
    mixer: object                # TiruraxDelta | TiruraxAttention
    ff: Optional[int]            # width of the dense feed-forward; None: the layer has none

    @classmethod
    def from_dict(cls, source, where):
        if not isinstance(source, dict):
            raise TiruraxConfigError(f"config.json: {where} must be an object")
        _known_keys(source, ("type", "mixer", "mlp"), where)
        kind = source.get("type")
        if kind not in MIXERS:
            raise TiruraxConfigError(f"config.json: {where}.type must be one of {sorted(MIXERS)}, "
                                     f"got {kind!r}")
        if not isinstance(source.get("mixer"), dict):
            raise TiruraxConfigError(f"config.json: {where} lacks the object 'mixer'")
        mixer = MIXERS[kind].from_dict(source["mixer"], where + ".mixer")
        mlp = source.get("mlp")
        ff = None
        if mlp is not None:
            if not isinstance(mlp, dict):
                raise TiruraxConfigError(f"config.json: {where}.mlp must be an object or null")
            _known_keys(mlp, ("kind", "ff"), where + ".mlp")
            if mlp.get("kind") != "dense":
                raise TiruraxConfigError(f"config.json: {where}.mlp.kind must be 'dense', "
                                         f"got {mlp.get('kind')!r}")
            ff = _int(mlp, "ff", where + ".mlp")
        return cls(mixer=mixer, ff=ff)

    def to_dict(self):
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"},
                "type": self.mixer.type}


@dataclass(frozen=True)
class TiruraxConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[TiruraxLayer, ...]

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "TiruraxConfig":
        # (keys of the top level that the decoder does not know are a file's own notes; inside
        # a layer an unknown key would change what is computed, and is refused)
        norm = source.get("norm")
        if not isinstance(norm, dict):
            raise TiruraxConfigError("config.json lacks the object 'norm'")
        _known_keys(norm, ("eps",), "norm")
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers:
            raise TiruraxConfigError("config.json: 'layers' must be a list of at least one layer")
        return cls(vocab=_int(source, "vocab", "the top level"),
                   width=_int(source, "width", "the top level"),
                   norm_eps=_number(norm, "eps", "norm"),
                   layers=tuple(TiruraxLayer.from_dict(layer, f"layers[{index}]")
                                for index, layer in enumerate(layers)))

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "layers": [layer.to_dict() for layer in self.layers],
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}

    # ------------------------------------------------------------------
    def _mixer_spec(self, mixer):
        if isinstance(mixer, TiruraxDelta):
            return GatedDeltaSpec(n_heads=mixer.heads, n_kv_heads=mixer.kv_heads,
                                  key_dim=mixer.dim, value_dim=mixer.vdim, conv_taps=mixer.conv,
                                  out_norm_eps=self.norm_eps, unit_eps=UNIT_EPS)
        return AttentionSpec(n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, head_dim=mixer.dim,
                             value_dim=mixer.vdim, qk_norm=True, qk_norm_eps=self.norm_eps,
                             qk_norm_scope="projection", qkv_bias=True, scale=mixer.scale, chunk=mixer.chunk,
                             distance_slope_range=DISTANCE_SLOPE_RANGE, sink=True,
                             position=PositionSpec(kind="none"))

    def model_spec(self) -> ModelSpec:
        norm = NormSpec(kind="rmsnorm", eps=self.norm_eps)
        layers = tuple(
            LayerSpec(block="outnorm", norm=norm, mixer=self._mixer_spec(layer.mixer),
                      feed_forward=None if layer.ff is None
                      else DenseMLPSpec(intermediate_size=layer.ff, activation="relu2"))
            for layer in self.layers)
        spec = ModelSpec(architecture=ARCHITECTURE, vocab_size=self.vocab, hidden_size=self.width,
                         layers=layers, schedule=default_schedule(len(layers)), final_norm=norm,
                         tie_word_embeddings=False, max_position_embeddings=MAX_POSITIONS,
                         bos_token_id=None, eos_token_id=None)
        spec.validate()
        return spec

    # ------------------------------------------------------------------
    _ATTENTION_NAMES = {
        "q_proj.weight": "q", "q_proj.bias": "q.b", "k_proj.weight": "k", "k_proj.bias": "k.b",
        "v_proj.weight": "v", "v_proj.bias": "v.b", "o_proj.weight": "o",
        "q_norm.weight": "q.norm", "k_norm.weight": "k.norm", "sink": "sink",
    }
    _DELTA_NAMES = {
        "q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v",
        "q_conv.weight": "q.conv", "k_conv.weight": "k.conv", "v_conv.weight": "v.conv",
        "beta_proj.weight": "b", "decay_proj.weight": "a", "decay_log_rate": "A_log",
        "decay_bias": "dt_bias", "gate_proj.weight": "g", "out_norm.weight": "norm",
        "o_proj.weight": "o",
    }
    _FFN_NAMES = {"up_proj.weight": "up", "down_proj.weight": "down"}

    def checkpoint_name(self, parameter: str) -> str:
        """Name of a model parameter in the checkpoint."""
        top = {"embed.weight": "embed", "final_norm.weight": "final.norm", "head.weight": "head",
               "head.bias": "head.b"}
        if parameter in top:
            return top[parameter]
        parts = parameter.split(".", 3)
        if parts[0] == "layers" and len(parts) == 4 and parts[1].isdigit() \
                and int(parts[1]) < len(self.layers):
            index, part, rest = int(parts[1]), parts[2], parts[3]
            if part in ("norm1", "norm2") and rest == "weight":
                return f"l{index}.{part}"
            if part == "mixer":
                table = (self._DELTA_NAMES if isinstance(self.layers[index].mixer, TiruraxDelta)
                         else self._ATTENTION_NAMES)
                if rest in table:
                    return f"l{index}.mix.{table[rest]}"
                if rest == "o_proj.bias":
                    return f"l{index}.mix.o.b"
            if part == "ffn":
                if rest in self._FFN_NAMES:
                    return f"l{index}.mlp.{self._FFN_NAMES[rest]}"
                if rest.endswith("_proj.bias"):
                    return f"l{index}.mlp.{rest[:-len('_proj.bias')]}.b"
        raise KeyError(f"Tirurax has no checkpoint tensor for parameter '{parameter}'")
