"""Typed configuration of the Zadenex decoder, read from config.json keys.

A Zadenex model is a list of layers, each with a mixer of its own kind and sizes and an
optional gated feed-forward; every sublayer has an RMS norm on its input and another on its
output, and what it adds to the stream is multiplied by `residual_mult`.  A span of layers
may run several times in a row with the same weights (`loop`).  config.json:

    architecture    "Zadenex"
    vocab, width    sizes of the table and of the stream
    embedding.scale the embedding rows are multiplied by it
    norm.eps        eps of every RMS norm
    residual_mult   multiplier of every sublayer's contribution
    loop            null, or {start, stop, times}: layers start .. stop - 1 run `times` times
    layers[i]       type     "mlstm" | "latent_attention" | "attention"
                    mixer    mlstm:            heads, dim, vdim, gate_cap
                             latent_attention: heads, dim, rot_dim, vdim, kv_rank, q_rank, scale,
                                               rot {base, dims}
                             attention:        heads, kv_heads, dim, vdim, scale, mask {size}
                    mlp      null, or {kind: "dense", ff}

Mixers: `mlstm` is the matrix memory with exponential gates (`parts.mlstm.MatrixMemory`);
`latent_attention` caches one latent and one rotated key part a position, with a sink in
the softmax and a sigmoid gate per head on the output (`parts.latent.LatentAttention`);
`attention` is grouped-query attention without rotation, with biased projections, scores
mixed over heads by a learned matrix, a sliding window and a 1 in the softmax's denominator
(`parts.attention.Attention` with those options).  The feed-forward is
down(gelu_tanh(gate x) * up x) with biases.  Checkpoint names: `embed`, `loop.in`, `loop.step`,
`l<i>.norm1`, `l<i>.norm1b`, `l<i>.norm2`, `l<i>.norm2b`, `l<i>.mix.*`, `l<i>.mlp.*`,
`final.norm`, `head`.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .specs import (AttentionSpec, GatedMLPSpec, LatentAttentionSpec, LayerSpec, LoopSpec,
                    MatrixMemorySpec, ModelSpec, NormSpec, PositionSpec, default_schedule,
                    looped_schedule)

ARCHITECTURE = "Zadenex"
# constants the design fixes
BOTTOM_EPS = 1e-6              # added to the matrix memory's denominator
MAX_POSITIONS = 1 << 30        # no table of positions: a sequence is as long as the cache allows


class ZadenexConfigError(ValueError):
    pass


def _int(source: Mapping[str, Any], key: str, where: str, least: int = 1) -> int:
    if key not in source:
        raise ZadenexConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or int(value) != value \
            or value < least or value > 2**31 - 1:
        raise ZadenexConfigError(f"config.json: {where}.{key} must be an integer of at least "
                                 f"{least}, got {value!r}")
    return int(value)


def _number(source: Mapping[str, Any], key: str, where: str) -> float:
    if key not in source:
        raise ZadenexConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) \
            or value <= 0:
        raise ZadenexConfigError(f"config.json: {where}.{key} must be a positive number, "
                                 f"got {value!r}")
    return float(value)


def _object(source: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = source.get(key)
    if not isinstance(value, dict):
        raise ZadenexConfigError(f"config.json: {where} lacks the object '{key}'")
    return value


def _known_keys(source: Mapping[str, Any], known, where: str) -> None:
    """Options this decoder does not implement are refused, never ignored."""
    extra = sorted(set(source) - set(known))
    if extra:
        raise ZadenexConfigError(f"config.json: {where} has keys this decoder does not know: {extra}")


@dataclass(frozen=True)
class ZadenexMatrixMemory:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    type = "mlstm"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "dim", "vdim", "gate_cap"), where)
        return cls(heads=_int(source, "heads", where), dim=_int(source, "dim", where),
                   vdim=_int(source, "vdim", where), gate_cap=_number(source, "gate_cap", where))

    def to_dict(self):
        return {"dim": self.dim, "gate_cap": self.gate_cap, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ZadenexLatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float
    rot_dims: int

    type = "latent_attention"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot"),
                    where)
        rot = _object(source, "rot", where)
        _known_keys(rot, ("base", "dims"), where + ".rot")
        mixer = cls(heads=_int(source, "heads", where), dim=_int(source, "dim", where),
                    rot_dim=_int(source, "rot_dim", where), vdim=_int(source, "vdim", where),
                    kv_rank=_int(source, "kv_rank", where), q_rank=_int(source, "q_rank", where),
                    scale=_number(source, "scale", where),
                    rot_base=_number(rot, "base", where + ".rot"),
                    rot_dims=_int(rot, "dims", where + ".rot"))
        if mixer.rot_dims != mixer.rot_dim or mixer.rot_dim % 2:
            raise ZadenexConfigError(f"config.json: {where}: the rotation covers the whole rotated "
                                     "part, so rot.dims must equal rot_dim, and both be even")
        return mixer

    def to_dict(self):
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank,
                "q_rank": self.q_rank, "rot": {"base": self.rot_base, "dims": self.rot_dims},
                "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class ZadenexAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]       # mask.size; None: every earlier position is visible

    type = "attention"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "kv_heads", "dim", "vdim", "scale", "mask"), where)
        mask = source.get("mask")
        window = None
        if mask is not None:
            if not isinstance(mask, dict):
                raise ZadenexConfigError(f"config.json: {where}.mask must be an object")
            _known_keys(mask, ("size",), where + ".mask")
            window = _int(mask, "size", where + ".mask")
        mixer = cls(heads=_int(source, "heads", where), kv_heads=_int(source, "kv_heads", where),
                    dim=_int(source, "dim", where), vdim=_int(source, "vdim", where),
                    scale=_number(source, "scale", where), window=window)
        if mixer.heads % mixer.kv_heads:
            raise ZadenexConfigError(f"config.json: {where}.heads must be a multiple of kv_heads")
        return mixer

    def to_dict(self):
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "scale": self.scale, "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


MIXERS = {"mlstm": ZadenexMatrixMemory, "latent_attention": ZadenexLatentAttention,
          "attention": ZadenexAttention}


@dataclass(frozen=True)
class ZadenexLayer:
    mixer: object                # one of the three mixer configurations
    ff: Optional[int]            # width of the gated feed-forward; None: the layer has none

    @classmethod
    def from_dict(cls, source, where):
        if not isinstance(source, dict):
            raise ZadenexConfigError(f"config.json: {where} must be an object")
        _known_keys(source, ("type", "mixer", "mlp"), where)
        kind = source.get("type")
        if kind not in MIXERS:
            raise ZadenexConfigError(f"config.json: {where}.type must be one of {sorted(MIXERS)}, "
                                     f"got {kind!r}")
        mixer = MIXERS[kind].from_dict(_object(source, "mixer", where), where + ".mixer")
        mlp = source.get("mlp")
        ff = None
        if mlp is not None:
            if not isinstance(mlp, dict):
                raise ZadenexConfigError(f"config.json: {where}.mlp must be an object or null")
            _known_keys(mlp, ("kind", "ff"), where + ".mlp")
            if mlp.get("kind") != "dense":
                raise ZadenexConfigError(f"config.json: {where}.mlp.kind must be 'dense', "
                                         f"got {mlp.get('kind')!r}")
            ff = _int(mlp, "ff", where + ".mlp")
        return cls(mixer=mixer, ff=ff)

    def to_dict(self):
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"},
                "type": self.mixer.type}


@dataclass(frozen=True)
class ZadenexConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    layers: Tuple[ZadenexLayer, ...]
    loop: Optional[Tuple[int, int, int]] = None      # (start, stop, times)

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "ZadenexConfig":
        # (keys of the top level that the decoder does not know are a file's own notes; inside
        # a layer an unknown key would change what is computed, and is refused)
        norm = _object(source, "norm", "the top level")
        _known_keys(norm, ("eps",), "norm")
        embedding = _object(source, "embedding", "the top level")
        _known_keys(embedding, ("scale",), "embedding")
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ZadenexConfigError("config.json: 'layers' must be a list of at least one layer")
        loop = source.get("loop")
        span = None
        if loop is not None:
            if not isinstance(loop, dict):
                raise ZadenexConfigError("config.json: 'loop' must be an object or null")
            _known_keys(loop, ("start", "stop", "times"), "loop")
            span = (_int(loop, "start", "loop", least=0), _int(loop, "stop", "loop"),
                    _int(loop, "times", "loop"))
            if not span[0] < span[1] <= len(layers):
                raise ZadenexConfigError(f"config.json: loop.start < loop.stop <= {len(layers)} "
                                         f"must hold, got {span[0]} and {span[1]}")
        return cls(vocab=_int(source, "vocab", "the top level"),
                   width=_int(source, "width", "the top level"),
                   norm_eps=_number(norm, "eps", "norm"),
                   embedding_scale=_number(embedding, "scale", "embedding"),
                   residual_mult=_number(source, "residual_mult", "the top level"),
                   layers=tuple(ZadenexLayer.from_dict(layer, f"layers[{index}]")
                                for index, layer in enumerate(layers)),
                   loop=span)

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers],
                "loop": None if self.loop is None else
                {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]},
                "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
                "vocab": self.vocab, "width": self.width}

    # ------------------------------------------------------------------
    def _mixer_spec(self, mixer):
        if isinstance(mixer, ZadenexMatrixMemory):
            return MatrixMemorySpec(n_heads=mixer.heads, key_dim=mixer.dim, value_dim=mixer.vdim,
                                    gate_cap=mixer.gate_cap, out_norm_eps=self.norm_eps,
                                    bottom_eps=BOTTOM_EPS)
        if isinstance(mixer, ZadenexLatentAttention):
            return LatentAttentionSpec(
                n_heads=mixer.heads, head_dim=mixer.dim, rot_dim=mixer.rot_dim,
                value_dim=mixer.vdim, kv_rank=mixer.kv_rank, q_rank=mixer.q_rank,
                scale=mixer.scale, norm_eps=self.norm_eps, sink=True, output_gate=True,
                position=PositionSpec(kind="rope_pairs", theta=mixer.rot_base, dim=mixer.rot_dims))
        return AttentionSpec(n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, head_dim=mixer.dim,
                             value_dim=mixer.vdim, qk_norm=False, qkv_bias=True, o_bias=True,
                             scale=mixer.scale, window=mixer.window, unit_sink=True,
                             talking_heads=True, position=PositionSpec(kind="none"))

    def model_spec(self) -> ModelSpec:
        norm = NormSpec(kind="rmsnorm", eps=self.norm_eps)
        layers = tuple(
            LayerSpec(block="sandwich", norm=norm, mixer=self._mixer_spec(layer.mixer),
                      feed_forward=None if layer.ff is None
                      else GatedMLPSpec(intermediate_size=layer.ff, activation="gelu_tanh",
                                        bias=True),
                      residual_scale=self.residual_mult)
            for layer in self.layers)
        loop = None if self.loop is None else LoopSpec(*self.loop)
        schedule = (default_schedule(len(layers)) if loop is None
                    else looped_schedule(len(layers), loop))
        spec = ModelSpec(architecture=ARCHITECTURE, vocab_size=self.vocab, hidden_size=self.width,
                         layers=layers, schedule=schedule, final_norm=norm,
                         tie_word_embeddings=False, max_position_embeddings=MAX_POSITIONS,
                         bos_token_id=None, eos_token_id=None,
                         embedding_scale=self.embedding_scale, loop=loop)
        spec.validate()
        return spec

    # ------------------------------------------------------------------
    _MIXER_NAMES = {
        "mlstm": {
            "q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v",
            "in_gate.weight": "i", "in_gate.bias": "i.b", "forget_gate.weight": "f",
            "forget_gate.bias": "f.b", "gate_proj.weight": "g", "out_norm.weight": "norm",
            "o_proj.weight": "o",
        },
        "latent_attention": {
            "q_down.weight": "dq", "q_down_norm.weight": "dq.norm", "q_up.weight": "uq",
            "kv_down.weight": "dkv", "kv_down_norm.weight": "dkv.norm", "k_up.weight": "uk",
            "v_up.weight": "uv", "sink": "sink", "gate_proj.weight": "g", "o_proj.weight": "o",
        },
        "attention": {
            "q_proj.weight": "q", "q_proj.bias": "q.b", "k_proj.weight": "k", "k_proj.bias": "k.b",
            "v_proj.weight": "v", "v_proj.bias": "v.b", "o_proj.weight": "o", "o_proj.bias": "o.b",
            "talk": "talk",
        },
    }
    _FFN_NAMES = {"gate_proj.weight": "gate", "gate_proj.bias": "gate.b", "up_proj.weight": "up",
                  "up_proj.bias": "up.b", "down_proj.weight": "down", "down_proj.bias": "down.b"}

    def checkpoint_name(self, parameter: str) -> str:
        """Name of a model parameter in the checkpoint."""
        top = {"embed.weight": "embed", "final_norm.weight": "final.norm", "head.weight": "head",
               "head.bias": "head.b", "loop.in.weight": "loop.in", "loop.step": "loop.step"}
        if parameter in top:
            return top[parameter]
        parts = parameter.split(".", 3)
        if parts[0] == "layers" and len(parts) == 4 and parts[1].isdigit() \
                and int(parts[1]) < len(self.layers):
            index, part, rest = int(parts[1]), parts[2], parts[3]
            if part in ("norm1", "norm1b", "norm2", "norm2b") and rest == "weight":
                return f"l{index}.{part}"
            if part == "mixer":
                table = self._MIXER_NAMES[self.layers[index].mixer.type]
                if rest in table:
                    return f"l{index}.mix.{table[rest]}"
            if part == "ffn" and rest in self._FFN_NAMES:
                return f"l{index}.mlp.{self._FFN_NAMES[rest]}"
        raise KeyError(f"Zadenex has no checkpoint tensor for parameter '{parameter}'")
