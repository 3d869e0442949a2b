"""Architecture-independent description of a decoder: what the engine builds from.

An architecture's own configuration (for example `Qwen3Config`) is translated
into a `ModelSpec`: a tuple of `LayerSpec`s, each naming its block arrangement,
norm, mixer and feed-forward with every size and constant as a field, plus a
`schedule` that says in which order layers run and which cache each run uses.
Parts are selected by the `kind` strings through `parts.registry`; nothing in
this file knows a model family.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    kind: str = "rmsnorm"
    eps: float = 1e-6


@dataclass(frozen=True)
class PositionSpec:
    """Position encoding of a mixer.  kind "rope": rotate-half pairs (i, i+dim/2)
    with angle = position / theta^(2i/dim); kind "none": no encoding."""
    kind: str = "rope"
    theta: float = 10000.0
    dim: int = 0
    max_positions: int = 0


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a key/value cache."""
    kind: str = "attention"
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    qk_norm: bool = False          # per-head RMSNorm of q and k before the rotation
    qk_norm_eps: float = 1e-6
    window: Optional[int] = None   # None: every earlier key; w: the last w keys
    scale: Optional[float] = None  # None: 1/sqrt(head_dim)
    position: PositionSpec = field(default_factory=PositionSpec)
    value_dim: Optional[int] = None     # None: values as wide as keys
    # biases of the q, k and v projections: None: taken when the checkpoint holds them,
    # True: the checkpoint must hold them, False: it must not
    qkv_bias: Optional[bool] = None
    # "head": RMSNorm of every head with one weight [head_dim]; "projection": one RMSNorm
    # over all heads of q (and of k) together, weights [heads * head_dim]
    qk_norm_scope: str = "head"
    # positions i >= j see each other only if i // chunk == j // chunk, counted from the
    # sequence's position 0 (None: no such blocks)
    chunk: Optional[int] = None
    # r: the score of query i and key j is lowered by 2^(-r (h + 1) / heads) * (i - j) for
    # head h (None: no distance term)
    distance_slope_range: Optional[float] = None
    # a learned number per head that joins the softmax's denominator as exp(sink), with no
    # key and no value
    sink: bool = False

    @property
    def q_width(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.n_kv_heads * self.head_dim

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def v_width(self) -> int:
        return self.n_kv_heads * self.v_dim

    @property
    def out_width(self) -> int:
        return self.n_heads * self.v_dim


@dataclass(frozen=True)
class GatedMLPSpec:
    """down(act(gate(x)) * up(x))."""
    kind: str = "gated_mlp"
    intermediate_size: int = 0
    activation: str = "silu"


@dataclass(frozen=True)
class DenseMLPSpec:
    """down(act(up(x))); activation "relu2" (the square of relu), "relu", "silu" or
    "gelu_tanh"."""
    kind: str = "dense_mlp"
    intermediate_size: int = 0
    activation: str = "relu2"


@dataclass(frozen=True)
class GatedDeltaSpec:
    """Gated delta rule: a recurrent mixer whose state is one [key_dim, value_dim] matrix per
    head, fed through short causal convolutions.  See `parts.delta`."""
    kind: str = "gated_delta"
    n_heads: int = 0              # value heads (one state each)
    n_kv_heads: int = 0           # query/key heads, shared by n_heads / n_kv_heads value heads
    key_dim: int = 0
    value_dim: int = 0
    conv_taps: int = 4            # taps of the causal convolution of q, k and v
    out_norm_eps: float = 1e-6    # eps of the RMS norm of each head's read-out
    unit_eps: float = 1e-6        # q and k become x / sqrt(sum(x^2) + unit_eps) per head

    @property
    def qk_width(self) -> int:
        return self.n_kv_heads * self.key_dim

    @property
    def v_width(self) -> int:
        return self.n_heads * self.value_dim


@dataclass(frozen=True)
class LayerSpec:
    block: str            # arrangement, e.g. "prenorm"
    norm: NormSpec
    mixer: object         # a spec with a .kind (AttentionSpec, or one a test registers)
    feed_forward: object  # a spec with a .kind (GatedMLPSpec, ...), or None: no feed-forward


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `cache` is the id of the cache entry the mixer uses;
    `writes_cache` False means it only reads an entry that another run wrote."""
    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    tie_word_embeddings: bool
    max_position_embeddings: int
    bos_token_id: Optional[int]   # None: the architecture names no such token
    eos_token_id: Optional[int]

    def validate(self) -> None:
        if not self.layers or not self.schedule:
            raise ValueError("a model needs at least one layer and one schedule entry")
        writers = {}
        for entry in self.schedule:
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule names layer {entry.layer} of {len(self.layers)}")
            if entry.writes_cache:
                if entry.cache in writers:
                    raise ValueError(f"cache entry {entry.cache} has two writers")
                writers[entry.cache] = entry.layer
        seen = set()
        for entry in self.schedule:
            if entry.writes_cache:
                seen.add(entry.cache)
            elif entry.cache not in seen:
                raise ValueError(
                    f"layer {entry.layer} reads cache entry {entry.cache} before it is written")


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    """Every layer once, in order, each with a cache entry of its own."""
    return tuple(ScheduleEntry(layer=i, cache=i) for i in range(n_layers))
