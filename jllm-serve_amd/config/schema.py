"""Typed description of a model: what config.json says, turned into per-layer specs.

The shapes follow the reference's records: ``Architecture.Core`` (model/Architecture.java:61-67),
``LayerSpec`` (model/LayerSpec.java:11-55), ``Attention.Gqa`` (model/Attention.java:48-115),
``Mlp.Dense`` (model/Mlp.java:7-22), ``RopeTable`` (model/RopeTable.java:20-52) and ``Scaling``
(model/Scaling.java:6-78). A family's switches are written into the per-layer specs, so nothing
below the parser ever looks at ``model_type`` (model/Architecture.java:17-20).

Every spec carries a ``kind`` string. The parts registry maps a kind to the class that runs it, so a
new mixer / feed-forward / norm / position encoding is a new spec class plus a registered part.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Sequence, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be turned into a model (the reference's IllegalArgumentException)."""


# --------------------------------------------------------------------------- position encodings


@dataclass(frozen=True)
class RopeScaling:
    """Frequency rescaling of a rotary table (model/Scaling.java:6-78)."""

    kind: str = "none"  # none | linear | llama3 | yarn
    factor: float = 1.0
    original_max_positions: int = 0
    low_freq_factor: float = 1.0  # llama3
    high_freq_factor: float = 4.0  # llama3
    beta_fast: float = 32.0  # yarn
    beta_slow: float = 1.0  # yarn
    mscale: float = 1.0  # yarn
    mscale_all_dim: float = 0.0  # yarn
    attention_factor: float = 0.0  # yarn: 0 = derive from factor
    truncate: bool = True  # yarn


@dataclass(frozen=True)
class RopeSpec:
    """One rotary table (model/RopeTable.java:20-52). ``pairing`` "half" rotates (i, i + rotary_dim/2)."""

    rotary_dim: int
    theta: float
    scaling: RopeScaling = RopeScaling()
    pairing: str = "half"
    kind: str = "rope"

    def __post_init__(self):
        # model/RopeTable.java:40-42
        if self.rotary_dim < 2 or self.rotary_dim % 2 != 0 or not (self.theta > 0):
            raise ConfigError(f"invalid rope table: rotary_dim={self.rotary_dim} theta={self.theta}")


# --------------------------------------------------------------------------- norms


@dataclass(frozen=True)
class NormSpec:
    """RMSNorm with a plain gain (no 1+w) and the model's eps (model/Families.java:663, :793)."""

    eps: float
    kind: str = "rmsnorm"


# --------------------------------------------------------------------------- mixers


@dataclass(frozen=True)
class GqaNames:
    """Where the tensors of an attention layer are found in the checkpoint, relative to the layer's prefix and
    without the ``.weight`` / ``.bias`` ending (the reference keeps such a table per family as conversion rules,
    model/ModelConverter.java:38-49). ``qkv``: one tensor stacked [q | k | v] along the output rows, in place of
    the three."""

    q: str = "self_attn.q_proj"
    k: str = "self_attn.k_proj"
    v: str = "self_attn.v_proj"
    o: str = "self_attn.o_proj"
    q_norm: str = "self_attn.q_norm"
    k_norm: str = "self_attn.k_norm"
    qkv: Optional[str] = None


@dataclass(frozen=True)
class GqaSpec:
    """Grouped-query attention of one layer (model/Attention.java:48-115).

    ``window`` 0 means every earlier key is visible; otherwise the query at position p sees keys
    [max(0, p + 1 - window), p] (model/Attention.java:68-71). ``position`` indexes ModelConfig.positions
    (None = no position encoding). ``qk_norm``: per-head RMSNorm of q and k before the rotation with
    gains shared by all heads (model/Families.java:168).
    """

    heads: int
    kv_heads: int
    head_dim: int
    scale: float
    window: int = 0
    position: Optional[int] = 0
    qk_norm: bool = False
    qk_norm_eps: float = 1e-6
    bias: bool = False
    out_bias: bool = False
    names: GqaNames = GqaNames()
    kind: str = "gqa"

    @property
    def q_dim(self) -> int:
        return self.heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.kv_heads * self.head_dim

    @property
    def group(self) -> int:
        return self.heads // self.kv_heads


# --------------------------------------------------------------------------- feed-forwards


@dataclass(frozen=True)
class GatedMlpNames:
    """Tensor names of a gated feed-forward under the layer's prefix, without ``.weight``. ``gate_up``: one tensor
    stacked [gate | up] along the output rows, in place of the two."""

    gate: str = "mlp.gate_proj"
    up: str = "mlp.up_proj"
    down: str = "mlp.down_proj"
    gate_up: Optional[str] = None


@dataclass(frozen=True)
class GatedMlpSpec:
    """Dense gated feed-forward: down(act(gate x) * up x) (model/Mlp.java:7-22)."""

    hidden: int
    activation: str = "silu"
    names: GatedMlpNames = GatedMlpNames()
    kind: str = "gated_mlp"


# --------------------------------------------------------------------------- layers and model


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: which mixer, which feed-forward, which norms, and how they are arranged.

    ``arrangement`` "prenorm": x += mixer(norm(x)); x += ffn(norm(x)) (model/LayerSpec.java:18-19,
    cpu/CpuBackend.java:959-969). ``prefix`` is the tensor-name prefix of the layer's weights; the names under it
    are data of the specs (here the two norms', in the mixer's and feed-forward's specs theirs), so a checkpoint
    that names or stacks its tensors differently is a matter of the parser.
    """

    mixer: Any
    ffn: Any
    norm: Any
    prefix: str
    arrangement: str = "prenorm"
    norm_in_name: str = "input_layernorm"  # under the prefix, without ``.weight``
    norm_post_name: str = "post_attention_layernorm"


@dataclass(frozen=True)
class ScheduleEntry:
    """One step of the layer schedule: run ``layer``; ``cache_from`` names an earlier schedule entry
    whose cache this run reads instead of writing one of its own (None = its own cache)."""

    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelNames:
    """The checkpoint's names of the tensors outside the layers."""

    embed: str = "model.embed_tokens.weight"
    final_norm: str = "model.norm.weight"
    head: str = "lm_head.weight"


@dataclass(frozen=True)
class ModelConfig:
    """The typed result of config.json (model/Architecture.java:61-67 plus model/Decoder.java:15-33)."""

    architecture: str
    model_type: str
    hidden: int
    vocab: int
    final_norm: Any
    layers: Tuple[LayerSpec, ...]
    positions: Tuple[Any, ...]
    schedule: Tuple[ScheduleEntry, ...]
    tie_embeddings: bool = False
    bos_token_id: int = -1
    eos_token_ids: Tuple[int, ...] = ()
    max_positions: int = 4096
    embed_scale: float = 1.0
    description: str = ""
    names: ModelNames = ModelNames()
    raw: Mapping[str, Any] = field(default_factory=dict, compare=False, repr=False)

    def __post_init__(self):
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ConfigError(f"schedule entry {i} names layer {e.layer}, the model has {n}")
            if e.cache_from is not None and not 0 <= e.cache_from < i:
                raise ConfigError(f"schedule entry {i} reads the cache of entry {e.cache_from}, which does not run before it")

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    return tuple(ScheduleEntry(i) for i in range(n_layers))


def flatten(values: Sequence[Any]) -> str:
    return ",".join(str(v) for v in values)
