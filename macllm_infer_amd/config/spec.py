"""Typed, format-neutral description of a decoder: which parts each layer is made of,
with every size and constant as a field, and the order in which layers run.

An architecture's config class (for example ``FalconH1Config``) lowers its own
``config.json`` keys to a ``ModelSpec``; the engine only ever sees the spec.  The
reference keeps the same split between a typed spec and family adapters
(src/architecture.rs:342-364 ``DecoderSpec``, :254-265 ``DecoderLayerSpec``,
:139-151 ``AttentionSpec``, :201-212 ``Mamba2Spec``, :51-62 ``RopeSpec``).

Every part spec carries a ``kind`` string; ``parts.registry`` maps kinds to the
classes that run them, so a new mixer, feed-forward, norm or position encoding is a
new spec dataclass plus a registered class, with no change here.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A configuration value is missing, malformed or unsupported; the message names the field."""


def _require(condition: bool, message: str) -> None:
    if not condition:
        raise ConfigError(message)


@dataclass(frozen=True)
class RopeSpec:
    """Half-split rotary position encoding of the first ``rotary_dim`` dims of a head
    (src/architecture.rs:44-62)."""
    theta: float
    rotary_dim: int
    kind: str = "rope"

    def validate(self, head_dim: int) -> None:
        _require(self.theta > 0 and self.theta == self.theta and self.theta != float("inf"),
                 f"rope theta must be finite and positive, got {self.theta}")
        _require(0 < self.rotary_dim <= head_dim and self.rotary_dim % 2 == 0,
                 f"rotary_dim {self.rotary_dim} must be even and in 2..={head_dim}")


@dataclass(frozen=True)
class NoPositionSpec:
    """No position encoding: q and k are used as projected."""
    kind: str = "none"

    def validate(self, head_dim: int) -> None:
        return None


@dataclass(frozen=True)
class RmsNormSpec:
    eps: float
    kind: str = "rmsnorm"

    def validate(self) -> None:
        _require(self.eps > 0, f"norm eps must be positive, got {self.eps}")


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query causal attention (src/architecture.rs:139-151).

    ``window``: None = every earlier key; w = the w most recent keys, the query's own
    included (a key is masked when query - key >= w, src/decoder.rs:4521-4526).
    Multipliers scale the normed input, the key projection's output and the output
    projection's output.
    """
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    position: object = field(default_factory=NoPositionSpec)
    window: Optional[int] = None
    qkv_bias: bool = False
    out_bias: bool = False
    in_multiplier: float = 1.0
    key_multiplier: float = 1.0
    out_multiplier: float = 1.0
    kind: str = "attention"

    def validate(self) -> None:
        _require(self.num_heads > 0 and self.num_kv_heads > 0,
                 "attention head counts must be positive")
        _require(self.num_heads % self.num_kv_heads == 0,
                 f"num_attention_heads {self.num_heads} is not a multiple of "
                 f"num_key_value_heads {self.num_kv_heads}")
        _require(self.head_dim > 0 and self.head_dim % 2 == 0,
                 f"head_dim {self.head_dim} must be positive and even")
        _require(self.scale > 0, "attention scale must be positive")
        _require(self.window is None or self.window > 0, "attention window must be positive")
        self.position.validate(self.head_dim)


@dataclass(frozen=True)
class Mamba2Spec:
    """Mamba2 state-space mixer (src/architecture.rs:201-212; checks :580-628).

    ``multipliers`` scale the five segments z, x, B, C, dt of the input projection.
    """
    num_heads: int
    head_dim: int
    state_size: int
    num_groups: int
    conv_kernel: int
    chunk_size: int
    norm_eps: float
    conv_bias: bool = True
    proj_bias: bool = False
    gated_norm: bool = False
    in_multiplier: float = 1.0
    out_multiplier: float = 1.0
    multipliers: Tuple[float, float, float, float, float] = (1.0, 1.0, 1.0, 1.0, 1.0)
    kind: str = "mamba2"

    @property
    def inner_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def conv_width(self) -> int:
        return self.inner_size + 2 * self.num_groups * self.state_size

    @property
    def projection_width(self) -> int:
        return self.inner_size + self.conv_width + self.num_heads

    def validate(self) -> None:
        for name in ("num_heads", "head_dim", "state_size", "num_groups", "conv_kernel", "chunk_size"):
            _require(getattr(self, name) > 0, f"mamba {name} must be positive")
        _require(self.num_heads % self.num_groups == 0,
                 f"mamba_n_heads {self.num_heads} is not a multiple of mamba_n_groups {self.num_groups}")
        _require(self.inner_size % self.num_groups == 0, "mamba inner size must divide into its groups")
        _require(len(self.multipliers) == 5, "ssm_multipliers must have 5 entries (z, x, B, C, dt)")
        _require(self.norm_eps > 0, "mamba norm eps must be positive")


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(SiLU(gate(x) * gate_multiplier) * up(x)) * down_multiplier (src/decoder.rs:261-306)."""
    intermediate_size: int
    bias: bool = False
    gate_multiplier: float = 1.0
    down_multiplier: float = 1.0
    kind: str = "swiglu"

    def validate(self) -> None:
        _require(self.intermediate_size > 0, "intermediate_size must be positive")


@dataclass(frozen=True)
class MixerSlot:
    """One mixer of a layer: the sub-path of its tensors and its spec."""
    name: str
    spec: object


@dataclass(frozen=True)
class LayerSpec:
    """One layer's parts and their arrangement.

    ``arrangement`` "parallel_prenorm": n = norm(h); h += sum of mixers(n);
    h += ffn(norm(h)) (src/decoder.rs:2658-2699).  One mixer gives the ordinary
    sequential pre-norm layer.  ``prefix`` is the tensor-name path of the layer;
    ``mixer_norm_name`` / ``ffn_norm_name`` / ``ffn_name`` the sub-paths below it
    (src/architecture.rs:1543-1567, :1639-1647).
    """
    prefix: str
    mixers: Tuple[MixerSlot, ...]
    ffn: object
    mixer_norm: object
    ffn_norm: object
    mixer_norm_name: str = "attn_norm"
    ffn_norm_name: str = "ffn_norm"
    ffn_name: str = "mlp"
    arrangement: str = "parallel_prenorm"


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named by
    several entries: its weights run again, with a cache of their own).  ``kv_from``
    names an earlier entry whose attention cache this run reads instead of writing one
    of its own (only mixers whose cache is token-proportional can do that)."""
    layer: int
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_context: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    tied_embeddings: bool = False
    embedding_multiplier: float = 1.0
    logit_multiplier: float = 1.0
    # logits <- cap * tanh(logits / cap) after their scaling (src/decoder.rs:3349-3355, 4791-4796); None: no cap
    logit_softcap: Optional[float] = None
    embedding_name: str = "model.embed_tokens"
    final_norm_name: str = "model.norm"
    lm_head_name: str = "lm_head"
    # other spellings under which checkpoints of this architecture store the same tensors:
    # (piece of a stored name, the piece it stands for here)
    tensor_aliases: Tuple[Tuple[str, str], ...] = ()
    # a checkpoint none of whose names starts with this gets it in front of all but the output head's
    root_namespace: str = "model."
    # ("part kind.spec field", the configuration file's key for it): for messages that name a field
    field_names: Tuple[Tuple[str, str], ...] = ()

    def validate(self) -> None:
        """Positivity, divisibility and bounds, field by field (src/architecture.rs:367-452)."""
        _require(self.hidden_size > 0, "hidden_size must be positive")
        _require(self.vocab_size > 0, "vocab_size must be positive")
        _require(0 < self.max_context <= (1 << 20),
                 f"max_position_embeddings {self.max_context} must be in 1..=2^20")
        _require(0 < len(self.layers) <= 4096, "num_hidden_layers must be in 1..=4096")
        _require(len(self.schedule) > 0, "the schedule of layers is empty")
        _require(self.logit_softcap is None or (0 < self.logit_softcap < float("inf")),
                 f"the cap on the logits must be finite and positive, got {self.logit_softcap}")
        self.final_norm.validate()
        for layer in self.layers:
            _require(len(layer.mixers) > 0, f"layer {layer.prefix} has no mixer")
            names = [slot.name for slot in layer.mixers]
            _require(len(set(names)) == len(names), f"layer {layer.prefix} names a mixer twice")
            for slot in layer.mixers:
                slot.spec.validate()
            layer.ffn.validate()
            layer.mixer_norm.validate()
            layer.ffn_norm.validate()
        for index, entry in enumerate(self.schedule):
            _require(0 <= entry.layer < len(self.layers),
                     f"schedule entry {index} names layer {entry.layer}, which does not exist")
            if entry.kv_from is not None:
                _require(0 <= entry.kv_from < index,
                         f"schedule entry {index} reads the cache of entry {entry.kv_from}, "
                         "which does not run before it")
                _require(self.schedule[entry.kv_from].kv_from is None,
                         f"schedule entry {index} reads the cache of an entry that owns none")
