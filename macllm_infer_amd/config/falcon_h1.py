"""Falcon-H1 configuration, read from the architecture's own ``config.json`` keys.

Each layer: pre-norm, then GQA attention with RoPE and a Mamba2 mixer in parallel on
the same normed input, summed into the residual; then a SwiGLU feed-forward
(src/decoder.rs:2658-2699).  The reference reaches this family only through GGUF
metadata (src/gguf_model.rs:471-636); the key names below are the config.json
spelling of the same quantities, and the checks mirror that builder's
(:488-494 head counts, :525-529 SSM sizes, :548-567 bias presence).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, fields
from typing import Optional, Tuple

from .spec import (AttentionSpec, ConfigError, LayerSpec, Mamba2Spec, MixerSlot, ModelSpec,
                   RmsNormSpec, RopeSpec, ScheduleEntry, SwiGLUSpec, _require)

_MISSING = object()

# The names of the reference's table (src/architecture.rs:1595-1647) are the model's own; these
# are the other spelling of the same tensors in checkpoints of the family.
TENSOR_ALIASES = ((".input_layernorm.", ".attn_norm."), (".pre_ff_layernorm.", ".ffn_norm."),
                  (".feed_forward.", ".mlp."), ("model.final_layernorm.", "model.norm."))


# the config.json keys behind the fields of the parts' specs, for messages about sizes the kernels refuse
FIELD_NAMES = (("attention.head_dim", "head_dim"), ("attention.num_heads", "num_attention_heads"),
               ("mamba2.conv_kernel", "mamba_d_conv"), ("mamba2.state_size", "mamba_d_state"),
               ("mamba2.num_heads", "mamba_n_heads"), ("mamba2.num_groups", "mamba_n_groups"),
               ("rmsnorm.hidden_size", "hidden_size"))


@dataclass(frozen=True)
class FalconH1Config:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    mamba_n_heads: int
    mamba_d_head: int
    mamba_d_ssm: int
    mamba_d_state: int
    mamba_n_groups: int = 1
    mamba_d_conv: int = 4
    mamba_chunk_size: int = 128
    mamba_conv_bias: bool = True
    mamba_proj_bias: bool = False
    mamba_rms_norm: bool = False
    attention_bias: bool = False
    mlp_bias: bool = False
    rms_norm_eps: float = 1e-5
    rope_theta: float = 1e11
    tie_word_embeddings: bool = False
    embedding_multiplier: float = 1.0
    lm_head_multiplier: float = 1.0
    attention_in_multiplier: float = 1.0
    attention_out_multiplier: float = 1.0
    key_multiplier: float = 1.0
    ssm_in_multiplier: float = 1.0
    ssm_out_multiplier: float = 1.0
    ssm_multipliers: Tuple[float, float, float, float, float] = (1.0, 1.0, 1.0, 1.0, 1.0)
    mlp_multipliers: Tuple[float, float] = (1.0, 1.0)
    eos_token_id: Optional[int] = None

    architecture_names = ("FalconH1ForCausalLM", "falcon_h1")

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, raw: dict) -> "FalconH1Config":
        def get(key, default=_MISSING):
            value = raw.get(key, default)
            if value is _MISSING or value is None and default is _MISSING:
                raise ConfigError(f"config.json: required key '{key}' is missing")
            return default if value is None else value

        def integer(key, default=_MISSING):
            value = get(key, default)
            if isinstance(value, bool) or not isinstance(value, int):
                raise ConfigError(f"config.json: '{key}' must be an integer, got {value!r}")
            return value

        def number(key, default):
            value = get(key, default)
            if isinstance(value, bool) or not isinstance(value, (int, float)):
                raise ConfigError(f"config.json: '{key}' must be a number, got {value!r}")
            return float(value)

        def flag(key, default):
            value = get(key, default)
            if not isinstance(value, bool):
                raise ConfigError(f"config.json: '{key}' must be true or false, got {value!r}")
            return value

        def vector(key, length):
            value = get(key, [1.0] * length)
            if (not isinstance(value, (list, tuple)) or len(value) != length
                    or any(isinstance(v, bool) or not isinstance(v, (int, float)) for v in value)):
                raise ConfigError(f"config.json: '{key}' must be a list of {length} numbers, got {value!r}")
            return tuple(float(v) for v in value)

        # Known keys whose other values would change the model and are not built.
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: 'rope_scaling' is not supported for Falcon-H1")
        if raw.get("sliding_window") not in (None, 0):
            raise ConfigError("config.json: 'sliding_window' is not supported for Falcon-H1")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"config.json: 'hidden_act' must be 'silu', got {raw.get('hidden_act')!r}")
        # the gated norm runs after the gate; the flag says nothing when there is no such norm
        if raw.get("mamba_norm_before_gate", False) and raw.get("mamba_rms_norm", False):
            raise ConfigError("config.json: 'mamba_norm_before_gate' = true together with 'mamba_rms_norm' is not "
                              "supported (the gated norm runs after the gate)")
        # the step size is softplus(dt + bias) as it comes (src/decoder.rs:2321-2324 has no clamp)
        limit = raw.get("time_step_limit")
        if limit is not None:
            if (not isinstance(limit, (list, tuple)) or len(limit) != 2
                    or any(isinstance(v, bool) or not isinstance(v, (int, float)) for v in limit)):
                raise ConfigError(f"config.json: 'time_step_limit' must be a pair of numbers, got {limit!r}")
            if float(limit[0]) > 0.0 or float(limit[1]) != float("inf"):
                raise ConfigError(f"config.json: 'time_step_limit' {list(limit)!r} is not supported: the step size "
                                  "is not clamped (only [0, inf])")
        # newer writers keep the rope settings in one table: {"rope_theta": ..., "rope_type": "default"}
        rope = raw.get("rope_parameters")
        rope_theta_default = 1e11
        if rope is not None:
            if not isinstance(rope, dict):
                raise ConfigError(f"config.json: 'rope_parameters' must be a table, got {rope!r}")
            if rope.get("rope_type", rope.get("type", "default")) != "default":
                raise ConfigError(f"config.json: 'rope_parameters.rope_type' "
                                  f"{rope.get('rope_type', rope.get('type'))!r} is not supported (only 'default')")
            if rope.get("rope_theta") is not None:
                inner = rope["rope_theta"]
                if isinstance(inner, bool) or not isinstance(inner, (int, float)):
                    raise ConfigError(f"config.json: 'rope_parameters.rope_theta' must be a number, got {inner!r}")
                if raw.get("rope_theta") is not None and float(raw["rope_theta"]) != float(inner):
                    raise ConfigError(f"config.json: 'rope_theta' {raw['rope_theta']!r} and "
                                      f"'rope_parameters.rope_theta' {inner!r} disagree")
                rope_theta_default = float(inner)

        hidden = integer("hidden_size")
        heads = integer("num_attention_heads")
        _require(heads > 0, "config.json: 'num_attention_heads' must be positive")
        mamba_heads = integer("mamba_n_heads")
        _require(mamba_heads > 0, "config.json: 'mamba_n_heads' must be positive")
        d_ssm = raw.get("mamba_d_ssm")
        d_head = raw.get("mamba_d_head")
        if d_ssm is None and d_head is None:
            raise ConfigError("config.json: one of 'mamba_d_ssm' and 'mamba_d_head' is required")
        if d_head is None:
            d_ssm = integer("mamba_d_ssm")
            _require(d_ssm % mamba_heads == 0,
                     f"config.json: 'mamba_d_ssm' {d_ssm} is not a multiple of 'mamba_n_heads' {mamba_heads}")
            d_head = d_ssm // mamba_heads
        else:
            d_head = integer("mamba_d_head")
            d_ssm = integer("mamba_d_ssm", mamba_heads * d_head)
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = eos[0] if eos else None
        config = cls(
            hidden_size=hidden,
            num_hidden_layers=integer("num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=integer("num_key_value_heads", heads),
            head_dim=integer("head_dim", hidden // heads),
            intermediate_size=integer("intermediate_size"),
            vocab_size=integer("vocab_size"),
            max_position_embeddings=integer("max_position_embeddings"),
            mamba_n_heads=mamba_heads,
            mamba_d_head=d_head,
            mamba_d_ssm=d_ssm,
            mamba_d_state=integer("mamba_d_state"),
            mamba_n_groups=integer("mamba_n_groups", 1),
            mamba_d_conv=integer("mamba_d_conv", 4),
            mamba_chunk_size=integer("mamba_chunk_size", 128),
            mamba_conv_bias=flag("mamba_conv_bias", True),
            mamba_proj_bias=flag("mamba_proj_bias", False),
            mamba_rms_norm=flag("mamba_rms_norm", False),
            attention_bias=flag("attention_bias", False),
            mlp_bias=flag("mlp_bias", False),
            rms_norm_eps=number("rms_norm_eps", 1e-5),
            rope_theta=number("rope_theta", rope_theta_default),
            tie_word_embeddings=flag("tie_word_embeddings", False),
            embedding_multiplier=number("embedding_multiplier", 1.0),
            lm_head_multiplier=number("lm_head_multiplier", 1.0),
            attention_in_multiplier=number("attention_in_multiplier", 1.0),
            attention_out_multiplier=number("attention_out_multiplier", 1.0),
            key_multiplier=number("key_multiplier", 1.0),
            ssm_in_multiplier=number("ssm_in_multiplier", 1.0),
            ssm_out_multiplier=number("ssm_out_multiplier", 1.0),
            ssm_multipliers=vector("ssm_multipliers", 5),
            mlp_multipliers=vector("mlp_multipliers", 2),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None,
        )
        config.validate()
        return config

    def to_dict(self) -> dict:
        out = {"architectures": ["FalconH1ForCausalLM"], "model_type": "falcon_h1"}
        for item in fields(self):
            value = getattr(self, item.name)
            out[item.name] = list(value) if isinstance(value, tuple) else value
        return out

    # ------------------------------------------------------------------ checks
    def validate(self) -> None:
        _require(self.mamba_d_ssm == self.mamba_n_heads * self.mamba_d_head,
                 f"config.json: 'mamba_d_ssm' {self.mamba_d_ssm} != mamba_n_heads*mamba_d_head "
                 f"{self.mamba_n_heads * self.mamba_d_head}")
        _require(self.mamba_d_conv >= 1, "config.json: 'mamba_d_conv' must be at least 1")
        for name in ("embedding_multiplier", "lm_head_multiplier", "attention_in_multiplier",
                     "attention_out_multiplier", "key_multiplier", "ssm_in_multiplier",
                     "ssm_out_multiplier"):
            value = getattr(self, name)
            _require(math.isfinite(value), f"config.json: '{name}' must be finite")
        _require(all(math.isfinite(v) for v in self.ssm_multipliers + self.mlp_multipliers),
                 "config.json: multipliers must be finite")
        self.to_model_spec().validate()

    # ------------------------------------------------------------------ lowering
    def to_model_spec(self) -> ModelSpec:
        norm = RmsNormSpec(eps=self.rms_norm_eps)
        attention = AttentionSpec(
            num_heads=self.num_attention_heads,
            num_kv_heads=self.num_key_value_heads,
            head_dim=self.head_dim,
            scale=1.0 / math.sqrt(self.head_dim),          # fixed 1/sqrt(dh), src/gguf_model.rs:584
            position=RopeSpec(theta=self.rope_theta, rotary_dim=self.head_dim),
            window=None,
            qkv_bias=self.attention_bias,
            out_bias=self.attention_bias,
            in_multiplier=self.attention_in_multiplier,
            key_multiplier=self.key_multiplier,
            out_multiplier=self.attention_out_multiplier,
        )
        mamba = Mamba2Spec(
            num_heads=self.mamba_n_heads,
            head_dim=self.mamba_d_head,
            state_size=self.mamba_d_state,
            num_groups=self.mamba_n_groups,
            conv_kernel=self.mamba_d_conv,
            chunk_size=self.mamba_chunk_size,
            norm_eps=self.rms_norm_eps,                    # the model's eps, src/decoder.rs:2138
            conv_bias=self.mamba_conv_bias,
            proj_bias=self.mamba_proj_bias,
            gated_norm=self.mamba_rms_norm,
            in_multiplier=self.ssm_in_multiplier,
            out_multiplier=self.ssm_out_multiplier,
            multipliers=self.ssm_multipliers,
        )
        ffn = SwiGLUSpec(intermediate_size=self.intermediate_size, bias=self.mlp_bias,
                         gate_multiplier=self.mlp_multipliers[0],
                         down_multiplier=self.mlp_multipliers[1])
        layers = tuple(
            LayerSpec(prefix=f"model.layers.{index}",
                      mixers=(MixerSlot("self_attn", attention), MixerSlot("mamba", mamba)),
                      ffn=ffn, mixer_norm=norm, ffn_norm=norm)
            for index in range(self.num_hidden_layers))
        return ModelSpec(
            architecture="FalconH1ForCausalLM",
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            max_context=self.max_position_embeddings,
            layers=layers,
            schedule=tuple(ScheduleEntry(layer=index) for index in range(self.num_hidden_layers)),
            final_norm=norm,
            tied_embeddings=self.tie_word_embeddings,
            embedding_multiplier=self.embedding_multiplier,
            logit_multiplier=self.lm_head_multiplier,
            tensor_aliases=TENSOR_ALIASES,
            field_names=FIELD_NAMES,
        )

    # ------------------------------------------------------------------ reports
    def kv_bytes_per_token(self, bytes_per_element: int) -> int:
        """K and V of every layer for one token (src/architecture.rs:677-695)."""
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * bytes_per_element

    def fixed_state_bytes(self, bytes_per_element: int) -> int:
        """Conv tail (activation dtype) + SSM state (float32) of every layer for one request
        (src/architecture.rs:758-789)."""
        conv_width = self.mamba_d_ssm + 2 * self.mamba_n_groups * self.mamba_d_state
        conv = (self.mamba_d_conv - 1) * conv_width * bytes_per_element
        ssm = self.mamba_n_heads * self.mamba_d_head * self.mamba_d_state * 4
        return self.num_hidden_layers * (conv + ssm)
