"""Typed configuration of the dense Qwen3 decoder (Qwen3ForCausalLM).

Keys, defaults and checks follow the reference's parser
(crates/core/src/config.rs): required sizes :186-198, head_dim default
:496-498, rope_theta required :536-545, rms_norm_eps default 1e-5 :583-585,
tie_word_embeddings default true :199-202, eos_token_id number or list
:266-274 with fallback 151643 :283-287, validate() :366-441.

Keys the reference does not read and this class does: `layer_types`,
`use_sliding_window`, `sliding_window`, `max_window_layers` (a window for some
layers). Keys of variants that this library does not hold (experts, vision,
scaled rotation) are refused instead of being ignored.
"""
from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..errors import ConfigError
from .base import Reader

_DEFAULT_EOS = 151643


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    eos_token_id: int
    # the fraction of a head that is rotated
    partial_rotary_factor: float = 1.0
    # (type, factor, original_max_position_embeddings, beta_fast, beta_slow); type default, linear or yarn
    rope_scaling: Tuple = ("default", 1.0, None, 32.0, 1.0)
    # one entry per layer: the number of keys a query sees, None = all of them
    layer_windows: Tuple[Optional[int], ...] = field(default=())
    model_type: str = "qwen3"

    @property
    def rotary_dims(self):
        """float32(head_dim) * float32(factor), cut to an integer (config.rs:525)."""
        import numpy as np
        return int(np.float32(self.head_dim) * np.float32(self.partial_rotary_factor))

    # derived sizes (crates/core/src/config.rs:303-319)
    @property
    def q_dim(self):
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self):
        return self.num_key_value_heads * self.head_dim

    @property
    def num_kv_groups(self):
        return self.num_attention_heads // self.num_key_value_heads

    @classmethod
    def from_dict(cls, raw):
        if isinstance(raw.get("text_config"), dict):
            raise ConfigError("config.json: nested text_config (a vision-language checkpoint) "
                              "is not supported by this library")
        for key in ("num_experts", "num_local_experts", "moe_intermediate_size"):
            if raw.get(key) is not None:
                raise ConfigError(f"config.json: {key} is set; expert feed-forwards are not "
                                  "part of this architecture here")
        # What the reference fixes in code for this family (no biases: crates/core/src/config.rs:508-512;
        # SwiGLU: crates/backends/backend_common/src/loader_common.rs:853) a config.json may contradict: the
        # reference never reads these keys and would run such a model wrongly; here it is refused.
        for key in ("attention_bias", "mlp_bias"):
            if raw.get(key) is True:
                raise ConfigError(f"config.json: {key} is true; this architecture has no biases here "
                                  "(stored bias tensors would be passed over)")
        if raw.get("hidden_act") not in (None, "silu", "swish"):
            raise ConfigError(f"config.json: hidden_act {raw.get('hidden_act')!r}; the feed-forward here is "
                              "silu(gate) * up")
        r = Reader(raw)
        rope_theta = r.number("rope_theta")
        rope_params = raw.get("rope_parameters")
        if rope_theta is None and isinstance(rope_params, dict):
            rope_theta = Reader(rope_params).number("rope_theta")
        if rope_theta is None:
            raise ConfigError("config.json: missing rope_theta")
        # crates/core/src/config.rs:547-580: the type from rope_parameters, else rope_scaling
        holder = rope_params if isinstance(rope_params, dict) else raw.get("rope_scaling")
        scaling = ("default", 1.0, None, 32.0, 1.0)
        if isinstance(holder, dict):
            kind = holder.get("rope_type", holder.get("type"))
            h = Reader(holder)
            factor = h.number("factor", 1.0)
            if kind == "linear":
                if factor > 1.0:                    # a factor of at most 1 is the plain rotation (:553-560)
                    scaling = ("linear", float(factor), None, 32.0, 1.0)
            elif kind == "yarn":
                scaling = ("yarn", float(factor), h.integer("original_max_position_embeddings"),
                           float(h.number("beta_fast", 32.0)), float(h.number("beta_slow", 1.0)))
            elif kind not in (None, "default"):
                # the reference falls back to the plain rotation here (:580); a model asking for
                # another scaling would then run with wrong angles, so this is an error instead
                raise ConfigError(f"config.json: rope scaling of type {kind!r} is not supported")
        # crates/core/src/config.rs:516-525: top level first, then rope_parameters; 1.0 if absent
        partial = r.number("partial_rotary_factor")
        if partial is None and isinstance(rope_params, dict):
            partial = Reader(rope_params).number("partial_rotary_factor")
        if partial is None:
            partial = 1.0
        hidden = r.integer("hidden_size", required=True)
        heads = r.integer("num_attention_heads", required=True)
        layers = r.integer("num_hidden_layers", required=True)
        if heads is not None and heads <= 0:
            raise ConfigError("num_attention_heads must be > 0")
        head_dim = r.integer("head_dim")
        if head_dim is None:
            head_dim = hidden // heads
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = eos[0] if eos else None
        if isinstance(eos, bool) or not isinstance(eos, int):
            eos = _DEFAULT_EOS
        cfg = cls(
            vocab_size=r.integer("vocab_size", required=True),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=r.integer("num_key_value_heads", required=True),
            head_dim=head_dim,
            intermediate_size=r.integer("intermediate_size", 0),
            max_position_embeddings=r.integer("max_position_embeddings", required=True),
            rope_theta=rope_theta,
            rms_norm_eps=r.number("rms_norm_eps", 1e-5),
            tie_word_embeddings=r.boolean("tie_word_embeddings", True),
            eos_token_id=eos,
            partial_rotary_factor=float(partial),
            rope_scaling=scaling,
            layer_windows=_layer_windows(r, layers),
            model_type=raw.get("model_type", "qwen3"),
        )
        cfg.validate()
        return cfg

    def validate(self):
        """The reference's checks, in its order and words (config.rs:366-407)."""
        if self.hidden_size <= 0:
            raise ConfigError("hidden_size must be > 0")
        if self.num_hidden_layers <= 0:
            raise ConfigError("num_layers must be > 0")
        if self.vocab_size <= 0:
            raise ConfigError("vocab_size must be > 0")
        if self.num_attention_heads <= 0:
            raise ConfigError("num_attention_heads must be > 0")
        if self.num_key_value_heads <= 0:
            raise ConfigError("num_key_value_heads must be > 0")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) must be divisible by "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim <= 0 or self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim ({self.head_dim}) must be > 0 and even (required by RoPE)")
        if self.intermediate_size <= 0:
            raise ConfigError("intermediate_size must be > 0")
        if not self.rms_norm_eps > 0.0:
            raise ConfigError("rms_norm_eps must be > 0")
        if not self.rope_theta > 0.0:
            raise ConfigError("rope_theta must be > 0")
        kind, factor, original, beta_fast, beta_slow = self.rope_scaling
        if kind not in ("default", "linear", "yarn") or not factor > 0.0:
            raise ConfigError(f"rope scaling {self.rope_scaling!r}: unknown type or a factor that is not > 0")
        if kind == "yarn" and (beta_fast == beta_slow or (original is not None and original <= 0)):
            raise ConfigError("yarn rope scaling needs beta_fast != beta_slow and original_max_position_embeddings > 0")
        if not 0.0 < self.partial_rotary_factor <= 1.0 or self.rotary_dims < 2 or self.rotary_dims % 2:
            raise ConfigError(f"partial_rotary_factor ({self.partial_rotary_factor}) must rotate an even number "
                              f"of at least 2 of the head's {self.head_dim} dimensions")
        if self.max_position_embeddings <= 0:
            raise ConfigError("max_position_embeddings must be > 0")
        if len(self.layer_windows) != self.num_hidden_layers:
            raise ConfigError("layer_windows must have one entry per layer")
        for w in self.layer_windows:
            if w is not None and w <= 0:
                raise ConfigError("sliding_window must be > 0")

    def to_dict(self):
        """config.json keys that give this configuration back through `from_dict`."""
        d = {
            "architectures": ["Qwen3ForCausalLM"],
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "partial_rotary_factor": self.partial_rotary_factor,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "eos_token_id": self.eos_token_id,
        }
        kind, factor, original, beta_fast, beta_slow = self.rope_scaling
        if kind == "linear":
            d["rope_scaling"] = {"rope_type": "linear", "factor": factor}
        elif kind == "yarn":
            d["rope_scaling"] = {"rope_type": "yarn", "factor": factor, "beta_fast": beta_fast, "beta_slow": beta_slow}
            if original is not None:
                d["rope_scaling"]["original_max_position_embeddings"] = original
        windows = [w for w in self.layer_windows if w is not None]
        if windows:
            if len(set(windows)) != 1:
                raise ConfigError("config.json can hold one sliding_window size only")
            d["sliding_window"] = windows[0]
            d["layer_types"] = ["full_attention" if w is None else "sliding_attention"
                                for w in self.layer_windows]
        return d


def _layer_windows(r, layers):
    """Per-layer window from `layer_types`, or from the older three keys.

    `layer_types[i]` is "full_attention" or "sliding_attention"; without it,
    layers from `max_window_layers` on slide when `use_sliding_window` is true.
    """
    if layers is None or layers <= 0:
        return ()
    window = r.integer("sliding_window")
    types = r.raw.get("layer_types")
    if types is not None:
        if not isinstance(types, list) or len(types) != layers:
            raise ConfigError("config.json: layer_types must list one type per layer")
        out = []
        for t in types:
            if t == "full_attention":
                out.append(None)
            elif t == "sliding_attention":
                if window is None:
                    raise ConfigError("config.json: sliding_attention layers need sliding_window")
                out.append(window)
            else:
                raise ConfigError(f"config.json: unknown layer type {t!r}")
        return tuple(out)
    if r.boolean("use_sliding_window", False) and window is not None:
        first = r.integer("max_window_layers", layers)
        return tuple(window if i >= first else None for i in range(layers))
    return tuple([None] * layers)
