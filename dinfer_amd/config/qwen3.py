"""Configuration of the Qwen3 dense architecture (``Qwen3ForCausalLM``).

Keys, defaults and rejections follow the reference's reader,
models/qwen3/src/config.rs:5-56: ten required keys, ``head_dim`` explicit (it is
not hidden_size / heads), ``hidden_act`` must be "silu", ``attention_bias`` must
be false, heads divisible by kv heads, ``eos_token_id`` a number or a list.

Two things go beyond the reference: ``rope_scaling`` is read so that a non-null
value is refused instead of silently ignored, and a sliding window is accepted
(the reference refuses it, config.rs:48) with the meaning the keys themselves
carry: with ``use_sliding_window`` the layers from index ``max_window_layers``
on attend to the last ``sliding_window`` keys only. Newer config.json files also
spell the pattern out layer by layer (``layer_types``: "full_attention" or
"sliding_attention"); it is read and must say what the three keys say, so a file
whose list and keys disagree is refused rather than run with one of the two.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .base import ConfigError, ModelConfig, key


@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    vocab_size: int = key(int)
    hidden_size: int = key(int)
    intermediate_size: int = key(int)
    num_hidden_layers: int = key(int)
    num_attention_heads: int = key(int)
    num_key_value_heads: int = key(int)
    head_dim: int = key(int)
    rms_norm_eps: float = key(float)
    rope_theta: float = key(float)
    max_position_embeddings: int = key(int)
    tie_word_embeddings: bool = key(bool, False)
    attention_bias: bool = key(bool, False)
    hidden_act: str = key(str, "silu")
    use_sliding_window: bool = key(bool, False)
    sliding_window: int | None = key(int, None, nullable=True)
    max_window_layers: int | None = key(int, None, nullable=True)
    eos_token_ids: tuple = field(default=())
    rope_scaling_present: bool = field(default=False)
    layer_types: tuple | None = field(default=None)

    ARCHITECTURE = "Qwen3ForCausalLM"

    @classmethod
    def extra_from_dict(cls, d: dict) -> dict:
        eos = d.get("eos_token_id")
        if eos is None:
            ids = ()
        elif isinstance(eos, bool):
            raise ConfigError(f"config key 'eos_token_id' must be a number or a list of numbers, got {eos!r}")
        elif isinstance(eos, int):
            ids = (eos,)
        elif isinstance(eos, list) and all(isinstance(x, int) and not isinstance(x, bool) for x in eos):
            ids = tuple(eos)
        else:
            raise ConfigError(f"config key 'eos_token_id' must be a number or a list of numbers, got {eos!r}")
        kinds = d.get("layer_types")
        if kinds is not None:
            if not isinstance(kinds, list) or not all(isinstance(x, str) for x in kinds):
                raise ConfigError(f"config key 'layer_types' must be a list of names, got {kinds!r}")
            kinds = tuple(kinds)
        return {"eos_token_ids": ids, "rope_scaling_present": d.get("rope_scaling") is not None, "layer_types": kinds}

    def extra_to_dict(self) -> dict:
        out = {"architectures": [self.ARCHITECTURE], "model_type": "qwen3"}
        if len(self.eos_token_ids) == 1:
            out["eos_token_id"] = self.eos_token_ids[0]
        elif self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.layer_types is not None:
            out["layer_types"] = list(self.layer_types)
        return out

    def check(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config key {name!r} must be positive, got {getattr(self, name)}")
        if self.hidden_act != "silu":
            raise ConfigError(f"unsupported hidden_act {self.hidden_act!r} (only 'silu')")
        if self.attention_bias:
            raise ConfigError("attention_bias = true is not supported")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not divisible by "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotary pairs)")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not (self.rope_theta > 0):
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        if self.rope_scaling_present:
            raise ConfigError("rope_scaling is not supported (must be null or absent)")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window <= 0:
                raise ConfigError(f"use_sliding_window needs a positive sliding_window, got {self.sliding_window}")
            if self.max_window_layers is None or not (0 <= self.max_window_layers <= self.num_hidden_layers):
                raise ConfigError("use_sliding_window needs max_window_layers in [0, num_hidden_layers], "
                                  f"got {self.max_window_layers}")
        if self.layer_types is not None:
            names = {"full_attention": False, "sliding_attention": True}
            unknown = sorted(set(self.layer_types) - set(names))
            if unknown:
                raise ConfigError(f"config key 'layer_types' names unknown kinds {unknown} (known: {sorted(names)})")
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError(f"config key 'layer_types' lists {len(self.layer_types)} layers, "
                                  f"num_hidden_layers is {self.num_hidden_layers}")
            derived = [self.layer_window(i) is not None for i in range(self.num_hidden_layers)]
            listed = [names[x] for x in self.layer_types]
            if listed != derived:
                i = next(i for i in range(len(listed)) if listed[i] != derived[i])
                raise ConfigError(f"config key 'layer_types' says layer {i} is {self.layer_types[i]!r}, but "
                                  f"use_sliding_window = {self.use_sliding_window}, max_window_layers = "
                                  f"{self.max_window_layers} make it {'sliding' if derived[i] else 'full'} attention")

    # sizes derived as the reference does (config.rs:66-77)
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def layer_window(self, layer: int) -> int | None:
        """The attention window of a layer, None for full causal attention."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None
