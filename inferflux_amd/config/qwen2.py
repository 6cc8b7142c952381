"""Configuration of the Qwen2 / Qwen2.5 dense decoder, from its config.json keys.

Keys the reference reads (runtime/backends/cuda/inferflux_cuda_executor.cpp:543-598):
hidden_size, num_hidden_layers, num_attention_heads, num_key_value_heads, head_dim,
intermediate_size, vocab_size, max_position_embeddings, rope_theta, model_type /
architectures[0], hidden_act, torch_dtype, rms_norm_eps.  The reference does not read
tie_word_embeddings, attention_bias or the sliding-window keys: it decides a tied
lm_head and the presence of q/k/v bias by tensor presence
(runtime/backends/cuda/native/weight_map.cpp:33-37, 55-58) and has no window.  Here the
keys are read, and the loader cross-checks them with the tensors in the file.

Sliding window (``use_sliding_window``, ``sliding_window``, ``max_window_layers``) has no
counterpart in the reference, so its meaning is fixed here: layers with index >=
``max_window_layers`` attend to the last ``sliding_window`` positions (the query's own
position included); layers below it attend to everything.  Parity of this rule with the
reference is unpinned, since the reference never windows.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, read_key


@dataclasses.dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-6
    tie_word_embeddings: bool = False
    attention_bias: bool = True
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: int = 0
    hidden_act: str = "silu"
    torch_dtype: str = "bfloat16"
    eos_token_id: Tuple[int, ...] = ()      # config.json gives one id or a list; every one of them ends a request
    bos_token_id: Optional[int] = None

    model_type: ClassVar[str] = "qwen2"
    architectures: ClassVar[Tuple[str, ...]] = ("Qwen2ForCausalLM",)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen2Config":
        hidden = read_key(d, "hidden_size", int)
        heads = read_key(d, "num_attention_heads", int)
        if heads <= 0:
            raise ConfigError("config.json: 'num_attention_heads' must be positive")
        # head_dim defaults to hidden/heads as in the reference (executor.cpp:555-559);
        # num_key_value_heads has no default there (0 when absent) -- here it defaults
        # to the number of query heads (plain multi-head attention).
        if "head_dim" in d and d["head_dim"] is not None:
            head_dim = read_key(d, "head_dim", int)
        else:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: no 'head_dim' and hidden_size {hidden} is not a multiple of "
                    f"num_attention_heads {heads}")
            head_dim = hidden // heads
        rope_scaling = d.get("rope_scaling")
        if rope_scaling not in (None, {}):
            raise ConfigError(f"config.json: 'rope_scaling' = {rope_scaling!r} is not supported (only null)")
        eos = d.get("eos_token_id")
        eos = [] if eos is None else (list(eos) if isinstance(eos, (list, tuple)) else [eos])
        if any(isinstance(e, bool) or not isinstance(e, int) or e < 0 for e in eos):
            raise ConfigError(f"config.json: 'eos_token_id' must be a token id or a list of them, got {d.get('eos_token_id')!r}")
        cfg = cls(
            vocab_size=read_key(d, "vocab_size", int),
            hidden_size=hidden,
            num_hidden_layers=read_key(d, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=read_key(d, "num_key_value_heads", int, heads),
            head_dim=head_dim,
            intermediate_size=read_key(d, "intermediate_size", int),
            max_position_embeddings=read_key(d, "max_position_embeddings", int),
            rope_theta=read_key(d, "rope_theta", float, 10000.0),
            rms_norm_eps=read_key(d, "rms_norm_eps", float, 1e-6),
            tie_word_embeddings=read_key(d, "tie_word_embeddings", bool, False),
            attention_bias=read_key(d, "attention_bias", bool, True),
            use_sliding_window=read_key(d, "use_sliding_window", bool, False),
            sliding_window=read_key(d, "sliding_window", int, None),
            max_window_layers=read_key(d, "max_window_layers", int, 0),
            hidden_act=read_key(d, "hidden_act", str, "silu"),
            torch_dtype=read_key(d, "torch_dtype", str, "bfloat16"),
            eos_token_id=tuple(dict.fromkeys(eos)),
            bos_token_id=read_key(d, "bos_token_id", int, None),
        )
        cfg.validate()
        return cfg

    def to_dict(self):
        out = super().to_dict()
        eos = list(self.eos_token_id)       # as config.json files spell it: null, one id, or a list
        out["eos_token_id"] = None if not eos else (eos[0] if len(eos) == 1 else eos)
        return out

    def validate(self) -> None:
        def positive(name):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{name}' must be positive, got {getattr(self, name)}")

        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            positive(name)
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even (rotary pairs)")
        if any(e >= self.vocab_size for e in self.eos_token_id):
            raise ConfigError(f"config.json: eos_token_id {list(self.eos_token_id)} outside the vocabulary of {self.vocab_size}")
        if not (self.rope_theta > 0):
            raise ConfigError(f"config.json: rope_theta must be positive, got {self.rope_theta}")
        if not (self.rms_norm_eps >= 0):
            raise ConfigError(f"config.json: rms_norm_eps must be >= 0, got {self.rms_norm_eps}")
        # The reference reads hidden_act and ignores it (always SiLU, executor.cpp:585-588);
        # another activation would silently compute the wrong model, so refuse it.
        if self.hidden_act != "silu":
            raise ConfigError(f"config.json: hidden_act '{self.hidden_act}' is not supported (only 'silu')")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window <= 0:
                raise ConfigError("config.json: use_sliding_window is true but 'sliding_window' is not a positive integer")
            if not (0 <= self.max_window_layers <= self.num_hidden_layers):
                raise ConfigError(
                    f"config.json: max_window_layers {self.max_window_layers} outside [0, {self.num_hidden_layers}]")

    def layer_window(self, layer: int) -> Optional[int]:
        """Number of positions layer ``layer`` attends to, or None for all of them."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None
