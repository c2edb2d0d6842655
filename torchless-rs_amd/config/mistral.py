"""`MistralConfig`: every key of a MistralForCausalLM config.json, typed.

The reference reads the same quantities from its own file header
(src/loader/parameters.rs:792-851) and a subset of the JSON keys
(src/loader/formats/safetensors.rs:701-809: hidden_size, intermediate_size,
num_hidden_layers, num_attention_heads, num_key_value_heads (default: heads),
vocab_size, max_position_embeddings, rope_theta, rms_norm_eps); it derives
head_dim as hidden/heads (src/model/mod.rs:143) and never applies
sliding_window on this path.  Here head_dim may be explicit, sliding_window
(null, absent or 0 = none) is honoured, and what cannot be served is refused.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, ModelConfig, take_bool, take_float, take_int

# keys that are read; anything else in the file is carried in `extra`
MAX_HEAD_DIM = 256          # the largest head the attention kernels take

_KNOWN = {
    "architectures", "model_type", "hidden_size", "intermediate_size", "num_hidden_layers",
    "num_attention_heads", "num_key_value_heads", "head_dim", "vocab_size",
    "max_position_embeddings", "rope_theta", "rms_norm_eps", "sliding_window", "hidden_act",
    "tie_word_embeddings", "torch_dtype", "dtype", "bos_token_id", "eos_token_id", "pad_token_id",
    "attention_dropout", "initializer_range", "use_cache", "transformers_version",
    "rope_scaling", "quantization_config", "attention_bias", "mlp_bias",
}


@dataclass
class MistralConfig(ModelConfig):
    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    vocab_size: int = 0
    max_position_embeddings: Optional[int] = None
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-5
    sliding_window: Optional[int] = None
    hidden_act: str = "silu"
    tie_word_embeddings: bool = False
    torch_dtype: Optional[str] = None
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)
    model_type: str = "mistral"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MistralConfig":
        archs = d.get("architectures") or ["MistralForCausalLM"]
        H = take_int(d, "hidden_size", required=True, minimum=1)
        nq = take_int(d, "num_attention_heads", required=True, minimum=1)
        nkv = take_int(d, "num_key_value_heads", default=nq, minimum=1)
        if "head_dim" in d and d["head_dim"] is not None:
            hd = take_int(d, "head_dim", minimum=2)
        else:
            if H % nq:
                raise ConfigError(
                    f"config.json: no 'head_dim' and hidden_size {H} is not a multiple of "
                    f"num_attention_heads {nq}")
            hd = H // nq
        if hd % 2:
            raise ConfigError(f"config.json: head_dim {hd} must be even for the rotation in pairs")
        if hd > MAX_HEAD_DIM:
            raise ConfigError(f"config.json: head_dim {hd} is not served (even sizes up to {MAX_HEAD_DIM})")
        if nq % nkv:
            raise ConfigError(
                f"config.json: num_attention_heads {nq} is not a multiple of "
                f"num_key_value_heads {nkv}")
        win = take_int(d, "sliding_window", default=None, allow_none=True, minimum=0)
        if win == 0:
            win = None
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act {act!r} is not served (only 'silu')")
        if d.get("rope_scaling") is not None:
            raise ConfigError("config.json: 'rope_scaling' is not served for this architecture")
        if d.get("quantization_config") is not None:
            raise ConfigError("config.json: quantized checkpoints are not served")
        if take_bool(d, "attention_bias") or take_bool(d, "mlp_bias"):
            raise ConfigError("config.json: projections with bias are not served")
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: List[int] = []
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = [eos]
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = list(eos)
        else:
            raise ConfigError(f"config.json: 'eos_token_id' must be an integer or a list, got {eos!r}")
        td = d.get("torch_dtype", d.get("dtype"))
        if td is not None and not isinstance(td, str):
            raise ConfigError(f"config.json: 'torch_dtype' must be a string, got {td!r}")
        return cls(
            architecture=archs[0],
            extra={k: v for k, v in d.items() if k not in _KNOWN},
            hidden_size=H,
            intermediate_size=take_int(d, "intermediate_size", required=True, minimum=1),
            num_hidden_layers=take_int(d, "num_hidden_layers", required=True, minimum=1),
            num_attention_heads=nq,
            num_key_value_heads=nkv,
            head_dim=hd,
            vocab_size=take_int(d, "vocab_size", required=True, minimum=1),
            max_position_embeddings=take_int(d, "max_position_embeddings", default=None,
                                             allow_none=True, minimum=1),
            rope_theta=take_float(d, "rope_theta", default=10000.0, positive=True),
            rms_norm_eps=take_float(d, "rms_norm_eps", default=1e-5, positive=True),
            sliding_window=win,
            hidden_act=act,
            tie_word_embeddings=take_bool(d, "tie_word_embeddings", False),
            torch_dtype=td,
            bos_token_id=take_int(d, "bos_token_id", default=None, allow_none=True),
            eos_token_ids=eos_ids,
            model_type=d.get("model_type", "mistral"),
        )

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture or "MistralForCausalLM"],
            "model_type": self.model_type,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "sliding_window": self.sliding_window,
            "hidden_act": self.hidden_act,
            "tie_word_embeddings": self.tie_word_embeddings,
        }
        if self.torch_dtype is not None:
            d["torch_dtype"] = self.torch_dtype
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 \
                else list(self.eos_token_ids)
        d.update(self.extra)
        return d
