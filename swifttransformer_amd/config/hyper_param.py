"""Typed hyper-parameters of the OPT architecture, read from config.json.

Counterpart of the reference's ``GptHyperParam`` and its ``GetOptHyperParam``
factory (src/csrc/model/gpt/gpt_hyper_param.h:8-28, :51-77).  The reference
selects a struct from a hard-coded name table
(src/examples/lib/common_gpt_hyper_params.h:105-116); here every size comes
from the model folder's own config.json keys and nothing is fixed per model
name.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any, Dict, Optional


class ConfigError(ValueError):
    """A config.json that cannot describe a model this engine can run."""


def _require_int(d: Dict[str, Any], key: str, minimum: int = 1) -> int:
    if key not in d:
        raise ConfigError(f"config.json lacks the key {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json: {key!r} must be an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json: {key!r} must be >= {minimum}, got {v}")
    return v


def _opt_bool(d: Dict[str, Any], key: str, default: bool) -> bool:
    v = d.get(key, default)
    if not isinstance(v, bool):
        raise ConfigError(f"config.json: {key!r} must be true or false, got {v!r}")
    return v


@dataclass(frozen=True)
class OptHyperParam:
    """Sizes and switches of one OPT model.

    The field names follow config.json.  ``position_offset`` is the number of
    leading rows of the learned position table that no position uses: the
    reference's converter drops them (scripts/lib/converter_lib.py:271), the
    engine keeps the table whole and adds the offset to the index.
    ``layer_norm_eps`` is 1e-5 in the reference (src/csrc/model/gpt/gpt_weight.h:63)
    and is taken from config.json when the key is there.
    """

    vocab_size: int
    max_position_embeddings: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    ffn_dim: int
    word_embed_proj_dim: int
    do_layer_norm_before: bool = True
    enable_bias: bool = True
    layer_norm_elementwise_affine: bool = True
    activation_function: str = "relu"
    tie_word_embeddings: bool = True
    remove_final_layer_norm: bool = False
    layer_norm_eps: float = 1e-5
    position_offset: int = 2
    eos_token_id: Optional[int] = 2
    bos_token_id: Optional[int] = 2
    pad_token_id: Optional[int] = 1
    torch_dtype: str = "bfloat16"
    architecture: str = "OPTForCausalLM"
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    # ---------------------------------------------------------------- derived
    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def num_kv_heads(self) -> int:
        # OPT is plain multi-head attention: GetOptHyperParam sets
        # num_kv_heads = num_heads (gpt_hyper_param.h:66-67).
        return self.num_attention_heads

    @property
    def has_projection(self) -> bool:
        return self.word_embed_proj_dim != self.hidden_size

    @property
    def has_final_norm(self) -> bool:
        return self.do_layer_norm_before and not self.remove_final_layer_norm

    # ------------------------------------------------------------- validation
    def validate(self) -> "OptHyperParam":
        if self.hidden_size % self.num_attention_heads != 0:
            # the reference asserts nh * hd == H (src/csrc/layer/attention.cc:82)
            raise ConfigError(
                f"hidden_size {self.hidden_size} is not a multiple of "
                f"num_attention_heads {self.num_attention_heads}")
        if self.activation_function != "relu":
            # OPT's feed-forward is ReLU (gpt_hyper_param.h:72)
            raise ConfigError(
                f"activation_function {self.activation_function!r} is not supported; "
                f"this architecture runs 'relu'")
        if self.layer_norm_eps <= 0:
            raise ConfigError(f"layer_norm_eps must be positive, got {self.layer_norm_eps}")
        if self.position_offset < 0:
            raise ConfigError("position_offset must be >= 0")
        return self

    # --------------------------------------------------------------- factories
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "OptHyperParam":
        hidden = _require_int(d, "hidden_size")
        archs = d.get("architectures") or ["OPTForCausalLM"]
        eps = d.get("layer_norm_eps", d.get("layer_norm_epsilon", 1e-5))
        if isinstance(eps, bool) or not isinstance(eps, (int, float)):
            raise ConfigError(f"config.json: layer_norm_eps must be a number, got {eps!r}")
        dtype = d.get("torch_dtype", d.get("dtype", "bfloat16")) or "bfloat16"
        known = {f.name for f in fields(cls)} | {
            "architectures", "_remove_final_layer_norm", "layer_norm_epsilon", "dtype"}
        hp = cls(
            vocab_size=_require_int(d, "vocab_size"),
            max_position_embeddings=_require_int(d, "max_position_embeddings"),
            hidden_size=hidden,
            num_hidden_layers=_require_int(d, "num_hidden_layers"),
            num_attention_heads=_require_int(d, "num_attention_heads"),
            ffn_dim=_require_int(d, "ffn_dim"),
            word_embed_proj_dim=(_require_int(d, "word_embed_proj_dim")
                                 if d.get("word_embed_proj_dim") is not None else hidden),
            do_layer_norm_before=_opt_bool(d, "do_layer_norm_before", True),
            enable_bias=_opt_bool(d, "enable_bias", True),
            layer_norm_elementwise_affine=_opt_bool(d, "layer_norm_elementwise_affine", True),
            activation_function=str(d.get("activation_function", "relu")),
            tie_word_embeddings=_opt_bool(d, "tie_word_embeddings", True),
            remove_final_layer_norm=_opt_bool(d, "_remove_final_layer_norm", False),
            layer_norm_eps=float(eps),
            position_offset=int(d.get("position_offset", 2)),
            eos_token_id=d.get("eos_token_id", 2),
            bos_token_id=d.get("bos_token_id", 2),
            pad_token_id=d.get("pad_token_id", 1),
            torch_dtype=str(dtype).replace("torch.", ""),
            architecture=str(archs[0]),
            extra={k: v for k, v in d.items() if k not in known},
        )
        return hp.validate()

    @classmethod
    def from_config_json(cls, path: str) -> "OptHyperParam":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    def to_config_dict(self) -> Dict[str, Any]:
        """The config.json that describes this model (inverse of ``from_dict``)."""
        return {
            "architectures": [self.architecture],
            "model_type": "opt",
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "ffn_dim": self.ffn_dim,
            "word_embed_proj_dim": self.word_embed_proj_dim,
            "do_layer_norm_before": self.do_layer_norm_before,
            "enable_bias": self.enable_bias,
            "layer_norm_elementwise_affine": self.layer_norm_elementwise_affine,
            "activation_function": self.activation_function,
            "tie_word_embeddings": self.tie_word_embeddings,
            "_remove_final_layer_norm": self.remove_final_layer_norm,
            "layer_norm_eps": self.layer_norm_eps,
            "eos_token_id": self.eos_token_id,
            "bos_token_id": self.bos_token_id,
            "pad_token_id": self.pad_token_id,
            "torch_dtype": self.torch_dtype,
        }

    def __str__(self) -> str:  # printable like gpt_hyper_param.h:30-49
        body = "\n".join(f"\t{f.name} = {getattr(self, f.name)}"
                         for f in fields(self) if f.name != "extra")
        return "OptHyperParam {\n" + body + "\n}"
