"""Named sizes of the OPT family, for runs with random weights where no config.json exists.

Counterpart of the reference's table of hyper-parameters by name
(src/examples/lib/common_gpt_hyper_params.h:9-68, looked up by ``str2hyperparam``
:105-130).  The numbers are those of the published OPT configurations; a model folder's
config.json always takes precedence over a name."""
from __future__ import annotations

from typing import Dict

from .hyper_param import OptHyperParam

#          name        layers hidden heads  ffn
_SIZES = {"opt_125m": (12, 768, 12, 3072),
          "opt_1.3b": (24, 2048, 32, 8192),
          "opt_2.7b": (32, 2560, 32, 10240),
          "opt_6.7b": (32, 4096, 32, 16384),
          "opt_13b": (40, 5120, 40, 20480),
          "opt_30b": (48, 7168, 56, 28672)}


def preset_names():
    return list(_SIZES)


def preset(name: str, **overrides) -> OptHyperParam:
    """Hyper-parameters of ``name`` (``opt_125m`` ... ``opt_30b``); keyword arguments replace fields."""
    key = name.lower().replace("-", "_")
    if key not in _SIZES:
        raise KeyError(f"invalid model name {name!r}; valid names: {' '.join(_SIZES)}")
    layers, hidden, heads, ffn = _SIZES[key]
    fields: Dict = dict(vocab_size=50272, max_position_embeddings=2048, hidden_size=hidden,
                        num_hidden_layers=layers, num_attention_heads=heads, ffn_dim=ffn,
                        word_embed_proj_dim=hidden)
    fields.update(overrides)
    return OptHyperParam(**fields).validate()
