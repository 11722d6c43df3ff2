"""Per-request sampling parameters."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class SamplingParams:
    """temperature 0 is greedy (the reference's only mode, src/csrc/model/gpt/gpt.cc:628-636);
    a positive temperature samples softmax(logits / temperature) with noise that depends
    only on (seed, index of the output token).  Generation ends at ``max_new_tokens``
    (the reference's MAX_DECODING_STEP, src/examples/run_gpt.cc:24), at the end token
    unless ``ignore_eos`` (src/examples/lib/inference_batch.cc:199-201), or when the
    model's positions are used up."""
    temperature: float = 0.0
    max_new_tokens: int = 128
    seed: int = 0
    eos_token_id: Optional[int] = None     # None: the model's own
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")
