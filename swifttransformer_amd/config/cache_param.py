"""Parameters of the paged cache: the engine-side counterpart of the
reference's ``GptPagedAttnParam{block_size, max_num_block_per_req}``
(src/csrc/model/gpt/gpt_pagedattn_param.h:7-10) plus the pool size that the
reference leaves to its caller (src/examples/run_gpt.cc:21)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True, eq=False)
class CacheParam:
    page_size: int = 16          # tokens per page ("block_size" in the reference)
    num_pages: object = 1024     # pages in every cache group's pool (an int, or {group index: int})
    max_seqs: int = 64           # live requests (state slots)
    max_pages_per_seq: int = 0   # 0: derived from the model's longest sequence

    def __post_init__(self):
        if self.page_size < 1:
            raise ValueError(f"page_size must be >= 1, got {self.page_size}")
        counts = self.num_pages.values() if isinstance(self.num_pages, dict) else [self.num_pages]
        if any(int(n) < 1 for n in counts):
            raise ValueError(f"num_pages must be >= 1, got {self.num_pages}")
        if self.max_seqs < 1:
            raise ValueError(f"max_seqs must be >= 1, got {self.max_seqs}")

    def pages_for(self, num_tokens: int) -> int:
        return -(-num_tokens // self.page_size)
