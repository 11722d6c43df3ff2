"""The description of a model as data: which parts each layer is made of, with
what sizes and constants, under which tensor names, and in which order the
layers run.  An architecture module turns its config.json into a ``ModelSpec``;
nothing below this file knows the architecture's name."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass
class PartSpec:
    kind: str                                    # name in the part registry of its category
    params: Dict[str, Any] = field(default_factory=dict)   # sizes and constants
    names: Dict[str, str] = field(default_factory=dict)    # logical tensor -> name in the file


@dataclass
class LayerSpec:
    """The parts of one layer.  The arrangement decides which of them it uses and how; a slot
    that its arrangement does not use is None (a block with one norm, or without feed-forward)."""
    arrangement: PartSpec        # how norms, mixer and feed-forward are wired (pre/post-norm)
    mixer_norm: Optional[PartSpec]
    mixer: PartSpec
    ffn_norm: Optional[PartSpec]
    feed_forward: Optional[PartSpec]


@dataclass
class ScheduleEntry:
    """One run of a layer.  ``cache`` names the cache this run uses (by default the
    layer's own); a run with ``write=False`` reads a cache that an earlier run of the
    same step has already filled with the step's tokens."""
    layer: int
    cache: int
    write: bool = True


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int            # longest sequence the model can run
    embedding: PartSpec
    position: PartSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: Optional[PartSpec]
    head: PartSpec
    eos_token_id: Optional[int] = None

    def validate(self) -> "ModelSpec":
        n = len(self.layers)
        written = set()
        for e in self.schedule:
            if not 0 <= e.layer < n:
                raise ValueError(f"the schedule names layer {e.layer}; there are {n} layers")
            if e.write:
                if e.cache in written:
                    raise ValueError(f"cache {e.cache} is written by two runs of one step")
                written.add(e.cache)
            elif e.cache not in written:
                raise ValueError(
                    f"layer {e.layer} reads cache {e.cache} before any run has written it")
        return self
