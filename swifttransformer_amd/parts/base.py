"""Interfaces of the parts a layer is put together from, and their registry.

Every part is constructed as ``cls(spec: PartSpec, hidden_size: int, dtype)``
and then offers:

  ``tensor_specs()``  the tensors it wants from the weight file;
  ``bind(tensors)``   receives them (on the device, storage types per
                      ``weights.loader``) and may fuse or re-lay them out.

Kinds of part and their calls (x_t: activations in the engine's storage type
[T, hidden]; x32: the float residual stream [T, hidden]):

  norm          ``forward(x32, out_t=bool, out_f32=bool, rows=None) -> (y_t, y32)``
  mixer         ``cache_need() -> CacheNeed | None``; ``use_position(position)``: the model's
                position part, told once after construction;
                ``forward(x_t, residual32, ctx, cache, write=True) -> x32`` (= residual + mix(x))
  feed_forward  ``forward(x_t, residual32, ctx) -> x32`` (= residual + ffn(x))
  position      ``embedding_addend(ctx)`` rows to add to the token embedding, or None;
                ``rotates`` (bool) and ``rotate(q, k, ctx)``: in-place change of the step's queries
                [T, heads*head_dim] and keys [T, kv_heads*head_dim] (views of the mixer's QKV
                output) before the keys are cached; mixers call it when ``rotates`` is true;
                ``biases_scores`` (bool) and ``score_slopes(num_heads) -> float32 [num_heads]``: an
                attention mixer adds slope * (key position - query position) to a head's scaled
                scores when ``biases_scores`` is true
  embedding     ``forward(ctx, position) -> x32``
  head          ``forward(y_t) -> logits float32 [R, vocab]``
  arrangement   ``forward(x32, layer, ctx, cache, write) -> x32``

Any part may also offer ``step_planner() -> (key, planner)``: ``planner(items, info)`` sees the
step's items on the host (slot, start, tokens of each) and a ``BatchInfo`` and returns a
``StepPlan`` of int32 work lists, or None; the packer sends them to the device with the batch and the part finds them in
``ctx.plans[key]``.  Parts with equal keys share one plan.  For a step that is recorded and
replayed the planner is asked for a plan of shared lengths (``BatchInfo.bucketed``).

A part gets its sizes and constants from ``spec.params`` only; which model it
sits in is not visible to it.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

from ..weights.loader import TensorSpec
from .spec import PartSpec

CATEGORIES = ("norm", "mixer", "feed_forward", "position", "embedding", "head", "arrangement")
_REGISTRY: Dict[str, Dict[str, Callable]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, cls: Callable) -> None:
    if category not in _REGISTRY:
        raise KeyError(f"unknown part category {category!r}; one of {CATEGORIES}")
    _REGISTRY[category][kind] = cls


def build_part(category: str, spec: PartSpec, hidden_size: int, dtype: torch.dtype):
    from . import builtin  # noqa: F401  (registers the built-in parts)
    try:
        cls = _REGISTRY[category][spec.kind]
    except KeyError:
        raise KeyError(f"no {category} part named {spec.kind!r}; registered: "
                       f"{sorted(_REGISTRY[category])}") from None
    return cls(spec, hidden_size, dtype)


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer asks of the cache manager for one cache.

    kind "paged_kv": keys and values in pages, ``num_kv_heads * head_dim`` elements
    per token each; ``window`` > 0 means only the last ``window`` tokens are ever
    read, so pages behind it are given back.
    kind "state": a fixed-size tensor per request (``state_shape``, ``state_dtype``),
    living in the request's state slot."""
    kind: str
    num_kv_heads: int = 0
    head_dim: int = 0
    window: int = 0
    state_shape: Tuple[int, ...] = ()
    state_dtype: Optional[torch.dtype] = None

    def group_key(self):
        return (self.kind, self.num_kv_heads, self.head_dim, self.window, self.state_shape,
                self.state_dtype)


@dataclass
class StepPlan:
    """What a part's planner made of a step's batch on the host: int32 arrays that travel to the
    device with the batch's own index arrays (``arrays``: numpy from the planner, device tensors
    in ``ctx.plans[key]``) and numbers the host keeps (``host``)."""
    arrays: Dict[str, Any] = field(default_factory=dict)
    host: Dict[str, int] = field(default_factory=dict)


@dataclass(frozen=True)
class BatchInfo:
    """What a planner is told about the step besides its items."""
    page_size: int
    max_pages: int          # width of the block tables the kernels will see
    # True: the plan is for a step that is recorded once and replayed for every batch of the same
    # shape.  Its arrays must then have lengths that many batches share (rounded up, the unused
    # entries filled with -1, which the kernels skip), and ``host`` must hold nothing but what
    # those lengths and the launch shapes follow from: two plans with equal ``host`` and equal
    # array lengths are replayed by one recording.
    bucketed: bool = False


def count_bucket(n: int) -> int:
    """A length that lists of about ``n`` entries share in recorded steps: ``n`` itself up to 8,
    then the next even number up to 16, the next multiple of 8 up to 64, of 32 beyond."""
    if n <= 8:
        return n
    if n <= 16:
        return n + (n & 1)
    if n <= 64:
        return -(-n // 8) * 8
    return -(-n // 32) * 32


class Part:
    def __init__(self, spec: PartSpec, hidden_size: int, dtype: torch.dtype):
        self.spec = spec
        self.hidden_size = hidden_size
        self.dtype = dtype

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        pass

    def param(self, key: str, default: Any = None) -> Any:
        if key in self.spec.params:
            return self.spec.params[key]
        if default is None:
            raise KeyError(f"{type(self).__name__}: spec lacks the parameter {key!r}")
        return default

    def name(self, logical: str) -> str:
        try:
            return self.spec.names[logical]
        except KeyError:
            raise KeyError(f"{type(self).__name__}: spec names no tensor for {logical!r}") from None


class Mixer(Part):
    graph_safe = True   # its forward launches only capturable work

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def use_position(self, position) -> None:
        """The model's position part (one for all layers), told once after construction."""
        self.position = position


class PositionEncoding(Part):
    rotates = False          # True: mixers must call ``rotate`` on their queries and keys
    biases_scores = False    # True: attention mixers must add ``score_slopes`` times the distance

    def embedding_addend(self, ctx):
        return None

    def rotate(self, q, k, ctx) -> None:
        return None

    def score_slopes(self, num_heads: int) -> Optional[torch.Tensor]:
        """float32 [num_heads] on the device: a head's scaled score of (query at p, key at j)
        gets slope * (j - p) added."""
        return None
