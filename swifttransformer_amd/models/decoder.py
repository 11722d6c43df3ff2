"""A decoder-only model put together from parts according to a ``ModelSpec``.

The run of a step follows the reference's ``Gpt<T>::forward``
(src/csrc/model/gpt/gpt.cc:507-657): embed the step's tokens, run the layers,
final norm, product with the head.  The reference normalises every row and then
gathers each request's last one (gpt.cc:614-624, :175-189); here only the wanted
rows are gathered (inside the norm's row index) because the norm and the head act
on rows independently.  Logits leave as float32."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..parts.base import CacheNeed, build_part
from ..parts.spec import ModelSpec
from ..weights.loader import TensorSpec, load_tensors


@dataclass
class Layer:
    arrangement: object
    mixer_norm: object
    mixer: object
    ffn_norm: object
    feed_forward: object

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward) if p is not None)


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"the engine runs in float32 or bfloat16, not {dtype}")
        self.spec = spec.validate()
        self.dtype = dtype
        H = spec.hidden_size
        self.hidden_size = H
        self.vocab_size = spec.vocab_size
        self.max_positions = spec.max_positions
        self.embedding = build_part("embedding", spec.embedding, H, dtype)
        self.position = build_part("position", spec.position, H, dtype)
        self.layers: List[Layer] = []
        opt = lambda category, ps: build_part(category, ps, H, dtype) if ps is not None else None
        for ls in spec.layers:
            layer = Layer(
                arrangement=build_part("arrangement", ls.arrangement, H, dtype),
                mixer_norm=opt("norm", ls.mixer_norm),
                mixer=build_part("mixer", ls.mixer, H, dtype),
                ffn_norm=opt("norm", ls.ffn_norm),
                feed_forward=opt("feed_forward", ls.feed_forward))
            needs = getattr(layer.arrangement, "needs", ())
            missing = [n for n in needs if getattr(layer, n) is None]
            if missing:
                raise ValueError(f"the arrangement {ls.arrangement.kind!r} needs the parts {missing}")
            if hasattr(layer.mixer, "use_position"):
                layer.mixer.use_position(self.position)
            self.layers.append(layer)
        self.final_norm = build_part("norm", spec.final_norm, H, dtype) if spec.final_norm else None
        self.head = build_part("head", spec.head, H, dtype)
        self.schedule = list(spec.schedule)
        self.weights_loaded = False

    # ------------------------------------------------------------------ weights
    def all_parts(self):
        yield self.embedding
        yield self.position
        for layer in self.layers:
            yield from layer.parts()
        if self.final_norm is not None:
            yield self.final_norm
        yield self.head

    def tensor_specs(self) -> List[TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self.all_parts():
            for s in p.tensor_specs():
                if s.name in specs and specs[s.name].shape != s.shape:
                    raise ValueError(f"two parts want {s.name} with different shapes")
                # a tensor wanted by two parts is required if either requires it
                if s.name not in specs or specs[s.name].optional:
                    specs[s.name] = s
        return list(specs.values())

    def load_weights(self, model_dir: str, device) -> None:
        tensors = load_tensors(model_dir, self.tensor_specs(), self.dtype, device)
        self.bind(tensors)

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self.all_parts():
            p.bind(tensors)
        self.weights_loaded = True

    # -------------------------------------------------------------------- cache
    def cache_needs(self) -> Dict[int, CacheNeed]:
        """cache id -> need, for every cache the schedule writes."""
        needs: Dict[int, CacheNeed] = {}
        for e in self.schedule:
            need = self.layers[e.layer].mixer.cache_need()
            if need is None:
                continue
            if e.cache in needs and needs[e.cache].group_key() != need.group_key():
                raise ValueError(f"cache {e.cache} is shared by layers with different needs")
            needs.setdefault(e.cache, need)
        return needs

    def step_planners(self) -> Dict[object, object]:
        """key -> planner of every part that wants work lists of its own packed with a step's
        batch (``engine.batch.pack_batch``).  Parts with equal keys share one plan."""
        out: Dict[object, object] = {}
        for p in self.all_parts():
            planner = getattr(p, "step_planner", None)
            if planner is not None:
                key, fn = planner()
                out.setdefault(key, fn)
        return out

    @property
    def graph_safe(self) -> bool:
        return all(getattr(layer.mixer, "graph_safe", False) for layer in self.layers)

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, caches, best: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run the step's tokens; returns float32 logits [num_wanted, vocab].

        ``caches``: cache id -> view object for this step (``cache.DeviceCache.view``).  ``best``
        (int32 [num_wanted]): receives the wanted rows' best tokens."""
        return self.forward_head(self.forward_layers(ctx, caches), ctx, best=best)

    def forward_layers(self, ctx, caches) -> torch.Tensor:
        """Embedding and the scheduled layers: the float residual stream [num_tokens, hidden]."""
        if not self.weights_loaded:
            # the reference refuses to run before weights are loaded (gptop_base.cc:47-49)
            raise RuntimeError("load the weights before running the model")
        ctx.position = self.position
        x32 = self.embedding.forward(ctx, self.position)
        for e in self.schedule:
            layer = self.layers[e.layer]
            K.arena.next_bank()      # what this run of a layer makes may be read until the next one ends
            x32 = layer.arrangement.forward(x32, layer, ctx, caches.get(e.cache), e.write)
        return x32

    def forward_head(self, x32: torch.Tensor, ctx, want_rows: Optional[torch.Tensor] = None,
                     keep: Optional[bool] = None, best: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Final norm on the wanted rows and the head: float32 logits [wanted, vocab].  ``want_rows``
        (default ``ctx.want_rows``): batch rows, int32 on the device.  ``keep`` (default: unless the
        step is a recorded one): the logits are a tensor of their own that later steps leave alone.
        ``best`` (int32 [wanted]): receives every row's best token, the lowest id on ties (from the
        head's own kernel where it finds them, else from the arg-max kernel)."""
        rows = ctx.want_rows if want_rows is None else want_rows
        n = rows.shape[0]
        if n == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=x32.device)
        K.arena.next_bank()
        if keep is None:
            keep = not ctx.static_shapes
        takes = getattr(self.head, "takes_norm", None)
        if self.final_norm is not None and takes is not None and takes(n, self.final_norm):
            # the head's kernel normalises the wanted rows itself and finds their best tokens
            y_t, fused_best = self.final_norm.as_input(x32, rows), best
        elif self.final_norm is not None:
            (y_t, _), fused_best = self.final_norm.forward(x32, out_t=True, rows=rows), None
        else:
            y32 = K.empty((n, self.hidden_size), torch.float32, x32.device)
            K.lookup(rows, x32, out_f32=y32)
            y_t, fused_best = (y32 if self.dtype == torch.float32 else K.cast(y32, self.dtype)), None
        if keep:
            with K.arena.outside():                 # a caller may keep these beyond the next step
                logits = self.head.forward(y_t, best=fused_best) if fused_best is not None else self.head.forward(y_t)
        else:                                       # a recorded step's logits keep their place
            logits = self.head.forward(y_t, best=fused_best) if fused_best is not None else self.head.forward(y_t)
        if best is not None and fused_best is None:
            K.sample(logits, out=best)
        return logits
