"""A second architecture, defined here and registered from outside the package, goes the whole
route of the built-in one: ``register_architecture`` -> a model folder written by
``write_random_model`` -> ``load_model`` by the name in config.json -> ``Engine.generate`` and
the trace replay.  Its hyper-parameter class, its spec builder and its parts (a mixer with state
of its own, a feed-forward with routing, a norm, an arrangement with one norm and parallel
branches) live in the tests; no file of the package names them.

The oracle inside this toy world is the model itself run without any history: the whole sequence
in one step of a fresh request."""
import io
import json
from dataclasses import dataclass, field
from typing import List

import numpy as np
import pytest
import torch

import tiny
from test_parts_gpu import RunningMeanMixer, ToyRoutedFeedForward, ToyScaleNorm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


class ParallelOneNorm:
    """A toy arrangement: x' = x + Mix(N(x)) + FFN(N(x)), one norm for both branches."""
    needs = ("mixer_norm", "feed_forward")

    def __init__(self, spec, hidden_size, dtype):
        self.spec, self.hidden_size, self.dtype = spec, hidden_size, dtype

    def tensor_specs(self):
        return []

    def bind(self, tensors):
        pass

    def forward(self, x32, layer, ctx, cache, write=True):
        a, _ = layer.mixer_norm.forward(x32, out_t=True)
        r32 = layer.mixer.forward(a, x32, ctx, cache, write)
        return layer.feed_forward.forward(a, r32, ctx)


@dataclass
class ToyHyperParam:
    """config.json keys of the toy architecture; ``layer_kinds`` chooses each layer's mixer,
    feed-forward and arrangement, ``schedule`` the order the layers run in."""
    vocab_size: int
    max_positions: int
    width: int
    heads: int
    inner: int
    experts: int
    norm_eps: float
    position_offset: int
    layer_kinds: List[str] = field(default_factory=list)      # "mean" | "attention" | "parallel"
    schedule: List[int] = field(default_factory=list)
    architecture: str = "ToyForCausalLM"
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, d):
        return cls(**{k: d[k] for k in ("vocab_size", "max_positions", "width", "heads", "inner", "experts",
                                        "norm_eps", "position_offset", "layer_kinds", "schedule")}).validate()

    def validate(self):
        assert self.width % self.heads == 0 and all(0 <= i < len(self.layer_kinds) for i in self.schedule)
        return self

    def to_config_dict(self):
        d = {k: getattr(self, k) for k in ("vocab_size", "max_positions", "width", "heads", "inner", "experts",
                                           "norm_eps", "position_offset", "layer_kinds", "schedule")}
        d["architectures"] = [self.architecture]
        return d


def build_toy_spec(hp: ToyHyperParam):
    from swifttransformer_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    H, hd = hp.width, hp.width // hp.heads
    ln = lambda n: PartSpec("layer_norm", {"eps": hp.norm_eps, "affine": True}, {"weight": f"{n}.g", "bias": f"{n}.b"})
    dense = lambda i: PartSpec("dense", {"inner": hp.inner, "activation": "relu", "bias": True},
                               {f"{n}.{t}": f"l{i}.{n}.{t}" for n in ("fc1", "fc2") for t in ("weight", "bias")})
    attn = lambda i: PartSpec("paged_attention", {"num_heads": hp.heads, "head_dim": hd, "scale": hd ** -0.5,
                                                  "bias": False},
                              {f"{n}.weight": f"l{i}.{n}" for n in ("q", "k", "v", "out")})
    layers = []
    for i, kind in enumerate(hp.layer_kinds):
        if kind == "mean":
            layers.append(LayerSpec(PartSpec("pre_norm"), ln(f"l{i}.n1"),
                                    PartSpec("running_mean", {}, {"weight": f"l{i}.toy"}),
                                    PartSpec("toy_scale", {"eps": hp.norm_eps}, {"gain": f"l{i}.n2.gain"}),
                                    PartSpec("toy_routed", {"experts": hp.experts, "inner": hp.inner},
                                             {"router": f"l{i}.router", "up": f"l{i}.up", "down": f"l{i}.down"})))
        elif kind == "attention":
            layers.append(LayerSpec(PartSpec("pre_norm"), ln(f"l{i}.n1"), attn(i), ln(f"l{i}.n2"), dense(i)))
        elif kind == "parallel":
            layers.append(LayerSpec(PartSpec("parallel_one_norm"), ln(f"l{i}.n1"), attn(i), None, dense(i)))
        else:
            raise ValueError(kind)
    return ModelSpec(
        hidden_size=H, vocab_size=hp.vocab_size, max_positions=hp.max_positions,
        embedding=PartSpec("token", {"vocab_size": hp.vocab_size, "embed_dim": H}, {"weight": "tok"}),
        position=PartSpec("learned", {"max_positions": hp.max_positions, "offset": hp.position_offset},
                          {"weight": "pos"}),
        layers=layers,
        # a layer named twice runs twice, each run with a cache (or state) of its own
        schedule=[ScheduleEntry(layer, cache) for cache, layer in enumerate(hp.schedule)],
        final_norm=ln("fn"),
        head=PartSpec("linear", {"vocab_size": hp.vocab_size, "embed_dim": H, "tied_to": "tok"}, {"weight": "lm"}),
        eos_token_id=None).validate()


def register_toy():
    from swifttransformer_amd.config.registry import register_architecture
    from swifttransformer_amd.parts import register_part
    register_part("mixer", "running_mean", RunningMeanMixer)
    register_part("norm", "toy_scale", ToyScaleNorm)
    register_part("feed_forward", "toy_routed", ToyRoutedFeedForward)
    register_part("arrangement", "parallel_one_norm", ParallelOneNorm)
    register_architecture("ToyForCausalLM", ToyHyperParam, build_toy_spec, short_name="toy",
                          presets=lambda name, **kw: ToyHyperParam(**dict(TOY_SIZES[name], **kw)).validate())


STATEFUL = dict(vocab_size=211, max_positions=96, width=64, heads=2, inner=48, experts=3, norm_eps=1e-5,
                position_offset=0, layer_kinds=["mean", "attention", "parallel"], schedule=[0, 1, 2, 0])
STATELESS = dict(vocab_size=150, max_positions=80, width=48, heads=3, inner=72, experts=1, norm_eps=1e-6,
                 position_offset=0, layer_kinds=["parallel", "attention"], schedule=[0, 1])


TOY_SIZES = {"toy_stateful": STATEFUL, "toy_stateless": STATELESS}


def write_toy(tmp_path, cfg, seed=4):
    from swifttransformer_amd.weights import write_random_model
    register_toy()
    return write_random_model(ToyHyperParam(**cfg).validate(), str(tmp_path / "toy"), seed=seed)


def whole_logits(model_dir, dtype, seqs):
    """Every sequence whole, in one step of a fresh request of a runner of its own: no history."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models import load_model
    runner = ModelRunner(load_model(model_dir, dtype, DEV), CacheParam(page_size=4, num_pages=64, max_seqs=2), DEV)
    out = []
    for i, s in enumerate(seqs):
        runner.admit(i)
        out.append(runner.step([StepEntry(i, s, list(range(len(s))))]).float().cpu().numpy())
        runner.finish(i)
    return out


def greedy_without_history(model_dir, dtype, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(whole_logits(model_dir, dtype, [toks])[0][-1].argmax()))
    return toks[len(prompt):]


def test_folder_of_a_registered_architecture_loads_by_name(tmp_path):
    from swifttransformer_amd.config.registry import hyper_param_from_dir, registered_architectures
    from swifttransformer_amd.models import load_model
    d = write_toy(tmp_path, STATEFUL)
    assert "ToyForCausalLM" in registered_architectures() and "OPTForCausalLM" in registered_architectures()
    assert json.load(open(f"{d}/config.json"))["architectures"] == ["ToyForCausalLM"]
    arch, hp = hyper_param_from_dir(d)
    assert arch.name == "ToyForCausalLM" and isinstance(hp, ToyHyperParam) and hp.schedule == [0, 1, 2, 0]
    model = load_model(d, torch.float32, DEV)
    needs = model.cache_needs()
    assert [needs[c].kind for c in sorted(needs)] == ["state", "paged_kv", "paged_kv", "state"]
    assert model.layers[2].ffn_norm is None and not model.graph_safe


def test_generate_with_slot_reuse_and_preemption_equals_no_history(tmp_path):
    """Five requests through two state slots and a pool that cannot hold two long ones: slots are
    taken over by later requests and a pre-empted request starts again in a slot that held state.
    Every admission clears the slot's state, so the tokens equal those computed without history."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d = write_toy(tmp_path, STATEFUL)
    prompts = [tiny.prompt(n, STATEFUL["vocab_size"], 40 + i) for i, n in enumerate((9, 30, 5, 17, 3))]
    n_new = 10
    eng = Engine(d, dtype="fp32", page_size=4, num_pages=13, max_seqs=2, max_batched_tokens=64, prefill_chunk=7)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=n_new, ignore_eos=True))
    assert eng.stats.preemptions > 0, "the pool was meant to run out"
    for p, o in zip(prompts, outs):
        assert o == greedy_without_history(d, torch.float32, p, n_new)
    eng.runner.manager.check_invariants()
    assert eng.runner.manager.num_free_slots == 2


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_replay_of_a_registered_architecture(tmp_path, dtype):
    """The replay program's loop on the toy folder: portions and single tokens of three requests,
    one left out of a step, pages and slots reused, against the same sequences without history."""
    from swifttransformer_amd.engine.trace import replay
    d = write_toy(tmp_path, STATEFUL)
    V = STATEFUL["vocab_size"]
    seqs = {"a": tiny.prompt(41, V, 1), "b": tiny.prompt(23, V, 2), "c": tiny.prompt(35, V, 3)}
    ref = dict(zip(seqs, whole_logits(d, DTYPES[dtype], list(seqs.values()))))
    cuts = {"a": [5, 1, 9, 2, 20, 1, 1, 2], "b": [2, 12, 1, 7, 1], "c": [30, 1, 1, 1, 2]}
    assert all(sum(cuts[r]) == len(seqs[r]) for r in seqs)
    steps, rows = [], {}
    done = {r: 0 for r in seqs}
    live = ["a", "b"]
    while live:
        entries, end = [], []
        for r in list(live):
            if r == "b" and len(steps) == 2:
                continue                                   # left out of one step
            c = cuts[r].pop(0)
            want = [0, c - 1] if c > 1 else [0]
            entries.append({"id": r, "tokens": seqs[r][done[r]:done[r] + c], "want": want})
            rows.setdefault(len(steps), []).extend((r, done[r] + x) for x in want)
            done[r] += c
            if not cuts[r]:
                end.append(r)
                live.remove(r)
                if r == "b":
                    live.append("c")                       # takes over b's slot and pages
        steps.append({"step": len(steps), "entries": entries, "end": end})
    text = "\n".join(json.dumps(s) for s in steps) + "\n"
    out = tmp_path / "out"
    assert replay(d, dtype, str(out), 128, io.StringIO(text), log=io.StringIO(), page_size=4, max_live=2) == 0
    for s, want in rows.items():
        got = np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(len(want), V)
        exp = np.stack([ref[r][p] for r, p in want])
        tol = 2e-5 + 1e-4 * np.abs(exp) if dtype == "float32" else 0.05 * exp.std() + 0.02 * np.abs(exp)
        assert (np.abs(got - exp) <= tol).all(), f"step {s}: max err {np.abs(got - exp).max():.3e}"
    index = json.load(open(out / "index.json"))
    assert [tuple(r) for r in index["rows"][str(2)]] == [(r, p) for r, p in rows[2]]


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_recorded_steps_with_padding_rows_and_position_offset_zero(tmp_path, dtype):
    """Nine requests decode in a recorded step of ten rows: the tenth is padding, whose position
    of -1 stays negative with a position table that starts at row 0.  The lookup adds nothing for
    it instead of reading before the table; the live rows equal the no-history logits."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models import load_model
    d = write_toy(tmp_path, STATELESS)
    V = STATELESS["vocab_size"]
    dt = DTYPES[dtype]
    seqs = [tiny.prompt(n, V, 60 + i) for i, n in enumerate((29, 12, 20, 9, 17, 31, 8, 25, 14))]
    ref = whole_logits(d, dt, seqs)
    model = load_model(d, dt, DEV)
    assert model.graph_safe and model.position.offset == 0
    runner = ModelRunner(model, CacheParam(page_size=4, num_pages=70, max_seqs=12), DEV, cache_fill=float("nan"))
    n_decode = 6
    for i, s in enumerate(seqs):
        runner.admit(i)
        runner.step([StepEntry(i, s[:len(s) - n_decode], [])])
    replays = runner.graph_replays           # (prompt steps of a shape seen before are replays too)
    for k in range(n_decode):
        logits = runner.step([StepEntry(i, [s[len(s) - n_decode + k]], [0]) for i, s in enumerate(seqs)])
        exp = np.stack([ref[i][len(s) - n_decode + k] for i, s in enumerate(seqs)])
        got = logits.float().cpu().numpy()
        tol = 2e-5 + 1e-4 * np.abs(exp) if dtype == "float32" else 0.05 * exp.std() + 0.02 * np.abs(exp)
        assert np.isfinite(got).all() and (np.abs(got - exp) <= tol).all(), f"decode step {k}"
    assert runner.graph_replays == replays + n_decode and runner._bucket(len(seqs)) == 10


def test_benchmark_command_line_runs_a_registered_architecture_by_name(capsys):
    """The benchmark command line with dummy weights knows no architecture of its own: a name
    whose family a registered architecture claims gets that architecture's sizes and model."""
    from swifttransformer_amd.cli.benchmark_all_input_same import main
    register_toy()
    assert main(["toy_stateless", "fp32", "smoke"]) == 0
    out = capsys.readouterr().out
    assert "Regression stage:" in out and "(4 tokens generated)" in out
    assert main(["toy_stateful", "bf16", "smoke"]) == 0
    assert main(["toy_unknown", "bf16", "smoke"]) == 1
