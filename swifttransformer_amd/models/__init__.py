"""Models by name: the registry maps an architecture's name to its hyper-parameter class and
its layout, and these three functions are the only routes from a configuration to a model:
from a folder (``load_model``), from typed hyper-parameters without weights (``build_model``),
and with random weights in memory (``random_model``).  The reference's counterparts are its
loader and ``initDummyWeight`` (src/csrc/model/gpt/gpt_weight.cc:235-326, :329-408)."""
from .decoder import DecoderModel
from . import opt  # noqa: F401  (registers OPTForCausalLM)
from .opt import build_opt_spec

__all__ = ["DecoderModel", "build_opt_spec", "build_model", "load_model", "random_model"]


def build_model(hyper_param, dtype) -> DecoderModel:
    """The model that ``hyper_param.architecture`` names, without weights."""
    from ..config.registry import resolve_architecture
    arch = resolve_architecture(hyper_param.architecture)
    model = DecoderModel(arch.build_spec(hyper_param), dtype)
    model.hyper_param = hyper_param
    return model


def load_model(model_dir: str, dtype, device="cuda:0") -> DecoderModel:
    """Build the model that ``model_dir``'s config.json names and load its weights."""
    import torch
    from ..config.registry import hyper_param_from_dir
    _arch, hp = hyper_param_from_dir(model_dir)
    model = build_model(hp, dtype)
    model.load_weights(model_dir, torch.device(device))
    return model


def random_model(hyper_param, dtype, seed: int = 0, device="cuda:0") -> DecoderModel:
    """The model of ``hyper_param`` with random weights generated on ``device``: tensor for tensor
    the values that ``weights.write_random_model(hyper_param, folder, seed)`` would write and
    ``load_model`` read back."""
    from ..weights.random_init import file_dtype_of, random_tensors
    model = build_model(hyper_param, dtype)
    model.bind(random_tensors(model.tensor_specs(), seed, dtype, device, file_dtype=file_dtype_of(hyper_param)))
    return model
