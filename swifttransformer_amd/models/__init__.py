from .decoder import DecoderModel
from . import opt  # noqa: F401  (registers OPTForCausalLM)
from .opt import build_opt_spec

__all__ = ["DecoderModel", "build_opt_spec", "load_model"]


def load_model(model_dir: str, dtype, device="cuda:0"):
    """Build the model that ``model_dir``'s config.json names and load its weights."""
    import torch
    from ..config.registry import hyper_param_from_dir
    arch, hp = hyper_param_from_dir(model_dir)
    model = DecoderModel(arch.build_spec(hp), dtype)
    model.hyper_param = hp
    model.load_weights(model_dir, torch.device(device))
    return model
