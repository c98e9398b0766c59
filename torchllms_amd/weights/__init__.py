from .loader import WeightError, load_weights, safetensors_files
from .names import NameRule, half_split_to_interleaved, interleaved_to_half_split, llama_name_rules

__all__ = [
    "NameRule", "WeightError", "half_split_to_interleaved", "interleaved_to_half_split",
    "llama_name_rules", "load_weights", "random_tensor", "random_tensors", "safetensors_files",
    "write_model_folder",
]

_RANDOM_INIT = ("random_tensor", "random_tensors", "write_model_folder")


def __getattr__(name):
    # ``random_init`` is also a program (``python -m torchllms_amd.weights.random_init``): imported here
    # eagerly it would already sit in sys.modules when the interpreter starts it as one
    if name in _RANDOM_INIT:
        from . import random_init

        return getattr(random_init, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
