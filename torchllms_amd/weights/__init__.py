from .loader import WeightError, load_weights, safetensors_files
from .names import NameRule, half_split_to_interleaved, interleaved_to_half_split, llama_name_rules
from .random_init import random_tensor, random_tensors, write_model_folder

__all__ = [
    "NameRule", "WeightError", "half_split_to_interleaved", "interleaved_to_half_split",
    "llama_name_rules", "load_weights", "random_tensor", "random_tensors", "safetensors_files",
    "write_model_folder",
]
