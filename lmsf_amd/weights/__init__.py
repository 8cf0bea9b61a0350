from .loader import WeightsError, check_against_declarations, collect_declarations, load_weights, \
    load_weights_from_generator
from .random_init import declared_tensors, random_tensor, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, list_weight_files, write_safetensors

__all__ = ["WeightsError", "check_against_declarations", "collect_declarations", "load_weights",
           "load_weights_from_generator", "declared_tensors", "random_tensor", "write_random_model",
           "SafetensorsError", "SafetensorsFile", "list_weight_files", "write_safetensors"]
