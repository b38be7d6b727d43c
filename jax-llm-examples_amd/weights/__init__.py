from .bindings import TensorBinding
from .loader import WeightsError, load_weights
from .random_init import init_random_, write_random_model
from .safetensors_io import SafetensorsFile, write_safetensors

__all__ = ["TensorBinding", "WeightsError", "load_weights", "init_random_", "write_random_model",
           "SafetensorsFile", "write_safetensors"]
