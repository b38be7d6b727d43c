"""A one-GPU inference engine for Llama 4 on AMD MI355X (gfx950)."""
__version__ = "0.1.0"

from .config import Llama4TextConfig, get_architecture, known_architectures, load_config, register_architecture
from .engine import Engine, ModelRunner, StepEntry, load_model, random_model
from .sampling import SamplingParams
from .weights import WeightsError, load_weights, write_random_model

__all__ = ["Llama4TextConfig", "get_architecture", "known_architectures", "load_config", "register_architecture",
           "Engine", "ModelRunner", "StepEntry", "load_model", "random_model", "SamplingParams", "WeightsError",
           "load_weights", "write_random_model"]
