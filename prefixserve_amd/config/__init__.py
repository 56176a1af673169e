from .llama import Llama3RopeScaling, LlamaConfig, UnsupportedModelError
from .registry import (Architecture, UnknownArchitectureError, architecture_of, read_model_dir,
                       register_architecture, registered_architectures)

__all__ = [
    "Architecture", "Llama3RopeScaling", "LlamaConfig", "UnknownArchitectureError", "UnsupportedModelError",
    "architecture_of", "read_model_dir", "register_architecture", "registered_architectures",
]
