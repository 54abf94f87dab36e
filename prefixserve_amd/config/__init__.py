from .fubelorn import FubelornConfig
from .gokolix import GokolixConfig
from .larupel import LarupelConfig
from .llama import Llama3RopeScaling, LlamaConfig, UnsupportedModelError
from .radivik import RadivikConfig
from .registry import (Architecture, UnknownArchitectureError, architecture_of, read_model_dir,
                       register_architecture, registered_architectures)

__all__ = [
    "Architecture", "FubelornConfig", "GokolixConfig", "LarupelConfig", "Llama3RopeScaling", "LlamaConfig", "RadivikConfig", "UnknownArchitectureError", "UnsupportedModelError",
    "architecture_of", "read_model_dir", "register_architecture", "registered_architectures",
]
