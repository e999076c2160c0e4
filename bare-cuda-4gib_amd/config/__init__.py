from .base import ModelConfig, field_from_json  # noqa: F401
from .registry import (  # noqa: F401
    Architecture, register_architecture, architecture_for, registered_architectures,
    load_config,
)
from .llama import LlamaConfig  # noqa: F401
