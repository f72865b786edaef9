from . import qwen3  # noqa: F401  (registers the architecture)
from .registry import (Architecture, config_from_dict, config_from_dir, known_architectures, lookup,
                       model_spec_for, register_architecture, unregister_architecture)
