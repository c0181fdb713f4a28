from . import qwen3  # noqa: F401  (registers the architecture)
from .registry import (ModelFamily, config_from_dict, family_of, load_config,
                       register_architecture, registered_architectures)
