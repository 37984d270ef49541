from .base import (ConfigError, Architecture, register_architecture, unregister_architecture,
                   registered_architectures, architecture_of, read_config_json, config_from_folder)
from .llama import LlamaConfig
from .presets import preset, preset_names
