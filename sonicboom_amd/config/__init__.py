from .base import ConfigError, read_config_json  # noqa: F401
from .qwen2 import Qwen2Config, RopeScaling  # noqa: F401
from .registry import (Architecture, architecture_of, load_config, register_architecture,  # noqa: F401
                       registered_architectures)
