from .llama import LlamaConfig, read_config_json  # noqa: F401
from .presets import preset, preset_names  # noqa: F401
from .registry import (  # noqa: F401
    Architecture,
    lookup_architecture,
    register_architecture,
    registered_architectures,
    spec_from_config,
)
