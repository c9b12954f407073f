from .loader import load_weights, open_weight_files  # noqa: F401
from .random_init import register_init_rule, registered_init_rules, write_random_model  # noqa: F401
from .safetensors_io import SafetensorsFile, write_safetensors  # noqa: F401
