from .loader import load_weights, open_weight_files  # noqa: F401
from .random_init import write_random_model  # noqa: F401
from .safetensors_io import SafetensorsFile, write_safetensors  # noqa: F401
