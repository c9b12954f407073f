"""Model descriptions and the generic decoder.  Importing the package
registers the architectures the library ships."""

from ..config.llama import LlamaConfig
from ..config.registry import register_architecture
from .decoder import DecoderModel  # noqa: F401
from .llama import llama_spec
from .spec import ModelSpec, ScheduleEntry  # noqa: F401

register_architecture("LlamaForCausalLM", LlamaConfig, llama_spec, replace=True)
