"""nnis_amd: a small decoder-inference library for one MI355X (gfx950).

Typed configuration and a registry of architectures, weights from safetensors
by name, layers put together from parts, a paged cache with a slot per
sequence, one step function, a generation loop with greedy and seeded
sampling, and hand-written HIP kernels underneath.
"""

from .errors import CacheFull, InvalidInput, KernelError, NnisError, Unsupported, WeightError  # noqa: F401

__all__ = [
    "load_model", "load_engine", "write_random_model", "generate",
    "NnisError", "InvalidInput", "Unsupported", "WeightError", "CacheFull", "KernelError",
]


def __getattr__(name):
    # heavy imports (torch) happen on first use
    if name in ("load_model", "load_engine", "generate"):
        from . import api

        return getattr(api, name)
    if name == "write_random_model":
        from . import models  # noqa: F401
        from .weights.random_init import write_random_model

        return write_random_model
    raise AttributeError(name)
