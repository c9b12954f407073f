"""Error types of the library.

The reference reports failures through one structured error with a kind
(invalid input, unsupported, io, driver) and a message
(/root/reference/crates/nnis-rt/src/error.rs:12-106).  The same kinds exist
here as exception classes so callers can tell a bad request from a model the
library does not run.
"""


class NnisError(Exception):
    """Base class of every error the library raises on purpose."""


class InvalidInput(NnisError, ValueError):
    """A request, configuration value or tensor that breaks a stated rule."""


class Unsupported(NnisError, NotImplementedError):
    """A valid thing that this library does not run (architecture, size, option)."""


class WeightError(NnisError):
    """A model folder whose tensors do not match what the model declares."""


class CacheFull(NnisError):
    """The cache has no free slot or page for what the step asks to hold."""


class KernelError(NnisError, RuntimeError):
    """The HIP extension is missing, failed to build, or refused an argument."""
