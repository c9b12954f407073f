"""What the parts need to know about where and how they run: the device, the
activation type, and the kernels.  ``float32`` means every tensor and every
operation in true 32-bit; ``bfloat16`` means bfloat16 activations and cache
with 32-bit accumulation, statistics, residual stream and logits.
"""

from __future__ import annotations

import torch

from ..errors import InvalidInput, KernelError

_NAMES = {
    "float32": torch.float32,
    "fp32": torch.float32,
    "f32": torch.float32,
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise InvalidInput(f"dtype must be float32 or bfloat16, got {name}")
        return name
    try:
        return _NAMES[str(name).lower()]
    except KeyError:
        raise InvalidInput(f"dtype must be float32 or bfloat16, got {name!r}") from None


class Runtime:
    """One runtime drives one GPU: it makes its device the current one, and
    every kernel is launched on that device's current stream.  A process that
    has bound its kernels to one GPU refuses a runtime on another."""

    def __init__(self, device="cuda:0", dtype="bfloat16"):
        self.device = torch.device(device)
        self.dtype = parse_dtype(dtype)
        if self.device.type != "cuda":
            raise KernelError(
                f"the engine runs on the GPU only (device {self.device}); there is no host path"
            )
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to this process; the engine has no host path")
        index = torch.cuda.current_device() if self.device.index is None else self.device.index
        count = torch.cuda.device_count()
        if not 0 <= index < count:
            raise InvalidInput(f"device ordinal {index} names no GPU of this process (it sees {count})")
        self.device = torch.device("cuda", index)
        from ..kernels import ops

        self.ops = ops
        ops.bind_device(index)  # refuses a second GPU in one process
        torch.cuda.set_device(index)  # launches, symbol addresses and new streams are the current device's
        ops.core()  # fails loudly here if the extension is neither built nor buildable

    def check_current(self) -> None:
        """Raises if the caller has made another GPU current since: a launch
        would then go to a stream of the wrong device."""
        current = torch.cuda.current_device()
        if current != self.device.index:
            raise InvalidInput(
                f"this engine runs on {self.device}, but the process's current device is cuda:{current}; "
                f"make it current again (torch.cuda.set_device({self.device.index})) before a step")

    @property
    def is_fp32(self) -> bool:
        return self.dtype == torch.float32

    def empty(self, *shape, dtype=None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)
