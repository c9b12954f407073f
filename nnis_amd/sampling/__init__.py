from .host import HostSampler, greedy_token  # noqa: F401
from .params import SamplingParams  # noqa: F401
from .rng import SplitMix64  # noqa: F401
