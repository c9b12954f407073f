"""Interfaces of the parts a decoder is put together from, and their registry.

A part is built from its own sizes and constants and from the checkpoint names
of its tensors; it never sees a model configuration and does not know which
model it is in.  A model description (``nnis_amd.models.spec``) names, layer
by layer, which part kinds to use and with which parameters; ``build_part``
turns one such entry into an object through the registry below.  A new mixer,
feed-forward, norm or position encoding is added by registering a class under
a new kind name; nothing else in the library keys on the kind.

The interfaces:

``Norm``
    ``forward(x, rt, rows=None)`` -> normed rows in the activation type;
    ``add_forward(residual, delta, rt, rows=None)`` -> the same after
    ``residual += delta`` (the sum is taken and kept in 32-bit).
``PositionEncoding``
    ``rotary()`` -> ``RotaryTables`` or ``None`` (consumed by attention
    mixers that rotate queries and keys); ``embed(x, ctx, rt)`` -> x, for
    encodings added to the token embedding (default: unchanged).
``Mixer``
    ``cache_request()`` -> what the cache must hold for one use of this mixer
    in the schedule (``KVRequest``, ``StateRequest`` or ``None``);
    ``forward(x, ctx, view, rt)`` -> y, where ``x`` is ``[tokens, width]`` in
    the activation type, ``ctx`` is the step's ``StepContext`` and ``view``
    is the cache's view for this schedule entry.  A mixer whose launches
    depend on the step's lengths says how (``decode_plan``, ``prompt_plan``);
    lists that it makes on the host for a step of prompts go through
    ``ctx.lists`` (``StepLists``), which is what lets the step be replayed.  A mixer that sets
    ``takes_pending_norm = True`` is handed a ``PendingNorm`` instead of ``x``
    and must consume it (``materialize()`` or ``fused(...)``).
``FeedForward``
    ``forward(x, ctx, rt)`` -> y, row-wise over the packed tokens; the same
    ``takes_pending_norm`` option.
``Block``
    ``forward(stream, ctx, view, rt)`` -> stream; the block owns the
    arrangement of norm, mixer and feed-forward around the residual stream.
"""

from __future__ import annotations

import inspect
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Tuple

from ..errors import InvalidInput


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part reads from the checkpoint.

    ``init`` names the rule by which the random-weights writer draws it
    (``weights/random_init.py``: ``register_init_rule``): ``"matrix"`` is
    N(0, 0.02), ``"gain"`` is 1 + N(0, 0.01), ``"zeros"`` is zeros; ``"index"``
    marks a table of integers, uniform in [0, ``high``), which is stored and
    kept as int32 whatever the activation type.  A part may register a rule
    of its own.  ``fallback`` names another checkpoint
    tensor that stands in when this one is absent (a tied head)."""

    name: str
    shape: Tuple[int, ...]
    init: str = "matrix"
    fallback: Optional[str] = None
    high: Optional[int] = None


@dataclass(frozen=True)
class KVRequest:
    """Keys and values of every token (``window is None``) or of the last
    ``window`` tokens, for ``kv_heads`` heads whose keys have ``head_dim``
    channels and whose values ``value_dim`` (None: as many as the keys)."""

    kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None

    @property
    def value_head_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateRequest:
    """A block of fixed shape per sequence, zero when the sequence starts.
    ``dtype`` is a torch dtype name; state is kept in it whatever the
    activation type is."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


class Part:
    """Common base: tensors in, bound device weights out.

    ``graph_safe`` says that ``forward`` only launches kernels that read the
    step's tokens, slots and positions from the context's device tensors (no
    host-side branching on them), so that a captured step can be replayed.  A
    part has to say so itself; the default is no."""

    graph_safe = False

    def tensors(self) -> List[TensorSpec]:
        return []

    def bind(self, weights: Dict[str, Any], rt: Any) -> None:
        """Receives the loaded tensors (by checkpoint name, on the device, in
        the stored type or widened for the 32-bit path) and keeps or repacks
        what it needs."""

    def weight_bytes(self) -> int:
        """Bytes of weights one step has to read through this part."""
        return 0

    def check(self, rt) -> None:
        """Raises ``Unsupported`` if the kernels this part would launch under
        ``rt`` do not take its sizes.  Asked when a model is put together,
        before any weight is read or any cache made, so that a size nobody
        runs is refused at load and not at the first step."""

    def decode_plan(self, batch: int, longest: int, rt):
        """How this part would launch a step of one token for each of
        ``batch`` sequences, the longest of ``longest`` tokens: anything that
        can be hashed and compared, or None if its launches do not depend on
        the lengths.  A captured step is replayed only for steps whose plans
        equal those it was captured with."""
        return None

    def prompt_plan(self, batch: int, rows: int, longest: int, rt):
        """The same for a step of prompts: ``batch`` sequences that bring
        ``rows`` tokens between them (rounded up as the engine rounds a
        replayed step's rows), the longest of ``longest`` tokens after it."""
        return None

    def held_buffers(self, rt):
        """Device memory beyond a step's own tensors that this part's kernels
        go through and that a captured step therefore has baked in (scratch
        that the part, or the kernels' wrapper for it, keeps between calls):
        a graph holds what this returns for as long as it lives."""
        return []

    def packed_sources(self):
        """[((address, shape) of a loaded tensor, its packed copy)] for the
        tensors this part packed when it was bound and no longer keeps in the
        checkpoint's order.  The model offers each to every other part
        (``adopt_packed``), so that a tensor two parts share is kept once."""
        return []

    def adopt_packed(self, source, packed) -> bool:
        """Takes another part's packed copy in place of the tensor at
        ``source`` if this part holds that tensor and can work from the
        packed order; says whether it did."""
        return False


class Norm(Part):
    def forward(self, x, rt, rows=None):
        raise NotImplementedError

    def add_forward(self, residual, delta, rt, rows=None):
        raise NotImplementedError

    def defer(self, x, delta, rt):
        """The norm of x (+ delta) as a value not computed yet; see ``PendingNorm``."""
        from .lazy import PendingNorm

        return PendingNorm(self, x, delta, rt)


@dataclass
class RotaryTables:
    cos: Any  # [positions, rot_dim/2] float32 on the device
    sin: Any
    rot_dim: int


class PositionEncoding(Part):
    def rotary(self) -> Optional[RotaryTables]:
        return None

    def embed(self, x, ctx, rt):
        return x


class Mixer(Part):
    def cache_request(self):
        return None

    def forward(self, x, ctx, view, rt):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x, ctx, rt):
        raise NotImplementedError


class Block(Part):
    def cache_request(self):
        return None

    def forward(self, stream, ctx, view, rt):
        raise NotImplementedError


# --------------------------------------------------------------------------
# registry of part kinds
# --------------------------------------------------------------------------

_PART_KINDS: Dict[Tuple[str, str], Callable[..., Part]] = {}
_ROLES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")


def register_part(role: str, kind: str, factory: Callable[..., Part], replace: bool = False) -> None:
    """Makes ``{"kind": kind, ...params}`` buildable for ``role``."""
    if role not in _ROLES:
        raise InvalidInput(f"unknown part role {role!r}; roles are {', '.join(_ROLES)}")
    key = (role, kind)
    if key in _PART_KINDS and not replace:
        raise InvalidInput(f"part kind {kind!r} is already registered for role {role!r}")
    _PART_KINDS[key] = factory


def build_part(role: str, spec: Dict[str, Any], **extra) -> Part:
    """``spec`` is ``{"kind": name, **parameters}``; ``extra`` carries objects
    the description cannot hold as data (the model's position encodings)."""
    if "kind" not in spec:
        raise InvalidInput(f"{role} description has no 'kind': {spec!r}")
    key = (role, spec["kind"])
    if key not in _PART_KINDS:
        known = sorted(kind for (r, kind) in _PART_KINDS if r == role)
        raise InvalidInput(f"unknown {role} kind {spec['kind']!r}; registered: {', '.join(known) or 'none'}")
    params = {k: v for k, v in spec.items() if k != "kind"}
    factory = _PART_KINDS[key]
    # context objects go only to factories that name them (a mixer without a
    # position encoding does not take ``positions``)
    accepted = inspect.signature(factory).parameters
    takes_any = any(p.kind is inspect.Parameter.VAR_KEYWORD for p in accepted.values())
    context = {k: v for k, v in extra.items() if takes_any or k in accepted}
    return factory(**params, **context)


def registered_kinds(role: str) -> List[str]:
    return sorted(kind for (r, kind) in _PART_KINDS if r == role)
