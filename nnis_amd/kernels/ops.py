"""Python face of the HIP kernels: checks operands against what a kernel and
its grid assume, then launches it on the current stream.  Every function here
runs hand-written device code; none has a host or library stand-in.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..cache.layout import k_page_shape, v_page_shape
from ..errors import KernelError, Unsupported
from . import lib as _lib

PAGE_TOKENS = 64

_VOID = ctypes.c_void_p
_INT = ctypes.c_int
_FLT = ctypes.c_float
_SIZE = ctypes.c_size_t
_U64 = ctypes.c_uint64

_CORE_SIGNATURES = {
    "nnis_embed": [_VOID, _VOID, _INT, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_embed_packed": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_step_tables": [_VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _VOID, _INT, _VOID, _VOID, _VOID, _VOID, _VOID],
    "nnis_rmsnorm": [_VOID, _INT, _VOID, _INT, _VOID, _INT, _VOID, _INT, _VOID, _INT, _INT, _FLT, _VOID],
    "nnis_rope_kv_write": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _INT,
                           _VOID, _INT, _INT, _INT, _INT, _INT, _VOID],
    "nnis_silu_mul": [_VOID, _INT, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_argmax": [_VOID, _VOID, _INT, _INT, _VOID, _VOID],
    "nnis_argmax_scratch": [_INT, _INT],
    "nnis_argmax_static": [_VOID, _VOID, _INT, _INT, _VOID],
    "nnis_gemm_ordered": [_VOID, _INT, _VOID, _INT, _VOID, _INT, _INT, _INT, _INT, _VOID],
    "nnis_gemm_bf16": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _VOID, _SIZE, _VOID],
    "nnis_gemm_fused": [_VOID, _VOID, _VOID, _VOID, _INT, _FLT, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT,
                        _VOID, _VOID, _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT, _VOID],
    "nnis_gemm_residual_parts": [_INT, _INT],
    "nnis_gemm_tile": [_INT, _INT, _INT],
    "nnis_gemm_takes_pair": [_INT, _INT, _INT, _SIZE],
    "nnis_gemm_residual": [_VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _INT, _VOID, _SIZE, _VOID, _VOID],
    "nnis_gemm_scaled": [_VOID, _VOID, _INT, _FLT, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT, _VOID, _VOID,
                         _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT, _VOID, _SIZE, _VOID],
    "nnis_gemm_residual_runs_fits": [_INT, _INT, _INT, _INT, _INT],
    "nnis_gemm_residual_runs": [_VOID, _INT, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _VOID,
                                _VOID],
    "nnis_pack_weight": [_VOID, _VOID, _INT, _INT, _VOID],
    "nnis_sample": [_VOID, _VOID, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _VOID],
}
_ATTN_SIGNATURES = {
    "nnis_attention_rows": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT,
                            _INT, _INT, _FLT, _VOID],
    "nnis_attention_prefill_tile_rows": [_INT, _INT, _INT],
    "nnis_attention_prefill_bf16": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _VOID, _VOID, _INT,
                                    _INT, _INT, _INT, _FLT, _INT, _INT, _VOID],
    "nnis_attention_prefill_max_waves": [_INT, _INT, _INT],
    "nnis_attention_decode_bf16": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _FLT,
                                   _INT, _INT, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_attention_combine": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID],
    "nnis_attention_decode_max_waves": [_INT, _INT],
}

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


def _pages_fit(k_pages: torch.Tensor, v_pages: torch.Tensor, kv_heads: int, head_dim: int) -> bool:
    """Key and value pages [pages, ...] in the cache's layout for these sizes, contiguous."""
    return (tuple(k_pages.shape[1:]) == k_page_shape(kv_heads, head_dim) and tuple(v_pages.shape[1:]) == v_page_shape(kv_heads, head_dim)
            and k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.shape[0] == v_pages.shape[0])


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}") from None


def bind(module: str, signatures):
    """Loads a kernel module (one that ``kernels.lib`` has built in, or one that a part registered there with
    ``register_module``) and declares its entry points: ``signatures`` maps a name to its argument types; every
    entry point returns an int, 0 or an error whose text ``nnis_last_error()`` holds (``check`` raises it)."""
    return _bind(module, signatures)


def stream() -> int:
    """The raw handle of the stream that launches go to (the last argument of every entry point)."""
    return _stream()


def check(lib, status: int) -> None:
    _check(lib, status)


def _bind(module: str, signatures):
    lib = _lib.load_module(module)
    if not getattr(lib, "_nnis_bound", False):
        for name, argtypes in signatures.items():
            fn = getattr(lib, name, None)
            if fn is None:
                continue  # a kernel that is not in this build; calling it raises below
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        lib._nnis_bound = True
    return lib


_core = None
_attn = {}


def core():
    global _core
    if _core is None:
        _core = _bind("core", _CORE_SIGNATURES)
    return _core


ATTENTION_MOST_CHANNELS = 256


def attention_check(head_dim: int) -> None:
    """Raises ``Unsupported`` for a head size that no attention kernel here takes."""
    if head_dim <= 0 or head_dim % 2 != 0 or head_dim > ATTENTION_MOST_CHANNELS:
        raise Unsupported(f"the attention kernels take an even head_dim up to {ATTENTION_MOST_CHANNELS}, got {head_dim}")


def attention_module(head_dim: int):
    if head_dim not in _attn:
        attention_check(head_dim)
        _attn[head_dim] = _bind(f"attn_hd{head_dim}", _ATTN_SIGNATURES)
    return _attn[head_dim]


def _check(lib, status: int) -> None:
    if status != 0:
        raise KernelError(lib.nnis_last_error().decode(errors="replace"))


_device_index: Optional[int] = None


def bind_device(index: int) -> None:
    """Names the one GPU whose streams this process's launches go to.  The
    runtime calls it when it is made (and makes that device current); a
    second runtime on another GPU is refused, because every launch below
    takes the bound device's current stream and the per-device arrays
    (``argmax_no_alloc``, the products' workspace) are looked up for it."""
    global _device_index
    if _device_index is not None and _device_index != int(index):
        raise KernelError(f"this process already runs its kernels on cuda:{_device_index}; a process drives one GPU "
                          f"(cuda:{int(index)} was asked for)")
    _device_index = int(index)


def bound_device() -> Optional[int]:
    return _device_index


def _stream() -> int:
    """The bound device's current stream (a raw handle:
    ``torch.cuda.current_stream().cuda_stream`` builds a Python stream object
    on every call, which cost a third of an operation's time on the host)."""
    if _device_index is None:
        bind_device(torch.cuda.current_device())  # kernels called without a runtime (tests of one kernel)
    return torch._C._cuda_getCurrentRawStream(_device_index)


def _dev(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise KernelError(f"{what} must live on the GPU; this library has no host path")
    if not t.is_contiguous():
        raise KernelError(f"{what} must be contiguous")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# ---------------------------------------------------------------------------

def embed(ids: torch.Tensor, table, out: torch.Tensor) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] widened to 32-bit; ids outside the table give a zero row.
    ``table``: a matrix [vocab, width], or the ``PackedWeight`` of one (a table that a head shares)."""
    _dev(ids, "ids"), _dev(table, "embedding table"), _dev(out, "out")
    tokens, width = out.shape
    if ids.dtype != torch.int32 or ids.numel() < tokens:
        raise KernelError(f"embed: ids must be int32 with at least {tokens} entries")
    if isinstance(table, PackedWeight):
        if table.shape[1] != width or out.dtype != torch.float32:
            raise KernelError(f"embed: packed table {table.shape} / out {tuple(out.shape)} {out.dtype} do not fit")
        lib = core()
        _check(lib, lib.nnis_embed_packed(ids.data_ptr(), table.data_ptr(), out.data_ptr(), tokens, width, table.shape[0], _stream()))
        return out
    if table.dim() != 2 or table.shape[1] != width or out.dtype != torch.float32:
        raise KernelError(f"embed: table {tuple(table.shape)} / out {tuple(out.shape)} {out.dtype} do not fit")
    lib = core()
    _check(lib, lib.nnis_embed(ids.data_ptr(), table.data_ptr(), _code(table), out.data_ptr(), tokens, width,
                               table.shape[0], _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = rmsnorm(x [+ delta]) * weight.  Without ``rows`` and with ``delta``
    the sum is written back into ``x`` (32-bit).  With ``rows`` (int32), output
    row r reads input row rows[r]."""
    _dev(x, "x"), _dev(weight, "norm weight"), _dev(out, "out")
    width = x.shape[-1]
    if weight.numel() != width or out.shape[-1] != width:
        raise KernelError(f"rmsnorm: width {width} against weight {tuple(weight.shape)} and out {tuple(out.shape)}")
    out_rows = out.numel() // width
    if rows is None:
        if x.numel() // width != out_rows:
            raise KernelError(f"rmsnorm: {x.numel() // width} input rows against {out_rows} output rows")
    else:
        _dev(rows, "rows")
        if rows.dtype != torch.int32 or rows.numel() < out_rows:
            raise KernelError("rmsnorm: rows must be int32 with one entry per output row")
    if delta is not None:
        _dev(delta, "delta")
        if delta.shape != x.shape:
            raise KernelError(f"rmsnorm: delta {tuple(delta.shape)} against x {tuple(x.shape)}")
    lib = core()
    _check(lib, lib.nnis_rmsnorm(x.data_ptr(), _code(x), _ptr(delta), _code(delta) if delta is not None else 0,
                                 weight.data_ptr(), _code(weight), out.data_ptr(), _code(out), _ptr(rows), out_rows,
                                 width, float(eps), _stream()))
    return out


def rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                  rot_dim: int, tok_slot: torch.Tensor, tok_pos: torch.Tensor, k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], block_table: Optional[torch.Tensor], heads: int, kv_heads: int,
                  head_dim: int) -> torch.Tensor:
    """Rotates queries and keys by their positions and writes keys and values
    into the pages of each token's slot.  ``k_pages`` and ``v_pages`` are
    ``[pages, *k_page_shape(kv_heads, head_dim)]`` and ``[pages,
    *v_page_shape(kv_heads, head_dim)]`` (``cache/layout.py``); both ``None``
    for a run that keeps no cache of its own."""
    _dev(qkv, "qkv"), _dev(q_out, "q_out"), _dev(tok_slot, "tok_slot"), _dev(tok_pos, "tok_pos")
    tokens = qkv.shape[0]
    if qkv.shape[1] != (heads + 2 * kv_heads) * head_dim or q_out.shape != (tokens, heads * head_dim):
        raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} / q_out {tuple(q_out.shape)} do not fit "
                          f"{heads}+2*{kv_heads} heads of {head_dim}")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or tok_slot.numel() < tokens or tok_pos.numel() < tokens:
        raise KernelError("rope_kv_write: tok_slot / tok_pos must be int32 with one entry per token")
    table_positions = 0
    if cos is not None:
        _dev(cos, "cos"), _dev(sin, "sin")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != rot_dim // 2:
            raise KernelError(f"rope_kv_write: tables {tuple(cos.shape)} do not fit rot_dim {rot_dim} in float32")
        table_positions = cos.shape[0]
    max_pages = 0
    cache_code = 0
    if k_pages is not None:
        _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table")
        if not _pages_fit(k_pages, v_pages, kv_heads, head_dim):
            raise KernelError(f"rope_kv_write: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
        if block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelError("rope_kv_write: block_table must be int32 [slots, pages]")
        max_pages = block_table.shape[1]
        cache_code = _code(k_pages)
    lib = core()
    _check(lib, lib.nnis_rope_kv_write(qkv.data_ptr(), _code(qkv), q_out.data_ptr(), _code(q_out), _ptr(cos), _ptr(sin),
                                       table_positions, rot_dim, tok_slot.data_ptr(), tok_pos.data_ptr(),
                                       _ptr(k_pages), _ptr(v_pages), cache_code, _ptr(block_table), max_pages, tokens,
                                       heads, kv_heads, head_dim, _stream()))
    return q_out


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(gate_up, "gate_up"), _dev(out, "out")
    tokens, inner = out.shape
    if gate_up.shape != (tokens, 2 * inner):
        raise KernelError(f"silu_mul: gate_up {tuple(gate_up.shape)} against out {tuple(out.shape)}")
    lib = core()
    _check(lib, lib.nnis_silu_mul(gate_up.data_ptr(), _code(gate_up), out.data_ptr(), _code(out), tokens, inner, _stream()))
    return out


STATIC_SCRATCH_WORDS = 65536  # NNIS_STATIC_SCRATCH_WORDS of csrc/nnis_noalloc.h


def argmax(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(logits, "logits"), _dev(out, "out")
    rows, vocab = logits.shape
    if logits.dtype != torch.float32 or out.dtype != torch.int32 or out.numel() < rows:
        raise KernelError("argmax: logits must be float32 [rows, vocab] and out int32 [rows]")
    if not logits.is_contiguous():
        raise KernelError("argmax: logits must be contiguous")
    lib = core()
    need = lib.nnis_argmax_scratch(rows, vocab)
    if need <= STATIC_SCRATCH_WORDS:
        # the array that the library holds on the GPU: nothing to allocate (calls follow one another on one stream)
        _check(lib, lib.nnis_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, _stream()))
        return out
    scratch = torch.empty(max(1, need), dtype=torch.float32, device=logits.device)
    _check(lib, lib.nnis_argmax(logits.data_ptr(), out.data_ptr(), rows, vocab, scratch.data_ptr(), _stream()))
    return out


def argmax_no_alloc(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``argmax`` for callers that cannot allocate: the first pass's results go
    through a fixed array that the library holds on the GPU (256 KB; enough
    for 2 * rows * ceil(vocab / 4096) <= 65,536 words, beyond that the call
    is refused).  Calls on one GPU share the array: keep them in order on one
    stream."""
    _dev(logits, "logits"), _dev(out, "out")
    rows, vocab = logits.shape
    if logits.dtype != torch.float32 or out.dtype != torch.int32 or out.numel() < rows:
        raise KernelError("argmax: logits must be float32 [rows, vocab] and out int32 [rows]")
    lib = core()
    _check(lib, lib.nnis_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, _stream()))
    return out


def gemm_ordered(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T, each element one ascending-k chain of
    32-bit fused multiply-adds."""
    _dev(x, "x"), _dev(w, "weight"), _dev(out, "out")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or out.shape != (m, n):
        raise KernelError(f"gemm: x {tuple(x.shape)} w {tuple(w.shape)} out {tuple(out.shape)} do not fit")
    lib = core()
    _check(lib, lib.nnis_gemm_ordered(x.data_ptr(), _code(x), w.data_ptr(), _code(w), out.data_ptr(), _code(out), m, n, k,
                                      _stream()))
    return out


class StepTables:
    """What a step's kernels would look up through each token's slot and
    position, gathered once by token (``step_tables``): ``cos`` / ``sin``
    float32 [tokens, rot_dim / 2], each token's rows of the rotation tables;
    ``page`` int32 [tokens], the cache page of each token's position (-1 for a
    padding row); ``pages`` int32 [tokens, pages a slot may hold], for a step
    of single tokens the pages of each token's sequence up to its position.
    Any of them is None where it was not asked for."""

    def __init__(self, tokens, cos=None, sin=None, page=None, pages=None):
        self.tokens, self.cos, self.sin, self.page, self.pages = tokens, cos, sin, page, pages


def step_tables(tok_slot: torch.Tensor, tok_pos: torch.Tensor, tokens: int, cos: Optional[torch.Tensor] = None,
                sin: Optional[torch.Tensor] = None, block_table: Optional[torch.Tensor] = None,
                sequence_pages: bool = False) -> StepTables:
    """One kernel at the start of a step; see ``StepTables``.  ``cos`` / ``sin``:
    rotation tables [positions, half]; ``block_table``: int32 [slots, pages];
    ``sequence_pages``: also each token's sequence's pages (a decode step).
    The positions live on the device, where nothing can refuse them: the
    caller sees to it that every position is below ``cos.shape[0]`` and
    below ``block_table.shape[1] * 64`` (the engine refuses a step beyond the
    model's positions before it launches anything, and its tables reach that
    far); the kernel's clamps of a position beyond either are a guard against
    reading out of bounds, not a result."""
    _dev(tok_slot, "tok_slot"), _dev(tok_pos, "tok_pos")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or min(tok_slot.numel(), tok_pos.numel()) < tokens:
        raise KernelError("step_tables: tok_slot / tok_pos must be int32 with one entry per token")
    out = StepTables(tokens)
    half = positions = max_pages = 0
    if cos is not None:
        _dev(cos, "cos"), _dev(sin, "sin")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2:
            raise KernelError("step_tables: rotation tables must be float32 [positions, half]")
        positions, half = cos.shape
        out.cos = torch.empty((tokens, half), dtype=torch.float32, device=cos.device)
        out.sin = torch.empty((tokens, half), dtype=torch.float32, device=cos.device)
    if block_table is not None:
        _dev(block_table, "block_table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelError("step_tables: block_table must be int32 [slots, pages]")
        max_pages = block_table.shape[1]
        out.page = torch.empty(tokens, dtype=torch.int32, device=block_table.device)
        if sequence_pages:
            out.pages = torch.empty((tokens, max_pages), dtype=torch.int32, device=block_table.device)
    lib = core()
    _check(lib, lib.nnis_step_tables(tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, _ptr(cos), _ptr(sin), half, positions,
                                     _ptr(block_table), max_pages, _ptr(out.cos), _ptr(out.sin), _ptr(out.page),
                                     _ptr(out.pages), _stream()))
    return out


def attention_rows(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                   block_table: torch.Tensor, tok_slot: torch.Tensor, tok_pos: torch.Tensor, heads: int, kv_heads: int,
                   head_dim: int, scale: float, window: int = 0) -> torch.Tensor:
    """Causal attention of each token over the cached keys of its slot up to
    its own position (32-bit arithmetic, any storage type)."""
    _dev(q, "q"), _dev(out, "out"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table")
    tokens = q.shape[0]
    if q.shape != (tokens, heads * head_dim) or out.shape != q.shape:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {heads} heads of {head_dim}")
    if not _pages_fit(k_pages, v_pages, kv_heads, head_dim):
        raise KernelError(f"attention: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
    if k_pages.dtype != v_pages.dtype:
        raise KernelError("attention: key and value pages differ in type")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or block_table.dtype != torch.int32:
        raise KernelError("attention: tok_slot, tok_pos and block_table must be int32")
    lib = attention_module(head_dim)
    _check(lib, lib.nnis_attention_rows(q.data_ptr(), _code(q), out.data_ptr(), _code(out), k_pages.data_ptr(),
                                        v_pages.data_ptr(), _code(k_pages), block_table.data_ptr(), block_table.shape[1],
                                        tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim,
                                        int(window), float(scale), _stream()))
    return out


# ---------------------------------------------------------------------------
# dispatch by operand types
# ---------------------------------------------------------------------------

class PackedWeight:
    """A bfloat16 weight [n, k] in the order the matrix-core products read it
    (``pack_weight``): strips of 16 rows, chunks of 64 k, both padded with
    zeros (and a strip to an odd number of chunks), a strip's chunk laid out
    as a wave's loads take it.  ``data`` is the
    flat packed storage; ``shape`` and ``dtype`` are the weight's own."""

    dtype = torch.bfloat16
    is_cuda = True

    def __init__(self, data: torch.Tensor, n: int, k: int):
        self.data = data
        self.shape = (int(n), int(k))

    @property
    def device(self):
        return self.data.device

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def is_contiguous(self) -> bool:
        return True


def packed_weight_elems(n: int, k: int) -> int:
    """Strips of 16 rows, each an odd number of chunks of 64 k (1024 elements) long."""
    return ((n + 15) // 16) * (((k + 63) // 64) | 1) * 1024


def packs(weight: torch.Tensor) -> bool:
    """Whether a weight is one that ``pack_weight`` takes."""
    return weight.is_cuda and weight.dim() == 2 and weight.dtype == torch.bfloat16 and weight.shape[1] % 8 == 0


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """The packed copy of a bfloat16 weight [n, k] (K a multiple of 8) that
    ``gemm_bf16``, ``gemm_fused``, ``gemm_residual`` and ``gemm_scaled`` take."""
    _dev(w, "weight")
    if not packs(w):
        raise KernelError(f"pack_weight takes a bfloat16 matrix whose K is a multiple of 8, got {w.dtype} {tuple(w.shape)}")
    n, k = w.shape
    data = torch.empty(packed_weight_elems(n, k), dtype=torch.bfloat16, device=w.device)
    lib = core()
    _check(lib, lib.nnis_pack_weight(w.data_ptr(), data.data_ptr(), n, k, _stream()))
    return PackedWeight(data, n, k)


def _packed(w, what: str) -> None:
    if not isinstance(w, PackedWeight):
        raise KernelError(f"{what}: the weight must be packed (pack_weight) for the matrix-core kernels")


# Where the tiled product cuts K among blocks (few tiles, a long K) the parts meet in this scratch: 256 blocks
# of 64 x 64 sums at most.  Kept per device; calls on one device share it, so they follow one another on one
# stream.  It is made outside a graph capture only: a capture that finds none goes without the cut.
GEMM_WORKSPACE_BYTES = 4 << 20
_gemm_workspaces = {}
PAIR_COUNTS = 1024  # 32-bit words kept behind the workspace for the strips' counts


def _gemm_workspace(device) -> Optional[torch.Tensor]:
    key = (device.type, device.index)
    held = _gemm_workspaces.get(key)
    if held is None and not torch.cuda.is_current_stream_capturing():
        # behind the workspace proper: the counts of the strips that two blocks share (`gemm_residual`), zero between calls
        held = _gemm_workspaces[key] = torch.zeros(GEMM_WORKSPACE_BYTES // 4 + PAIR_COUNTS, dtype=torch.float32, device=device)
    return held


def gemm_takes_pair(m: int, n: int, k: int) -> bool:
    """Whether ``gemm_residual`` gives a product of these sizes to two blocks a strip (the kernel whose blocks
    meet in the workspace and count in the words behind it)."""
    return bool(core().nnis_gemm_takes_pair(int(m), int(n), int(k), GEMM_WORKSPACE_BYTES))


def gemm_pair_counts(device) -> Optional[torch.Tensor]:
    """The strips' counts of the products with two blocks a strip on ``device`` (int32 [PAIR_COUNTS]; None
    before the first product there): every word is zero whenever no such product is running."""
    work = _gemm_workspace(torch.device(device))
    return None if work is None else work[GEMM_WORKSPACE_BYTES // 4:].view(torch.int32)


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, split: int = 0) -> torch.Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T on the matrix cores: bfloat16 operands,
    32-bit accumulation, bfloat16 or float32 output.  ``w``: a ``PackedWeight``."""
    _packed(w, "gemm_bf16")
    _dev(x, "x"), _dev(out, "out")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or out.shape != (m, n):
        raise KernelError(f"gemm: x {tuple(x.shape)} w {tuple(w.shape)} out {tuple(out.shape)} do not fit")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_bf16 takes bfloat16 operands, got {x.dtype} and {w.dtype}")
    lib = core()
    work = _gemm_workspace(x.device)
    _check(lib, lib.nnis_gemm_bf16(x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out), m, n, k, int(split), _ptr(work),
                                   GEMM_WORKSPACE_BYTES if work is not None else 0, _stream()))
    return out


EPILOGUE_STORE, EPILOGUE_SILU, EPILOGUE_ROPE = 0, 1, 2
FUSED_MAX_TOKENS = 16  # beyond a tile of 16 tokens every wave re-reads too much of x: the separate kernels win


def gemm_fused(x_in: torch.Tensor, delta: Optional[torch.Tensor], x_out: Optional[torch.Tensor], norm_weight: torch.Tensor,
               eps: float, w: torch.Tensor, y: torch.Tensor, epilogue: int = EPILOGUE_STORE, rope: Optional[dict] = None,
               split: int = 0):
    """y = epilogue( W . rmsnorm(x_in + delta) ) for a few tokens (callers
    keep to ``FUSED_MAX_TOKENS``; the kernel itself takes up to 64), in one
    kernel; ``x_out`` receives x_in + delta.  ``epilogue``: store; SiLU(gate) *
    up for a weight of gate rows followed by up rows; or rotate-half RoPE with
    the write of keys and values into the cache (``rope``: cos, sin, tok_slot,
    tok_pos, k_pages, v_pages, block_table, heads, kv_heads, head_dim)."""
    _packed(w, "gemm_fused")
    m, k = x_in.shape
    n = w.shape[0]
    _dev(x_in, "x"), _dev(norm_weight, "norm weight"), _dev(y, "y")
    if x_in.dtype != torch.float32 or w.dtype != torch.bfloat16 or y.dtype != torch.bfloat16 or w.shape[1] != k:
        raise KernelError("gemm_fused: x must be float32 [m, k], the weight bfloat16 [n, k] and y bfloat16")
    if norm_weight.numel() != k:
        raise KernelError(f"gemm_fused: norm weight of {norm_weight.numel()} for width {k}")
    if delta is not None:
        _dev(delta, "delta"), _dev(x_out, "x_out")
        if delta.shape != x_in.shape or delta.dtype != torch.bfloat16 or x_out.shape != x_in.shape or x_out.dtype != torch.float32:
            raise KernelError("gemm_fused: delta must be bfloat16 and x_out float32, both shaped like x")
    r = _check_epilogue("gemm_fused", m, n, y, epilogue, rope)
    lib = core()
    bt = r.get("block_table")
    _check(lib, lib.nnis_gemm_fused(
        x_in.data_ptr(), _ptr(delta), _ptr(x_out) if delta is not None else None, norm_weight.data_ptr(), _code(norm_weight),
        float(eps), w.data_ptr(), m, n, k, int(epilogue), y.data_ptr(), _ptr(r.get("cos")), _ptr(r.get("sin")),
        r["cos"].shape[0] if r.get("cos") is not None else 0, _ptr(r.get("tok_slot")), _ptr(r.get("tok_pos")),
        _ptr(r.get("k_pages")), _ptr(r.get("v_pages")), _ptr(bt), bt.shape[1] if bt is not None else 0,
        r.get("heads", 0), r.get("kv_heads", 0), r.get("head_dim", 0), *_step_table_pointers(r), int(split), _stream()))
    return y


def _step_table_pointers(rope: dict):
    """(tok_cos, tok_sin, tok_page) of a rotating epilogue's ``tables`` (a ``StepTables``), or three nulls."""
    tables = rope.get("tables")
    if tables is None or tables.cos is None or tables.page is None:
        return None, None, None
    return tables.cos.data_ptr(), tables.sin.data_ptr(), tables.page.data_ptr()


def _check_epilogue(what: str, m: int, n: int, y: torch.Tensor, epilogue: int, rope: Optional[dict]) -> dict:
    """Checks y and the rotating epilogue's arguments against the sizes; returns the arguments (or {})."""
    expect = {EPILOGUE_STORE: (m, n), EPILOGUE_SILU: (m, n // 2)}.get(epilogue)
    r = rope or {}
    if epilogue == EPILOGUE_ROPE:
        expect = (m, r["heads"] * r["head_dim"])
        for name in ("cos", "sin", "tok_slot", "tok_pos"):
            _dev(r[name], name)
        if r["cos"].dtype != torch.float32 or r["cos"].shape != r["sin"].shape or r["cos"].shape[1] != r["head_dim"] // 2:
            raise KernelError(f"{what}: rotation tables must be float32 [positions, head_dim / 2]")
        if r["tok_slot"].dtype != torch.int32 or r["tok_pos"].dtype != torch.int32 or min(r["tok_slot"].numel(), r["tok_pos"].numel()) < m:
            raise KernelError(f"{what}: tok_slot / tok_pos must be int32 with one entry per token")
        tables = r.get("tables")
        if tables is not None and tables.cos is not None:
            if (tables.tokens < m or tables.cos.shape[1] != r["head_dim"] // 2 or tables.cos.dtype != torch.float32
                    or (r.get("k_pages") is not None and tables.page is None)):
                raise KernelError(f"{what}: the step's tables do not fit {m} tokens with heads of {r['head_dim']}")
        if r.get("k_pages") is not None:
            kp, vp, bt = r["k_pages"], r["v_pages"], r["block_table"]
            _dev(kp, "k_pages"), _dev(vp, "v_pages"), _dev(bt, "block_table")
            if (kp.dtype != torch.bfloat16 or vp.dtype != torch.bfloat16 or bt.dtype != torch.int32
                    or not _pages_fit(kp, vp, r["kv_heads"], r["head_dim"])):
                raise KernelError(f"{what}: cache pages must be bfloat16 in the cache's layout, the block table int32")
    if expect is None or tuple(y.shape) != expect or y.dtype != torch.bfloat16 or not y.is_contiguous():
        raise KernelError(f"{what}: y {tuple(y.shape)} {y.dtype} does not fit epilogue {epilogue} (expected bfloat16 {expect})")
    return r


# tiles of the tiled product (``tile`` of gemm_residual; 16 times as much as a ``split`` of gemm_bf16 / gemm_scaled)
TILE_64x128, TILE_64x64, TILE_256x256, TILE_256x192, TILE_128x128, TILE_256x128, TILE_128x192 = 2, 3, 4, 5, 6, 7, 8


def gemm_tile(m: int, n: int, k: int) -> int:
    """The tile (``TILE_*``) that the tiled kernel takes for a product of m rows with n weight rows of k."""
    return core().nnis_gemm_tile(int(m), int(n), int(k))


def gemm_residual_parts(m: int, n: int) -> int:
    """Rows of the ``ss`` scratch that ``gemm_residual`` may fill for these sizes."""
    return core().nnis_gemm_residual_parts(int(m), int(n))


def gemm_residual(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, gain: torch.Tensor, scaled: torch.Tensor,
                  ss: torch.Tensor, tile: int = 0) -> int:
    """The projection that ends a part of a pre-norm block: ``resid`` (float32
    [m, n]) takes x @ w^T in, in place, and the norm that follows is prepared:
    ``scaled`` = bfloat16(resid * gain) and, in ``ss`` [parts, m], parts of
    each row's sum of squares.  Returns how many parts were written; the
    norm's 1 / sqrt(mean + eps) is taken by ``gemm_scaled``, which reads them.
    ``x`` may be the ``KeyRuns`` of a decode attention (where ``fits``): the
    kernel then adds the runs up itself on its way.  ``tile`` (for tests and
    tuning): 0 lets the sizes choose, ``TILE_64x128``, ``TILE_64x64``,
    ``TILE_256x256``, ``TILE_256x192``, ``TILE_128x128``, ``TILE_256x128`` and
    ``TILE_128x192`` ask for the tiled kernel with that tile."""
    _packed(w, "gemm_residual")
    m, k = x.shape
    n = w.shape[0]
    runs = x if isinstance(x, KeyRuns) else None
    for t, what in ((x if runs is None else x.partial, "x"), (resid, "resid"), (gain, "gain"), (scaled, "scaled"),
                    (ss, "ss")):
        _dev(t, what)
        if not t.is_contiguous():
            raise KernelError(f"gemm_residual: {what} must be contiguous")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k:
        raise KernelError("gemm_residual: x must be bfloat16 [m, k] and the weight bfloat16 [n, k]")
    if resid.dtype != torch.float32 or tuple(resid.shape) != (m, n) or scaled.dtype != torch.bfloat16 or tuple(scaled.shape) != (m, n):
        raise KernelError("gemm_residual: resid must be float32 [m, n] and scaled bfloat16 [m, n]")
    if gain.numel() != n:
        raise KernelError(f"gemm_residual: norm weight of {gain.numel()} for width {n}")
    if ss.dtype != torch.float32 or ss.numel() < m:
        raise KernelError("gemm_residual: ss must be float32 [rows, m] (gemm_residual_parts(m, n) rows are always enough)")
    lib = core()
    parts = ctypes.c_int(0)
    if runs is not None:
        if not runs.fits(n):
            raise KernelError("gemm_residual: these key runs are not taken; add them up first (KeyRuns.combine)")
        _check(lib, lib.nnis_gemm_residual_runs(runs.partial.data_ptr(), runs.runs, runs.heads, runs.head_dim, runs.tok_slot.data_ptr(),
                                                w.data_ptr(), resid.data_ptr(), gain.data_ptr(), _code(gain), scaled.data_ptr(),
                                                ss.data_ptr(), ss.numel() // m, m, n, ctypes.addressof(parts), _stream()))
        return parts.value
    work = _gemm_workspace(x.device)
    _check(lib, lib.nnis_gemm_residual(x.data_ptr(), w.data_ptr(), resid.data_ptr(), gain.data_ptr(), _code(gain),
                                       scaled.data_ptr(), ss.data_ptr(), ss.numel() // m, m, n, k, ctypes.addressof(parts),
                                       int(tile), _ptr(work), GEMM_WORKSPACE_BYTES if work is not None else 0,
                                       work.data_ptr() + GEMM_WORKSPACE_BYTES if work is not None else None, _stream()))
    return parts.value


def gemm_scaled(scaled: torch.Tensor, ss: torch.Tensor, parts: int, eps: float, w: torch.Tensor, y: torch.Tensor,
                epilogue: int = EPILOGUE_STORE, rope: Optional[dict] = None, split: int = 0) -> torch.Tensor:
    """y = epilogue( (W . scaled) / sqrt(sum of the parts of ss / k + eps) ):
    the second half of an RMSNorm whose first half ``gemm_residual`` took, with
    the epilogues of ``gemm_fused``."""
    _packed(w, "gemm_scaled")
    m, k = scaled.shape
    n = w.shape[0]
    for t, what in ((scaled, "scaled"), (ss, "ss"), (y, "y")):
        _dev(t, what)
    if scaled.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k or not scaled.is_contiguous():
        raise KernelError("gemm_scaled: scaled must be bfloat16 [m, k] and the weight bfloat16 [n, k]")
    if ss.dtype != torch.float32 or parts <= 0 or ss.numel() < parts * m:
        raise KernelError("gemm_scaled: ss must be float32 [parts, m]")
    r = _check_epilogue("gemm_scaled", m, n, y, epilogue, rope)
    lib = core()
    work = _gemm_workspace(scaled.device)
    bt = r.get("block_table")
    _check(lib, lib.nnis_gemm_scaled(
        scaled.data_ptr(), ss.data_ptr(), int(parts), float(eps), w.data_ptr(), m, n, k, int(epilogue), y.data_ptr(),
        _ptr(r.get("cos")), _ptr(r.get("sin")), r["cos"].shape[0] if r.get("cos") is not None else 0, _ptr(r.get("tok_slot")),
        _ptr(r.get("tok_pos")), _ptr(r.get("k_pages")), _ptr(r.get("v_pages")), _ptr(bt), bt.shape[1] if bt is not None else 0,
        r.get("heads", 0), r.get("kv_heads", 0), r.get("head_dim", 0), *_step_table_pointers(r), int(split), _ptr(work),
        GEMM_WORKSPACE_BYTES if work is not None else 0, _stream()))
    return y


def linear(x: torch.Tensor, weight, out: torch.Tensor) -> torch.Tensor:
    """out = x @ weight^T.  A packed weight (bfloat16) takes the matrix-core
    kernels; a weight as the checkpoint has it (32-bit, or a width the 16-byte
    loads cannot take) the ordered 32-bit product."""
    if isinstance(weight, PackedWeight):
        if x.dtype != torch.bfloat16 or x.data_ptr() % 16 != 0 or out.data_ptr() % 16 != 0:
            raise KernelError(f"linear: a packed weight multiplies bfloat16 rows on 16-byte boundaries, got {x.dtype}")
        return gemm_bf16(x, weight, out)
    return gemm_ordered(x, weight, out)


def _check_pages(q, out, k_pages, v_pages, block_table, heads, kv_heads, head_dim):
    tokens = q.shape[0]
    if q.shape != (tokens, heads * head_dim) or out.shape != q.shape:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {heads} heads of {head_dim}")
    if not _pages_fit(k_pages, v_pages, kv_heads, head_dim):
        raise KernelError(f"attention: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
    if block_table.dtype != torch.int32 or block_table.dim() != 2:
        raise KernelError("attention: block_table must be int32 [slots, pages]")
    for t, what in ((q, "q"), (out, "out"), (k_pages, "k_pages"), (v_pages, "v_pages")):
        _dev(t, what)
        if t.dtype != torch.bfloat16:
            raise KernelError(f"attention: the matrix-core kernels take bfloat16, {what} is {t.dtype}")


def prefill_tile_rows(heads: int, kv_heads: int, head_dim: int, columns: int = 0) -> int:
    """Query rows per work item of ``attention_prefill_bf16`` for these sizes.
    ``columns``: the most 16-column tiles (query tiles x heads of a group) a
    wave carries; 0 for as many as the head size allows."""
    return attention_module(head_dim).nnis_attention_prefill_tile_rows(heads, kv_heads, columns)


def prefill_max_waves(heads: int, kv_heads: int, head_dim: int, columns: int = 0) -> int:
    return attention_module(head_dim).nnis_attention_prefill_max_waves(heads, kv_heads, columns)


def attention_prefill_bf16(q, out, k_pages, v_pages, block_table, tile_seq, tile_row0, seq_slot, seq_start, seq_pos0,
                           heads, kv_heads, head_dim, scale, window=0, waves=1, columns=0):
    """Causal attention of whole runs of new tokens over the cache, on the
    matrix cores.  ``tile_seq``/``tile_row0`` (int32) name, per work item, a
    sequence of the step and the first of ``prefill_tile_rows`` rows of its
    new tokens; ``seq_start`` [batch + 1] gives each sequence's packed rows."""
    _check_pages(q, out, k_pages, v_pages, block_table, heads, kv_heads, head_dim)
    for t in (tile_seq, tile_row0, seq_slot, seq_start, seq_pos0):
        _dev(t, "step metadata")
        if t.dtype != torch.int32:
            raise KernelError("attention: step metadata must be int32")
    tiles = tile_seq.numel()
    if tile_row0.numel() != tiles or seq_start.numel() != seq_slot.numel() + 1 or seq_pos0.numel() != seq_slot.numel():
        raise KernelError("attention: step metadata arrays do not fit each other")
    lib = attention_module(head_dim)
    _check(lib, lib.nnis_attention_prefill_bf16(q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
                                                block_table.data_ptr(), block_table.shape[1], tile_seq.data_ptr(),
                                                tile_row0.data_ptr(), tiles, seq_slot.data_ptr(), seq_start.data_ptr(),
                                                seq_pos0.data_ptr(), heads, kv_heads, head_dim, int(window), float(scale),
                                                int(waves), int(columns), _stream()))
    return out


def attention_decode_bf16(q, out, k_pages, v_pages, block_table, tok_slot, tok_pos, heads, kv_heads, head_dim, scale,
                          window=0, splits=1, partial=None, waves=1, kernel="auto", keep_runs=False, token_pages=None):
    """One query token per sequence over its cached keys.  The keys are cut
    into ``splits`` runs, each a block of ``waves`` waves that deal its pages
    among themselves and merge in LDS; the runs are summed by a second kernel.
    ``partial``: float32 scratch of tokens * heads * splits * (head_dim + 4)
    when splits > 1 (``decode_scratch`` keeps one per device).  ``keep_runs``
    (with splits > 1): the second kernel is left out and a ``KeyRuns`` is
    returned in place of ``out`` -- the projection that follows adds the runs
    up itself (``gemm_residual``), or ``KeyRuns.combine()`` does.  ``kernel``:
    "keys" (keys on lanes; groups of up to 4 heads of up to 128 channels),
    "columns" (heads in the columns of a tile; any group the head size
    carries) or "auto", which takes "keys" where it fits.  ``token_pages``
    (int32 [tokens, pages], ``StepTables.pages``): each token's sequence's
    pages, read in place of the block table's row of the token's slot."""
    _check_pages(q, out, k_pages, v_pages, block_table, heads, kv_heads, head_dim)
    tokens = q.shape[0]
    table = block_table
    if token_pages is not None:
        _dev(token_pages, "token_pages")
        if token_pages.dtype != torch.int32 or token_pages.dim() != 2 or token_pages.shape[0] < tokens:
            raise KernelError("attention: token_pages must be int32 [tokens, pages]")
        table = token_pages
    for t in (tok_slot, tok_pos):
        _dev(t, "step metadata")
        if t.dtype != torch.int32 or t.numel() < tokens:
            raise KernelError("attention: tok_slot / tok_pos must be int32 with one entry per token")
    if splits > 1:
        if partial is None or partial.dtype != torch.float32 or partial.numel() < tokens * heads * splits * (head_dim + 4):
            raise KernelError("attention: splits need float32 scratch of tokens * heads * splits * (head_dim + 4)")
        _dev(partial, "partial")
    lib = attention_module(head_dim)
    _check(lib, lib.nnis_attention_decode_bf16(q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
                                               table.data_ptr(), table.shape[1], tok_slot.data_ptr(),
                                               tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim, int(window),
                                               float(scale), int(splits), int(waves), _ptr(partial) if splits > 1 else None,
                                               _DECODE_KERNELS[kernel], 0 if (keep_runs and splits > 1) else 1,
                                               1 if token_pages is not None else 0, _stream()))
    if keep_runs and splits > 1:
        return KeyRuns(partial, int(splits), tokens, heads, head_dim, tok_slot, out)
    return out


# Up to this many tokens a decode step leaves its runs of keys to the output projection; beyond, every block of
# the projection making the same activations again costs more than the kernel between the two.
KEY_RUNS_MOST_TOKENS = 4


class KeyRuns:
    """What the decode attention leaves when it cuts the keys into runs and is
    told not to add them up: per (token, head, run) the run's outputs, its
    softmax reference and its sum, in ``partial`` (the device's decode scratch:
    valid until the next decode attention on this device).  A stand-in for the
    attention's output [tokens, heads * head_dim] in bfloat16."""

    dtype = torch.bfloat16

    def __init__(self, partial, runs, tokens, heads, head_dim, tok_slot, out):
        self.partial, self.runs, self.tokens, self.heads, self.head_dim = partial, runs, tokens, heads, head_dim
        self.tok_slot, self.out = tok_slot, out
        self.shape = (tokens, heads * head_dim)

    def fits(self, rows_out: int) -> bool:
        """Whether ``gemm_residual`` takes these runs for a weight of ``rows_out`` rows."""
        return bool(core().nnis_gemm_residual_runs_fits(self.tokens, int(rows_out), self.heads, self.head_dim, self.runs))

    def combine(self) -> torch.Tensor:
        """The attention's output, added up by the kernel of its own."""
        lib = attention_module(self.head_dim)
        _check(lib, lib.nnis_attention_combine(self.partial.data_ptr(), self.out.data_ptr(), self.tok_slot.data_ptr(), self.tokens,
                                               self.heads, self.head_dim, self.runs, _stream()))
        return self.out


_DECODE_KERNELS = {"auto": 0, "columns": 1, "keys": 2}
_decode_scratch = {}  # per device: the scratch in use


def decode_scratch(device, floats: int) -> torch.Tensor:
    """Scratch of the split decode attention, kept per device.  Calls on one
    device share it, so they must follow one another on one stream.  A call
    that needs more gets a larger tensor, made outside a graph capture only
    (the run that warms a graph up sizes it), and the smaller one is let go:
    kernels already on the stream are ahead of whoever gets its memory next,
    and a captured graph, which has the address it was captured with baked in
    and goes on writing there on every replay, holds the tensor itself for as
    long as it lives (``Part.held_buffers``, ``engine/graph.py``)."""
    key = (device.type, device.index)
    held = _decode_scratch.get(key)
    if held is None or held.numel() < floats:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("attention: the decode scratch would have to grow inside a graph capture")
        held = _decode_scratch[key] = torch.empty(max(floats, 2 * held.numel() if held is not None else 1 << 16),
                                                   dtype=torch.float32, device=device)
    return held


def decode_scratch_held(device):
    """The scratch a decode attention launched now would use (None: none made yet)."""
    return _decode_scratch.get((device.type, device.index))


def decode_max_waves(heads: int, kv_heads: int, head_dim: int) -> int:
    return attention_module(head_dim).nnis_attention_decode_max_waves(heads, kv_heads)


def decode_plan(batch: int, kv_heads: int, longest: int, max_waves: int = 4, width: int = 0):
    """(splits, waves) of a decode step's attention.  A block of 4 waves deals
    a sequence's pages among its waves.  Cutting the keys into runs for more
    blocks costs a second kernel that sums the runs (dearer the more runs), so
    it pays only from about 9 pages on; then a wave gets 1 to 2 pages, in at
    most 8 runs and about a thousand waves on the chip.  Powers of two.
    ``width`` (query heads x head size, 0: unknown) says what a run costs to
    sum: beyond 1024 runs pay from 17 pages on and a wave gets 2 to 4 pages
    (32 heads of 64, 128 to 2k keys, tokens/s with the one rule and the other:
    batch 8 on 4 key-value heads 5,654 against 5,497, batch 1 862 against 852;
    batch 1 on 32 key-value heads 700 against 682).
    Measured on 9 query / 3 key-value heads of 64 (microseconds a layer, runs
    of 1/2/4/8/16): batch 1 at 1k keys 7.9/8.3/8.7/10.7, at 8k 30/20/15/14/17;
    batch 8 at 2k 11.6/11.0/9.5/9.3/13.6; batch 32 at 4k 27/25/31/34/45.  And
    on whole decode steps of 30 such layers (milliseconds, runs of 1/2/4/8 with
    4 waves): batch 1 at 1k keys 0.839/0.822/0.790/0.775, at 128 to 2k
    0.957/0.882/0.823/0.790, at 256 keys 0.724/0.742/0.741/0.749; batch 8 at 1k
    0.943/0.952/0.919/0.914, at 128 to 2k 1.051/0.968/0.910/0.890, at 512 keys
    0.874/0.900/0.881/0.893."""
    pages = (longest + 63) // 64
    waves = 1
    while waves * 2 <= min(max_waves, pages):
        waves *= 2
    splits = 1
    first, each = (8, 4) if 0 < width <= 1024 else (16, 8)  # runs from more than `first` pages on, about `each` pages a run
    if pages > first:
        wanted = min(8, (pages + each - 1) // each)
        room = max(1, 1024 // max(1, batch * kv_heads * waves))
        while splits * 2 <= room and splits < wanted:
            splits *= 2
    if splits == 1 and batch * kv_heads >= 2048:
        # eight and more blocks a compute unit: two waves a block read as fast as four or faster (batch 64 on 32
        # key-value heads of 64, whole steps: 1,000 to 1,100 keys each 16,230 tokens/s against 15,900, 128 to 2k
        # 15,620 either way); at four blocks a unit four waves are faster (batch 32: 12,010 against 11,600)
        waves = min(waves, 2)
    return splits, waves


# The prefill attention's plan: the waves of a block, and the most column tiles (query tiles x heads of a group) a
# wave carries, 0 for as many as the head size allows.  Fewer columns make more and lighter work items, which a step
# of few tokens needs to fill the chip, and read keys and values more often, which a long one pays for.  Measured on
# one sequence, microseconds a layer, as it was (2, 4, 8 waves from 128, 512, 1,024 tokens on, always the widest
# tiles) against these plans: 9/3 heads of 64 at 128 / 512 / 768 tokens 16.9 / 11.7 / 11.0 against 9.8 / 9.7 / 10.1;
# 32/32 heads at 128 / 512 / 1,024 10.9 / 12.9 / 22.5 against 9.4 / 11.1 / 16.7; 32/4 heads 10.3 / 12.1 / 22.3
# against 9.6 / 10.8 / 17.3.  From 1,024 tokens on 9/3 heads are fastest with the widest tiles and 8 waves (12.9
# against 13.3), from 1,536 on all three are (9/3: 14.9 against 22.9 with two columns).  Whole prompt steps, ms:
# TinyLlama shape 128 / 1,024 tokens 1.68 / 4.31 -> 1.60 / 4.19, 135M shape 128 / 256 1.04 / 1.32 -> 0.99 / 1.23.
PREFILL_MANY_ROWS = 65536  # rows x query heads from which a step has work items enough for the widest tiles
PREFILL_SOME_ROWS = 16384  # ... from which a step of 1,024 to 1,279 tokens still gains by two columns
# Items of four columns (up to 64 channels, any group but 3) merge the states of 8 waves through 72 KB of LDS: worth it
# while a step's items are few (16 heads of 64 at 2,048 tokens 26 us a layer against 37 with 4 waves, 16/4 heads of 48
# 25 against 39; 32 heads at 1,024 tokens 21 against 25), not beyond (32 heads at 1,536 tokens 41 against 35, 64/8 heads
# at 2,048 83 against 73).
PREFILL_EIGHT_WAVES_MOST = 40960


def prefill_plan(longest: int, rows: int, heads: int, head_dim: int = 64, kv_heads: int = 0):
    """(waves of a block, column option) of the prefill attention for a step of ``rows`` rows (what the engine
    plans for: a step's tokens rounded up as a replayed step's are) whose longest sequence has ``longest``
    (``kv_heads``: 0 for as many as ``heads``)."""
    plan_class = prefill_plan_class(longest)
    size = rows * heads
    # A step with work items for about twice the waves that the chip holds (two a SIMD up to 64 channels, one
    # beyond; an item is 16 rows x 4, 2 or 1 columns) gives each item to one wave, which needs no merge and pays an
    # item's first loads once.  One sequence, microseconds a layer with one wave against the plan by length: 32
    # heads of 64 at 8,192 tokens 349 against 467; 64/8 heads of 64 at 4,096 180 against 243; 32/8 heads of 128 at
    # 2,048 66 against 102, at 8,192 833 against 1,306; 16 heads of 96 at 8,192 259 against 349.  Up to 64 channels a
    # step of half that size has the items with two columns: 32 heads at 4,096 tokens 119 against 137, 64/8 heads at
    # 2,048 64 against 74, 16 heads at 8,192 213 against 243, and from three eighths on 32 heads at 3,072 83 against
    # 93 -- where two columns divide a group's heads (of 9/3 heads they would leave a quarter of the columns empty:
    # 227 against 145 at 8,192; 24/8 heads of 64 at 8,192 tokens have items of three columns for twice the chip's
    # waves: 276 with one wave an item against 345).  At a quarter (32 heads at 2,048 tokens) the kernel alone took 49
    # against 47 to 56 and whole prompts 2 to 3% longer: not taken there.
    # With fewer items the waves of a block deal an item's keys: 9/3 heads of 64 at 8,192 tokens 141 with 8 waves,
    # 193 with one.
    group = heads // kv_heads if kv_heads else 1
    wide = (3 if group == 3 else 4) if head_dim <= 64 else (2 if head_dim <= 128 else 1)  # (a group of 3 heads fills 3 columns)
    # (Since the waves of a block that holds a long item and a short one are shared out by their pages also in
    # odd numbers -- 3 + 1 of 4 -- the blocks of 4 waves hold out longer: 32 heads of 64 at 3,072 tokens 68 us
    # against 78 with one wave an item of two columns, equal at 4,096; 32/8 heads of 128 at 2,048 tokens 58
    # against 66 with one wave an item, at 4,096 200 against 179.)
    many = 2 * (2048 if head_dim <= 64 else 1024) * 16 * wide
    if size >= (2 * many if 64 < head_dim <= 128 else many):
        return 1, 0
    if head_dim <= 64 and 2 * size >= many and (group == 1 or group % 2 == 0):
        return 1, 2
    waves = (1, 2, 4, 8, 8)[plan_class]
    if waves == 8 and head_dim <= 64 and group != 3 and size > PREFILL_EIGHT_WAVES_MOST:
        waves = 4
    if plan_class == 0 or plan_class == 4 or size >= PREFILL_MANY_ROWS:
        return waves, 0
    if plan_class == 3:
        if size < PREFILL_SOME_ROWS:
            return 8, 0
        return (4, 0) if group == 3 else (4, 2)  # (two columns would leave a group of 3 heads a quarter of them empty)
    return waves, plan_class  # 2 waves and one column from 128 tokens on, 4 waves and two columns from 512 on


def prefill_plan_class(longest: int) -> int:
    """Steps whose longest sequence falls into the same class launch the same prefill attention kernels
    (``attention`` picks the waves of a block, and the column option, by these thresholds)."""
    return 4 if longest >= 1280 else (3 if longest >= 1024 else (2 if longest >= 512 else (1 if longest >= 128 else 0)))


PREFILL_CLASS_LENGTH = (1, 128, 512, 1024, 1280)  # a length of each class


def _prefill_tile_arrays(new_tokens, first_positions, rows: int):
    """``prefill_tile_items`` as two int64 arrays (a step of thousands of tokens has hundreds of tiles: arrays,
    not a loop, while the GPU waits for the host)."""
    import numpy as np

    counts, pos0 = np.asarray(new_tokens, dtype=np.int64), np.asarray(first_positions, dtype=np.int64)
    tiles = (counts + rows - 1) // rows  # of each sequence
    seq = np.repeat(np.arange(counts.size, dtype=np.int64), tiles)
    row0 = (np.arange(int(tiles.sum()), dtype=np.int64) - np.repeat(np.cumsum(tiles) - tiles, tiles)) * rows
    last_key = pos0[seq] + np.minimum(row0 + rows, counts[seq])  # one beyond the last key that the tile's last row reads
    order = np.lexsort((-row0, -seq, -last_key))  # most keys first; among equals the later sequence, the later row
    return seq[order], row0[order]


def prefill_tile_items(new_tokens, first_positions, rows: int):
    """Work items (sequence of the step, first row) of a prefill step for tiles of ``rows`` query rows: those
    with the most keys first."""
    seq, row0 = _prefill_tile_arrays(new_tokens, first_positions, rows)
    return seq.tolist(), row0.tolist()


NO_ROWS = 1 << 24  # first row of a work item that has none: it lies beyond any sequence's tokens


def prefill_tile_list(new_tokens, first_positions, padded, rows: int):
    """``prefill_tile_items`` as one int32 array [2, items] (row 0 the sequences, row 1 the first rows), the form in
    which a step keeps its work lists (``StepContext.lists``).  ``padded``: None, or (sequences, rows of the step)
    of a step that runs from fixed buffers: the list then has as many items as any step of that shape can have
    (rows of the step / rows of a tile + sequences), those beyond the step's own with no rows."""
    import numpy as np

    seqs, row0s = _prefill_tile_arrays(new_tokens, first_positions, rows)
    count = len(seqs)
    if padded is not None:
        count = padded[1] // rows + padded[0]
        if len(seqs) > count:
            raise KernelError(f"{len(seqs)} work items for a step of {padded[0]} sequences and {padded[1]} rows")
    out = np.empty((2, count), dtype=np.int32)
    out[0, :len(seqs)], out[0, len(seqs):] = seqs, 0
    out[1, :len(seqs)], out[1, len(seqs):] = row0s, NO_ROWS
    return out


def attention(q: torch.Tensor, out: torch.Tensor, view, ctx, heads: int, kv_heads: int, head_dim: int, scale: float,
              window: int = 0, keep_runs: bool = False, tables: Optional[StepTables] = None, plan=None):
    """Attention of the step's tokens over the cache ``view``: bfloat16 with a
    head size in steps of 16 runs on the matrix cores (one kernel for single
    tokens, one for runs of tokens); anything else takes the 32-bit kernel.
    ``keep_runs``: a decode step whose keys are cut into runs may return them
    as ``KeyRuns`` instead of the output (see ``attention_decode_bf16``).
    ``plan``: (runs, waves) of a step of single tokens (``decode_plan``), or
    (waves, columns) of a step of prompts (``prefill_plan``); None: as those
    functions choose for the step's planned sizes."""
    fast = (q.dtype == torch.bfloat16 and view.k_pages.dtype == torch.bfloat16 and head_dim % 16 == 0)
    if fast and ctx.decode and heads // kv_heads <= 16 * (4 if head_dim <= 64 else (2 if head_dim <= 128 else 1)):
        splits, waves = plan or decode_plan(ctx.batch, kv_heads, ctx.planned_len, width=heads * head_dim)
        waves = min(waves, decode_max_waves(heads, kv_heads, head_dim))
        partial = None
        if splits > 1:
            partial = decode_scratch(q.device, q.shape[0] * heads * splits * (head_dim + 4))
        return attention_decode_bf16(q, out, view.k_pages, view.v_pages, view.block_table, ctx.tok_slot, ctx.tok_pos, heads,
                                     kv_heads, head_dim, scale, window, splits, partial, waves,
                                     keep_runs=keep_runs and q.shape[0] <= KEY_RUNS_MOST_TOKENS,
                                     token_pages=tables.pages if tables is not None else None)
    if fast and not ctx.decode:
        # A tile's keys are a chain of dependent loads: the longest tile sets the kernel's time.  The waves of
        # a block deal the keys among themselves (their merge lives in LDS).
        waves, columns = plan or prefill_plan(ctx.planned_len, ctx.planned_rows, heads, head_dim, kv_heads)
        waves = min(waves, prefill_max_waves(heads, kv_heads, head_dim, columns))
        rows = prefill_tile_rows(heads, kv_heads, head_dim, columns)
        tiles = ctx.lists.device_list(("attention_tiles", rows), lambda new, first, padded: prefill_tile_list(new, first, padded, rows))
        return attention_prefill_bf16(q, out, view.k_pages, view.v_pages, view.block_table, tiles[0], tiles[1],
                                      ctx.seq_slot, ctx.seq_start, ctx.seq_pos0, heads, kv_heads, head_dim, scale, window,
                                      waves, columns)
    return attention_rows(q, out, view.k_pages, view.v_pages, view.block_table, ctx.tok_slot, ctx.tok_pos, heads,
                          kv_heads, head_dim, scale, window)


def sample(logits: torch.Tensor, weights: torch.Tensor, row_slot: torch.Tensor, rng: torch.Tensor,
           temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, out: torch.Tensor, by_slot: bool = False,
           best: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Seeded sampling per row; rows whose slot is negative are skipped (their
    ``out`` stays as it is).  ``rng`` is int64 [slots] holding each sequence's
    SplitMix64 state; ``weights`` is float64 scratch of at least [rows, vocab].
    ``temperature``, ``top_k`` and ``top_p`` hold a value per row, or, with
    ``by_slot``, per slot (like ``rng``).  ``best`` (int32 [rows], may be
    ``out``) holds an index of each row's maximum where the caller has it
    (``argmax``); without it the maxima are found here.  A row with a
    non-finite logit gets -1."""
    for t, what in ((logits, "logits"), (weights, "weights"), (row_slot, "row_slot"), (rng, "rng"),
                    (temperature, "temperature"), (top_k, "top_k"), (top_p, "top_p"), (out, "out")):
        _dev(t, what)
    rows, vocab = logits.shape
    if logits.dtype != torch.float32 or weights.dtype != torch.float64 or weights.numel() < rows * vocab:
        raise KernelError("sample: logits must be float32 and weights float64 scratch of [rows, vocab]")
    if rng.dtype != torch.int64 or row_slot.dtype != torch.int32 or top_k.dtype != torch.int32 or out.dtype != torch.int32:
        raise KernelError("sample: rng must be int64; row_slot, top_k and out int32")
    if temperature.dtype != torch.float32 or top_p.dtype != torch.float32:
        raise KernelError("sample: temperature and top_p must be float32")
    if min(row_slot.numel(), out.numel()) < rows:
        raise KernelError("sample: per-row arrays are shorter than the rows")
    needed = rng.numel() if by_slot else rows
    if min(temperature.numel(), top_k.numel(), top_p.numel()) < needed:
        raise KernelError("sample: temperature, top_k and top_p need a value per " + ("slot" if by_slot else "row"))
    if best is None:
        best = argmax(logits, torch.empty(rows, dtype=torch.int32, device=logits.device))
    else:
        _dev(best, "best")
        if best.dtype != torch.int32 or best.numel() < rows:
            raise KernelError("sample: best must be int32 [rows]")
    lib = core()
    _check(lib, lib.nnis_sample(logits.data_ptr(), weights.data_ptr(), rows, vocab, row_slot.data_ptr(), rng.data_ptr(),
                                temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), 1 if by_slot else 0,
                                best.data_ptr(), out.data_ptr(), _stream()))
    return out
