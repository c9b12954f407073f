"""The plain host references of the kernels' operations (``csrc/reference.cpp``:
scalar C++ in a fixed order of 32-bit arithmetic), on numpy arrays.  What the
device kernels are compared with in the tests; the product never calls them,
and they need no GPU.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import numpy as np

from ..errors import KernelError
from . import lib as _lib

_F = ctypes.POINTER(ctypes.c_float)
_I = ctypes.POINTER(ctypes.c_int)
_U64 = ctypes.POINTER(ctypes.c_uint64)
_INT, _FLT, _SIZE = ctypes.c_int, ctypes.c_float, ctypes.c_size_t
_SIGNATURES = {
    "nnis_ref_embed": [_I, _F, _F, _INT, _INT, _INT],
    "nnis_ref_rmsnorm": [_F, _F, _F, _INT, _INT, _FLT],
    "nnis_ref_rope_tables": [_F, _F, _INT, _INT, _FLT],
    "nnis_ref_rope_rotate_half": [_F, _F, _F, _F, _I, _INT, _INT, _INT, _INT, _INT],
    "nnis_ref_attention": [_F, _F, _F, _F, _INT, _INT, _INT, _INT, _INT, _FLT, _INT],
    "nnis_ref_silu_mul": [_F, _F, _F, _SIZE],
    "nnis_ref_gemm": [_F, _F, _F, _INT, _INT, _INT],
    "nnis_ref_residual_add": [_F, _F, _SIZE],
    "nnis_ref_argmax": [_F, _I, _INT, _INT],
    "nnis_ref_splitmix64": [_U64, _U64, _INT],
    "nnis_ref_sample": [_F, _INT, _FLT, _INT, _FLT, _U64, _I],
}
_handle = None


def _library():
    global _handle
    if _handle is None:
        handle = _lib.load_module("reference")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes, fn.restype = argtypes, ctypes.c_int
        _handle = handle
    return _handle


def _f(array) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=np.float32)


def _i(array) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=np.int32)


def _p(array: np.ndarray, kind):
    return array.ctypes.data_as(kind)


def _check(status: int) -> None:
    if status != 0:
        raise KernelError(_library().nnis_last_error().decode(errors="replace"))


def embed(ids, table) -> np.ndarray:
    ids, table = _i(ids), _f(table)
    out = np.empty((ids.size, table.shape[1]), dtype=np.float32)
    _check(_library().nnis_ref_embed(_p(ids, _I), _p(table, _F), _p(out, _F), ids.size, table.shape[1], table.shape[0]))
    return out


def rmsnorm(x, weight, eps: float) -> np.ndarray:
    x, weight = _f(x), _f(weight)
    out = np.empty_like(x)
    _check(_library().nnis_ref_rmsnorm(_p(x, _F), _p(weight, _F), _p(out, _F), x.shape[0], x.shape[1], float(eps)))
    return out


def rope_tables(positions: int, rot_dim: int, theta: float) -> Tuple[np.ndarray, np.ndarray]:
    cos = np.empty((positions, rot_dim // 2), dtype=np.float32)
    sin = np.empty_like(cos)
    _check(_library().nnis_ref_rope_tables(_p(cos, _F), _p(sin, _F), positions, rot_dim, float(theta)))
    return cos, sin


def rope_rotate_half(x, cos, sin, positions, rot_dim: Optional[int] = None) -> np.ndarray:
    """x: [tokens, heads, head_dim]; cos / sin: the tables [positions, rot_dim / 2]; positions: each token's."""
    x, cos, sin, positions = _f(x), _f(cos), _f(sin), _i(positions)
    tokens, heads, head_dim = x.shape
    out = np.empty_like(x)
    _check(_library().nnis_ref_rope_rotate_half(_p(x, _F), _p(out, _F), _p(cos, _F), _p(sin, _F), _p(positions, _I), tokens, heads,
                                                head_dim, 2 * cos.shape[1] if rot_dim is None else rot_dim, cos.shape[0]))
    return out


def attention(q, k, v, scale: float, first: int = 0, window: int = 0) -> np.ndarray:
    """q: [tokens, heads, head_dim], the queries at positions first ..; k, v: [first + tokens, kv_heads, head_dim]."""
    q, k, v = _f(q), _f(k), _f(v)
    tokens, heads, head_dim = q.shape
    if k.shape != v.shape or k.shape[0] != first + tokens or k.shape[2] != head_dim:
        raise KernelError(f"reference attention: q {q.shape}, k {k.shape}, v {v.shape}, first {first} do not fit")
    out = np.empty_like(q)
    _check(_library().nnis_ref_attention(_p(q, _F), _p(k, _F), _p(v, _F), _p(out, _F), tokens, first, heads, k.shape[1], head_dim,
                                         float(scale), int(window)))
    return out


def silu_mul(gate, up) -> np.ndarray:
    gate, up = _f(gate), _f(up)
    out = np.empty_like(gate)
    _check(_library().nnis_ref_silu_mul(_p(gate, _F), _p(up, _F), _p(out, _F), gate.size))
    return out


def gemm(x, w) -> np.ndarray:
    """x [m, k] times w [n, k] transposed, every output one ascending chain of fused multiply-adds."""
    x, w = _f(x), _f(w)
    out = np.empty((x.shape[0], w.shape[0]), dtype=np.float32)
    _check(_library().nnis_ref_gemm(_p(x, _F), _p(w, _F), _p(out, _F), x.shape[0], w.shape[0], x.shape[1]))
    return out


def residual_add(residual, delta) -> np.ndarray:
    out, delta = _f(residual).copy(), _f(delta)
    _check(_library().nnis_ref_residual_add(_p(out, _F), _p(delta, _F), out.size))
    return out


def argmax(logits) -> np.ndarray:
    logits = _f(logits)
    out = np.empty(logits.shape[0], dtype=np.int32)
    _check(_library().nnis_ref_argmax(_p(logits, _F), _p(out, _I), logits.shape[0], logits.shape[1]))
    return out


class Generator:
    """A sequence's SplitMix64 state."""

    def __init__(self, seed: int):
        self.state = np.array([seed & ((1 << 64) - 1)], dtype=np.uint64)

    def next_u64(self, draws: int = 1) -> np.ndarray:
        out = np.empty(draws, dtype=np.uint64)
        _check(_library().nnis_ref_splitmix64(_p(self.state, _U64), _p(out, _U64), draws))
        return out


def sample(logits, generator: Generator, temperature: float = 1.0, top_k: Optional[int] = None, top_p: Optional[float] = None) -> int:
    logits = _f(logits)
    token = np.zeros(1, dtype=np.int32)
    _check(_library().nnis_ref_sample(_p(logits, _F), logits.size, float(temperature), int(top_k or 0), float(top_p or 0.0),
                                      _p(generator.state, _U64), _p(token, _I)))
    return int(token[0])
