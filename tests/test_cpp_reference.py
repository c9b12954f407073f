"""The plain C++ references of the kernels' operations (``nnis_amd/csrc/reference.cpp``), pinned twice: by the
vectors the reference's own tests hold, and by the tests' plain Python model, which is written from the same
formulas in another language with another library's sums.  (The GPU tests then compare kernels with these:
``tests/test_gpu_kernels.py``.)  The host compiler builds the module on first use; no GPU is needed."""

import math

import numpy as np
import pytest
import torch

import plain_llama as P
from nnis_amd.errors import KernelError
from nnis_amd.kernels import reference as R


def test_rmsnorm():
    # /root/reference/crates/nnis-model/src/kernels.rs:470-488
    x = np.array([[1.0, -2.0, 3.0, -4.0], [2.0, 1.0, -1.0, 0.5]], dtype=np.float32)
    w = np.array([0.5, 1.0, 1.5, 2.0], dtype=np.float32)
    got = R.rmsnorm(x, w, 1e-5)
    assert abs(got[0, 0] - 0.18257406) < 1e-6 and abs(got[1, 2] - (-1.19999616)) < 1e-6
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal((7, 100)).astype(np.float32) * 3, 1 + 0.1 * rng.standard_normal(100).astype(np.float32)
    want = P.rms_norm(torch.from_numpy(x).double(), torch.from_numpy(w).double(), 3e-6).numpy()
    assert np.abs(R.rmsnorm(x, w, 3e-6) - want).max() < 1e-5


def test_rotation_tables_and_pairing():
    for positions, rot_dim, theta in ((64, 16, 10000.0), (300, 64, 100000.0), (50, 6, 500000.0)):
        cos, sin = R.rope_tables(positions, rot_dim, theta)
        want_cos, want_sin = P.rope_tables(positions, rot_dim, theta)
        assert np.array_equal(cos, want_cos) and np.array_equal(sin, want_sin)  # the same 32-bit steps: bit for bit
    # /root/reference/crates/nnis-model/src/runtime_kernels.rs:306-341: 2 heads of 4, table row 1
    x = np.array([1.0, 2.0, 3.0, 4.0, -1.0, 0.5, 2.0, -3.0], dtype=np.float32).reshape(1, 2, 4)
    cos = np.array([[9.0, 9.0], [0.5, -0.25]], dtype=np.float32)
    sin = np.array([[9.0, 9.0], [0.25, 0.75]], dtype=np.float32)
    got = R.rope_rotate_half(x, cos, sin, [1]).ravel()
    assert np.allclose(got, [-0.25, -3.5, 1.75, 0.5, -1.0, 2.125, 0.75, 1.125], atol=1e-6)
    # part of a head rotated, the rest passed through; against the plain model on its first channels
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 3, 24)).astype(np.float32)
    cos, sin = R.rope_tables(40, 16, 1000.0)
    positions = [0, 7, 7, 39, 2]
    got = R.rope_rotate_half(x, cos, sin, positions, rot_dim=16)
    want = P.rope_rotate_half(torch.from_numpy(x[..., :16]).double(), torch.from_numpy(cos[positions]).double(),
                              torch.from_numpy(sin[positions]).double()).numpy()
    assert np.abs(got[..., :16] - want).max() < 1e-6 and np.array_equal(got[..., 16:], x[..., 16:])
    with pytest.raises(KernelError, match="beyond the tables"):
        R.rope_rotate_half(x, cos, sin, [0, 1, 2, 3, 40])


def test_attention():
    # /root/reference/crates/nnis-model/src/kernels.rs:501-558: two cached positions, scale 1, grouped heads
    k = np.array([[[1.0, 0.0], [1.0, 1.0]], [[0.0, 1.0], [-1.0, 1.0]]], dtype=np.float32)
    v = np.array([[[10.0, 0.0], [1.0, 2.0]], [[0.0, 20.0], [3.0, 4.0]]], dtype=np.float32)
    e, e2 = math.e, math.exp(2.0)
    q = np.array([[[1.0, 0.0], [0.0, 1.0], [1.0, 0.0], [0.0, 1.0]]], dtype=np.float32)  # the query at position 1
    out = R.attention(q, k, v, 1.0, first=1).ravel()
    want = [10 * e / (e + 1), 20 / (e + 1), 10 / (e + 1), 20 * e / (e + 1), (e2 + 3) / (e2 + 1), (2 * e2 + 4) / (e2 + 1), 2.0, 3.0]
    assert np.allclose(out, want, atol=2e-5)
    # a whole sequence, and its tail alone over the same keys, against the plain model; a window against a mask
    rng = np.random.default_rng(2)
    t, heads, kv_heads, hd = 23, 6, 2, 16
    q = rng.standard_normal((t, heads, hd)).astype(np.float32)
    k, v = rng.standard_normal((t, kv_heads, hd)).astype(np.float32), rng.standard_normal((t, kv_heads, hd)).astype(np.float32)
    scale = 1 / math.sqrt(hd)
    want = P.causal_attention(torch.from_numpy(q).double(), torch.from_numpy(k).double(), torch.from_numpy(v).double(), scale).numpy()
    assert np.abs(R.attention(q, k, v, scale) - want).max() < 1e-5
    assert np.abs(R.attention(q[15:], k, v, scale, first=15) - want[15:]).max() < 1e-5
    window = 5
    scores = np.einsum("thd,phd->thp", q.astype(np.float64), np.repeat(k, heads // kv_heads, axis=1).astype(np.float64)) * scale
    place = np.arange(t)
    counts = (place[None, :] <= place[:, None]) & (place[None, :] > place[:, None] - window)
    scores = np.where(counts[:, None, :], scores, -np.inf)
    weights = np.exp(scores - scores.max(-1, keepdims=True))
    weights /= weights.sum(-1, keepdims=True)
    want = np.einsum("thp,phd->thd", weights, np.repeat(v, heads // kv_heads, axis=1).astype(np.float64))
    assert np.abs(R.attention(q, k, v, scale, window=window) - want).max() < 1e-5


def test_products_gating_and_the_stream():
    rng = np.random.default_rng(3)
    x, w = rng.standard_normal((5, 300)).astype(np.float32), rng.standard_normal((7, 300)).astype(np.float32)
    got = R.gemm(x, w)
    assert np.abs(got - x.astype(np.float64) @ w.astype(np.float64).T).max() < 1e-4
    # one ascending chain of fused multiply-adds: reproduced step by step in 64-bit with one rounding a step
    chain = np.float32(0.0)
    for a, b in zip(x[2], w[4]):
        chain = np.float32(np.float64(a) * np.float64(b) + np.float64(chain))
    assert got[2, 4] == chain
    # the checkpoint's [out, in] orientation (/root/reference/crates/nnis-model/src/safetensors_loader.rs:1063-1072)
    assert np.array_equal(R.gemm([[1.0, 0.0, -1.0]], [[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]]), [[-2.0, -2.0]])
    gate, up = rng.standard_normal(1000).astype(np.float32) * 4, rng.standard_normal(1000).astype(np.float32)
    want = (P.silu(torch.from_numpy(gate).double()) * torch.from_numpy(up).double()).numpy()
    assert (np.abs(R.silu_mul(gate, up) - want) <= 1e-6 * (1 + np.abs(want))).all()
    assert R.silu_mul([0.0], [5.0])[0] == 0.0 and abs(R.silu_mul([1.0], [1.0])[0] - 1 / (1 + math.exp(-1))) < 1e-7  # SiLU on the gate
    assert np.array_equal(R.residual_add([1.0, 2.0], [0.5, -2.0]), [1.5, 0.0])
    table = rng.standard_normal((11, 6)).astype(np.float32)
    assert np.array_equal(R.embed([3, 0, 10, 3, 11, -1], table), np.stack([table[3], table[0], table[10], table[3], np.zeros(6), np.zeros(6)]))


def test_selection():
    logits = np.array([[0.1, 0.7, 0.7, -1.0], [5.0, 5.0, 5.0, 5.0], [-3.0, -2.0, -1.0, -0.5]], dtype=np.float32)
    assert R.argmax(logits).tolist() == [1, 0, 3]  # the lowest index on ties
    # the generator: /root/reference/crates/nnis-model/src/sampling.rs:261-284, against the plain one draw for draw
    for seed in (0, 7, (1 << 64) - 1):
        mine, plain = R.Generator(seed), P.PlainSplitMix64(seed)
        assert [int(u) for u in mine.next_u64(5)] == [plain.next_u64() for _ in range(5)]
    rng = np.random.default_rng(4)
    for options in (dict(), dict(temperature=0.7), dict(top_k=5), dict(top_p=0.8), dict(temperature=1.3, top_k=40, top_p=0.5)):
        row = rng.standard_normal(200).astype(np.float32) * 3
        row[17] = row[90] = row.max()  # a tie at the top: the lower id comes first
        mine, plain = R.Generator(11), P.PlainSplitMix64(11)
        for _ in range(30):
            assert R.sample(row, mine, **options) == P.plain_sample(row, plain, **options)
    with pytest.raises(KernelError, match="not finite"):
        R.sample(np.array([0.0, np.inf], dtype=np.float32), R.Generator(1))
