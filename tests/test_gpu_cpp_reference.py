"""The 32-bit kernels against the plain C++ references of the same operations
(``nnis_amd/csrc/reference.cpp``, which ``tests/test_cpp_reference.py`` pins on
the CPU): the ordered product bit for bit, the others within the rounding of
sums taken in another order; selection token for token."""

import math

import numpy as np
import pytest
import torch

from nnis_amd.kernels import reference as R
from test_gpu_kernels import _empty_pages, _i32, _ops, _paged, _read_pages

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m, n, k", [(1, 960, 576), (7, 63, 17), (65, 130, 176), (3, 100, 1100)])
def test_the_ordered_product_equals_the_plain_chain_bit_for_bit(m, n, k):
    ops = _ops()
    rng = np.random.default_rng(m + n + k)
    x, w = rng.standard_normal((m, k)).astype(np.float32), rng.standard_normal((n, k)).astype(np.float32)
    y = torch.empty(m, n, device="cuda")
    ops.gemm_ordered(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), y)
    assert np.array_equal(y.cpu().numpy(), R.gemm(x, w))


def test_norm_rotation_gating_and_embedding():
    ops = _ops()
    rng = np.random.default_rng(5)
    x, w = rng.standard_normal((9, 1020)).astype(np.float32) * 4, (1 + 0.2 * rng.standard_normal(1020)).astype(np.float32)
    out = torch.empty(9, 1020, device="cuda")
    ops.rmsnorm(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), 3e-6, out)
    want = R.rmsnorm(x, w, 3e-6)
    assert (np.abs(out.cpu().numpy() - want) <= 1e-6 * (1 + np.abs(want))).all()

    gate_up = rng.standard_normal((5, 2 * 130)).astype(np.float32) * 3
    out = torch.empty(5, 130, device="cuda")
    ops.silu_mul(torch.from_numpy(gate_up).cuda(), out)
    want = R.silu_mul(gate_up[:, :130], gate_up[:, 130:])
    assert (np.abs(out.cpu().numpy() - want) <= 2e-6 * (1 + np.abs(want))).all()

    table = rng.standard_normal((77, 36)).astype(np.float32)
    ids = [0, 76, 5, 5, -1, 77]
    out = torch.full((len(ids), 36), 9.0, device="cuda")
    ops.embed(_i32(ids), torch.from_numpy(table).cuda(), out)
    assert np.array_equal(out.cpu().numpy(), R.embed(ids, table))

    # rotation of queries and keys by their positions (part of a head), and the write into the pages
    heads, kv_heads, head_dim, rot_dim = 3, 1, 48, 32
    tokens, slots, positions = 4, [1, 1, 0, 1], [63, 64, 5, 130]
    cos, sin = R.rope_tables(256, rot_dim, 50000.0)
    qkv = rng.standard_normal((tokens, (heads + 2 * kv_heads) * head_dim)).astype(np.float32)
    block_table = torch.tensor([[3, 0, 0], [9, 4, 6]], dtype=torch.int32)
    k_pages, v_pages = _empty_pages(10, kv_heads, head_dim, torch.float32, 7.0, 7.0, "cuda")
    q_out = torch.empty(tokens, heads * head_dim, device="cuda")
    ops.rope_kv_write(torch.from_numpy(qkv).cuda(), q_out, torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda(), rot_dim,
                      _i32(slots), _i32(positions), k_pages, v_pages, block_table.cuda(), heads, kv_heads, head_dim)
    parts = qkv.reshape(tokens, heads + 2 * kv_heads, head_dim)
    want = R.rope_rotate_half(parts[:, :heads + kv_heads], cos, sin, positions, rot_dim=rot_dim)
    assert np.abs(q_out.cpu().numpy().reshape(tokens, heads, head_dim) - want[:, :heads]).max() <= 1e-6
    k_plain, v_plain = _read_pages(k_pages, v_pages, head_dim)
    for t in range(tokens):
        page, inside = block_table[slots[t], positions[t] // 64].item(), positions[t] % 64
        assert np.abs(k_plain[page, :, inside].numpy() - want[t, heads:]).max() <= 1e-6
        assert np.array_equal(v_plain[page, :, inside].numpy(), parts[t, heads + kv_heads:])


@pytest.mark.parametrize("heads, kv_heads, head_dim, window", [(4, 2, 16, 0), (9, 3, 64, 0), (6, 1, 40, 100)])
def test_attention_over_the_cache(heads, kv_heads, head_dim, window):
    """Sequences of unequal length in pages handed out in reverse order; queries at their ends and in the middle."""
    ops = _ops()
    rng = np.random.default_rng(heads * head_dim)
    lengths = [300, 1, 65]
    ks = [rng.standard_normal((n, kv_heads, head_dim)).astype(np.float32) for n in lengths]
    vs = [rng.standard_normal((n, kv_heads, head_dim)).astype(np.float32) for n in lengths]
    scale = 1.0 / math.sqrt(head_dim)
    k_pages, v_pages, table = _paged([torch.from_numpy(k) for k in ks], [torch.from_numpy(v) for v in vs], torch.float32, kv_heads, head_dim)
    queries = [(0, 299), (1, 0), (2, 64), (0, 130)]
    q = rng.standard_normal((len(queries), heads, head_dim)).astype(np.float32)
    out = torch.empty(len(queries), heads * head_dim, device="cuda")
    ops.attention_rows(torch.from_numpy(q).reshape(len(queries), -1).cuda(), out, k_pages, v_pages, table, _i32([s for s, _ in queries]),
                       _i32([p for _, p in queries]), heads, kv_heads, head_dim, scale, window)
    out = out.cpu().numpy().reshape(len(queries), heads, head_dim)
    for row, (slot, pos) in enumerate(queries):
        want = R.attention(q[row:row + 1], ks[slot][:pos + 1], vs[slot][:pos + 1], scale, first=pos, window=window)[0]
        assert np.abs(out[row] - want).max() <= 2e-6, (row, np.abs(out[row] - want).max())


@pytest.mark.parametrize("vocab", [1000, 49152])
def test_selection_token_for_token(vocab):
    ops = _ops()
    rng = np.random.default_rng(vocab)
    logits = (rng.standard_normal((6, vocab)) * 3).astype(np.float32)
    logits[2, 17] = logits[2, 900] = logits[2].max() + 1.0  # a tie at the top
    dev = torch.from_numpy(logits).cuda()
    best = torch.empty(6, dtype=torch.int32, device="cuda")
    ops.argmax(dev, best)
    assert np.array_equal(best.cpu().numpy(), R.argmax(logits))
    # seeded draws: every row a sequence of its own (a slot), three draws each, with the options of its slot
    options = [dict(temperature=1.0), dict(temperature=0.7), dict(temperature=1.0, top_k=40), dict(temperature=1.0, top_p=0.8),
               dict(temperature=1.3, top_k=50, top_p=0.5), dict(temperature=0.9, top_p=0.95)]
    seeds = [3, 5, 7, 11, 13, (1 << 63) + 9]
    rng_state = torch.tensor([s if s < (1 << 63) else s - (1 << 64) for s in seeds], dtype=torch.int64, device="cuda")
    temperature = torch.tensor([o["temperature"] for o in options], dtype=torch.float32, device="cuda")
    top_k = torch.tensor([o.get("top_k", 0) for o in options], dtype=torch.int32, device="cuda")
    top_p = torch.tensor([o.get("top_p", 0.0) for o in options], dtype=torch.float32, device="cuda")
    weights = torch.empty(6, vocab, dtype=torch.float64, device="cuda")
    generators = [R.Generator(seed) for seed in seeds]
    for _ in range(3):
        out = torch.empty(6, dtype=torch.int32, device="cuda")
        ops.sample(dev, weights, _i32(list(range(6))), rng_state, temperature, top_k, top_p, out, by_slot=True)
        want = [R.sample(logits[r], generators[r], **options[r]) for r in range(6)]
        assert out.cpu().tolist() == want
