"""Each kernel alone against a plain 32-bit (or 64-bit) reference of the same
operation, at sizes other than the engine's, with inputs made so that a fault
shows: a far key among hundreds, a window's edge, a slot of the cache, pages
out of order."""

import math

import numpy as np
import pytest
import torch

import plain_llama as P
from nnis_amd.errors import KernelError

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _ops():
    from nnis_amd.kernels import ops

    return ops


def _i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed(dtype):
    ops = _ops()
    table = torch.randn(777, 130).to(DT[dtype])
    ids = [0, 776, 5, 5, -1, 777, 300]
    out = torch.full((len(ids), 130), 9.0, device="cuda")
    ops.embed(_i32(ids), table.cuda(), out)
    want = torch.stack([table[i].float() if 0 <= i < 777 else torch.zeros(130) for i in ids])
    assert torch.equal(out.cpu(), want)


@pytest.mark.parametrize("width", [5, 576, 4100])
@pytest.mark.parametrize("x_dtype, w_dtype, out_dtype", [("float32", "float32", "float32"), ("float32", "bfloat16", "bfloat16"),
                                                         ("bfloat16", "float32", "bfloat16"), ("float32", "float32", "bfloat16")])
def test_rmsnorm(width, x_dtype, w_dtype, out_dtype):
    ops = _ops()
    torch.manual_seed(width)
    x = (torch.randn(7, width) * 4).to(DT[x_dtype])
    w = (1 + 0.2 * torch.randn(width)).to(DT[w_dtype])
    out = torch.empty(7, width, dtype=DT[out_dtype], device="cuda")
    ops.rmsnorm(x.cuda(), w.cuda(), 1e-6, out)
    want = P.rms_norm(x.double(), w.double(), 1e-6)
    tol = 1e-6 if out_dtype == "float32" else 1e-2
    assert ((out.cpu().double() - want).abs() <= tol * (1 + want.abs())).all()
    if x_dtype == "bfloat16":
        with pytest.raises(KernelError, match="32-bit"):
            ops.rmsnorm(x.cuda(), w.cuda(), 1e-6, out, delta=x.cuda())


@pytest.mark.parametrize("m, n, k", [(1, 1, 1), (1, 960, 576), (7, 63, 17), (65, 130, 176), (200, 70, 600), (3, 1000, 96)])
@pytest.mark.parametrize("x_dtype, w_dtype, y_dtype", [("float32", "float32", "float32"), ("bfloat16", "bfloat16", "bfloat16"),
                                                       ("bfloat16", "bfloat16", "float32"), ("bfloat16", "float32", "bfloat16")])
def test_gemm_ordered(m, n, k, x_dtype, w_dtype, y_dtype):
    ops = _ops()
    torch.manual_seed(m * 1000 + n + k)
    x = torch.randn(m, k).to(DT[x_dtype])
    w = torch.randn(n, k).to(DT[w_dtype])
    y = torch.empty(m, n, dtype=DT[y_dtype], device="cuda")
    ops.gemm_ordered(x.cuda(), w.cuda(), y)
    want = x.double() @ w.double().t()
    scale = (x.double().abs() @ w.double().abs().t())  # bounds the rounding of a sum of k products
    tol = 2e-7 * math.sqrt(k) if y_dtype == "float32" else 4e-3
    assert ((y.cpu().double() - want).abs() <= tol * scale + 1e-30).all()
    if (x_dtype, w_dtype, y_dtype) == ("float32", "float32", "float32"):
        # one ascending chain of fused multiply-adds per element: reproduce it exactly for one row
        chain = np.zeros(n, dtype=np.float64)
        for kk in range(k):  # float64 holds every 32-bit product exactly; round after each step
            chain = (x[0, kk].double().item() * w[:, kk].double().numpy() + chain).astype(np.float32).astype(np.float64)
        assert np.array_equal(y[0].cpu().numpy().astype(np.float64), chain)
    # a row's result does not depend on the other rows
    if m > 1:
        alone = torch.empty(1, n, dtype=DT[y_dtype], device="cuda")
        ops.gemm_ordered(x[m - 1:].contiguous().cuda(), w.cuda(), alone)
        assert torch.equal(alone[0], y[m - 1])


def _paged(k_seqs, v_seqs, dtype, kv_heads, head_dim, page_order=None, pages=32, max_pages=12):
    """Lays sequences out in pages the way the cache does.  k_seqs[i]: [len, kv_heads, head_dim]."""
    k_pages = torch.full((pages, kv_heads, 64, head_dim), 77.0, dtype=dtype)
    v_pages = torch.full((pages, kv_heads, head_dim, 64), -55.0, dtype=dtype)
    table = torch.zeros(len(k_seqs), max_pages, dtype=torch.int32)
    order = list(page_order or range(pages))
    for slot, (k, v) in enumerate(zip(k_seqs, v_seqs)):
        for page_index in range((k.shape[0] + 63) // 64):
            page = order.pop()
            table[slot, page_index] = page
            chunk = slice(page_index * 64, min(k.shape[0], page_index * 64 + 64))
            n = chunk.stop - chunk.start
            k_pages[page, :, :n, :] = k[chunk].transpose(0, 1).to(dtype)
            v_pages[page, :, :, :n] = v[chunk].permute(1, 2, 0).to(dtype)
    return k_pages.cuda(), v_pages.cuda(), table.cuda()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads, kv_heads, head_dim", [(4, 2, 16), (3, 1, 32), (9, 3, 64), (5, 5, 80), (8, 2, 128)])
def test_attention_over_pages(dtype, heads, kv_heads, head_dim):
    """Queries at the end of three sequences of unequal length (and one in the
    middle of a sequence), pages handed out in reverse order."""
    ops = _ops()
    torch.manual_seed(heads * head_dim)
    lengths = [700, 1, 65]
    ks = [torch.randn(n, kv_heads, head_dim) for n in lengths]
    vs = [torch.randn(n, kv_heads, head_dim) for n in lengths]
    scale = 1.0 / math.sqrt(head_dim)
    # a far key among hundreds: position 3 of sequence 0 answers the last query of head 0 and nothing else does
    q_last = torch.randn(heads, head_dim)
    ks[0][3, 0] = q_last[0] * (12.0 / scale / q_last[0].pow(2).sum())
    if dtype == "bfloat16":
        ks = [k.bfloat16().float() for k in ks]
        vs = [v.bfloat16().float() for v in vs]
    k_pages, v_pages, table = _paged(ks, vs, DT[dtype], kv_heads, head_dim)
    queries = [(0, 699, q_last), (1, 0, torch.randn(heads, head_dim)), (2, 64, torch.randn(heads, head_dim)),
               (0, 130, torch.randn(heads, head_dim)), (-1, 5, torch.randn(heads, head_dim))]
    q = torch.stack([qq for _, _, qq in queries]).to(DT[dtype])
    out = torch.full((len(queries), heads * head_dim), 3.0, dtype=DT[dtype], device="cuda")
    ops.attention_rows(q.reshape(len(queries), -1).cuda(), out, k_pages, v_pages, table, _i32([s for s, _, _ in queries]),
                       _i32([p for _, p, _ in queries]), heads, kv_heads, head_dim, scale)
    out = out.cpu().float().view(len(queries), heads, head_dim)
    tol = 2e-5 if dtype == "float32" else 2e-2
    for row, (slot, pos, _) in enumerate(queries):
        if slot < 0:
            assert (out[row] == 0).all()  # a padding row
            continue
        full_q = torch.zeros(pos + 1, heads, head_dim)
        full_q[pos] = q[row].float()
        want = P.causal_attention(full_q, ks[slot][:pos + 1], vs[slot][:pos + 1], scale)[pos]
        assert (out[row] - want).abs().max().item() <= tol, (row, (out[row] - want).abs().max().item())
    # the far key dominates head 0 of the first query: its value comes back almost alone
    assert (out[0, 0] - vs[0][3, 0]).abs().max().item() < 0.05


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_window_edge(dtype):
    """With a window of w the query at p reads keys p-w+1 .. p: a loud key just
    outside changes nothing, the same key just inside takes over."""
    ops = _ops()
    heads, kv_heads, head_dim, window, pos = 2, 1, 32, 100, 300
    torch.manual_seed(5)
    scale = 1.0 / math.sqrt(head_dim)
    q = torch.randn(1, heads, head_dim)
    loud = q[0, 0] * (15.0 / scale / q[0, 0].pow(2).sum())
    for where, inside in ((pos - window, False), (pos - window + 1, True)):
        k, v = torch.randn(pos + 1, kv_heads, head_dim), torch.randn(pos + 1, kv_heads, head_dim)
        k[where, 0] = loud
        if dtype == "bfloat16":
            k, v = k.bfloat16().float(), v.bfloat16().float()
        k_pages, v_pages, table = _paged([k], [v], DT[dtype], kv_heads, head_dim)
        out = torch.empty(1, heads * head_dim, dtype=DT[dtype], device="cuda")
        ops.attention_rows(q.reshape(1, -1).to(DT[dtype]).cuda(), out, k_pages, v_pages, table, _i32([0]), _i32([pos]), heads,
                           kv_heads, head_dim, scale, window=window)
        lo = pos - window + 1
        full_q = torch.zeros(window, heads, head_dim)
        full_q[-1] = q[0].to(DT[dtype]).float()
        want = P.causal_attention(full_q, k[lo:], v[lo:], scale)[-1]
        got = out.cpu().float().view(heads, head_dim)
        assert (got - want).abs().max().item() <= (2e-5 if dtype == "float32" else 2e-2)
        assert ((got[0] - v[where, 0]).abs().max().item() < 0.05) == inside


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads, kv_heads, head_dim, rot_dim", [(4, 2, 16, 16), (3, 1, 32, 32), (2, 2, 48, 16), (1, 1, 64, 0)])
def test_rope_and_cache_write(dtype, heads, kv_heads, head_dim, rot_dim):
    ops = _ops()
    torch.manual_seed(rot_dim + heads)
    tokens = 6
    slots = [2, 2, 0, -1, 1, 2]
    positions = [63, 64, 5, 9, 130, 200]
    width = (heads + 2 * kv_heads) * head_dim
    qkv = torch.randn(tokens, width).to(DT[dtype])
    table = torch.tensor([[3, 0, 0, 0], [9, 4, 6, 0], [1, 7, 2, 5]], dtype=torch.int32)
    k_pages = torch.full((10, kv_heads, 64, head_dim), 7.0, dtype=DT[dtype], device="cuda")
    v_pages = torch.full((10, kv_heads, head_dim, 64), 7.0, dtype=DT[dtype], device="cuda")
    q_out = torch.full((tokens, heads * head_dim), 5.0, dtype=DT[dtype], device="cuda")
    cos = sin = None
    if rot_dim:
        c, s = P.rope_tables(256, rot_dim, 10000.0)
        cos, sin = torch.from_numpy(c).cuda(), torch.from_numpy(s).cuda()
    ops.rope_kv_write(qkv.cuda(), q_out, cos, sin, rot_dim, _i32(slots), _i32(positions), k_pages, v_pages, table.cuda(),
                      heads, kv_heads, head_dim)
    x = qkv.float().view(tokens, heads + 2 * kv_heads, head_dim)
    rotated = x[:, :heads + kv_heads].clone()
    if rot_dim:
        pos = torch.tensor(positions)
        turned = P.rope_rotate_half(rotated[..., :rot_dim], torch.from_numpy(c)[pos], torch.from_numpy(s)[pos])
        rotated = torch.cat([turned, rotated[..., rot_dim:]], dim=-1)
    tol = 1e-6 if dtype == "float32" else 1e-2
    touched_k = torch.zeros(10, 64, dtype=torch.bool)
    for t in range(tokens):
        if slots[t] < 0:
            assert (q_out[t] == 5.0).all()
            continue
        assert (q_out[t].cpu().float().view(heads, head_dim) - rotated[t, :heads]).abs().max() <= tol
        page, inside = table[slots[t], positions[t] // 64].item(), positions[t] % 64
        touched_k[page, inside] = True
        assert (k_pages[page, :, inside, :].cpu().float() - rotated[t, heads:]).abs().max() <= tol
        assert torch.equal(v_pages[page, :, :, inside].cpu().float(), x[t, heads + kv_heads:])  # values are copied as they are
    # nothing else in the cache was written
    assert (k_pages.cpu().float()[~touched_k.unsqueeze(1).expand(-1, kv_heads, -1)] == 7.0).all()
    assert (v_pages.cpu().float().transpose(2, 3)[~touched_k.unsqueeze(1).expand(-1, kv_heads, -1)] == 7.0).all()
    # a run that keeps no cache rotates the queries only
    q_only = torch.empty_like(q_out)
    ops.rope_kv_write(qkv.cuda(), q_only, cos, sin, rot_dim, _i32([0] * tokens), _i32(positions), None, None, None,
                      heads, kv_heads, head_dim)
    assert (q_only.cpu().float().view(tokens, heads, head_dim) - rotated[:, :heads]).abs().max() <= tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_silu_mul(dtype):
    ops = _ops()
    gate_up = (torch.randn(13, 2 * 177) * 3).to(DT[dtype])
    out = torch.empty(13, 177, dtype=DT[dtype], device="cuda")
    ops.silu_mul(gate_up.cuda(), out)
    want = P.silu(gate_up[:, :177].double()) * gate_up[:, 177:].double()
    assert ((out.cpu().double() - want).abs() <= (1e-6 if dtype == "float32" else 1e-2) * (1 + want.abs())).all()


@pytest.mark.parametrize("vocab", [1, 63, 1000, 49152, 50001])
def test_argmax(vocab):
    ops = _ops()
    torch.manual_seed(vocab)
    logits = torch.randn(5, vocab)
    if vocab >= 63:
        logits[0, 40] = logits[0, 7] = 9.0  # a tie: the lower index wins
        logits[1, vocab - 1] = 11.0
        logits[2] = 0.5  # all equal: index 0
        logits[3, 3] = float("nan")
        logits[3, 20] = 30.0
    out = torch.empty(5, dtype=torch.int32, device="cuda")
    ops.argmax(logits.cuda(), out)
    want = [int(np.nanargmax(row)) for row in logits.numpy()]
    assert out.cpu().tolist() == want
    if vocab >= 63:
        assert want[:3] == [7, vocab - 1, 0]


def test_refusals():
    ops = _ops()
    f = lambda *shape, dtype=torch.float32: torch.zeros(*shape, dtype=dtype, device="cuda")  # noqa: E731
    with pytest.raises(KernelError):
        ops.gemm_ordered(f(3, 8), f(5, 9), f(3, 5))
    with pytest.raises(KernelError, match="GPU"):
        ops.gemm_ordered(torch.zeros(3, 8), f(5, 8), f(3, 5))
    with pytest.raises(KernelError, match="float32 or bfloat16"):
        ops.gemm_ordered(f(3, 8, dtype=torch.float16), f(5, 8), f(3, 5))
    with pytest.raises(KernelError, match="head_dim"):
        ops.attention_module(7)
    with pytest.raises(KernelError):
        ops.silu_mul(f(4, 11), f(4, 5))
    with pytest.raises(KernelError):
        ops.argmax(f(4, 11), torch.zeros(4, dtype=torch.int64, device="cuda"))
