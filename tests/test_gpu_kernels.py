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


@pytest.mark.parametrize("width", [5, 64, 576, 1020, 4100, 8192, 9000])
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


@pytest.mark.parametrize("m", [1, 8, 16, 17, 40, 64, 65, 130, 300])
@pytest.mark.parametrize("n, k", [(576, 576), (960, 576), (1000, 96), (70, 176), (3072, 64), (64, 1536), (17, 8), (200, 1096),
                                  (2050, 2312)])  # the last: large weights, few columns -- K is cut among blocks beyond 16 tokens
@pytest.mark.parametrize("y_dtype", ["bfloat16", "float32"])
def test_gemm_bf16_on_the_matrix_cores(m, n, k, y_dtype):
    """Skinny (M <= 64) and tiled kernels at sizes with tails in every
    dimension.  Integer-valued operands make the 32-bit sums exact, so any
    misplaced or dropped product shows as a whole-number error."""
    ops = _ops()
    torch.manual_seed(m + n + k)
    x = torch.randint(-3, 4, (m, k)).to(torch.bfloat16)
    w = torch.randint(-3, 4, (n, k)).to(torch.bfloat16)
    y = torch.full((m, n), 7.0, dtype=DT[y_dtype], device="cuda")
    ops.gemm_bf16(x.cuda(), ops.pack_weight(w.cuda()), y)
    want = x.double() @ w.double().t()
    if y_dtype == "float32":
        assert torch.equal(y.cpu().double(), want)
    else:
        assert torch.equal(y.cpu(), want.to(torch.bfloat16))
    # and with ordinary values, against the 64-bit product
    x = torch.randn(m, k).to(torch.bfloat16)
    w = torch.randn(n, k).to(torch.bfloat16)
    ops.gemm_bf16(x.cuda(), ops.pack_weight(w.cuda()), y)
    want = x.double() @ w.double().t()
    scale = x.double().abs() @ w.double().abs().t()
    tol = 1e-6 * math.sqrt(k) if y_dtype == "float32" else 4e-3
    assert ((y.cpu().double() - want).abs() <= tol * scale + 1e-30).all()


@pytest.mark.parametrize("n,k", [(16, 64), (5, 8), (37, 88), (130, 200), (960, 576)])
def test_packed_weight_order(n, k):
    """Element (row, c) of a weight lies in strip row / 16, chunk c / 64, half c % 16 / 8, lane
    16 * (c % 64 / 16) + row % 16, place c % 8; what pads the last strip and chunk is zeros."""
    ops = _ops()
    w = torch.randn(n, k).bfloat16()
    packed = ops.pack_weight(w.cuda())
    assert packed.shape == (n, k) and packed.data.numel() == ops.packed_weight_elems(n, k)
    strips, chunks = (n + 15) // 16, ((k + 63) // 64) | 1  # a strip is padded to an odd number of chunks
    got = packed.data.cpu().view(strips, chunks, 2, 4, 16, 8)  # [strip][chunk][half][k group][row][8]
    padded = torch.zeros(strips * 16, chunks * 64, dtype=torch.bfloat16)
    padded[:n, :k] = w
    want = padded.view(strips, 16, chunks, 4, 2, 8).permute(0, 2, 4, 3, 1, 5)  # [strip][row][chunk][k group][half][8] ->
    assert torch.equal(got, want.contiguous())


def test_gemm_bf16_refuses_what_it_cannot_load():
    ops = _ops()
    x = torch.zeros(4, 12, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(6, 12, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(KernelError, match="multiple of 8"):
        ops.pack_weight(w)
    assert not ops.packs(w)
    with pytest.raises(KernelError, match="must be packed"):  # a weight in the checkpoint's order is not taken for a packed one
        ops.gemm_bf16(x, w, torch.zeros(4, 6, dtype=torch.bfloat16, device="cuda"))
    out = torch.zeros(4, 6, dtype=torch.bfloat16, device="cuda")
    ops.linear(x + 1, w + 1, out)  # a weight that is not packed takes the ordered product
    assert (out == 12).all()


MFMA_SHAPES = [(4, 2, 16), (3, 3, 16), (3, 1, 32), (6, 2, 48), (6, 6, 48), (4, 2, 48), (9, 3, 64), (2, 2, 64), (5, 5, 80),
               (4, 1, 112), (8, 2, 128), (32, 1, 64), (40, 2, 16), (8, 1, 64), (12, 2, 32), (2, 1, 192), (3, 3, 256)]


def _small_decode_call(heads, kv_heads, head_dim):
    """Arguments of a one-token decode call over one page (for calls that are to be refused)."""
    k_pages, v_pages = _empty_pages(1, kv_heads, head_dim, torch.bfloat16, 0.0, 0.0, "cuda")
    q = torch.zeros(1, heads * head_dim, dtype=torch.bfloat16, device="cuda")
    return (q, torch.empty_like(q), k_pages, v_pages, _i32([[0]]), _i32([0]), _i32([0]), heads, kv_heads, head_dim, 1.0)


def _plain_rows(q_rows, ks, vs, scale, window=0):
    """q_rows: list of (slot, pos, q[heads, hd]) -> plain attention output per row."""
    out = []
    for slot, pos, q in q_rows:
        lo = max(0, pos + 1 - window) if window else 0
        full_q = torch.zeros(pos + 1 - lo, *q.shape)
        full_q[-1] = q
        out.append(P.causal_attention(full_q, ks[slot][lo:pos + 1], vs[slot][lo:pos + 1], scale)[-1])
    return torch.stack(out)


@pytest.mark.parametrize("heads, kv_heads, head_dim", MFMA_SHAPES)
@pytest.mark.parametrize("splits, waves", [(1, 1), (4, 1), (16, 2), (1, 8), (2, 4)])
@pytest.mark.parametrize("kernel", ["columns", "keys"])
def test_decode_attention_on_the_matrix_cores(heads, kv_heads, head_dim, splits, waves, kernel):
    ops = _ops()
    if kernel == "keys" and (heads // kv_heads > 4 or head_dim > 128):  # refused, in words
        with pytest.raises(Exception, match="keys on lanes"):
            ops.attention_decode_bf16(*_small_decode_call(heads, kv_heads, head_dim), kernel="keys")
        return
    torch.manual_seed(heads + head_dim)
    lengths = [700, 1, 65, 33]
    ks = [torch.randn(n, kv_heads, head_dim).bfloat16().float() for n in lengths]
    vs = [torch.randn(n, kv_heads, head_dim).bfloat16().float() for n in lengths]
    scale = 1.0 / math.sqrt(head_dim)
    q_last = torch.randn(heads, head_dim)
    ks[0][3, 0] = (q_last[0] * (12.0 / scale / q_last[0].pow(2).sum())).bfloat16().float()  # a far key among hundreds
    k_pages, v_pages, table = _paged(ks, vs, torch.bfloat16, kv_heads, head_dim)
    rows = [(0, 699, q_last), (1, 0, torch.randn(heads, head_dim)), (-1, 9, torch.randn(heads, head_dim)),
            (2, 64, torch.randn(heads, head_dim)), (3, 31, torch.randn(heads, head_dim))]
    rows = [(s, p, q.bfloat16().float()) for s, p, q in rows]
    q = torch.stack([q for _, _, q in rows]).bfloat16().reshape(len(rows), -1).cuda()
    out = torch.full((len(rows), heads * head_dim), 3.0, dtype=torch.bfloat16, device="cuda")
    partial = torch.full((len(rows) * heads * splits * (head_dim + 4),), float("nan"), dtype=torch.float32, device="cuda")
    waves = min(waves, ops.decode_max_waves(heads, kv_heads, head_dim))
    ops.attention_decode_bf16(q, out, k_pages, v_pages, table, _i32([s for s, _, _ in rows]), _i32([p for _, p, _ in rows]),
                              heads, kv_heads, head_dim, scale, 0, splits, partial, waves, kernel)
    got = out.cpu().float().view(len(rows), heads, head_dim)
    live = [i for i, (s, _, _) in enumerate(rows) if s >= 0]
    want = _plain_rows([rows[i] for i in live], ks, vs, scale)
    assert (got[live] - want).abs().max().item() <= 2e-2
    assert (got[2] == 3.0).all()  # the padding row is left alone
    assert (got[0, 0] - vs[0][3, 0]).abs().max().item() < 0.05
    # a window: the row at position 699 reads keys 600..699 only
    ops.attention_decode_bf16(q, out, k_pages, v_pages, table, _i32([s for s, _, _ in rows]), _i32([p for _, p, _ in rows]),
                              heads, kv_heads, head_dim, scale, 100, splits, partial, waves, kernel)
    got = out.cpu().float().view(len(rows), heads, head_dim)
    want = _plain_rows([rows[i] for i in live], ks, vs, scale, window=100)
    assert (got[live] - want).abs().max().item() <= 2e-2


@pytest.mark.parametrize("heads, kv_heads, head_dim", MFMA_SHAPES)
def test_prefill_attention_on_the_matrix_cores(heads, kv_heads, head_dim):
    """Three sequences in one step: a whole prompt, a continuation that starts
    at position 70, and a single token; every new row against the plain
    attention over its sequence's keys up to its own position."""
    ops = _ops()
    torch.manual_seed(heads * 3 + head_dim)
    sequences = [(2, 0, 130), (0, 70, 37), (1, 0, 1)]  # (slot, first new position, new tokens)
    total = {slot: pos0 + n for slot, pos0, n in sequences}
    ks = [torch.randn(total[s], kv_heads, head_dim).bfloat16().float() for s in range(3)]
    vs = [torch.randn(total[s], kv_heads, head_dim).bfloat16().float() for s in range(3)]
    scale = 1.0 / math.sqrt(head_dim)
    k_pages, v_pages, table = _paged(ks, vs, torch.bfloat16, kv_heads, head_dim)
    rows = [(slot, pos0 + i, torch.randn(heads, head_dim).bfloat16().float()) for slot, pos0, n in sequences for i in range(n)]
    # one loud key: row 100 of the first sequence must find key 17 (head 0)
    loud_q = rows[100][2][0]
    ks[2][17, 0] = (loud_q * (12.0 / scale / loud_q.pow(2).sum())).bfloat16().float()
    k_pages, v_pages, table = _paged(ks, vs, torch.bfloat16, kv_heads, head_dim)
    q = torch.stack([q for _, _, q in rows]).bfloat16().reshape(len(rows), -1).cuda()
    out = torch.full((len(rows), heads * head_dim), 3.0, dtype=torch.bfloat16, device="cuda")
    tile = ops.prefill_tile_rows(heads, kv_heads, head_dim)
    assert tile in (16, 32, 64)
    items = [(seq, row0) for seq, (_, _, n) in enumerate(sequences) for row0 in range(0, n, tile)]
    starts = [0, 130, 167, 168]
    starts = [0, 130, 167, 168]
    for window, waves, columns in ((0, 1, 0), (40, 1, 0), (0, 8, 0), (40, 2, 0), (0, 8, 1), (40, 4, 2), (0, 1, 2)):
        waves = min(waves, ops.prefill_max_waves(heads, kv_heads, head_dim, columns))
        tile = ops.prefill_tile_rows(heads, kv_heads, head_dim, columns)
        items = [(seq, row0) for seq, (_, _, n) in enumerate(sequences) for row0 in range(0, n, tile)]
        ops.attention_prefill_bf16(q, out, k_pages, v_pages, table, _i32([s for s, _ in items]), _i32([r for _, r in items]),
                                   _i32([s for s, _, _ in sequences]), _i32(starts), _i32([p for _, p, _ in sequences]),
                                   heads, kv_heads, head_dim, scale, window, waves, columns)
        got = out.cpu().float().view(len(rows), heads, head_dim)
        want = _plain_rows(rows, ks, vs, scale, window=window)
        error = (got - want).abs().amax(dim=(1, 2))
        assert error.max().item() <= 2e-2, (window, int(error.argmax()), error.max().item())
        if window == 0:
            assert (got[100, 0] - vs[2][17, 0]).abs().max().item() < 0.05


@pytest.mark.parametrize("heads, kv_heads, head_dim, splits, rows_out", [(9, 3, 64, 4, 576), (4, 2, 16, 8, 70), (8, 2, 128, 2, 1024),
                                                                         (5, 5, 80, 3, 200)])
def test_residual_projection_adds_up_key_runs(heads, kv_heads, head_dim, splits, rows_out):
    """A decode attention that leaves its runs of keys, and the projection that
    adds them up on its way: the stream, the prepared norm and its sums are
    those of the path with the kernel of its own between the two, bit for bit
    (a padding row's aside: nobody reads it)."""
    ops = _ops()
    torch.manual_seed(heads + head_dim + splits)
    lengths = [700, 1, 65, 33]
    ks = [torch.randn(n, kv_heads, head_dim).bfloat16().float() for n in lengths]
    vs = [torch.randn(n, kv_heads, head_dim).bfloat16().float() for n in lengths]
    k_pages, v_pages, table = _paged(ks, vs, torch.bfloat16, kv_heads, head_dim)
    slots, positions = [0, 1, -1, 2, 3], [699, 0, 9, 64, 31]
    live = [i for i, s in enumerate(slots) if s >= 0]
    m, k = len(slots), heads * head_dim
    q = torch.randn(m, k).bfloat16().cuda()
    out = torch.zeros(m, k, dtype=torch.bfloat16, device="cuda")
    partial = torch.full((m * heads * splits * (head_dim + 4),), float("nan"), dtype=torch.float32, device="cuda")
    waves = min(2, ops.decode_max_waves(heads, kv_heads, head_dim))
    runs = ops.attention_decode_bf16(q, out, k_pages, v_pages, table, _i32(slots), _i32(positions), heads, kv_heads, head_dim,
                                     1.0 / math.sqrt(head_dim), 0, splits, partial, waves, keep_runs=True)
    assert isinstance(runs, ops.KeyRuns) and runs.shape == (m, k) and runs.fits(rows_out)
    w = (torch.randn(rows_out, k) / math.sqrt(k)).bfloat16().cuda()
    packed = ops.pack_weight(w)
    gain = (1 + 0.3 * torch.randn(rows_out)).bfloat16().cuda()
    resid = torch.randn(m, rows_out).cuda()

    def project(x):
        mine = resid.clone()
        scaled = torch.zeros(m, rows_out, dtype=torch.bfloat16, device="cuda")
        ss = torch.zeros(ops.gemm_residual_parts(m, rows_out), m, device="cuda")
        parts = ops.gemm_residual(x, packed, mine, gain, scaled, ss)
        return mine[live].cpu(), scaled[live].cpu(), ss[:parts][:, live].cpu()

    fused = project(runs)
    added = runs.combine()
    assert added.data_ptr() == out.data_ptr()
    want = _plain_rows([(slots[i], positions[i], q[i].float().cpu().view(heads, head_dim)) for i in live], ks, vs, 1.0 / math.sqrt(head_dim))
    assert (added[live].cpu().float().view(len(live), heads, head_dim) - want).abs().max().item() <= 2e-2
    apart = project(added)
    for got, expected in zip(fused, apart):
        assert torch.equal(got, expected)
    # runs that the projection does not take: too many of them, or too many tokens
    assert not ops.KeyRuns(partial, 9, m, heads, head_dim, _i32(slots), out).fits(rows_out)
    assert not ops.KeyRuns(partial, splits, 65, heads, head_dim, _i32(slots), out).fits(rows_out)


@pytest.mark.parametrize("heads, kv_heads, head_dim, lengths", [(9, 3, 64, (1500, 700, 90)), (8, 8, 16, (1300, 1000, 100))])
def test_prefill_attention_with_more_items_than_compute_units(heads, kv_heads, head_dim, lengths):
    """Steps of so many tiles that a block takes two of them, a long one and
    then a short one.  The second sequence goes on from position 100.  One
    loud key far back for a row of the shortest tiles and one for a row of
    the longest."""
    ops = _ops()
    torch.manual_seed(heads + head_dim)
    sequences = [(1, 0, lengths[0]), (2, 100, lengths[1]), (0, 0, lengths[2])]  # (slot, first new position, new tokens)
    total = {slot: pos0 + n for slot, pos0, n in sequences}
    ks = [torch.randn(total[s], kv_heads, head_dim).bfloat16().float() for s in range(3)]
    vs = [torch.randn(total[s], kv_heads, head_dim).bfloat16().float() for s in range(3)]
    scale = 1.0 / math.sqrt(head_dim)
    queries = {slot: torch.zeros(total[slot], heads, head_dim) for slot in total}
    for slot, pos0, n in sequences:
        queries[slot][pos0:] = torch.randn(n, heads, head_dim).bfloat16().float()
    loud = [(0, 40, 3), (1, lengths[0] - 2, 70)]  # (slot, position of the row, position of the key), head 0
    for slot, row, key in loud:
        loud_q = queries[slot][row, 0]
        ks[slot][key, 0] = (loud_q * (14.0 / scale / loud_q.pow(2).sum())).bfloat16().float()
    pages = sum((n + 63) // 64 for n in total.values())
    k_pages, v_pages, table = _paged(ks, vs, torch.bfloat16, kv_heads, head_dim, pages=pages, max_pages=max(total.values()) // 64 + 1)
    q = torch.cat([queries[slot][pos0:] for slot, pos0, _ in sequences]).bfloat16().reshape(sum(lengths), -1).cuda()
    want = torch.cat([P.causal_attention(queries[slot], ks[slot], vs[slot], scale)[pos0:] for slot, pos0, _ in sequences])
    starts = [0, lengths[0], lengths[0] + lengths[1], sum(lengths)]
    tile = ops.prefill_tile_rows(heads, kv_heads, head_dim)
    items = sorted(((pos0 + min(row0 + tile, n), seq, row0) for seq, (_, pos0, n) in enumerate(sequences)
                    for row0 in range(0, n, tile)), reverse=True)  # longest first, as the engine hands them over
    group_chunks = kv_heads * -(-(heads // kv_heads) // max(1, min(heads // kv_heads, 4)))
    assert len(items) * group_chunks > 256 + 32  # more than the compute units of the chip: the grid folds
    for waves in (8, 2, 1):  # (one wave: each item whole, a block's two one after the other)
        waves = min(waves, ops.prefill_max_waves(heads, kv_heads, head_dim))
        out = torch.full((sum(lengths), heads * head_dim), 3.0, dtype=torch.bfloat16, device="cuda")
        ops.attention_prefill_bf16(q, out, k_pages, v_pages, table, _i32([s for _, s, _ in items]), _i32([r for _, _, r in items]),
                                   _i32([s for s, _, _ in sequences]), _i32(starts), _i32([p for _, p, _ in sequences]),
                                   heads, kv_heads, head_dim, scale, 0, waves)
        got = out.cpu().float().view(sum(lengths), heads, head_dim)
        error = (got - want).abs().amax(dim=(1, 2))
        assert error.max().item() <= 2e-2, (waves, int(error.argmax()), error.max().item())
        for slot, row, key in loud:
            seq = [s for s, _, _ in sequences].index(slot)
            packed = starts[seq] + row - sequences[seq][1]
            assert (got[packed, 0] - vs[slot][key, 0]).abs().max().item() < 0.05


@pytest.mark.parametrize("heads, kv_heads, head_dim", [(9, 3, 64), (32, 4, 64), (4, 4, 32)])
def test_attention_beyond_64_pages(heads, kv_heads, head_dim):
    """A sequence of 4,500 tokens (71 pages: a wave that walks them all comes
    to the end of its first run of page numbers and has to fetch the next),
    with a loud key in the very first page and one beyond page 64, for one
    token of a decode step (one wave and one run, several waves, several runs,
    both kernels) and for the last rows of a prompt step."""
    ops = _ops()
    torch.manual_seed(heads + head_dim)
    length = 4500
    scale = 1.0 / math.sqrt(head_dim)
    ks = [torch.randn(length, kv_heads, head_dim).bfloat16().float(), torch.randn(70, kv_heads, head_dim).bfloat16().float()]
    vs = [torch.randn(length, kv_heads, head_dim).bfloat16().float(), torch.randn(70, kv_heads, head_dim).bfloat16().float()]
    group = heads // kv_heads
    q_last = torch.randn(heads, head_dim).bfloat16().float()
    # head 0 finds key 5 (page 0); the first head of the last group finds key 4,230 (page 66)
    far_head = heads - group
    ks[0][5, 0] = (q_last[0] * (14.0 / scale / q_last[0].pow(2).sum())).bfloat16().float()
    ks[0][4230, kv_heads - 1] = (q_last[far_head] * (14.0 / scale / q_last[far_head].pow(2).sum())).bfloat16().float()
    k_pages, v_pages, table = _paged(ks, vs, torch.bfloat16, kv_heads, head_dim, pages=80, max_pages=72)
    rows = [(0, length - 1, q_last), (1, 69, torch.randn(heads, head_dim).bfloat16().float())]
    q = torch.stack([q for _, _, q in rows]).bfloat16().reshape(len(rows), -1).cuda()
    want = _plain_rows(rows, ks, vs, scale)
    kernels = ["columns"] + (["keys"] if group <= 4 else [])
    for kernel in kernels:
        for splits, waves in ((1, 1), (1, 4), (8, 4), (2, 1)):
            waves = min(waves, ops.decode_max_waves(heads, kv_heads, head_dim))
            out = torch.full((len(rows), heads * head_dim), 3.0, dtype=torch.bfloat16, device="cuda")
            partial = torch.full((len(rows) * heads * splits * (head_dim + 4),), float("nan"), dtype=torch.float32, device="cuda")
            ops.attention_decode_bf16(q, out, k_pages, v_pages, table, _i32([0, 1]), _i32([length - 1, 69]), heads, kv_heads,
                                      head_dim, scale, 0, splits, partial, waves, kernel)
            got = out.cpu().float().view(len(rows), heads, head_dim)
            assert (got - want).abs().max().item() <= 2e-2, (kernel, splits, waves, (got - want).abs().max().item())
            assert (got[0, 0] - vs[0][5, 0]).abs().max().item() < 0.05, (kernel, splits, waves)
            assert (got[0, far_head] - vs[0][4230, kv_heads - 1]).abs().max().item() < 0.05, (kernel, splits, waves)
    # a prompt step: the sequence's last 40 tokens are new, the 4,460 before them are in the cache
    new = 40
    pos0 = length - new
    q_rows = torch.randn(new, heads, head_dim).bfloat16().float()
    q_rows[-1] = q_last
    prompt_rows = [(0, pos0 + i, q_rows[i]) for i in range(new)]
    want = _plain_rows(prompt_rows, ks, vs, scale)
    qp = q_rows.bfloat16().reshape(new, -1).cuda()
    for waves in (1, 8):
        waves = min(waves, ops.prefill_max_waves(heads, kv_heads, head_dim))
        tile = ops.prefill_tile_rows(heads, kv_heads, head_dim)
        items = [(0, row0) for row0 in range(0, new, tile)]
        out = torch.full((new, heads * head_dim), 3.0, dtype=torch.bfloat16, device="cuda")
        ops.attention_prefill_bf16(qp, out, k_pages, v_pages, table, _i32([s for s, _ in items]), _i32([r for _, r in items]),
                                   _i32([0]), _i32([0, new]), _i32([pos0]), heads, kv_heads, head_dim, scale, 0, waves)
        got = out.cpu().float().view(new, heads, head_dim)
        assert (got - want).abs().max().item() <= 2e-2, (waves, (got - want).abs().max().item())
        assert (got[-1, 0] - vs[0][5, 0]).abs().max().item() < 0.05
        assert (got[-1, far_head] - vs[0][4230, kv_heads - 1]).abs().max().item() < 0.05


def test_step_tables_and_the_kernels_that_read_them():
    """The step's tables against plain indexing, padding rows included; the decode attention reading each token's
    pages from them gives what it gives through slots and the block table; the rotating projection that takes
    rotation rows and pages from them writes the same queries and the same cache."""
    ops = _ops()
    torch.manual_seed(11)
    heads, kv_heads, head_dim = 6, 2, 64
    half = head_dim // 2
    lengths = [300, 70, 1, 129]
    ks = [torch.randn(n, kv_heads, head_dim).bfloat16().float() for n in lengths]
    vs = [torch.randn(n, kv_heads, head_dim).bfloat16().float() for n in lengths]
    k_pages, v_pages, table = _paged(ks, vs, torch.bfloat16, kv_heads, head_dim)
    cos, sin = (torch.from_numpy(t).cuda() for t in P.rope_tables(512, head_dim, 10000.0))
    slots, positions = [2, -1, 0, 3, 1, -1], [0, 0, 299, 128, 69, 0]
    tables = ops.step_tables(_i32(slots), _i32(positions), len(slots), cos, sin, table, sequence_pages=True)
    host_table = table.cpu()
    for row, (slot, pos) in enumerate(zip(slots, positions)):
        if slot < 0:
            assert tables.page[row].item() == -1 and tables.pages[row, 0].item() == 0
            assert bool((tables.cos[row] == 1).all()) and bool((tables.sin[row] == 0).all())
            continue
        assert torch.equal(tables.cos[row], cos[pos]) and torch.equal(tables.sin[row], sin[pos])
        assert tables.page[row].item() == host_table[slot, pos // 64].item()
        assert torch.equal(tables.pages[row, :pos // 64 + 1].cpu(), host_table[slot, :pos // 64 + 1])
    only_pages = ops.step_tables(_i32(slots), _i32(positions), len(slots), block_table=table)
    assert only_pages.cos is None and only_pages.pages is None and torch.equal(only_pages.page, tables.page)

    scale = 1.0 / math.sqrt(head_dim)
    q = torch.randn(len(slots), heads * head_dim).bfloat16().cuda()
    for kernel in ("keys", "columns"):
        for splits, waves in ((1, 1), (4, 2)):
            outs = []
            for token_pages in (None, tables.pages):
                out = torch.zeros(len(slots), heads * head_dim, dtype=torch.bfloat16, device="cuda")
                partial = torch.zeros(len(slots) * heads * splits * (head_dim + 4), dtype=torch.float32, device="cuda")
                ops.attention_decode_bf16(q, out, k_pages, v_pages, table, _i32(slots), _i32(positions), heads, kv_heads, head_dim,
                                          scale, 0, splits, partial, waves, kernel, token_pages=token_pages)
                outs.append(out.cpu())
            live = [i for i, s in enumerate(slots) if s >= 0]
            assert torch.equal(outs[0][live], outs[1][live]), (kernel, splits, waves)

    # the rotating projection: 6 tokens, one a padding row, written at the positions above
    m, k, eps = len(slots), 96, 1e-5
    n = (heads + 2 * kv_heads) * head_dim
    x = torch.randn(m, k)
    gain = (1 + 0.1 * torch.randn(k)).bfloat16()
    w = ops.pack_weight((torch.randn(n, k) / math.sqrt(k)).bfloat16().cuda())
    results = []
    for with_tables in (False, True):
        kp, vp = k_pages.clone(), v_pages.clone()
        rope = dict(cos=cos, sin=sin, tok_slot=_i32(slots), tok_pos=_i32(positions), k_pages=kp, v_pages=vp, block_table=table,
                    heads=heads, kv_heads=kv_heads, head_dim=head_dim, tables=tables if with_tables else None)
        y = torch.zeros(m, heads * head_dim, dtype=torch.bfloat16, device="cuda")
        ops.gemm_fused(x.cuda(), None, None, gain.cuda(), eps, w, y, ops.EPILOGUE_ROPE, rope)
        results.append((y.cpu(), kp.cpu(), vp.cpu()))
    live = [i for i, s in enumerate(slots) if s >= 0]
    assert torch.equal(results[0][0][live], results[1][0][live])
    assert torch.equal(results[0][1], results[1][1]) and torch.equal(results[0][2], results[1][2])
    assert not torch.equal(results[1][1], k_pages.cpu())  # and the cache was written


@pytest.mark.parametrize("hint", [32, 48, 64, 80, 96, 112, 128])
def test_gemm_tiled_over_many_blocks(hint):
    """Each tile of the tiled kernel (64 x 128, 64 x 64, 256 x 256, 256 x 192, 128 x 128, 256 x 128, 128 x 192) over a grid of hundreds of blocks in
    bands and groups, with a ragged edge in every dimension; whole-number
    operands, so a block that took another's rows or columns shows."""
    ops = _ops()
    torch.manual_seed(hint)
    m, n, k = 2300, 1100, 584
    x = torch.randint(-3, 4, (m, k)).to(torch.bfloat16)
    w = torch.randint(-3, 4, (n, k)).to(torch.bfloat16)
    y = torch.full((m, n), 7.0, dtype=torch.float32, device="cuda")
    ops.gemm_bf16(x.cuda(), ops.pack_weight(w.cuda()), y, hint)
    assert torch.equal(y.cpu().double(), x.double() @ w.double().t())


@pytest.mark.parametrize("m", [1, 8, 19, 64, 67, 100, 300])
@pytest.mark.parametrize("n, k", [(576, 576), (100, 72), (2048, 1536), (48, 8), (64, 176), (3072, 576), (2080, 2304)])
@pytest.mark.parametrize("gain_dtype", ["bfloat16", "float32"])
def test_residual_projection_prepares_the_norm(m, n, k, gain_dtype):
    """resid += x . w^T in place; scaled = bfloat16(resid * gain); the parts of
    ss add up to each row's sum of squares."""
    ops = _ops()
    torch.manual_seed(m + n + k)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    resid = torch.randn(m, n) * 2
    gain = (1 + 0.3 * torch.randn(n)).to(DT[gain_dtype])
    want = resid.double() + x.double() @ w.double().t()
    resid_gpu = resid.cuda()
    scaled = torch.full((m, n), 9.0, dtype=torch.bfloat16, device="cuda")
    rows = ops.gemm_residual_parts(m, n)
    ss = torch.full((rows + 1, m), 7.0, device="cuda")
    parts = ops.gemm_residual(x.cuda(), ops.pack_weight(w.cuda()), resid_gpu, gain.cuda(), scaled, ss)
    assert 0 < parts <= rows
    assert (ss[parts:] == 7.0).all()  # nothing beyond the parts it names
    got = resid_gpu.cpu().double()
    assert ((got - want).abs() <= 1e-5 * (1 + want.abs())).all(), (got - want).abs().max().item()
    # scaled is the rounding of the 32-bit product of the new residual and the gain
    exact = (resid_gpu.cpu() * gain.float()).bfloat16()
    assert torch.equal(scaled.cpu(), exact)
    total = ss[:parts].cpu().double().sum(dim=0)
    assert ((total - got.pow(2).sum(dim=1)).abs() <= 1e-5 * got.pow(2).sum(dim=1)).all()


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n, k", [(2048, 5632), (1990, 5128), (48, 8192), (2048, 5120)])
def test_residual_projection_with_two_blocks_a_strip(m, n, k):
    """Up to 16 tokens on few strips and a long K (from 5,120 on): two blocks share each strip, and the second
    to be done adds the sums of the first to its own.  Three calls in a row on the same stream, with a tiled
    product that cuts its K into parts (and fills the workspace they share) between them: each is right, and
    the strips' counts are back at zero."""
    ops = _ops()
    assert ops.gemm_takes_pair(m, n, k)  # the kernel under test is the one that runs (and not at sizes beside its rule)
    assert not ops.gemm_takes_pair(17, n, k) and not ops.gemm_takes_pair(m, n, 5056) and not ops.gemm_takes_pair(m, 2064, k)
    torch.manual_seed(m + n + k)
    gain = (1 + 0.3 * torch.randn(n)).bfloat16()
    other_x = torch.randn(64, 4096).bfloat16().cuda()
    other_w = ops.pack_weight((torch.randn(2048, 4096) / 64).bfloat16().cuda())
    other_y = torch.empty(64, 2048, dtype=torch.bfloat16, device="cuda")
    rows = ops.gemm_residual_parts(m, n)
    for call in range(3):
        x = torch.randn(m, k).bfloat16()
        w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
        resid = torch.randn(m, n) * 2
        want = resid.double() + x.double() @ w.double().t()
        resid_gpu = resid.cuda()
        scaled = torch.full((m, n), 9.0, dtype=torch.bfloat16, device="cuda")
        ss = torch.full((rows + 1, m), 7.0, device="cuda")
        parts = ops.gemm_residual(x.cuda(), ops.pack_weight(w.cuda()), resid_gpu, gain.cuda(), scaled, ss)
        ops.gemm_bf16(other_x, other_w, other_y)  # 64 tokens on 2048 x 4096: K in parts, through the workspace
        assert 0 < parts <= rows and (ss[parts:] == 7.0).all()
        got = resid_gpu.cpu().double()
        assert ((got - want).abs() <= 1e-5 * (1 + want.abs())).all(), (call, (got - want).abs().max().item())
        assert torch.equal(scaled.cpu(), (resid_gpu.cpu() * gain.float()).bfloat16())
        total = ss[:parts].cpu().double().sum(dim=0)
        assert ((total - got.pow(2).sum(dim=1)).abs() <= 1e-5 * got.pow(2).sum(dim=1)).all()
        counts = ops.gemm_pair_counts(resid_gpu.device)
        assert counts.numel() == ops.PAIR_COUNTS and int(counts.abs().sum()) == 0


@pytest.mark.parametrize("tile", ["TILE_64x128", "TILE_64x64", "TILE_256x256", "TILE_256x192", "TILE_128x128", "TILE_256x128", "TILE_128x192"])
@pytest.mark.parametrize("m, n, k", [(70, 600, 136), (530, 300, 72), (300, 1100, 584)])
def test_residual_projection_with_every_tile(tile, m, n, k):
    """The tiled kernel's residual epilogue with each tile shape (several row
    and column blocks, ragged edges): the stream, the prepared operand and the
    parts of the sums of squares, one per wave column."""
    ops = _ops()
    torch.manual_seed(m + n)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    resid = torch.randn(m, n) * 2
    gain = (1 + 0.3 * torch.randn(n)).bfloat16()
    want = resid.double() + x.double() @ w.double().t()
    resid_gpu = resid.cuda()
    scaled = torch.full((m, n), 9.0, dtype=torch.bfloat16, device="cuda")
    rows = ops.gemm_residual_parts(m, n)
    ss = torch.full((rows + 1, m), 7.0, device="cuda")
    parts = ops.gemm_residual(x.cuda(), ops.pack_weight(w.cuda()), resid_gpu, gain.cuda(), scaled, ss, getattr(ops, tile))
    width = {"TILE_64x128": 64, "TILE_64x64": 32, "TILE_256x256": 128, "TILE_256x192": 96, "TILE_128x128": 64, "TILE_256x128": 64, "TILE_128x192": 96}[tile]  # columns of a wave
    if parts != 2 * ((n + 2 * width - 1) // (2 * width)):  # few tiles and a long K: K went in parts, summed per 64 columns
        assert tile in ("TILE_64x128", "TILE_64x64") and k >= 512 and parts == (n + 63) // 64
        width = 64
    assert (ss[parts:] == 7.0).all()
    got = resid_gpu.cpu().double()
    assert ((got - want).abs() <= 1e-5 * (1 + want.abs())).all(), (got - want).abs().max().item()
    assert torch.equal(scaled.cpu(), (resid_gpu.cpu() * gain.float()).bfloat16())
    for part in range(parts):
        columns = got[:, part * width:(part + 1) * width]
        assert ((ss[part].cpu().double() - columns.pow(2).sum(dim=1)).abs() <= 1e-5 * (1e-3 + columns.pow(2).sum(dim=1))).all(), part


@pytest.mark.parametrize("m", [1, 8, 16, 17, 40, 64, 65, 200, 300])
@pytest.mark.parametrize("k", [64, 96, 576, 1096])
@pytest.mark.parametrize("with_delta", [False, True, "prepared"])
@pytest.mark.parametrize("gain_dtype", ["bfloat16", "float32"])
def test_fused_norm_projection(m, k, with_delta, gain_dtype):
    """Residual sum + RMSNorm + projection in one kernel, with each epilogue,
    against the plain functions one after another.  "prepared": the sum and
    the first half of the norm are taken by the projection before (here one by
    the identity, so that it adds ``delta`` itself), the second half by the
    kernel under test."""
    ops = _ops()
    prepared = with_delta == "prepared"
    with_delta = bool(with_delta)
    if m > 64 and not prepared:
        pytest.skip("the kernel that takes the sum and the norm itself is for up to 64 tokens")
    torch.manual_seed(m * 7 + k)
    eps = 2e-5
    x = torch.randn(m, k) * 2
    delta = torch.randn(m, k).bfloat16() if with_delta else None
    gain = (1 + 0.3 * torch.randn(k)).to(DT[gain_dtype])
    summed = x + (delta.float() if with_delta else 0)
    normed = P.rms_norm(summed.double(), gain.double(), eps)

    if prepared:
        resid = x.cuda()
        scaled = torch.empty(m, k, dtype=torch.bfloat16, device="cuda")
        ss = torch.empty(ops.gemm_residual_parts(m, k), m, device="cuda")
        parts = ops.gemm_residual(delta.cuda(), ops.pack_weight(torch.eye(k).bfloat16().cuda()), resid, gain.cuda(), scaled, ss)
        assert torch.equal(resid.cpu(), summed)

    def run(w, y, epilogue, rope=None):
        if prepared:
            ops.gemm_scaled(scaled, ss, parts, eps, ops.pack_weight(w.cuda()), y, epilogue, rope)
            return y.cpu().double()
        x_out = torch.full((m, k), 9.0, device="cuda") if with_delta else None
        ops.gemm_fused(x.cuda(), delta.cuda() if with_delta else None, x_out, gain.cuda(), eps, ops.pack_weight(w.cuda()), y, epilogue, rope)
        if with_delta:
            assert torch.equal(x_out.cpu(), summed)  # the residual sum, exactly, written once
        return y.cpu().double()

    def close(got, want, what):
        assert ((got - want).abs() <= 2e-2 * (1 + want.abs())).all(), (what, (got - want).abs().max().item())

    # store, with a ragged last strip
    n = 70
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    close(run(w, torch.empty(m, n, dtype=torch.bfloat16, device="cuda"), ops.EPILOGUE_STORE), normed @ w.double().t(), "store")
    # gate rows, then up rows
    inner = 88
    w = (torch.randn(2 * inner, k) / math.sqrt(k)).bfloat16()
    both = normed @ w.double().t()
    close(run(w, torch.empty(m, inner, dtype=torch.bfloat16, device="cuda"), ops.EPILOGUE_SILU),
          P.silu(both[:, :inner]) * both[:, inner:], "silu")
    # queries, keys, values: rotation and the cache
    heads, kv_heads, head_dim = 3, 2, 32
    w = (torch.randn((heads + 2 * kv_heads) * head_dim, k) / math.sqrt(k)).bfloat16()
    qkv = (normed @ w.double().t()).view(m, heads + 2 * kv_heads, head_dim)
    cos_np, sin_np = P.rope_tables(512, head_dim, 10000.0)
    slots = [(i * 5) % 7 - (1 if i % 9 == 4 else 0) * 100 for i in range(m)]  # some padding rows
    slots = [s if s >= 0 else -1 for s in slots]
    positions = [(i * 37) % 320 for i in range(m)]  # no two tokens at one position (37 and 320 share no factor)
    table = torch.arange(7 * 5, dtype=torch.int32).view(7, 5).flip(0).contiguous()
    k_pages, v_pages = _empty_pages(35, kv_heads, head_dim, torch.bfloat16, 7.0, 7.0, "cuda")
    rope = dict(cos=torch.from_numpy(cos_np).cuda(), sin=torch.from_numpy(sin_np).cuda(), tok_slot=_i32(slots),
                tok_pos=_i32(positions), k_pages=k_pages, v_pages=v_pages, block_table=table.cuda(), heads=heads,
                kv_heads=kv_heads, head_dim=head_dim)
    got_q = run(w, torch.empty(m, heads * head_dim, dtype=torch.bfloat16, device="cuda"), ops.EPILOGUE_ROPE, rope)
    pos = torch.tensor(positions)
    turned = P.rope_rotate_half(qkv[:, :heads + kv_heads], torch.from_numpy(cos_np)[pos].double(), torch.from_numpy(sin_np)[pos].double())
    close(got_q.view(m, heads, head_dim), turned[:, :heads], "queries")
    seen = {}
    for t in range(m):  # a later token of the same slot and position overwrites an earlier one
        if slots[t] >= 0:
            seen[(slots[t], positions[t])] = t
    k_plain, v_plain = _read_pages(k_pages, v_pages, head_dim)
    for (slot, position), t in seen.items():
        page, inside = table[slot, position // 64].item(), position % 64
        close(k_plain[page, :, inside, :].double(), turned[t, heads:], "keys")
        close(v_plain[page, :, inside, :].double(), qkv[t, heads + kv_heads:], "values")
    written = sum(1 for _ in seen)
    assert int((k_plain != 7.0).any(dim=-1).sum()) <= written * kv_heads
    assert int((v_plain != 7.0).any(dim=-1).sum()) <= written * kv_heads


@pytest.mark.parametrize("hint", [32, 48, 64, 80, 96, 112, 128])
@pytest.mark.parametrize("m", [65, 200, 530])
def test_scaled_projection_with_every_tile(hint, m):
    """The tiled kernel's epilogues with each of its tile shapes (the hint picks
    one): pairs of strips in a wave, one or two of them."""
    ops = _ops()
    torch.manual_seed(hint + m)
    k, eps = 96, 1e-5
    v = torch.randn(m, k) * 2
    gain = (1 + 0.3 * torch.randn(k)).bfloat16()
    normed = P.rms_norm(v.double(), gain.double(), eps)
    resid = v.cuda()
    scaled = torch.empty(m, k, dtype=torch.bfloat16, device="cuda")
    ss = torch.empty(ops.gemm_residual_parts(m, k), m, device="cuda")
    parts = ops.gemm_residual(torch.zeros(m, 8, dtype=torch.bfloat16, device="cuda"), ops.pack_weight(torch.zeros(k, 8, dtype=torch.bfloat16, device="cuda")),
                              resid, gain.cuda(), scaled, ss)

    def close(got, want, what):
        assert ((got - want).abs() <= 2e-2 * (1 + want.abs())).all(), (what, (got - want).abs().max().item())

    n = 300
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    y = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    close(ops.gemm_scaled(scaled, ss, parts, eps, ops.pack_weight(w.cuda()), y, ops.EPILOGUE_STORE, None, hint).cpu().double(), normed @ w.double().t(), "store")
    inner = 200
    w = (torch.randn(2 * inner, k) / math.sqrt(k)).bfloat16()
    both = normed @ w.double().t()
    y = torch.empty(m, inner, dtype=torch.bfloat16, device="cuda")
    close(ops.gemm_scaled(scaled, ss, parts, eps, ops.pack_weight(w.cuda()), y, ops.EPILOGUE_SILU, None, hint).cpu().double(),
          P.silu(both[:, :inner]) * both[:, inner:], "silu")
    heads, kv_heads, head_dim = 5, 2, 64
    w = (torch.randn((heads + 2 * kv_heads) * head_dim, k) / math.sqrt(k)).bfloat16()
    qkv = (normed @ w.double().t()).view(m, heads + 2 * kv_heads, head_dim)
    cos_np, sin_np = P.rope_tables(1024, head_dim, 10000.0)
    positions = [(i * 37) % 1024 for i in range(m)]  # no two tokens at one place
    slots = [0 if i % 11 else -1 for i in range(m)]
    table = _i32([[3, 1, 0, 2, 15, 14, 4, 5, 13, 6, 12, 7, 11, 8, 10, 9]])
    k_pages, v_pages = _empty_pages(16, kv_heads, head_dim, torch.bfloat16, 7.0, 7.0, "cuda")
    rope = dict(cos=torch.from_numpy(cos_np).cuda(), sin=torch.from_numpy(sin_np).cuda(), tok_slot=_i32(slots),
                tok_pos=_i32(positions), k_pages=k_pages, v_pages=v_pages, block_table=table, heads=heads,
                kv_heads=kv_heads, head_dim=head_dim)
    y = torch.empty(m, heads * head_dim, dtype=torch.bfloat16, device="cuda")
    got_q = ops.gemm_scaled(scaled, ss, parts, eps, ops.pack_weight(w.cuda()), y, ops.EPILOGUE_ROPE, rope, hint).cpu().double()
    pos = torch.tensor(positions)
    turned = P.rope_rotate_half(qkv[:, :heads + kv_heads], torch.from_numpy(cos_np)[pos].double(), torch.from_numpy(sin_np)[pos].double())
    close(got_q.view(m, heads, head_dim), turned[:, :heads], "queries")
    k_plain, v_plain = _read_pages(k_pages, v_pages, head_dim)
    written = 0
    for t in range(m):
        if slots[t] < 0:
            continue
        written += 1
        page, inside = table[0, positions[t] // 64].item(), positions[t] % 64
        close(k_plain[page, :, inside, :].double(), turned[t, heads:], "keys")
        close(v_plain[page, :, inside, :].double(), qkv[t, heads + kv_heads:], "values")
    assert int((k_plain != 7.0).any(dim=-1).sum()) <= written * kv_heads  # padding rows wrote nothing


@pytest.mark.parametrize("m", [1, 8, 16, 30])
@pytest.mark.parametrize("n, paired", [(8192, False), (11264, False), (32000, False), (2 * 4096, True), (2 * 5632, True), (2 * 14336, True)])
def test_prepared_projection_on_wide_weights(n, paired, m):
    """Few tokens on a prepared operand over hundreds to thousands of strips of 16 weight rows, where the
    number of waves that share a strip's K goes from 8 to 4, 2 and 1 with the width: every width the rule
    tells apart, with the sizes' own choice."""
    ops = _ops()
    torch.manual_seed(n + m)
    k, eps = 2048, 1e-5
    v = torch.randn(m, k) * 2
    gain = (1 + 0.3 * torch.randn(k)).bfloat16()
    normed = P.rms_norm(v.double(), gain.double(), eps)
    scaled = torch.empty(m, k, dtype=torch.bfloat16, device="cuda")
    ss = torch.empty(ops.gemm_residual_parts(m, k), m, device="cuda")
    parts = ops.gemm_residual(torch.zeros(m, 8, dtype=torch.bfloat16, device="cuda"), ops.pack_weight(torch.zeros(k, 8, dtype=torch.bfloat16, device="cuda")),
                              v.cuda(), gain.cuda(), scaled, ss)
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    both = normed @ w.double().t()
    if paired:
        want = P.silu(both[:, :n // 2]) * both[:, n // 2:]
        y = torch.empty(m, n // 2, dtype=torch.bfloat16, device="cuda")
        got = ops.gemm_scaled(scaled, ss, parts, eps, ops.pack_weight(w.cuda()), y, ops.EPILOGUE_SILU).cpu().double()
    else:
        want = both
        y = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
        got = ops.gemm_scaled(scaled, ss, parts, eps, ops.pack_weight(w.cuda()), y, ops.EPILOGUE_STORE).cpu().double()
    assert ((got - want).abs() <= 2e-2 * (1 + want.abs())).all(), (got - want).abs().max().item()


def _k_index(head_dim):
    """[64 tokens, head_dim] -> offset of each (token, channel) in a page's keys of one head."""
    t = torch.arange(64).view(64, 1)
    c = torch.arange(head_dim).view(1, head_dim)
    return (c // 8) * 512 + t * 8 + c % 8


def _v_index(head_dim):
    t = torch.arange(64).view(64, 1)
    c = torch.arange(head_dim).view(1, head_dim)
    return ((((c // 16) * 2 + t // 32) * 4 + (t % 32) // 8) * 16 + c % 16) * 8 + t % 8


def _empty_pages(pages, kv_heads, head_dim, dtype, k_fill, v_fill, device="cpu"):
    k_pages = torch.full((pages, kv_heads, (head_dim + 7) // 8, 64, 8), k_fill, dtype=dtype, device=device)
    v_pages = torch.full((pages, kv_heads, (head_dim + 15) // 16, 2, 4, 16, 8), v_fill, dtype=dtype, device=device)
    return k_pages, v_pages


def _read_pages(k_pages, v_pages, head_dim):
    """Pages back in plain order: keys and values as [pages, kv_heads, 64 tokens, head_dim]."""
    pages, kv_heads = k_pages.shape[:2]
    k = k_pages.cpu().float().reshape(pages, kv_heads, -1)[:, :, _k_index(head_dim)]
    v = v_pages.cpu().float().reshape(pages, kv_heads, -1)[:, :, _v_index(head_dim)]
    return k, v


def _paged(k_seqs, v_seqs, dtype, kv_heads, head_dim, page_order=None, pages=32, max_pages=12):
    """Lays sequences out in pages the way the cache does.  k_seqs[i]: [len, kv_heads, head_dim]."""
    k_pages, v_pages = _empty_pages(pages, kv_heads, head_dim, dtype, 77.0, -55.0)
    k_flat, v_flat = k_pages.view(pages, kv_heads, -1), v_pages.view(pages, kv_heads, -1)
    k_index, v_index = _k_index(head_dim), _v_index(head_dim)
    table = torch.zeros(len(k_seqs), max_pages, dtype=torch.int32)
    order = list(page_order or range(pages))
    for slot, (k, v) in enumerate(zip(k_seqs, v_seqs)):
        for page_index in range((k.shape[0] + 63) // 64):
            page = order.pop()
            table[slot, page_index] = page
            chunk = slice(page_index * 64, min(k.shape[0], page_index * 64 + 64))
            n = chunk.stop - chunk.start
            k_flat[page][:, k_index[:n]] = k[chunk].transpose(0, 1).to(dtype)
            v_flat[page][:, v_index[:n]] = v[chunk].transpose(0, 1).to(dtype)
    return k_pages.cuda(), v_pages.cuda(), table.cuda()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads, kv_heads, head_dim", [(4, 2, 16), (3, 1, 32), (9, 3, 64), (5, 5, 80), (8, 2, 128), (2, 1, 192), (3, 3, 256)])
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
    k_pages, v_pages = _empty_pages(10, kv_heads, head_dim, DT[dtype], 7.0, 7.0, "cuda")
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
    k_plain, v_plain = _read_pages(k_pages, v_pages, head_dim)  # [pages, kv_heads, 64, head_dim]
    for t in range(tokens):
        if slots[t] < 0:
            assert (q_out[t] == 5.0).all()
            continue
        assert (q_out[t].cpu().float().view(heads, head_dim) - rotated[t, :heads]).abs().max() <= tol
        page, inside = table[slots[t], positions[t] // 64].item(), positions[t] % 64
        touched_k[page, inside] = True
        assert (k_plain[page, :, inside, :] - rotated[t, heads:]).abs().max() <= tol
        assert torch.equal(v_plain[page, :, inside, :], x[t, heads + kv_heads:])  # values are copied as they are
    # nothing else in the cache was written (padding of a page's last chunk included)
    assert (k_plain[~touched_k.unsqueeze(1).expand(-1, kv_heads, -1)] == 7.0).all()
    assert (v_plain[~touched_k.unsqueeze(1).expand(-1, kv_heads, -1)] == 7.0).all()
    assert int((k_pages != 7.0).sum()) <= int(touched_k.sum()) * kv_heads * head_dim
    assert int((v_pages != 7.0).sum()) <= int(touched_k.sum()) * kv_heads * head_dim
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
    if vocab > 9000:
        logits[4, 8999] = logits[4, 100] = 12.0  # a tie between two blocks' shares of the row
    out = torch.empty(5, dtype=torch.int32, device="cuda")
    ops.argmax(logits.cuda(), out)
    want = [int(np.nanargmax(row)) for row in logits.numpy()]
    assert out.cpu().tolist() == want
    if vocab >= 63:
        assert want[:3] == [7, vocab - 1, 0]
    if vocab > 9000:
        assert want[4] == 100


def test_refusals():
    ops = _ops()
    f = lambda *shape, dtype=torch.float32: torch.zeros(*shape, dtype=dtype, device="cuda")  # noqa: E731
    with pytest.raises(KernelError, match="ss has 1 rows"):  # scratch too small for the parts it would write
        ops.gemm_residual(f(70, 176, dtype=torch.bfloat16), ops.pack_weight(f(64, 176, dtype=torch.bfloat16)), f(70, 64),
                          f(64, dtype=torch.bfloat16), f(70, 64, dtype=torch.bfloat16), f(1, 70))
    with pytest.raises(KernelError):
        ops.gemm_ordered(f(3, 8), f(5, 9), f(3, 5))
    with pytest.raises(KernelError, match="GPU"):
        ops.gemm_ordered(torch.zeros(3, 8), f(5, 8), f(3, 5))
    with pytest.raises(KernelError, match="float32 or bfloat16"):
        ops.gemm_ordered(f(3, 8, dtype=torch.float16), f(5, 8), f(3, 5))
    from nnis_amd.errors import Unsupported

    for head_dim in (7, 258, 0):  # a size nobody runs: said as such (the model's check at load raises the same)
        with pytest.raises(Unsupported, match="head_dim"):
            ops.attention_module(head_dim)
    with pytest.raises(KernelError):
        ops.silu_mul(f(4, 11), f(4, 5))
    with pytest.raises(KernelError):
        ops.argmax(f(4, 11), torch.zeros(4, dtype=torch.int64, device="cuda"))


def test_the_tiles_that_products_are_given():
    """The tiled kernel's choice of tile by the product's sizes, at the sizes its rules were measured on (the
    library's own host code: no launch)."""
    ops = _ops()
    T = ops
    for (m, n, k), tile in {
        (2048, 16384, 2048): T.TILE_256x256,  # two full rounds of large tiles
        (2048, 6144, 2048): T.TILE_256x192,   # 256 blocks of 192 columns, where 256 columns make 192
        (1024, 11264, 2048): T.TILE_256x192,  # 236 blocks
        (512, 16384, 2048): T.TILE_256x128,   # 256 blocks where tiles of 256 x 192 make 172
        (384, 16384, 2048): T.TILE_256x128,   # rows that fill three quarters of their blocks: enough for a three-stage tile
        (320, 16384, 2048): T.TILE_64x128,    # ... and rows that do not (the blocks of 128 rows would be 384: a round and a half)
        (4096, 4096, 4096): T.TILE_256x256,   # a large tile that fills its round stays
        (4096, 2048, 8192): T.TILE_256x128,   # 256 blocks, one a compute unit, where large tiles would be 176
        (2048, 4096, 14336): T.TILE_256x128,
        (2048, 2048, 8192): T.TILE_128x128,   # 256 blocks of 128 rows where 256 rows make 128
        (2048, 2048, 512): T.TILE_64x128,     # ... over a short K the small tiles
        (2048, 2560, 2048): T.TILE_128x192,   # 224 tiles, where 256 x 128 makes 160 and 128 x 128 a round and a quarter
        (1536, 2560, 2048): T.TILE_128x128,
        (2048, 3072, 2048): T.TILE_128x192,   # a full round of 128 x 192 before three quarters of one of 256 x 128
        (1536, 4096, 4096): T.TILE_256x128,   # three quarters of a round (eleven sixteenths are enough)
        (1024, 6144, 2048): T.TILE_128x192,
        (2048, 1536, 2048): T.TILE_128x128,
        (3072, 2048, 4096): T.TILE_256x128,   # (192 blocks, where 128 x 128 would make a round and a half)
        (1024, 2048, 2048): T.TILE_64x64,     # no more than one wide block a compute unit: the narrow tile
        (2048, 576, 1536): T.TILE_64x64,
        (2048, 3072, 576): T.TILE_64x128,
    }.items():
        assert ops.gemm_tile(m, n, k) == tile, (m, n, k, ops.gemm_tile(m, n, k))
