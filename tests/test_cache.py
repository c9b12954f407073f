"""The cache's bookkeeping on the host: no slot or page is lost, held twice or
freed twice; a refused growth changes nothing; slots given back are used again;
state of fixed size starts at zero.  Behaviours kept from the reference's cache
tests (/root/reference/crates/nnis-rt/src/kv_cache.rs:501-629: overflow leaves
the length unchanged, reset reuses)."""

import random

import pytest
import torch

from nnis_amd.cache import FreeList, PageTable, SequenceCache, pages_for
from nnis_amd.errors import CacheFull, InvalidInput
from nnis_amd.parts.base import KVRequest, StateRequest


def test_free_list_never_loses_or_doubles():
    pool = FreeList(5, "slot")
    taken = [pool.take() for _ in range(5)]
    assert sorted(taken) == [0, 1, 2, 3, 4] and pool.free == 0
    with pytest.raises(CacheFull):
        pool.take()
    pool.give_back(3)
    with pytest.raises(InvalidInput, match="not held"):
        pool.give_back(3)  # freed twice
    with pytest.raises(InvalidInput):
        pool.give_back(17)  # never given
    assert pool.take() == 3  # used again
    rng = random.Random(0)
    held = set(pool.held)
    for _ in range(2000):
        if held and (rng.random() < 0.5 or pool.free == 0):
            item = rng.choice(sorted(held))
            pool.give_back(item)
            held.remove(item)
        else:
            item = pool.take()
            assert item not in held  # never held twice
            held.add(item)
        assert pool.free + len(held) == 5 and held == set(pool.held)
    with pytest.raises(InvalidInput):
        FreeList(0, "slot")


def test_pages_follow_lengths():
    assert [pages_for(n) for n in (0, 1, 64, 65, 128, 129)] == [0, 1, 1, 2, 2, 3]
    table = PageTable(pages=4, slots=3, max_pages_per_slot=3)
    assert table.grow(0, 1) == [0] and table.grow(0, 64) == [] and table.grow(0, 65) == [1]
    assert table.grow(1, 100) == [0, 1]
    with pytest.raises(CacheFull):
        table.grow(2, 1)
    assert table.rows[0] != table.rows[1] and not set(table.rows[0]) & set(table.rows[1])
    table.release(0)
    assert table.pool.free == 2 and 0 not in table.rows
    table.grow(2, 128)
    with pytest.raises(CacheFull, match="at most 3 pages"):
        PageTable(pages=8, slots=1, max_pages_per_slot=3).grow(0, 64 * 4)


def _cache(max_tokens=512, extra=()):
    requests = [(0, KVRequest(2, 16)), (1, KVRequest(2, 16)), (2, KVRequest(1, 32, window=100)), *extra]
    return SequenceCache(requests, {3: 1}, max_tokens=max_tokens, max_positions=300, dtype=torch.float32, device="cpu")


def test_groups_have_storage_of_their_own():
    cache = _cache(extra=[(4, StateRequest((3, 5)))])
    assert len(cache.kv_groups) == 2  # all keys / a window of them
    full, windowed = cache.kv_groups
    # [entries, pages, kv_heads, ...]: keys in chunks of 8 channels, values in tiles of 16 channels
    assert full.k.shape == (2, 8, 2, 2, 64, 8) and full.v.shape == (2, 8, 2, 1, 2, 4, 16, 8)
    assert windowed.k.shape == (1, 8, 1, 4, 64, 8) and windowed.request.window == 100
    assert cache.view(0).k_pages.data_ptr() != cache.view(1).k_pages.data_ptr()
    shared = cache.view(3)  # reads entry 1's cache
    assert shared.read_only and shared.k_pages.data_ptr() == cache.view(1).k_pages.data_ptr()
    assert not cache.view(1).read_only
    assert cache.view(4).state.shape == (8, 3, 5)
    assert cache.bytes_per_token() == 2 * 2 * 2 * 16 * 4 + 2 * 1 * 1 * 32 * 4


def test_slots_are_given_back_and_used_again():
    cache = _cache(max_tokens=256)  # 4 pages, 4 slots
    a, b = cache.acquire(), cache.acquire()
    cache.grow({a: 70, b: 5})
    assert cache.length(a) == 70 and cache.length(b) == 5 and cache.live_tokens() == 75
    assert cache.kv_groups[0].table.pool.free == 1
    # a refused growth changes nothing: neither lengths nor pages
    with pytest.raises(CacheFull):
        cache.grow({a: 60, b: 60})
    assert cache.length(a) == 70 and cache.length(b) == 5 and cache.kv_groups[0].table.pool.free == 1
    with pytest.raises(CacheFull, match="positions end at 300"):
        cache.check_room({a: 231})
    pages_of_a = list(cache.kv_groups[0].table.rows[a])
    row = cache.kv_groups[0].block_table[a, :2].tolist()
    assert row == pages_of_a  # the device table follows the host's
    cache.release(a)
    with pytest.raises(InvalidInput):
        cache.release(a)
    with pytest.raises(InvalidInput):
        cache.length(a)
    again = cache.acquire()
    assert again == a and cache.length(again) == 0  # the slot is used again, empty
    cache.grow({again: 128})
    assert sorted(cache.kv_groups[0].table.rows[again]) == sorted(pages_of_a)  # and so are its pages
    for slot in (again, b):
        cache.release(slot)
    assert all(g.table.pool.free == 4 for g in cache.kv_groups) and cache.slots.free == 4


def test_state_starts_at_zero():
    cache = _cache(extra=[(4, StateRequest((2,), "float32"))])
    region = cache.add_state_region("extra", (), torch.int64)
    slot = cache.acquire()
    cache.view(4).state[slot] = 7.0
    region[slot] = 99
    cache.release(slot)
    assert cache.acquire() == slot
    assert cache.view(4).state[slot].abs().sum() == 0 and region[slot] == 0
    with pytest.raises(InvalidInput):
        cache.add_state_region("extra", (), torch.int64)


@pytest.mark.parametrize("head_dim", [16, 24, 64, 80])
def test_a_page_holds_every_key_and_value_once(head_dim):
    """The page orders are one-to-one: every (token, channel) has a place of
    its own inside the page, 8 channels of a key lie together and so do 8
    tokens of a value channel."""
    from nnis_amd.cache.layout import k_offset, k_page_shape, v_offset, v_page_shape

    k_size = 1
    for n in k_page_shape(1, head_dim):
        k_size *= n
    v_size = 1
    for n in v_page_shape(1, head_dim):
        v_size *= n
    k_places = {k_offset(t, c) for t in range(64) for c in range(head_dim)}
    v_places = {v_offset(c, t) for t in range(64) for c in range(head_dim)}
    assert len(k_places) == len(v_places) == 64 * head_dim
    assert max(k_places) < k_size and max(v_places) < v_size
    assert k_size == 64 * 8 * ((head_dim + 7) // 8) and v_size == 64 * 16 * ((head_dim + 15) // 16)
    for t in (0, 37, 63):
        for c in range(0, head_dim - 7, 8):
            assert [k_offset(t, c + i) - k_offset(t, c) for i in range(8)] == list(range(8))
    for c in (0, head_dim - 1):
        for t in range(0, 64, 8):
            assert [v_offset(c, t + i) - v_offset(c, t) for i in range(8)] == list(range(8))
    # a wave's loads: lane = token reads 16 consecutive bytes of a chunk after its neighbour's
    assert k_offset(5, 8) - k_offset(4, 8) == 8
    # lane (r, g) of a value load: channel 16 t + r, tokens 32 h + 8 g ..; consecutive lanes r, then g
    assert v_offset(1, 0) - v_offset(0, 0) == 8 and v_offset(0, 8) - v_offset(15, 0) == 8


def test_one_more_token_each_is_all_or_nothing():
    cache = _cache(max_tokens=192)  # 3 pages, 3 slots
    a, b = cache.acquire(), cache.acquire()
    cache.grow({a: 64, b: 63})
    free = cache.kv_groups[0].table.pool.free
    assert cache.grow_by_one([a, b]) == [64, 63]  # a starts its second page, b fills its first
    assert cache.length(a) == 65 and cache.length(b) == 64
    assert cache.kv_groups[0].table.pool.free == free - 1
    assert cache.kv_groups[0].block_table[a, :2].tolist() == cache.kv_groups[0].table.rows[a]
    # b needs a page now and none is left: nothing changes, a included
    with pytest.raises(CacheFull):
        cache.grow_by_one([a, b])
    assert cache.length(a) == 65 and cache.length(b) == 64 and cache.kv_groups[0].table.pool.free == 0
    with pytest.raises(InvalidInput, match="not held"):
        cache.grow_by_one([a, 7])
    assert cache.length(a) == 65
    cache.release(b)
    c = cache.acquire()
    for _ in range(64):
        cache.grow_by_one([c])  # the page that b gave back
    assert cache.length(c) == 64 and cache.kv_groups[0].table.pool.free == 0
    lone = SequenceCache([(0, KVRequest(1, 16))], {}, max_tokens=640, max_positions=70, dtype=torch.float32, device="cpu")
    s = lone.acquire()
    lone.grow({s: 69})
    assert lone.grow_by_one([s]) == [69]
    with pytest.raises(CacheFull, match="positions end at 70"):
        lone.grow_by_one([s])
    assert lone.length(s) == 70


def test_truncate_gives_pages_back_and_keeps_the_rest():
    # the rules of /root/reference/crates/nnis-rt/src/kv_cache.rs:69-83,170-192,509-545 on pages
    cache = _cache(max_tokens=512)  # 8 pages
    a, b = cache.acquire(), cache.acquire()
    cache.grow({a: 200, b: 65})
    full = cache.kv_groups[0]
    first_pages = list(full.table.rows[a])
    assert len(first_pages) == 4 and full.table.pool.free == 2
    # longer than what is held: refused, nothing changes
    with pytest.raises(InvalidInput, match="cannot be truncated to 201"):
        cache.truncate(a, 201)
    with pytest.raises(InvalidInput):
        cache.truncate(a, -1)
    assert cache.length(a) == 200 and full.table.pool.free == 2
    cache.truncate(a, 200)  # to its own length: nothing to do
    assert full.table.rows[a] == first_pages
    cache.truncate(a, 70)  # 4 pages -> 2, in every group
    assert cache.length(a) == 70 and cache.length(b) == 65
    assert full.table.rows[a] == first_pages[:2]
    assert all(g.table.pool.free == 4 for g in cache.kv_groups)
    assert not set(first_pages[2:]) & set(full.table.pool.held)
    # the next tokens are appended at the new length, on pages taken anew (lowest first: those just given back)
    cache.grow({a: 100})
    assert cache.length(a) == 170 and full.table.rows[a][:2] == first_pages[:2]
    assert sorted(full.table.rows[a][2:]) == sorted(first_pages[2:])[:1]
    assert full.block_table[a, :3].tolist() == full.table.rows[a]
    # within a page: no page moves
    cache.truncate(a, 129)
    assert len(full.table.rows[a]) == 3
    cache.truncate(a, 128)
    assert len(full.table.rows[a]) == 2
    with pytest.raises(InvalidInput, match="not held"):
        cache.truncate(7, 0)
    # nothing is lost, held twice or freed twice
    for slot in (a, b):
        cache.release(slot)
    assert all(g.table.pool.free == 8 and not g.table.pool.held for g in cache.kv_groups)


def test_reset_empties_a_slot_that_stays_held():
    """Lengths, pages and the layers' own state go; what somebody else keeps
    for the sequence in the slot's state regions (a sampler's generator and
    options) stays: a sampled sequence goes on after a reset
    (kv_cache.rs:170-172 only sets lengths to 0)."""
    cache = _cache(max_tokens=256, extra=[(4, StateRequest((3,)))])
    region = cache.add_state_region("extra", (2,), torch.float32)
    a = cache.acquire()
    cache.grow({a: 130})
    region[a] = 3.0
    cache.view(4).state[a] = 5.0
    cache.reset(a)
    assert cache.length(a) == 0 and a in cache.slots.held
    assert all(g.table.pool.free == 4 for g in cache.kv_groups)
    assert cache.view(4).state[a].abs().sum() == 0  # the mixer's state starts over
    assert bool((region[a] == 3.0).all())  # the sampler's does not
    cache.release(a)
    assert cache.acquire() == a and region[a].abs().sum() == 0  # a new sequence in the slot starts from zero everywhere
    cache.grow({a: 256})  # the whole cache again
    assert cache.length(a) == 256
    cache.release(a)
    with pytest.raises(InvalidInput):
        cache.reset(a)


def test_fixed_size_state_refuses_truncation():
    cache = _cache(extra=[(4, StateRequest((3,)))])
    a = cache.acquire()
    cache.grow({a: 10})
    with pytest.raises(InvalidInput, match="fixed-size state"):
        cache.truncate(a, 5)
    assert cache.length(a) == 10
    cache.truncate(a, 10)  # nothing is wound back: allowed
    cache.reset(a)  # starts the sequence over, state zeroed
    assert cache.length(a) == 0


def test_free_list_hands_out_the_lowest_whatever_came_back():
    from nnis_amd.cache.allocator import FreeList

    pool = FreeList(6, "thing")
    taken = [pool.take() for _ in range(6)]
    assert taken == [0, 1, 2, 3, 4, 5]
    for item in (4, 1, 5, 2):
        pool.give_back(item)
    assert [pool.take() for _ in range(4)] == [1, 2, 4, 5]
    with pytest.raises(CacheFull):
        pool.take()
    pool.give_back(3)
    with pytest.raises(InvalidInput):
        pool.give_back(3)
    assert pool.free == 1 and pool.held == frozenset({0, 1, 2, 4, 5})


def test_values_may_be_narrower_than_keys():
    cache = SequenceCache([(0, KVRequest(2, 32, value_dim=16)), (1, KVRequest(2, 32))], {}, max_tokens=128, max_positions=128,
                          dtype=torch.float32, device="cpu")
    assert len(cache.kv_groups) == 2  # a need of its own, storage of its own
    narrow = cache.kv_groups[0]
    assert narrow.k.shape[2:] == (2, 4, 64, 8) and narrow.v.shape[2:] == (2, 1, 2, 4, 16, 8)
    assert narrow.bytes_per_token() == 2 * (32 + 16) * 4 and cache.kv_groups[1].bytes_per_token() == 2 * 64 * 4


def test_roll_back_returns_what_a_failed_step_took():
    """A step whose launch failed after the cache grew: lengths and pages as
    before, also where fixed-size state makes ``truncate`` refuse; a slot that
    is not held, or a length not below the present one, is left alone."""
    cache = _cache(max_tokens=512, extra=[(4, StateRequest((3,)))])
    a, b = cache.acquire(), cache.acquire()
    cache.grow({a: 70, b: 10})
    free = [g.table.pool.free for g in cache.kv_groups]
    before = {a: cache.length(a), b: cache.length(b)}
    cache.grow({a: 200, b: 1})
    cache.roll_back(before)
    assert {a: cache.length(a), b: cache.length(b)} == before
    assert [g.table.pool.free for g in cache.kv_groups] == free
    cache.roll_back({a: 500, 99: 0})  # nothing to undo
    assert cache.length(a) == 70
    cache.grow({a: 1})
    assert cache.length(a) == 71  # and the sequence goes on where it was


def test_one_more_is_checked_without_a_change():
    cache = _cache(max_tokens=192)
    a, b = cache.acquire(), cache.acquire()
    cache.grow({a: 64, b: 64})
    cache.check_one_more([a])  # one page is free
    with pytest.raises(CacheFull):
        cache.check_one_more([a, b])  # both start a page, one is left
    assert cache.length(a) == 64 and cache.length(b) == 64
    checked = cache.check_one_more([a])
    assert cache.grow_by_one([a], checked) == [64] and cache.length(a) == 65
    with pytest.raises(InvalidInput, match="not held"):
        cache.check_one_more([7])


def test_positions_end_for_a_model_without_keys():
    """A model that keeps only fixed-size state is stopped at its last position too."""
    cache = SequenceCache([(0, StateRequest((2,)))], {}, max_tokens=1024, max_positions=100, dtype=torch.float32, device="cpu")
    a = cache.acquire()
    cache.grow({a: 99})
    cache.grow_by_one([a])
    with pytest.raises(CacheFull, match="positions end at 100"):
        cache.grow({a: 1})
    with pytest.raises(CacheFull, match="positions end at 100"):
        cache.grow_by_one([a])
    assert cache.length(a) == 100


class _Event:
    """Stands in for the event behind a flush: counts who waits for it."""

    def __init__(self):
        self.recorded = self.waited = 0

    def record(self):
        self.recorded += 1

    def synchronize(self):
        self.waited += 1


def test_a_row_is_not_rewritten_before_its_copy_has_left():
    """The block table's rows go to the device by copies that do not wait;
    whoever writes into the pinned rows again waits for the last flush first,
    and only then (no wait where nothing is pending)."""
    cache = _cache(max_tokens=512)
    group = cache.kv_groups[0]
    group._flushed = event = _Event()
    a = cache.acquire()
    cache.grow({a: 10})  # first pages: nothing pending yet
    assert (event.recorded, event.waited) == (1, 0)
    cache.grow({a: 20})  # no new page: no flush, no wait
    assert (event.recorded, event.waited) == (1, 0)
    cache.grow({a: 60})  # a new page: the row is written again, after the first flush has left
    assert (event.recorded, event.waited) == (2, 1)
    cache.release(a)
    b = cache.acquire()  # the same slot, another sequence
    assert b == a
    cache.grow({b: 1})
    assert (event.recorded, event.waited) == (3, 2)
    cache.grow_by_one([b])  # inside its page
    assert (event.recorded, event.waited) == (3, 2)


@pytest.mark.parametrize("seed", range(8))
def test_operations_drawn_from_a_seed(seed):
    """Four hundred operations in an order drawn from the seed -- sequences start, grow by prompts and by single
    tokens (checked first, all or nothing), are cut back, reset, rolled back and ended -- against a model of the
    lengths kept here.  After each one: every group holds exactly the pages its lengths need, no page twice, the
    rows that the kernels read name them, and what is free and what is held add up."""
    rng = random.Random(seed)
    cache = _cache(max_tokens=10 * 64)
    lengths = {}

    def check():
        assert {s: cache.length(s) for s in lengths} == lengths and set(cache.slots.held) == set(lengths)
        assert cache.live_tokens() == sum(lengths.values())
        for group in cache.kv_groups:
            seen = []
            for slot, n in lengths.items():
                row = group.table.rows.get(slot, [])
                assert len(row) == pages_for(n)
                assert group.block_table_host[slot, :len(row)].tolist() == row
                seen += row
            assert len(seen) == len(set(seen)) and set(seen) == set(group.table.pool.held)
            assert group.table.pool.free + len(seen) == 10

    for _ in range(400):
        action = rng.random()
        if not lengths or (action < 0.12 and len(lengths) < cache.max_slots):
            lengths[cache.acquire()] = 0
        elif action < 0.2:
            slot = rng.choice(sorted(lengths))
            cache.release(slot)
            del lengths[slot]
        elif action < 0.3:
            slot = rng.choice(sorted(lengths))
            keep = rng.randint(0, lengths[slot])
            cache.truncate(slot, keep)
            lengths[slot] = keep
        elif action < 0.35:
            slot = rng.choice(sorted(lengths))
            cache.reset(slot)
            lengths[slot] = 0
        elif action < 0.65:  # prompts: some sequences grow by any number of tokens, together or not at all
            some = [s for s in sorted(lengths) if rng.random() < 0.6] or [rng.choice(sorted(lengths))]
            growth = {s: rng.choice([1, 2, 63, 64, 65, rng.randint(1, 200)]) for s in some}
            fits = (all(lengths[s] + n <= 300 for s, n in growth.items())
                    and sum(pages_for(lengths[s] + n) - pages_for(lengths[s]) for s, n in growth.items()) <= cache.kv_groups[0].table.pool.free)
            before = dict(lengths)
            try:
                cache.check_room(growth)
                cache.grow(growth)
                assert fits
                for s, n in growth.items():
                    lengths[s] += n
                if rng.random() < 0.2:  # the step failed in flight: everything goes back
                    cache.roll_back(before)
                    lengths = before
            except (CacheFull, InvalidInput):
                assert not fits
        else:  # one token each
            some = [s for s in sorted(lengths) if rng.random() < 0.7] or [rng.choice(sorted(lengths))]
            fits = (all(lengths[s] + 1 <= 300 for s in some)
                    and sum(1 for s in some if lengths[s] % 64 == 0) <= cache.kv_groups[0].table.pool.free)
            try:
                checked = cache.check_one_more(some)
                assert fits
                assert cache.grow_by_one(some, checked if rng.random() < 0.5 else None) == [lengths[s] for s in some]
                for s in some:
                    lengths[s] += 1
            except (CacheFull, InvalidInput):
                assert not fits
        check()
    for slot in list(lengths):
        cache.release(slot)
    assert all(g.table.pool.free == 10 and not g.table.pool.held for g in cache.kv_groups) and not cache.slots.held
