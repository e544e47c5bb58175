"""The cache manager on the host: pages on demand, reuse, windows, state slots; no page is
lost, held twice or freed twice under random orders of requests (no GPU)."""

import random

import numpy as np
import pytest


from liyab_amd import Busy, ContextFull, InvalidArgument, OutOfPages
from liyab_amd.cache import UNMAPPED, CacheManager, KVSpec, PagePool


def manager(num_pages=64, page_size=16, max_positions=1024, max_requests=8, window=0, groups=None):
    groups = groups or [(KVSpec(4, 16, window), [0, 1])]
    return CacheManager(groups, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                        max_positions=max_positions)


def test_the_reference_tests_page_counts():
    """tests/test_kv_cache.cpp:129-149 with 16-token pages and a 1,024 limit."""
    m = manager()
    m.open("r")
    assert m.pages_in_use() == 0
    m.reserve([("r", 1)])
    assert m.pages_in_use() == 1
    m.reserve([("r", 100)])
    assert m.pages_in_use() == 7  # ceil(100 / 16)
    with pytest.raises(ContextFull):
        m.reserve([("r", 1025)])
    m.commit("r", 100)
    m.truncate("r", 20)  # pages starting at >= 32 are returned
    assert m.pages_in_use() == 2
    before = set(m.block_table("r"))
    m.reserve([("r", 100)])
    assert m.pages_in_use() == 7 and m.groups[0].pool.peak_in_use == 7  # freed pages were used again
    assert before <= set(m.block_table("r"))
    m.close("r")
    assert m.pages_in_use() == 0
    m.check()


def test_reserve_is_all_or_nothing_across_requests():
    m = manager(num_pages=5)
    m.open("a")
    m.open("b")
    m.reserve([("a", 40)])  # 3 pages
    m.commit("a", 40)
    assert not m.can_reserve([("a", 50), ("b", 20)])  # 1 + 2 > 2 free
    with pytest.raises(OutOfPages):
        m.reserve([("a", 50), ("b", 20)])
    assert m.pages_in_use() == 3 and m.block_table("b") == [] and len(m.block_table("a")) == 3
    assert m.can_reserve([("a", 48), ("b", 16)])  # a needs none (48 fits 3 pages), b one
    m.reserve([("a", 49), ("b", 16)])
    assert m.pages_in_use() == 5 and m.free_pages() == 0
    assert not m.can_reserve([], new_lengths=[1]) and m.can_reserve([], new_lengths=[0])
    m.check()


def test_finished_requests_pages_are_used_again_first():
    m = manager(num_pages=8)
    m.open("a")
    m.reserve([("a", 64)])
    pages_a = list(m.block_table("a"))
    m.commit("a", 64)
    m.close("a")
    m.open("b")
    m.reserve([("b", 33)])
    assert set(m.block_table("b")) <= set(pages_a) and m.groups[0].pool.peak_in_use == 4
    assert m.slot_of_position("b", 0, 17) == m.block_table("b")[1] * 16 + 1
    m.check()


def test_misuse_is_refused():
    m = manager(max_requests=2)
    m.open("a")
    with pytest.raises(InvalidArgument):
        m.open("a")
    m.open("b")
    with pytest.raises(Busy):
        m.open("c")
    m.reserve([("a", 10)])
    with pytest.raises(InvalidArgument):
        m.commit("a", 17)  # past the reserved pages
    m.commit("a", 10)
    with pytest.raises(InvalidArgument):
        m.reserve([("a", 5)])
    with pytest.raises(InvalidArgument):
        m.truncate("a", 11)
    with pytest.raises(KeyError):
        m.close("zzz")
    pool = PagePool(2)
    p = pool.allocate(1)
    pool.release(p)
    with pytest.raises(AssertionError):
        pool.release(p)  # freed twice
    with pytest.raises(OutOfPages):
        pool.allocate(3)


def test_state_slots():
    m = manager(max_requests=3)
    slots = [m.open(r) for r in "abc"]
    assert sorted(slots) == [0, 1, 2] and m.free_slots() == 0
    m.close("b")
    assert m.open("d") == slots[1]  # the freed slot is used again
    m.check()


def test_window_group_gives_back_pages_the_window_has_passed():
    spec_all, spec_win = KVSpec(2, 16, 0), KVSpec(2, 16, 40)
    m = CacheManager([(spec_all, [0, 2]), (spec_win, [1, 3])], page_size=16, num_pages=[64, 6], max_requests=4,
                     max_positions=1024)
    assert m.group_of_layer == {0: 0, 2: 0, 1: 1, 3: 1}
    m.open("r")
    length = 0
    for n in (30, 30, 1, 1, 50, 1, 1, 1, 7, 33):
        m.reserve([("r", length + n)])
        length += n
        m.commit("r", length)
        # group 0 keeps everything
        assert m.pages_in_use(0) == -(-length // 16)
        # group 1 keeps exactly the pages a query at position >= length can still see
        first_needed = max(0, length - 40 + 1)
        table = m.block_table("r", 1)
        for lp, page in enumerate(table):
            assert (page == UNMAPPED) == ((lp + 1) * 16 <= first_needed), (length, lp)
        m.check()
    assert m.groups[1].pool.peak_in_use <= 6
    m.close("r")
    assert m.pages_in_use(0) == 0 and m.pages_in_use(1) == 0
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    window = rng.choice([0, 0, 24, 70])
    m = CacheManager([(KVSpec(2, 16, 0), [0]), (KVSpec(2, 16, window), [1])], page_size=rng.choice([4, 16]),
                     num_pages=[rng.randint(20, 60), rng.randint(20, 60)], max_requests=5, max_positions=300)
    live, n = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.15 and len(live) < 5:
            rid = f"r{n}"
            n += 1
            m.open(rid)
            live[rid] = 0
        elif op < 0.75 and live:
            k = rng.randint(1, min(3, len(live)))
            wants = [(rid, live[rid] + rng.choice([1, 1, 1, 2, 9, 40])) for rid in rng.sample(sorted(live), k)]
            used = [m.pages_in_use(g) for g in range(2)]
            try:
                m.reserve(wants)
            except (OutOfPages, ContextFull):
                assert [m.pages_in_use(g) for g in range(2)] == used  # nothing changed
            else:
                for rid, length in wants:
                    m.commit(rid, length)
                    live[rid] = length
        elif op < 0.85 and live and window == 0:
            rid = rng.choice(sorted(live))
            live[rid] = rng.randint(0, live[rid])
            m.truncate(rid, live[rid])
        elif live:
            rid = rng.choice(sorted(live))
            m.close(rid)
            del live[rid]
        m.check()
        for rid, length in live.items():
            assert m.length(rid) == length
            assert sum(p != UNMAPPED for p in m.block_table(rid, 0)) >= -(-length // m.page_size)
    for rid in list(live):
        m.close(rid)
    m.check()
    assert m.pages_in_use(0) == 0 and m.pages_in_use(1) == 0 and m.free_slots() == 5


@pytest.mark.parametrize("seed", range(8))
def test_native_manager_does_what_the_plain_one_does(seed):
    """The same random operations on the native manager and on the plain Python one: the same
    pages in the same places, the same counters, the same refusals."""
    import plain_cache

    rng = random.Random(100 + seed)
    window = rng.choice([0, 24, 70])
    page_size = rng.choice([4, 16])
    pages = [rng.randint(10, 40), rng.randint(10, 40)]
    specs = [(KVSpec(2, 16, 0), [0]), (KVSpec(2, 16, window), [1])]
    kw = dict(page_size=page_size, num_pages=pages, max_requests=4, max_positions=200)
    a = CacheManager(specs, **kw)
    b = plain_cache.CacheManager([(plain_cache.KVSpec(2, 16, 0), [0]), (plain_cache.KVSpec(2, 16, window), [1])], **kw)
    live, n = {}, 0

    def both(op):
        """Runs op on both managers; they must agree on the outcome."""
        out = []
        for m in (a, b):
            try:
                out.append(("ok", op(m)))
            except (OutOfPages, ContextFull, InvalidArgument, Busy) as e:
                out.append((type(e).__name__, None))
        assert out[0] == out[1], out
        return out[0][0] == "ok"

    for _ in range(500):
        op = rng.random()
        if op < 0.15:
            rid = f"r{n}"
            n += 1
            if both(lambda m: m.open(rid)):
                live[rid] = 0
        elif op < 0.7 and live:
            k = rng.randint(1, min(3, len(live)))
            wants = [(rid, live[rid] + rng.choice([0, 1, 1, 2, 9, 40, 120])) for rid in rng.sample(sorted(live), k)]
            if both(lambda m: m.reserve(wants)):
                for rid, length in wants:
                    if rng.random() < 0.9:
                        both(lambda m: m.commit(rid, length))
                        live[rid] = length
        elif op < 0.8 and live:
            rid = rng.choice(sorted(live))
            to = rng.randint(0, live[rid] + 1)
            if both(lambda m: m.truncate(rid, to)):
                live[rid] = to
        elif live:
            rid = rng.choice(sorted(live))
            both(lambda m: m.close(rid))
            del live[rid]
        a.check()
        b.check()
        assert a.free_slots() == b.free_slots()
        for g in range(2):
            assert a.free_pages(g) == b.free_pages(g) and a.groups[g].pool.peak_in_use == b.groups[g].pool.peak_in_use
            assert np.array_equal(a.table_rows(g), b.table_rows(g))
        for rid, length in live.items():
            assert a.length(rid) == b.length(rid) == length and a.slot(rid) == b.slot(rid)
            assert [a.block_table(rid, g) for g in range(2)] == [b.block_table(rid, g) for g in range(2)]
            assert a.pages_needed(rid, length + 33) == b.pages_needed(rid, length + 33)


@pytest.mark.parametrize("seed,page_size,window", [(0, 16, 0), (1, 4, 0), (2, 24, 0), (3, 8, 20), (4, 48, 100)])
def test_a_steps_metadata_names_only_pages_and_slots_of_the_pool(seed, page_size, window):
    """Random stories of requests through the step metadata's native layout (liyab_step_shape /
    liyab_step_fill): every page id a block table carries to the device is -1 or a page of the
    pool, every slot a position of a page of the pool, and the slot of a token is its page's
    place in the table. The kernels follow these words without asking. Some steps carry padding rows
    behind their tokens: token 0 at position 0 of the first request, with slot -1, which the kernels skip."""
    import ctypes

    from liyab_amd import host

    rng = random.Random(seed)
    num_pages, max_positions, vocab = 40, 300, 1000
    groups = [(KVSpec(2, 16, 0), [0]), (KVSpec(2, 16, window), [1])] if window else [(KVSpec(2, 16, 0), [0, 1])]
    m = CacheManager(groups, page_size=page_size, num_pages=num_pages, max_requests=6, max_positions=max_positions)
    lib = host.lib()
    ip = lambda a: a.ctypes.data_as(host.IP)  # noqa: E731
    live, next_id, steps = {}, 0, 0
    for _ in range(400):
        if len(live) < 6 and (not live or rng.random() < 0.3):
            m.open(next_id)
            live[next_id] = 0
            next_id += 1
        batch = [r for r in live if rng.random() < 0.7] or [next(iter(live))]
        q = [min(rng.choice([1, 1, 1, 2, 5, 17, 60]), max_positions - live[r]) for r in batch]
        batch, q = [r for r, n in zip(batch, q) if n > 0], [n for n in q if n > 0]
        if batch:
            slots = np.array([m.slot(r) for r in batch], dtype=np.intc)
            q_lens = np.array(q, dtype=np.intc)
            try:
                new_lengths = m.reserve_more(slots, q_lens)
            except OutOfPages:
                victim = rng.choice(list(live))
                m.close(victim)
                del live[victim]
                continue
            wants = np.zeros(len(batch), dtype=np.intc)
            shape = host.StepShape()
            pad = rng.choice([0, 0, 1, 15, 63])
            host.check(lib.liyab_step_shape(m.handle, len(batch), ip(slots), ip(q_lens), ip(wants), pad, ctypes.byref(shape)))
            assert shape.n_tokens == int(q_lens.sum()) and shape.n_rows == shape.n_tokens + pad
            block = np.full(shape.total, -12345, dtype=np.int32)
            tokens = np.array([rng.randrange(vocab) for _ in range(int(q_lens.sum()))], dtype=np.int64)
            host.check(lib.liyab_step_fill(m.handle, ctypes.byref(shape), ip(slots), ip(q_lens),
                                           tokens.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), ip(wants), ip(np.zeros(1, dtype=np.intc)),
                                           vocab, block.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))))
            S, N, W = len(batch), int(q_lens.sum()), shape.max_blocks
            positions = block[shape.off_positions:shape.off_positions + N]
            tok_seq = block[shape.off_tok_seq:shape.off_tok_seq + N]
            assert positions.min() >= 0 and positions.max() < W * page_size
            for g in range(shape.n_groups):
                bt = block[shape.off_block_tables[g]:shape.off_block_tables[g] + S * W].reshape(S, W)
                sl = block[shape.off_slots[g]:shape.off_slots[g] + N]
                assert bt.min() >= -1 and bt.max() < num_pages
                assert sl.min() >= 0 and sl.max() < num_pages * page_size
                assert (sl == bt[tok_seq, positions // page_size] * page_size + positions % page_size).all()
                assert (block[shape.off_slots[g] + N:shape.off_slots[g] + N + pad] == -1).all()
            for off in (shape.off_token_ids, shape.off_positions, shape.off_tok_seq):
                assert (block[off + N:off + N + pad] == 0).all()
            assert (block != -12345).all()  # every word of the block is written
            m.commit_slots(slots, new_lengths)
            for r, n in zip(batch, new_lengths):
                live[r] = int(n)
            steps += 1
        for r in [r for r in live if live[r] >= max_positions or rng.random() < 0.03]:
            m.close(r)
            del live[r]
        m.check()
    assert steps > 200
