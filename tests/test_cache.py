"""The cache manager's books: no page lost, held twice or freed twice, under
random orders of requests; pages behind a window come back and are used again."""

import random

import pytest

from rvllm_amd.cache import CacheBookkeepingError, CacheManager, OutOfPages, PagePool, StateSlots
from rvllm_amd.parts.base import KVNeed, StateNeed


def make(window=8, page_size=4, num_pages=16, max_requests=4, extra_state=False):
    needs = [KVNeed(2, 16, window), KVNeed(2, 16, None), KVNeed(1, 32, window)]
    if extra_state:
        needs.append(StateNeed((4,)))
    return CacheManager(needs, page_size, num_pages, max_requests)


def test_layers_group_by_need():
    m = make(extra_state=True)
    assert set(m.groups) == {"window8", "full"}
    assert m.groups["window8"].layers == [0, 2] and m.groups["full"].layers == [1]
    assert m.layer_group == ["window8", "full", "window8", None] and m.state_layers == [3]


def test_pool_refuses_double_free_and_foreign_free():
    pool = PagePool("g", 4)
    pages = pool.take("a", 2)
    assert pages == [0, 1]
    pool.give_back("a", [0])
    with pytest.raises(CacheBookkeepingError):
        pool.give_back("a", [0])  # twice
    with pytest.raises(CacheBookkeepingError):
        pool.give_back("b", [1])  # not the owner
    with pytest.raises(OutOfPages):
        pool.take("b", 4)
    assert pool.free_count == 3  # the refused request took nothing
    assert pool.take("b", 1) == [0]  # the page just given back is used again first
    pool.check()


def test_window_pages_come_back_and_full_pages_stay():
    m = make(window=8, page_size=4, num_pages=16)
    m.add_request("r")
    m.extend("r", 10)
    assert m.table("r", "full") == [0, 1, 2] and m.table("r", "window8") == [0, 1, 2]
    m.commit("r", 10)
    # the next token is at 10 and sees 3..10: page 0 (positions 0..3) is still needed
    assert m.table("r", "window8") == [0, 1, 2]
    m.extend("r", 12)
    m.commit("r", 12)
    # next token at 12 sees 5..12: page 0 has been passed
    assert m.table("r", "window8") == [-1, 1, 2] and m.free_pages()["window8"] == 14
    m.extend("r", 13)
    # the page given back is the first to be used again
    assert m.table("r", "window8") == [-1, 1, 2, 0]
    m.commit("r", 13)
    assert m.table("r", "full") == [0, 1, 2, 3]
    m.check()
    m.release("r")
    assert m.free_pages() == {"window8": 16, "full": 16}
    m.check()


def test_reference_ring_vectors_scaled_down():
    """The reference pins which slots a sliding layer uses around the wrap of
    its ring (v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:6357-6381: with
    window 1024 a token at 1023/1024/1025 sees at most 1024 keys).  Here the
    same edge in pages: with window 8 and pages of 4, the first page is kept
    while the next token's position is at most 10 and given back from 11 on."""
    for length, kept in [(8, 0), (10, 0), (11, 1), (12, 1), (15, 2)]:
        m = make(window=8, page_size=4)
        assert m.groups["window8"].first_kept_page(length) == kept
        assert m.groups["full"].first_kept_page(length) == 0


def test_out_of_pages_takes_nothing():
    m = make(num_pages=4, page_size=4)
    m.add_request("a")
    m.extend("a", 12)
    m.add_request("b")
    with pytest.raises(OutOfPages):
        m.extend("b", 8)
    assert m.table("b", "full") == [] and m.table("b", "window8") == []
    assert not m.can_extend([("b", 8)]) and m.can_extend([("b", 4)])
    with pytest.raises(OutOfPages):
        m.require([("a", 16), ("b", 4)])  # together they do not fit
    m.check()


def test_a_step_gets_all_its_pages_or_none():
    m = make(num_pages=6, page_size=4)
    for rid in "abc":
        m.add_request(rid)
    m.extend_all([("a", 8), ("b", 5), ("c", 1)])  # 2 + 2 + 1 pages of 6
    assert [len(m.table(r, "full")) for r in "abc"] == [2, 2, 1]
    for rid, n in (("a", 8), ("b", 5), ("c", 1)):
        m.commit(rid, n)
    with pytest.raises(OutOfPages):
        m.extend_all([("a", 9), ("b", 9)])  # one page each, one is left
    assert [len(m.table(r, "full")) for r in "abc"] == [2, 2, 1] and m.free_pages()["full"] == 1
    with pytest.raises(ValueError, match="cannot extend"):
        m.extend_all([("a", 7)])
    with pytest.raises(KeyError):
        m.extend_all([("nobody", 1)])
    m.extend_all([("c", 4), ("a", 9)])  # c needs none
    assert m.free_pages()["full"] == 0
    m.check()


def test_a_reservation_says_what_the_whole_list_says():
    """The tally a scheduler keeps while it plans a step: asked one request at a time, it answers as
    ``can_extend`` does for everything planned so far and the one more, for live requests and new ones, with pools
    that run out of pages and of slots, and after a request that was not planned gave its pages back in between."""
    rng = random.Random(5)
    refused = accepted = 0
    for trial in range(80):
        m = make(num_pages=rng.choice([6, 10, 24]), page_size=4, max_requests=rng.choice([3, 6]))
        live = []
        for i in range(rng.randrange(0, 4)):
            length = rng.randrange(1, 14)
            if m.can_extend([(f"old{i}", length)]):
                m.add_request(f"old{i}")
                m.extend(f"old{i}", length)
                m.commit(f"old{i}", length)
                live.append(f"old{i}")
        tally, planned = m.reservation(), []
        candidates = [(rid, m.length(rid) + rng.randrange(1, 30)) for rid in live] + \
                     [(f"new{j}", rng.randrange(1, 30)) for j in range(5)]
        rng.shuffle(candidates)
        gone = set()
        for rid, new_len in candidates:
            if rid in gone:
                continue
            want = m.can_extend(planned + [(rid, new_len)])
            assert tally.fits(rid, new_len) == want, (trial, rid, new_len)
            if want:
                accepted += 1
                if not m.has_request(rid):
                    m.add_request(rid)  # as a scheduler admits what it has planned
                tally.add(rid, new_len)
                planned.append((rid, new_len))
            else:
                refused += 1
                unplanned = [r for r in live if r not in gone and all(r != p for p, _ in planned)]
                if unplanned and rng.random() < 0.5:
                    m.release(unplanned[-1])  # set back: its pages count as free from now on
                    gone.add(unplanned[-1])
        m.check()
    assert refused > 20 and accepted > 20


def test_commit_without_pages_is_caught():
    m = make()
    m.add_request("a")
    with pytest.raises(CacheBookkeepingError):
        m.commit("a", 5)


def test_slots():
    m = make(max_requests=2)
    a, b = m.add_request("a"), m.add_request("b")
    assert {a.slot, b.slot} == {0, 1}
    with pytest.raises(OutOfPages):
        m.add_request("c")
    m.release("a")
    assert m.add_request("c").slot == a.slot
    with pytest.raises(KeyError):
        m.add_request("c")
    s = StateSlots(1)
    s.take("x")
    with pytest.raises(CacheBookkeepingError):
        s.give_back("y", 0)


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    window, page_size = rng.choice([(8, 4), (5, 16), (70, 16), (3, 4)])
    m = make(window=window, page_size=page_size, num_pages=rng.choice([6, 12, 40]), max_requests=4)
    wname = f"window{window}"
    live: dict[str, int] = {}
    counter = 0
    for _ in range(400):
        action = rng.random()
        if (action < 0.2 and len(live) < 4) or not live:
            counter += 1
            name = f"r{counter}"
            m.add_request(name)
            live[name] = 0
        elif action < 0.3:
            name = rng.choice(list(live))
            m.release(name)
            del live[name]
        else:
            name = rng.choice(list(live))
            new_len = live[name] + rng.choice([1, 1, 1, 2, 7, 30])
            try:
                m.extend(name, new_len)
            except OutOfPages:
                m.check()
                victim = rng.choice(list(live))
                m.release(victim)
                del live[victim]
                continue
            m.commit(name, new_len)
            live[name] = new_len
            # every position the next token can see has a page; nothing older is held
            first_visible = max(0, new_len - window + 1)
            table = m.table(name, wname)
            for pos in range(first_visible, new_len):
                assert table[pos // page_size] >= 0
            for i in range(first_visible // page_size):
                assert table[i] == -1
            assert all(p >= 0 for p in m.table(name, "full")[: -(-new_len // page_size)])
        m.check()
    for name in list(live):
        m.release(name)
    m.check()
    assert all(free == g.pool.num_pages for free, g in zip(m.free_pages().values(), m.groups.values()))


def test_block_table_grows_and_forgets_what_a_window_passed():
    """The array behind a table doubles as it grows; passing pages returns each
    page once and looks only at entries that were not passed before."""
    import numpy as np

    from rvllm_amd.cache.pages import BlockTable

    t = BlockTable()
    assert len(t) == 0 and t == [] and t.held() == []
    t.extend(range(100, 140))  # beyond the first allocation
    assert len(t) == 40 and t[0] == 100 and t[-1] == 139 and t[38:] == [138, 139]
    assert np.asarray(t).dtype == np.int32 and np.asarray(t).tolist() == list(range(100, 140))
    assert t.pass_up_to(3) == [100, 101, 102] and t.passed == 3
    assert t.pass_up_to(2) == [] and t.pass_up_to(3) == []
    assert t.pass_up_to(5) == [103, 104] and t[:6] == [-1, -1, -1, -1, -1, 105]
    t.extend([7])
    assert t.held() == list(range(105, 140)) + [7]
    assert t.pass_up_to(1000) == list(range(105, 140)) + [7] and t.held() == [] and t.passed == 41
    adopted = BlockTable([-1, -1, 5, 6], passed=2)
    assert adopted.held() == [5, 6] and adopted.pass_up_to(3) == [5]


def test_commit_at_a_long_context_looks_at_new_pages_only():
    """A window group's commit does not walk the whole table each step."""
    m = CacheManager([KVNeed(2, 16, 8)], page_size=4, num_pages={"window8": 8}, max_requests=1)
    m.add_request("r")
    length = 0
    for _ in range(300):
        length += 3
        m.extend("r", length)
        m.commit("r", length)
        m.check()
    table = m.table("r", "window8")
    assert table.passed == m.groups["window8"].first_kept_page(length) and len(table.held()) <= 4
