"""The cache manager on the host: no page lost, held twice or freed twice,
under random orders of requests; lowest-free allocation; windows; rollback."""
import random

import pytest

from imparo_amd.cache import (PagePool, CacheManager, PagedSpec, PagedArray, PAGE, FixedSpec, OutOfPages, CacheError,
                              kv_spec)


def test_lowest_free_page_always():
    # the reference's sequence (/root/reference/crates/imparo-kv/src/alloc.rs:147-276):
    # 0,1,2,3; free 2 and 0; next 0, 2, 4
    p = PagePool(8)
    assert [p.alloc() for _ in range(4)] == [0, 1, 2, 3]
    p.free(2)
    p.free(0)
    assert [p.alloc() for _ in range(3)] == [0, 2, 4]
    assert p.high_water == 5


def test_ascending_after_churn_and_purity():
    rng = random.Random(0)
    p = PagePool(64)
    held = set()
    for _ in range(2000):
        if held and (rng.random() < 0.5 or p.n_free == 0):
            page = rng.choice(sorted(held))
            p.free(page)
            held.remove(page)
        else:
            page = p.alloc()
            assert page == min(set(range(64)) - held)      # a function of the free set only
            held.add(page)
    for page in sorted(held):
        p.free(page)
    assert [p.alloc() for _ in range(64)] == list(range(64))


def test_double_free_and_exhaustion():
    p = PagePool(2)
    a = p.alloc()
    p.alloc()
    with pytest.raises(OutOfPages):
        p.alloc()
    p.free(a)
    with pytest.raises(CacheError, match="freed twice"):
        p.free(a)
    with pytest.raises(CacheError):
        p.free(9)


def test_scrambled_placement_is_a_permutation():
    p = PagePool(16)
    p.scramble(3)
    got = [p.alloc() for _ in range(16)]
    assert sorted(got) == list(range(16)) and got != list(range(16))
    p.free(got[5])
    assert p.alloc() == got[5]


SITES = [FixedSpec((2, 8)), kv_spec(2, 16), FixedSpec((2, 8)), kv_spec(2, 16), kv_spec(2, 16, window=10), None]


def test_groups_follow_the_specs():
    m = CacheManager(SITES, page_size=4, n_pages=10, n_slots=3)
    assert len(m.groups) == 2
    assert m.groups[0].sites == [1, 3] and m.groups[1].sites == [4]
    assert m.fixed_sites == [0, 2] and m.group_of_site == {1: 0, 3: 0, 4: 1}


def test_reserve_commit_release():
    m = CacheManager(SITES, page_size=4, n_pages=10, n_slots=3)
    assert m.admit("a") == 0 and m.admit("b") == 1
    m.reserve("a", 9)
    m.commit("a", 9)
    assert m.table(0, "a") == [0, 1, 2] and m.length["a"] == 9
    m.reserve("b", 4)
    m.commit("b", 4)
    assert m.table(0, "b") == [3]
    m.reserve("a", 10)           # still inside page 2
    m.commit("a", 10)
    assert m.table(0, "a") == [0, 1, 2]
    m.release("a")
    assert m.free_pages()[0] == 9
    assert m.admit("c") == 0      # slot reused
    m.reserve("c", 5)
    assert m.table(0, "c") == [0, 1]    # pages reused, lowest first
    m.check()
    with pytest.raises(CacheError):
        m.release("zzz")
    with pytest.raises(CacheError):
        m.admit("b")


def test_reserve_is_all_or_nothing():
    m = CacheManager(SITES, page_size=4, n_pages=4, n_slots=2)
    m.admit("a")
    m.reserve("a", 8)
    m.commit("a", 8)
    m.admit("b")
    before = (m.free_pages(), list(m.table(0, "b")), list(m.table(1, "b")))
    with pytest.raises(OutOfPages):
        m.reserve("b", 12)       # needs 3 pages, 2 are free
    assert (m.free_pages(), m.table(0, "b"), m.table(1, "b")) == before
    got = m.reserve("b", 8)
    m.rollback("b", got)
    assert (m.free_pages(), m.table(0, "b"), m.table(1, "b")) == before
    m.check()


def test_slots_run_out():
    m = CacheManager(SITES, page_size=4, n_pages=4, n_slots=1)
    m.admit("a")
    with pytest.raises(OutOfPages, match="slots"):
        m.admit("b")


def test_a_window_gives_pages_back_as_it_passes_them():
    m = CacheManager([kv_spec(1, 16, window=10), kv_spec(1, 16)], page_size=4, n_pages=64, n_slots=1)
    m.admit("a")
    for n in range(1, 41):
        m.reserve("a", n)
        m.commit("a", n)
        win, full = m.table(0, "a"), m.table(1, "a")
        # the next query sits at position n and reads keys n+1-10 .. n
        lo = max(0, n + 1 - 10)
        for idx, page in enumerate(win):
            needed = (idx + 1) * 4 > lo
            assert (page >= 0) == needed, (n, idx, win)
        assert all(p >= 0 for p in full)
        assert m.held_pages("a")[0] <= 10 // 4 + 2
        m.check()
    # a long portion keeps what its own first query needs
    m.release("a")
    m.admit("b")
    m.reserve("b", 30)
    assert all(p >= 0 for p in m.table(0, "b"))
    m.commit("b", 30)
    assert m.table(0, "b")[:5] == [-1] * 5      # keys below 21 are behind the window of position 30
    m.reserve("b", 50)
    assert m.table(0, "b")[5] >= 0


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_never_lose_or_share_a_page(seed):
    rng = random.Random(seed)
    m = CacheManager(SITES, page_size=4, n_pages=24, n_slots=4)
    live = {}
    next_id = 0
    for _ in range(1500):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            rid = f"r{next_id}"
            next_id += 1
            m.admit(rid)
            live[rid] = 0
        elif action < 0.85 and live:
            rid = rng.choice(sorted(live))
            grow = rng.choice([1, 1, 1, 2, 7, 19])
            try:
                got = m.reserve(rid, live[rid] + grow)
            except OutOfPages:
                m.check()
                continue
            if rng.random() < 0.1:
                m.rollback(rid, got)
            else:
                live[rid] += grow
                m.commit(rid, live[rid])
        elif live:
            rid = rng.choice(sorted(live))
            m.release(rid)
            del live[rid]
        m.check()
        for rid, n in live.items():
            assert m.length[rid] == n
            assert len(m.table(0, rid)) == (n + 3) // 4 or len(m.table(0, rid)) >= (n + 3) // 4
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.free_pages() == [24, 24] and m.slots.n_free == 4


def test_pack_lays_out_a_step():
    """The native packer: tokens | positions | row_of_token | seg_start | seg_len | slot | row lists |
    want | tables, positions counted from each request's length before the step."""
    m = CacheManager([kv_spec(1, 16), FixedSpec((4,)), kv_spec(1, 16, window=6)], page_size=4, n_pages=16, n_slots=4)
    m.admit("a"), m.admit("b"), m.admit("c")
    m.reserve("a", 9), m.commit("a", 9)
    m.reserve("a", 10), m.reserve("b", 3), m.reserve("c", 1)
    arr, lay = m.pack(["a", "b", "c"], [[7], [1, 2, 3], [4]], [[0], [2, 0], []])
    T, R, W, G, P = (lay[k] for k in "TRWGP")
    assert (T, R, W, G) == (5, 3, 3, 2) and P == 3 and lay["n_single"] == 2 and lay["n_multi"] == 1
    assert lay["max_seg_len"] == 3 and lay["max_context"] == 10
    a = arr.tolist()
    assert a[0:5] == [7, 1, 2, 3, 4]                      # tokens
    assert a[5:10] == [9, 0, 1, 2, 0]                     # positions
    assert a[10:15] == [0, 1, 1, 1, 2]                    # row of token
    assert a[15:18] == [0, 1, 4] and a[18:21] == [1, 3, 1] and a[21:24] == [0, 1, 2]   # start, len, slot
    assert a[24:27] == [0, 2, 1]                          # rows with one token, then the others
    assert a[27:30] == [0, 3, 1]                          # wanted places as indices into the batch
    tables = arr[30:].reshape(G, R, P).tolist()
    assert tables[0] == [m.table(0, "a"), m.table(0, "b") + [-1, -1], m.table(0, "c") + [-1, -1]]
    assert tables[1][0] == m.table(1, "a") and tables[1][0][0] == -1      # behind the window of 6 at length 9
    fixed, lay2 = m.pack(["a"], [[7]], [[0]], table_width=8)
    assert lay2["P"] == 8 and fixed[-8:].tolist() == m.table(1, "a") + [-1] * 5
    with pytest.raises(CacheError):
        m.pack(["zzz"], [[1]], [[0]])


def snapshot(m, names):
    return (m.free_pages(), m.slots.n_free, sorted(n for n in names if m.is_live(n)),
            {n: [m.table(g, n) for g in range(len(m.groups))] for n in names if m.is_live(n)},
            {n: m.length[n] for n in names if m.is_live(n)})


def test_a_whole_step_is_booked_in_one_call():
    """begin_step admits, reserves and checks for the whole batch; end_step commits it. The
    result is what admit/reserve/commit give one request at a time."""
    from imparo_amd.cache import native as N
    specs = [kv_spec(1, 16), FixedSpec((4,)), kv_spec(1, 16, window=6)]
    m = CacheManager(specs, page_size=4, n_pages=16, n_slots=3)
    one = CacheManager(specs, page_size=4, n_pages=16, n_slots=3)
    steps = [(["a", "b"], [[1] * 9, [2] * 3]), (["b", "a", "c"], [[5], [6, 7], [8] * 5]), (["c", "a"], [[1], [2]])]
    for names, toks in steps:
        b = m.batch(names, toks, [[0]] * len(names))
        assert m.begin_step(b, vocab=10, max_position=64) == (0, -1)
        new = [n for n, s in zip(names, b.new_slots.tolist()) if s >= 0]
        for n, t in zip(names, toks):
            if not one.is_live(n):
                assert n in new and one.admit(n) == int(b.new_slots[names.index(n)])
            else:
                assert n not in new
            one.reserve(n, one.length[n] + len(t))
        assert b.widest == max(len(one.table(g, n)) for n in names for g in range(2))
        arr, lay = m.pack_batch(b)
        arr1, lay1 = one.pack(names, toks, [[0]] * len(names))
        assert lay == lay1 and arr.tolist() == arr1.tolist()
        m.end_step(b)
        for n, t in zip(names, toks):
            one.commit(n, one.length[n] + len(t))
        assert snapshot(m, "abc") == snapshot(one, "abc")
        m.check()
    # what is wrong with a batch is said before anything is touched
    before = snapshot(m, "abcd")
    for names, toks, want, code, row in (
            (["a", "d", "a"], [[1], [1], [1]], [[0], [0], [0]], N.E_TWICE, 2),
            (["a", "d"], [[1], []], [[0], []], N.E_EMPTY, 1),
            (["d", "a"], [[1], [1] * 60], [[0], [0]], N.E_POSITIONS, 1),
            (["d", "a"], [[1, 10], [1]], [[0], [0]], N.E_TOKEN, 0),
            (["d", "a"], [[1, -1], [1]], [[0], [0]], N.E_TOKEN, 0),
            (["d", "a"], [[1], [1, 2]], [[0], [2]], N.E_WANT, 1)):
        assert m.begin_step(m.batch(names, toks, want), vocab=10, max_position=64) == (code, row)
        assert snapshot(m, "abcd") == before
    with pytest.raises(CacheError, match="32 bits"):
        m.batch(["a"], [[2 ** 40]], [[0]])


def test_a_step_that_does_not_fit_changes_nothing():
    m = CacheManager([kv_spec(1, 16), kv_spec(1, 16, window=6)], page_size=4, n_pages=6, n_slots=2)
    b = m.batch(["a"], [[1] * 10], [[9]])
    assert m.begin_step(b, 10, 64) == (0, -1)
    m.end_step(b)
    before = snapshot(m, "abc")
    # a's 6 more fit (1 page of 3 free), new b's 12 do not: neither advances, b is not admitted
    with pytest.raises(OutOfPages, match="pages"):
        m.begin_step(m.batch(["a", "b"], [[1] * 6, [1] * 12], [[0], [0]]), 10, 64)
    assert snapshot(m, "abc") == before
    # slots: b fits, c finds no slot; b leaves again
    with pytest.raises(OutOfPages, match="slots"):
        m.begin_step(m.batch(["b", "c", "a"], [[1], [1], [1]], [[0], [0], [0]]), 10, 64)
    assert snapshot(m, "abc") == before
    # a step that was booked and then did not run
    b = m.batch(["a", "b"], [[1] * 3, [1] * 4], [[0], [0]])
    assert m.begin_step(b, 10, 64) == (0, -1)
    assert m.is_live("b") and snapshot(m, "abc") != before
    m.abort_step(b)
    assert snapshot(m, "abc") == before
    m.check()


# ---- what a paged site keeps is the mixer's to declare; pools are sized per group
def test_a_paged_spec_names_its_arrays_and_their_page_layout():
    spec = kv_spec(2, 16, window=10, v_transposed=True)
    assert [a.name for a in spec.arrays] == ["k", "v"]
    assert spec.arrays[0].shape(5, 8) == (5, 2, 8, 16) and spec.arrays[1].shape(5, 8) == (5, 2, 16, 8)
    assert spec.bytes_per_position(2) == 2 * 2 * 16 * 2
    # a latent of 24 values a position in float32 beside a narrow key: no K/V pair of one shape
    other = PagedSpec((PagedArray("latent", (PAGE, 24), float32=True), PagedArray("key", (1, PAGE, 8))))
    assert other.bytes_per_position(2) == 24 * 4 + 8 * 2
    assert other != spec and other == PagedSpec(other.arrays)
    with pytest.raises(ValueError, match="twice"):
        PagedSpec((PagedArray("a", (PAGE, 4)), PagedArray("a", (PAGE, 2))))
    with pytest.raises(ValueError, match="positions"):
        PagedSpec((PagedArray("a", (4, 4)),))


def test_every_group_has_a_pool_of_its_own_size():
    specs = [kv_spec(1, 16), FixedSpec((4,)), kv_spec(1, 16, window=6), kv_spec(1, 16)]
    groups = CacheManager.groups_of(specs)
    assert [(s.window, sites) for s, sites in groups] == [(None, [0, 3]), (6, [2])]
    m = CacheManager(specs, page_size=4, n_pages=[10, 3], n_slots=2)
    assert [g.pool.n_pages for g in m.groups] == [10, 3]
    m.admit("a")
    m.reserve("a", 11)                 # 3 pages in both groups
    m.commit("a", 11)                  # the window's group gives one back
    assert m.free_pages() == [7, 1]
    with pytest.raises(OutOfPages):    # 5 more pages: the small pool cannot, and the large one keeps its pages
        m.reserve("a", 31)
    assert m.free_pages() == [7, 1]
    m.check()
    with pytest.raises(ValueError, match="pool sizes"):
        CacheManager(specs, page_size=4, n_pages=[10], n_slots=2)


def test_pool_sizes_from_a_budget_in_bytes():
    from imparo_amd.engine import Engine
    import torch
    specs = [FixedSpec((2, 64)), kv_spec(8, 64), None, kv_spec(8, 64), kv_spec(8, 64, window=128)]
    # a page of 64 positions: 2 * 8 * 64 values per position and site, 2 bytes each, three sites in two groups
    per_page = 64 * (2 * 8 * 64 * 2) * 3
    assert Engine.pool_sizes(specs, 64, torch.bfloat16, None, 10 * per_page + 5, None) == [10, 10]
    assert Engine.pool_sizes(specs, 64, torch.float32, None, 10 * per_page, None) == [5, 5]
    assert Engine.pool_sizes(specs, 64, torch.bfloat16, 1000, None, None) == [16, 16]
    assert Engine.pool_sizes(specs, 64, torch.bfloat16, None, None, 7) == [7, 7]
    assert Engine.pool_sizes(specs, 64, torch.bfloat16, None, None, [7, 3]) == [7, 3]
    with pytest.raises(ValueError, match="one page"):
        Engine.pool_sizes(specs, 64, torch.bfloat16, None, per_page - 1, None)
    with pytest.raises(ValueError, match="num_pages"):
        Engine.pool_sizes(specs, 64, torch.bfloat16, None, None, [7])


def test_fixed_specs_name_one_array_or_several():
    from imparo_amd.cache import FixedArray, FixedSpec
    one = FixedSpec((2, 64), 0.5)
    assert one.all_arrays() == (FixedArray("state", (2, 64), "float32", 0.5),)
    two = FixedSpec(arrays=(FixedArray("r", (4, 4)), FixedArray("s", (8,), "bfloat16")))
    assert [a.name for a in two.all_arrays()] == ["r", "s"] and two != one
    with pytest.raises(ValueError, match="either one float32 array"):
        FixedSpec()
    with pytest.raises(ValueError, match="either one float32 array"):
        FixedSpec((3,), arrays=(FixedArray("r", (3,)),))
    with pytest.raises(ValueError, match="twice"):
        FixedSpec(arrays=(FixedArray("r", (3,)), FixedArray("r", (4,))))
    with pytest.raises(ValueError, match="other than zero"):
        FixedArray("s", (8,), "bfloat16", init=1.0)
    with pytest.raises(ValueError, match="dtype"):
        FixedArray("s", (8,), "float16")
