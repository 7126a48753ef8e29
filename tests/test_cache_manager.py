"""The cache manager (CPU): no page lost, held twice or freed twice, under random orders."""
import random

import numpy as np
import pytest

from photon_infer_amd import CacheError, OutOfPagesError
from photon_infer_amd.cache import CacheManager, PagePool


def test_pool_is_lifo_and_all_or_nothing():
    pool = PagePool(6)
    a = pool.allocate(4)
    assert a == [0, 1, 2, 3] and pool.num_free == 2
    with pytest.raises(OutOfPagesError):
        pool.allocate(3)
    assert pool.num_free == 2                      # nothing was taken
    pool.free([1, 3])
    assert pool.allocate(2) == [3, 1]              # the page given back last comes first


def test_pool_detects_double_free_and_bad_ids():
    pool = PagePool(4)
    a = pool.allocate(2)
    pool.free([a[0]])
    with pytest.raises(CacheError, match="twice"):
        pool.free([a[0]])
    with pytest.raises(CacheError, match="twice"):
        pool.free([a[1], a[1]])
    assert pool.is_allocated(a[1])                 # the failed call changed nothing
    with pytest.raises(CacheError, match="outside"):
        pool.free([17])


def make(windows=(None,), page=4, pages=16, slots=4, max_len=64):
    return CacheManager(list(windows), page, pages, slots, max_len)


def test_pages_on_demand_and_block_table():
    m = make()
    slot = m.admit("a")
    assert m.pages_needed("a", 5) == [2]
    m.reserve("a", 5)
    m.commit("a", 5)
    assert m.length("a") == 5 and m.free_pages() == 14
    assert m.pages_needed("a", 3) == [0] and m.pages_needed("a", 4) == [1]
    row = m.table_rows(0, [slot])[0]
    assert list(row[:2]) == [0, 1] and (row[2:] == -1).all()
    m.check_invariants()
    m.release("a")
    assert m.free_pages() == 16 and m.num_live == 0
    m.check_invariants()


def test_pages_are_used_again_at_once():
    m = make(pages=4)
    m.admit("a"); m.reserve("a", 16); m.commit("a", 16)
    held = set(m.table_rows(0, [m.slot("a")])[0][:4].tolist())
    m.admit("b")
    with pytest.raises(OutOfPagesError):
        m.reserve("b", 1)
    m.release("a")
    m.reserve("b", 9)
    assert set(m.table_rows(0, [m.slot("b")])[0][:3].tolist()) <= held
    m.check_invariants()


def test_errors():
    m = make(slots=2, max_len=8)
    m.admit("a")
    with pytest.raises(CacheError, match="already live"):
        m.admit("a")
    m.admit("b")
    with pytest.raises(CacheError, match="no free slot"):
        m.admit("c")
    with pytest.raises(CacheError, match="not live"):
        m.reserve("zzz", 1)
    with pytest.raises(CacheError, match="limit"):
        m.reserve("a", 9)
    m.reserve("a", 4)
    with pytest.raises(CacheError, match="held for"):
        m.commit("a", 5)
    m.release("a")
    with pytest.raises(CacheError, match="not live"):
        m.release("a")
    m.check_invariants()


def test_reserve_is_all_or_nothing_across_groups():
    m = CacheManager([None, 8], 4, [16, 2], 4, 64)
    m.admit("a")
    with pytest.raises(OutOfPagesError, match="group 1"):
        m.reserve("a", 12)                 # group 1 has 2 pages, 3 needed
    assert m.free_pages(0) == 16 and m.free_pages(1) == 2
    m.check_invariants()


def test_window_group_gives_pages_back_when_the_window_has_passed():
    W, page = 6, 4
    m = CacheManager([None, W], page, [32, 32], 2, 128)
    s = m.admit("a")
    length = 0
    for n in [5, 1, 1, 7, 1, 1, 1, 2, 9, 1]:
        m.reserve("a", n)
        # every key a query of this step may read is still there
        first_key = max(0, length - W + 1)
        row = m.table_rows(1, [s])[0]
        assert (row[first_key // page: -(-(length + n) // page)] >= 0).all()
        m.commit("a", n)
        length += n
        first_needed = max(0, length - W + 1) // page
        row = m.table_rows(1, [s])[0]
        assert (row[:first_needed] == -1).all()                    # passed pages are gone
        assert (m.table_rows(0, [s])[0][: -(-length // page)] >= 0).all()   # the full group keeps all
        assert 32 - m.free_pages(1) == -(-length // page) - first_needed
        m.check_invariants()
    m.release("a")
    assert m.free_pages(0) == 32 and m.free_pages(1) == 32


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_never_lose_or_double_a_page(seed):
    rng = random.Random(seed)
    m = CacheManager([None, 5], 4, [24, 12], 4, 96)
    live, lengths = [], {}
    nxt = 0
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and m.free_slots:
            rid = f"r{nxt}"; nxt += 1
            m.admit(rid); live.append(rid); lengths[rid] = 0
        elif op < 0.85 and live:
            rid = rng.choice(live)
            n = rng.choice([1, 1, 1, 2, 3, 7, 16])
            if lengths[rid] + n > 96:
                continue
            if m.can_reserve(rid, n):
                m.reserve(rid, n); m.commit(rid, n); lengths[rid] += n
            else:
                with pytest.raises(OutOfPagesError):
                    m.reserve(rid, n)
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            m.release(rid); del lengths[rid]
        m.check_invariants()
        for rid in live:
            assert m.length(rid) == lengths[rid]
    for rid in live:
        m.release(rid)
    m.check_invariants()
    assert m.free_pages(0) == 24 and m.free_pages(1) == 12 and m.free_slots == 4


def test_native_cache_manager_under_address_and_undefined_sanitizers(tmp_path):
    """The host-side C++ of the cache manager, compiled whole with a random workload
    (tests/cpp/cache_sanitize.cpp) under -fsanitize=address,undefined and run on the CPU: any
    out-of-bounds access, use after free, leak or undefined operation ends it with a report."""
    import os
    import subprocess

    from photon_infer_amd.errors import KernelLibraryMissing
    from photon_infer_amd.ops import build

    driver = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "cache_sanitize.cpp")
    try:
        exe = build.build_host_program([driver, "runtime/cache.cpp"], str(tmp_path / "cache_sanitize"), "address,undefined")
    except KernelLibraryMissing as e:
        if "sanitize" in str(e) or "asan" in str(e) or "ubsan" in str(e):
            pytest.skip(f"this compiler has no sanitizer runtimes: {e}")
        raise
    env = dict(os.environ)
    # the environment is left as it is: where it preloads libraries of its own, the sanitizer's
    # runtime is not the first in the list, which it is told to accept
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0:verify_asan_link_order=0"
    r = subprocess.run([exe, "60"], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.strip() == "ok 60 seeds"
