"""The cache manager: pages and slots are never lost, held twice or freed twice, under
random orders of requests; windows give pages back; the pool's contract."""

import random

import pytest
import torch

from distie_amd.cache import GONE, BlockPool, CacheManager, OutOfBlocks, pages_needed
from distie_amd.parts import FixedState, PagedKV


def test_pages_needed_vectors():
    # worker/tests/test_kv_cache.py:43-50
    assert [pages_needed(n, 16) for n in (0, 1, 16, 17)] == [0, 1, 1, 2]
    with pytest.raises(ValueError):
        pages_needed(1, 0)


def test_pool_contract():
    # core/tests/test_block_pool.py:15-35, core/tests/test_block_pool.cpp:16-65
    pool = BlockPool(4)
    assert pool.allocate(3) == [0, 1, 2]
    assert pool.utilization == 0.75 and pool.num_free == 1 and pool.num_used == 3
    with pytest.raises(RuntimeError):
        pool.allocate(2)                       # all or nothing
    assert pool.num_free == 1
    pool.free([1])
    assert pool.allocate(1) == [1]             # the id given back last goes out first
    for bad in ([5], [-1], [3], [0, 0]):
        with pytest.raises(ValueError):
            pool.free(bad)
        assert pool.num_used == 3              # an invalid free changes nothing
    with pytest.raises(ValueError):
        pool.free([2, 9])
    assert pool.is_held(2)
    pool.free([0, 1, 2])
    with pytest.raises(ValueError):
        pool.free([0])                         # double free
    with pytest.raises(ValueError):
        BlockPool(0)


def test_pool_threads():
    import threading

    pool = BlockPool(64)
    errors = []

    def work():
        try:
            for _ in range(500):
                try:
                    ids = pool.allocate(3)
                except RuntimeError:
                    continue
                pool.free(ids)
        except Exception as exc:  # noqa: BLE001
            errors.append(exc)

    threads = [threading.Thread(target=work) for _ in range(8)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errors and pool.num_free == 64


@pytest.mark.parametrize("sanitizers", ["address,undefined", "thread"])
def test_pool_under_sanitizers(tmp_path, sanitizers):
    """The C++ id pool, driven from eight threads through its C interface (tests/pool_driver.cpp), built with
    the host compiler's sanitizers: no report, exit status 0."""
    import os
    import shutil
    import subprocess
    from pathlib import Path

    compiler = shutil.which(os.environ.get("CXX", "g++"))
    if compiler is None:
        pytest.skip("no host compiler")
    here = Path(__file__).resolve().parent
    source = here.parent / "distie_amd" / "csrc" / "block_pool.cpp"
    binary = tmp_path / "pool_driver"
    static = ["-static-libasan"] if "address" in sanitizers else ["-static-libtsan"]
    build = subprocess.run([compiler, "-std=c++17", "-O1", "-g", "-pthread", f"-fsanitize={sanitizers}",
                            "-fno-sanitize-recover=all", *static, str(source), str(here / "pool_driver.cpp"),
                            "-o", str(binary)], capture_output=True, text=True)
    if build.returncode != 0 and "sanitize" in build.stderr.lower() + build.stdout.lower():
        pytest.skip("the host compiler has no runtime for these sanitizers")
    assert build.returncode == 0, build.stderr
    run = subprocess.run([str(binary)], capture_output=True, text=True, timeout=120)   # runtimes linked statically
    assert run.returncode == 0 and "pool driver: fine" in run.stdout, run.stdout + run.stderr
    assert "Sanitizer" not in run.stderr, run.stderr


def manager(block=4, pages=12, slots=4, window=6):
    needs = [PagedKV(2, 16), PagedKV(2, 16, window), PagedKV(2, 16), None, FixedState.of((3,))]
    return CacheManager(needs, block, pages, slots, allocate=False)


def test_groups_by_need():
    m = manager()
    assert len(m.groups) == 2
    assert m.groups[0].layers == [0, 2] and m.groups[1].layers == [1]
    assert m.layer(0)["mixer"].group == 0 and m.layer(1)["mixer"].group == 1 and m.layer(3)["mixer"].group == -1


def test_page_bytes_counts_every_layer_and_tensor():
    needs = [PagedKV(2, 16), PagedKV(2, 16, 6), PagedKV(2, 16), None, FixedState.of((3,))]
    m = CacheManager(needs, 4, 12, 4)
    per_page = CacheManager.page_bytes(needs, m.block_size, torch.float32)
    paged = sum(t.numel() * t.element_size() for g in m.groups for t in g.tensors.values())
    assert per_page * (m.num_blocks + 1) == paged
    assert CacheManager.page_bytes(needs, m.block_size, torch.bfloat16) * 2 == per_page
    assert CacheManager.page_bytes([None, FixedState.of((3,))], 4) == 0


def test_reserve_commit_release_and_window():
    m = manager(block=4, pages=12, window=6)
    m.add("a")
    m.reserve("a", 10)
    assert [len(t) for t in m.request("a").tables] == [3, 3]
    m.commit("a", 10)
    # 10 cached, window 6: the next query (position 10) reads keys 5..10 -> page 0 is passed
    assert [p == GONE for p in m.request("a").tables[1]] == [True, False, False]
    assert m.free_pages() == [9, 10]
    m.reserve("a", 1)          # position 10 is in page 2: nothing new
    m.commit("a", 1)
    assert m.free_pages() == [9, 10]
    m.reserve("a", 9)          # positions 11..19 -> pages 2..4
    assert m.free_pages() == [7, 8]
    m.commit("a", 9)           # 20 cached: keys from 15 -> pages 0..2 passed
    assert [p == GONE for p in m.request("a").tables[1]] == [True, True, True, False, False]
    assert m.free_pages() == [7, 10]
    m.check()
    m.release("a")
    assert m.free_pages() == [12, 12] and m.slots.num_free == 4
    with pytest.raises(KeyError):
        m.release("a")


def test_reserve_is_all_or_nothing_across_groups():
    m = manager(block=4, pages=3, window=100)
    m.add("a")
    m.reserve("a", 8)
    m.add("b")
    with pytest.raises(OutOfBlocks):
        m.reserve("b", 5)
    assert m.free_pages() == [1, 1] and m.request("b").tables == [[], []]
    assert not m.can_reserve("b", 5) and m.can_reserve("b", 4)
    m.check()


def test_slots_run_out_and_come_back():
    m = manager(slots=2)
    m.add("a")
    m.add("b")
    with pytest.raises(OutOfBlocks):
        m.add("c")
    with pytest.raises(ValueError):
        m.add("a")
    m.release("a")
    assert m.add("c").slot == 0


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    m = manager(block=rng.choice([2, 4, 8]), pages=rng.randint(10, 30), slots=4, window=rng.randint(1, 20))
    m.device = "cpu"
    m.bind_tables(64)              # the tables as the kernels read them: kept up to date entry by entry

    def tables_follow():
        """After the changed entries went along with a step, a live request's row holds what its list holds,
        wherever a kernel may look (from the first page a query can still read)."""
        for g, group in enumerate(m.groups):
            index, value = m.take_changes(g)
            if index:
                assert len(set(index)) == len(index)
                group.table.view(-1)[torch.tensor(index)] = torch.tensor(value, dtype=torch.int32)
            assert group.table[m.sink_slot, 0] == group.sink_page
            for rid in m.live():
                entry = m.request(rid)
                assert group.table[entry.slot, :len(entry.tables[g])].tolist() == entry.tables[g]

    live = {}
    n = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            rid = f"r{n}"
            n += 1
            m.add(rid)
            live[rid] = 0
        elif action < 0.8 and live:
            rid = rng.choice(list(live))
            count = rng.choice([1, 1, 1, 2, 5, 17])
            if m.can_reserve(rid, count):
                m.reserve(rid, count)
                m.commit(rid, count)
                live[rid] += count
            else:
                with pytest.raises(OutOfBlocks):
                    m.reserve(rid, count)
        elif action < 0.9 and live:
            rid = rng.choice(list(live))
            m.reset(rid)
            live[rid] = 0
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        if rng.random() < 0.3:
            tables_follow()
        for rid, cached in live.items():
            entry = m.request(rid)
            assert entry.num_cached == cached
            full, windowed = entry.tables
            assert len(full) == pages_needed(cached, m.block_size) and GONE not in full
            # every page a query at the next position may read is there
            first = max(0, cached - m.groups[1].requirement.window + 1) // m.block_size
            assert all(p != GONE for p in windowed[first:])
    tables_follow()
    for rid in list(live):
        m.release(rid)
    assert m.free_pages() == [m.num_blocks] * 2 and m.slots.num_free == 4
