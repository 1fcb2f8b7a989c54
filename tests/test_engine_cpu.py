"""The engine's logic (batching, cache groups, windows, page reuse) on the CPU test double,
against the plain implementation."""

import pytest
import torch

import plain_qwen2 as plain
from distie_amd.engine.batch import StepEntry
from engine_util import FP32_TOL, oracle, build_runner, make_model_dir, random_ids, replay_cut, replay_whole
from torch_ops import TorchOps

CONFIGS = {"A": (plain.TINY_A, 4), "B": (plain.TINY_B, 8), "C": (plain.TINY_C, 16)}


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def setup(request, tmp_path_factory):
    cfg, block = CONFIGS[request.param]
    folder, weights = make_model_dir(tmp_path_factory.mktemp("m" + request.param), cfg, seed=11)
    return cfg, block, folder, weights


def test_whole_prompt(setup):
    cfg, block, folder, weights = setup
    runner = build_runner(folder, TorchOps(), block_size=block)
    ids = random_ids(cfg, 45, 1)
    want = oracle(weights, cfg, ids)
    got = replay_whole(runner, "a", ids)
    assert (got - want).abs().max() < FP32_TOL
    runner.cache.check()
    assert all(f == runner.cache.num_blocks for f in runner.cache.free_pages())


@pytest.mark.parametrize("cuts", [[13], [2, 3, 5, 7, 2, 11, 4], [40, 2, 2], [1, 1, 1, 30]])
def test_cuttings(setup, cuts):
    cfg, block, folder, weights = setup
    runner = build_runner(folder, TorchOps(), block_size=block)
    ids = random_ids(cfg, 50, 2)
    want = oracle(weights, cfg, ids)
    got = replay_cut(runner, "a", ids, cuts)
    assert (got - want).abs().max() < FP32_TOL
    runner.cache.check()


def test_mixed_batches_with_page_reuse(setup):
    cfg, block, folder, weights = setup
    lengths = [37, 50, 21, 44, 30, 26]
    # enough pages for four live requests, so pages are used again by later ones
    pages = sum(-(-n // block) for n in sorted(lengths)[-4:])
    runner = build_runner(folder, TorchOps(), block_size=block, num_blocks=pages, num_slots=4)
    reqs = {f"r{i}": random_ids(cfg, n, 10 + i) for i, n in enumerate(lengths)}
    want = {r: oracle(weights, cfg, ids) for r, ids in reqs.items()}
    got = {r: [] for r in reqs}
    at = {r: 0 for r in reqs}
    waiting = list(reqs)
    live = []
    gen = torch.Generator().manual_seed(5)
    step = 0
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries = []
        for r in live:
            left = len(reqs[r]) - at[r]
            decode = left <= 6
            n = 1 if decode else min(left, int(torch.randint(2, 9, (1,), generator=gen)))
            if step % 3 == 2 and r == live[0] and len(live) > 1:
                continue  # a request may sit out a step
            entries.append(StepEntry(r, reqs[r][at[r]:at[r] + n], list(range(n))))
        logits = runner.step(entries)
        row = 0
        for e in entries:
            n = len(e.tokens)
            got[e.request_id].append(logits[row:row + n])
            row += n
            at[e.request_id] += n
        for r in list(live):
            if at[r] == len(reqs[r]):
                runner.finish(r)
                live.remove(r)
        runner.cache.check()
        step += 1
    for r in reqs:
        assert (torch.cat(got[r]).float() - want[r]).abs().max() < FP32_TOL, r
    assert all(f == pages for f in runner.cache.free_pages())


def test_window_pages_are_given_back_and_never_read(tmp_path):
    cfg = plain.TINY_B
    folder, weights = make_model_dir(tmp_path, cfg, seed=3)
    runner = build_runner(folder, TorchOps(), block_size=4, num_blocks=16)
    ids = random_ids(cfg, 60, 4)
    want = oracle(weights, cfg, ids)
    got = replay_cut(runner, "a", ids, [9, 5, 2, 17])
    assert (got - want).abs().max() < FP32_TOL
    runner2 = build_runner(folder, TorchOps(), block_size=4, num_blocks=16)
    runner2.step([StepEntry("x", ids[:30], [])])
    entry = runner2.cache.request("x")
    full, windowed = entry.tables
    assert all(p >= 0 for p in full) and len(full) == 8
    # window 8, 30 cached: the next query (position 30) reads keys 23..30 -> pages 5.. stay
    assert [p >= 0 for p in windowed] == [False] * 5 + [True] * 3
    assert runner2.cache.free_pages() == [8, 13]


def test_wanted_rows_and_empty_want(setup):
    cfg, block, folder, weights = setup
    runner = build_runner(folder, TorchOps(), block_size=block)
    a, b = random_ids(cfg, 9, 7), random_ids(cfg, 12, 8)
    assert runner.step([StepEntry("a", a[:5], []), StepEntry("b", b[:7], [])]) is None
    logits = runner.step([StepEntry("a", a[5:], [3, 0]), StepEntry("b", b[7:], [4])])
    wa, wb = oracle(weights, cfg, a), oracle(weights, cfg, b)
    assert (logits[0] - wa[8]).abs().max() < FP32_TOL
    assert (logits[1] - wa[5]).abs().max() < FP32_TOL
    assert (logits[2] - wb[11]).abs().max() < FP32_TOL


class _CountingTable(list):
    """A request's block table that counts the entries anyone looks at."""

    touched = 0

    def __getitem__(self, key):
        got = super().__getitem__(key)
        _CountingTable.touched += len(got) if isinstance(key, slice) else 1
        return got

    def __iter__(self):
        _CountingTable.touched += len(self)
        return super().__iter__()


def test_filling_a_step_does_not_grow_with_the_contexts():
    """64 requests, decoding or with a portion of 40 tokens: what the host looks at to describe the step is the
    same at 2,000 and at 32,000 cached tokens a request, since the block tables live on the device and only
    changed entries travel. Counted in table entries touched and entries sent, not in seconds."""
    import numpy as np

    from distie_amd.cache import CacheManager
    from distie_amd.engine.batch import BatchBuilder
    from distie_amd.parts import PagedKV

    def work(context, new):
        cache = CacheManager([PagedKV(1, 16), PagedKV(1, 16, 4096)], 16, 64 * (context // 16 + 8), 64, device="cpu",
                             allocate=False)
        builder = BatchBuilder(cache, 40000, "cpu", 100)
        entries = []
        for r in range(64):
            cache.add(r)
            cache.reserve(r, context)
            cache.commit(r, context)
            entries.append(StepEntry(r, [1] * new, [0]))
        builder.flush_tables()
        for r in range(64):
            cache.reserve(r, new)
            state = cache.request(r)
            state.tables = [_CountingTable(t) for t in state.tables]
        host = np.empty(int(builder.layout(64 * new, 64, 64)[-1]), dtype=np.int32)
        sent = sum(len(cache.groups[g].changed) for g in range(2))
        _CountingTable.touched = 0
        builder.fill(host, entries)
        builder.flush_tables()
        return _CountingTable.touched, sent

    for new in (1, 40):
        short, long = work(2000 - 8, new), work(32000 - 8, new)
        assert short == long, (new, short, long)
        touched, sent = short
        assert touched <= 64 * 2 * (new // 16 + 2) and sent <= 64 * 2 * (new // 16 + 1)


def test_the_fields_of_a_step_as_numbers():
    """The reference's vector of its batch description (worker/tests/test_qwen2_batch.py:50-59): two requests
    at pages of 4 tokens, "a" with 2 new tokens behind none in pages [3, 0], "b" with 1 new token behind 5
    in pages [1, 5] -> positions [0, 1, 5], slots [12, 13, 21], prefix sums [0, 2, 3], tables [[3, 0], [1, 5]],
    last rows [1, 2], longest portion 2, longest context 6. Here the cached lengths travel as they are
    ([2, 6]; the reference sends their prefix sums [0, 2, 8]) and the tables are rows of the device table
    named by each request's state slot."""
    import numpy as np

    from distie_amd.cache import CacheManager
    from distie_amd.engine.batch import BatchBuilder
    from distie_amd.parts import PagedKV

    cache = CacheManager([PagedKV(2, 8), PagedKV(2, 8)], 4, 8, 4, device="cpu")
    builder = BatchBuilder(cache, 16, "cpu", 100)
    assert builder.table_width == 4
    (group,) = cache.groups
    held = group.pool.allocate(8)                       # every page is taken, so the chosen ones are held
    group.pool.free([p for p in held if p not in (3, 0, 1, 5)])
    a, b = cache.add("a"), cache.add("b")
    for entry, pages, cached in ((a, [3, 0], 0), (b, [1, 5], 5)):
        entry.tables[0] = list(pages)
        entry.num_cached = cached
        for i, page in enumerate(pages):
            cache._note(group, entry.slot, i, page)
    cache.check()
    entries = [StepEntry("a", [7, 8], [1]), StepEntry("b", [9], [0])]
    host = np.full(64, -7, dtype=np.int32)
    offsets, T, B, R, max_q, max_kv, cu_q, past = builder.fill(host, entries)
    assert (T, B, R, max_q, max_kv) == (3, 2, 2, 2, 6)
    field = lambda i: host[offsets[i]:offsets[i + 1]].tolist()
    assert field(0) == [7, 8, 9]                        # token ids
    assert field(1) == [0, 1, 5]                        # positions
    assert field(2) == [0, 0, 1]                        # request of each token
    assert field(3) == [0, 2, 3]                        # prefix sums of the new tokens
    assert field(4) == [2, 6]                           # cached after the step
    assert field(5) == [a.slot, b.slot]                 # state slots = rows of the device tables
    assert field(6) == [1, 2]                           # rows whose logits are wanted: the last of each
    assert field(7) == [12, 13, 21]                     # page * 4 + place in the page
    assert cu_q.tolist() == [0, 2, 3] and past.tolist() == [0, 5]
    assert int(offsets[-1]) == 3 * 3 + 3 + 2 + 2 + 2 + 3
    # the device tables: the changed entries go along, rows by state slot, -1 where nothing is held
    ids, meta, want = builder.build(entries)
    table = meta.groups[0].block_table
    assert table[a.slot].tolist() == [3, 0, -1, -1] and table[b.slot].tolist() == [1, 5, -1, -1]
    assert table[cache.sink_slot, 0] == group.sink_page == 8
    assert meta.table_rows.tolist() == [a.slot, b.slot] and want.tolist() == [1, 2]
    assert meta.positions.tolist() == [0, 1, 5] and meta.groups[0].slots.tolist() == [12, 13, 21]
    assert (meta.max_q, meta.max_kv, meta.all_decode) == (2, 6, False)
    # two rows of padding, as a captured step of four would have: position 0 of the sink page and slot
    offsets, T, B, R, *_ = builder.fill(host, [StepEntry("b", [9], [0])], pad_requests=2, want_all=True)
    field = lambda i: host[offsets[i]:offsets[i + 1]].tolist()
    assert (T, B, R) == (3, 3, 3)
    assert field(1) == [5, 0, 0] and field(3) == [0, 1, 2, 3] and field(4) == [6, 1, 1]
    assert field(5) == [b.slot, 4, 4] and field(6) == [0, 1, 2] and field(7) == [21, 32, 32]
    # a mixed step padded to 8 tokens and 4 requests, the last row of every request wanted: the first padding
    # request takes the tokens that are left, at positions 0.. of the sink page
    b.tables[0] = [1, 5]
    offsets, T, B, R, max_q, max_kv, *_ = builder.fill(host, [StepEntry("b", [9], [0]), StepEntry("a", [7, 8], [])],
                                                       pad_requests=2, pad_tokens=3, want_last=True)
    field = lambda i: host[offsets[i]:offsets[i + 1]].tolist()
    assert (T, B, R, max_q, max_kv) == (8, 4, 4, 4, 6)
    assert field(1) == [5, 0, 1, 0, 1, 2, 3, 0] and field(2) == [0, 1, 1, 2, 2, 2, 2, 3]
    assert field(3) == [0, 1, 3, 7, 8] and field(4) == [6, 2, 4, 1] and field(5) == [b.slot, a.slot, 4, 4]
    assert field(6) == [0, 2, 6, 7] and field(7) == [21, 12, 13, 32, 33, 34, 35, 32]
    with pytest.raises(ValueError):
        builder.fill(host, [StepEntry("b", [9], [0])], pad_tokens=2)
    # what the reference refuses (test_qwen2_batch.py:61-68): a table too short for the new tokens, an empty step
    b.tables[0] = [1]
    with pytest.raises(ValueError):
        builder.fill(host, [StepEntry("b", [9], [0])])
    with pytest.raises(ValueError):
        builder.fill(host, [])
