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


def test_filling_a_step_does_not_grow_with_the_contexts():
    """64 requests that decode: what the host does to describe the step is the same at 2,000 and at 32,000
    cached tokens a request, since the block tables live on the device and only changed entries travel."""
    import time

    import numpy as np

    from distie_amd.cache import CacheManager
    from distie_amd.engine.batch import BatchBuilder
    from distie_amd.parts import PagedKV

    def seconds(context):
        cache = CacheManager([PagedKV(1, 16), PagedKV(1, 16, 4096)], 16, 64 * (context // 16 + 2), 64, device="cpu",
                             allocate=False)
        builder = BatchBuilder(cache, 40000, "cpu", 100)
        entries = []
        for r in range(64):
            cache.add(r)
            cache.reserve(r, context)
            cache.commit(r, context)
            cache.reserve(r, 1)
            entries.append(StepEntry(r, [1], [0]))
        builder.flush_tables()
        host = np.empty(int(builder.layout(64, 64, 64)[-1]), dtype=np.int32)
        best = 1e9
        for _ in range(5):
            began = time.perf_counter()
            for _ in range(20):
                builder.fill(host, entries)
                builder.flush_tables()
            best = min(best, time.perf_counter() - began)
        return best

    short, long = seconds(2000), seconds(32000)
    assert long < 1.5 * short + 1e-3, (short, long)
