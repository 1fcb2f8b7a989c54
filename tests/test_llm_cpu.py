"""The entry point end to end on the CPU test double: greedy generation against the plain
implementation, concurrent == sequential, a tight pool with preemption == a roomy one,
cancel, a failing step, trace (worker/tests/test_batched_engine.py:85-144,
worker/tests/test_torch_engine.py:100-130)."""

import pytest
import torch

import plain_qwen2 as plain
from distie_amd import LLM, SamplingParams
from engine_util import check_generation, make_model_dir, oracle, plain_uniform, random_ids
from torch_ops import TorchOps


def plain_greedy(weights, cfg, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(oracle(weights, cfg, ids)[-1].argmax()))
    return ids[len(prompt):]


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    cfg = plain.TINY_B
    folder, weights = make_model_dir(tmp_path_factory.mktemp("llm"), cfg, seed=21)
    return cfg, folder, weights


def engine(folder, **options):
    options.setdefault("block_size", 8)
    options.setdefault("num_blocks", 64)
    return LLM(folder, dtype="fp32", ops=TorchOps(), **options)


def test_greedy_generation_matches_the_plain_implementation(tiny):
    cfg, folder, weights = tiny
    llm = engine(folder, token_budget=7)      # prompts of 9, 23 and 40 are cut into portions of <= 7
    prompts = [random_ids(cfg, n, 30 + n) for n in (1, 9, 23, 40)]
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=12))
    for prompt, out in zip(prompts, outs):
        assert out.token_ids == plain_greedy(weights, cfg, prompt, 12)
        assert out.finished and out.finish_reason == "length"
        assert out.time_to_first_token_ms > 0 and out.total_latency_ms >= out.time_to_first_token_ms
    llm.cache.check()
    assert llm.cache.free_pages() == [64, 64]


def test_concurrent_equals_sequential_and_a_tight_pool_preempts_yet_agrees(tiny):
    cfg, folder, weights = tiny
    prompts = [random_ids(cfg, n, 50 + n) for n in (5, 11, 17, 8)]
    params = SamplingParams(max_new_tokens=10)
    together = [o.token_ids for o in engine(folder).generate(prompts, params)]
    one = engine(folder)
    alone = [one.generate([p], params)[0].token_ids for p in prompts]
    assert together == alone
    tight = engine(folder, num_blocks=8)      # 8 pages of 8 tokens for four requests of up to 27 tokens
    outs = tight.generate(prompts, params)
    assert [o.token_ids for o in outs] == together
    assert sum(o.preemptions for o in outs) > 0
    tight.cache.check()
    assert tight.cache.free_pages() == [8, 8]


def test_temperature_sampling_is_repeatable_and_depends_on_the_seed(tiny):
    cfg, folder, _ = tiny
    prompts = [random_ids(cfg, 6, 1), random_ids(cfg, 9, 2)]
    a = engine(folder).generate(prompts, SamplingParams(max_new_tokens=12, temperature=0.7, seed=5))
    b = engine(folder).generate(list(reversed(prompts)), SamplingParams(max_new_tokens=12, temperature=0.7, seed=5))
    c = engine(folder).generate(prompts, SamplingParams(max_new_tokens=12, temperature=0.7, seed=6))
    assert [o.token_ids for o in a] == [o.token_ids for o in reversed(b)]      # not a matter of batch order
    assert [o.token_ids for o in a] != [o.token_ids for o in c]
    greedy = engine(folder).generate(prompts, SamplingParams(max_new_tokens=12))
    assert [o.token_ids for o in a] != [o.token_ids for o in greedy]


def test_eos_stops_and_is_emitted(tiny):
    cfg, folder, weights = tiny
    prompt = random_ids(cfg, 7, 3)
    want = plain_greedy(weights, cfg, prompt, 6)
    out = engine(folder).generate([prompt], SamplingParams(max_new_tokens=6, eos_id=want[2]))[0]
    assert out.token_ids == want[:3] and out.finish_reason == "stop"
    out = engine(folder).generate([prompt], SamplingParams(max_new_tokens=6, eos_id=want[2], ignore_eos=True))[0]
    assert out.token_ids == want


def test_cancel_frees_blocks(tiny):
    cfg, folder, _ = tiny
    llm = engine(folder)
    a = llm.add_request(random_ids(cfg, 9, 4), SamplingParams(max_new_tokens=50))
    b = llm.add_request(random_ids(cfg, 5, 5), SamplingParams(max_new_tokens=4))
    llm.run_step()
    llm.abort(a)
    while llm.has_work():
        llm.run_step()
    assert llm._outputs[a].finish_reason == "abort" and len(llm._outputs[a].token_ids) == 1
    assert llm._outputs[b].finish_reason == "length"
    assert llm.cache.free_pages() == [64, 64] and llm.cache.slots.num_free == llm.cache.num_slots


def test_request_larger_than_the_pool(tiny):
    cfg, folder, _ = tiny
    llm = engine(folder, num_blocks=2)
    with pytest.raises(RuntimeError, match="out of KV blocks"):
        llm.generate([random_ids(cfg, 30, 6)], SamplingParams(max_new_tokens=4))


def test_a_failing_step_reaches_its_requests_and_frees(tiny):
    cfg, folder, _ = tiny
    llm = engine(folder)
    calls = {"n": 0}
    real = llm.ops.silu_mul

    def flaky(x):
        calls["n"] += 1
        if calls["n"] == 4:
            raise RuntimeError("injected kernel failure")
        return real(x)

    llm.ops.silu_mul = flaky
    outs = llm.generate([random_ids(cfg, 4, 7)], SamplingParams(max_new_tokens=5))
    assert outs[0].finish_reason == "error" and "injected" in outs[0].error
    assert llm.cache.free_pages() == [64, 64]
    llm.ops.silu_mul = real
    assert llm.generate([random_ids(cfg, 4, 7)], SamplingParams(max_new_tokens=2))[0].finish_reason == "length"


def test_trace_free_running_and_forced(tiny):
    cfg, folder, weights = tiny
    llm = engine(folder)
    prompt = random_ids(cfg, 8, 8)
    want = plain_greedy(weights, cfg, prompt, 5)
    trace = llm.trace(prompt, 5)
    assert trace.token_ids == want and trace.logits.shape == (5, cfg["vocab_size"])
    full = oracle(weights, cfg, prompt + want)
    assert (trace.logits - full[len(prompt) - 1:len(prompt) + 4]).abs().max() < 1e-4
    forced = [3, 1, 4, 1, 5]
    trace = llm.trace(prompt, 5, forced_ids=forced)
    full = oracle(weights, cfg, prompt + forced)
    assert (trace.logits - full[len(prompt) - 1:len(prompt) + 4]).abs().max() < 1e-4
    with pytest.raises(ValueError):
        llm.trace([], 3)
    with pytest.raises(ValueError):
        llm.trace(prompt, 3, forced_ids=[1])
    assert llm.cache.free_pages() == [64, 64]


def test_steps_planned_ahead_change_nothing(tiny):
    """Decoding steps are launched before the tokens of the step before have reached the host: the
    same tokens as step by step, with requests that end at different lengths, one that stops at an
    end-of-sequence token (its row of the step after is computed for nothing), sampling with a
    temperature, a pool so tight that planning ahead has to give way to preemption, prompts in portions
    (the next portion goes into the step planned ahead) and fewer seats than requests (a waiting
    request is admitted by a step planned ahead)."""
    cfg, folder, weights = tiny
    prompts = [random_ids(cfg, n, 70 + n) for n in (3, 12, 7, 20)]
    stop = plain_greedy(weights, cfg, prompts[1], 9)[5]
    params = [SamplingParams(max_new_tokens=9), SamplingParams(max_new_tokens=14, eos_id=stop),
              SamplingParams(max_new_tokens=2), SamplingParams(max_new_tokens=11, temperature=0.8, seed=3)]
    for options in ({}, {"num_blocks": 7}, {"token_budget": 5}, {"max_seqs": 2}, {"max_seqs": 2, "token_budget": 4},
                    {"max_seqs": 3, "token_budget": 6, "num_blocks": 8}):
        plain_loop = engine(folder, lookahead=False, **options)
        want = plain_loop.generate(prompts, params)
        assert plain_loop.steps_ahead == 0
        ahead = engine(folder, **options)
        got = ahead.generate(prompts, params)
        assert ahead.steps_ahead > 0
        assert ahead._ahead is None and ahead._ahead_failed is None      # nothing is kept of a step launched for nothing
        assert [o.token_ids for o in got] == [o.token_ids for o in want]
        assert [o.finish_reason for o in got] == [o.finish_reason for o in want]
        assert got[1].finish_reason == "stop" and got[0].finish_reason == "length"
        ahead.cache.check()
        pages = options.get("num_blocks", 64)
        assert ahead.cache.free_pages() == [pages, pages] and ahead.cache.slots.num_free == ahead.cache.num_slots
        # the engine is as good as new: a second round gives the same
        again = ahead.generate(prompts, params)
        assert [o.token_ids for o in again] == [o.token_ids for o in want]


def test_abort_and_arrival_while_a_step_is_ahead(tiny):
    cfg, folder, weights = tiny
    llm = engine(folder)
    a = llm.add_request(random_ids(cfg, 6, 1), SamplingParams(max_new_tokens=30))
    b = llm.add_request(random_ids(cfg, 4, 2), SamplingParams(max_new_tokens=8))
    for _ in range(3):
        llm.run_step()
    assert llm._ahead is not None            # a step is in flight beyond the tokens the host has seen
    llm.abort(a)
    late_prompt = random_ids(cfg, 5, 3)
    c = llm.add_request(late_prompt, SamplingParams(max_new_tokens=6))
    while llm.has_work():
        llm.run_step()
    assert llm._outputs[a].finish_reason == "abort"
    assert llm._outputs[b].token_ids == plain_greedy(weights, cfg, random_ids(cfg, 4, 2), 8)
    assert llm._outputs[c].token_ids == plain_greedy(weights, cfg, late_prompt, 6)
    llm.cache.check()
    assert llm.cache.free_pages() == [64, 64] and llm.cache.slots.num_free == llm.cache.num_slots


def test_the_uniform_numbers_are_splitmix64():
    """The generator is pinned from outside: the output function of splitmix64 turns the state
    0x9E3779B97F4A7C15 (its first state from seed 0) into 0xE220A8397B1DCDAF, the published first value
    of that generator. The seed that makes (seed * G + K) equal that state reaches it through the kernel's
    own arithmetic; the independent copy of the tests agrees everywhere else."""
    from distie_amd.sampling import derive_seed, uniform_of

    G, K, M = 0x9E3779B97F4A7C15, 0x94D049BB133111EB, 1 << 64
    seed = ((G - K) * pow(G, -1, M)) % M
    assert uniform_of(seed, 0) == (0xE220A8397B1DCDAF >> 40) / 2 ** 24
    for s_, n in ((0, 0), (1, 0), (0, 1), (5, 17), (2 ** 63 + 11, 2 ** 40), (2 ** 64 - 1, 3)):
        assert uniform_of(s_, n) == plain_uniform(s_, n)
    seeds = [derive_seed(0, i) for i in range(100)] + [derive_seed(1, i) for i in range(100)]
    assert len(set(seeds)) == 200 and all(0 <= s_ < M for s_ in seeds)


def test_sampled_tokens_are_the_plain_draws_token_by_token(tiny):
    """Greedy and temperature requests mixed in one batch, prompts in portions: every token is
    argmax / the inverse of the cumulative sum at the request's own n-th uniform number, given the
    tokens before it, whatever else runs beside it."""
    cfg, folder, weights = tiny
    prompts = [random_ids(cfg, n, 90 + n) for n in (1, 9, 23, 40)]
    params = [SamplingParams(max_new_tokens=12, temperature=0.7, seed=11), SamplingParams(max_new_tokens=12),
              SamplingParams(max_new_tokens=12, temperature=0.7, seed=12), SamplingParams(max_new_tokens=12)]
    for options in ({"token_budget": 7}, {"token_budget": 7, "lookahead": False}, {"num_blocks": 9}):
        outs = engine(folder, **options).generate(prompts, params)
        for prompt, sp, out in zip(prompts, params, outs):
            assert len(out.token_ids) == 12
            assert check_generation(weights, cfg, prompt, out.token_ids, sp.temperature, sp.seed or 0, tol=1e-6) == 0


def test_requests_without_a_seed_draw_from_streams_of_their_own(tiny):
    cfg, folder, _ = tiny
    prompt = random_ids(cfg, 6, 1)
    params = SamplingParams(max_new_tokens=8, temperature=1.5)
    llm = engine(folder)
    first = [o.token_ids for o in llm.generate([prompt] * 3, params)]
    assert len({tuple(t) for t in first}) == 3                     # three samples of one prompt differ
    later = [o.token_ids for o in llm.generate([prompt] * 3, params)]
    assert later != first                                          # and so do later ones of the same engine
    assert [o.token_ids for o in engine(folder).generate([prompt] * 3, params)] == first     # a rerun repeats
    assert [o.token_ids for o in engine(folder, seed=1).generate([prompt] * 3, params)] != first
    # an explicit seed is taken as it is: the same stream for every request that names it
    fixed = SamplingParams(max_new_tokens=8, temperature=1.5, seed=4)
    same = [o.token_ids for o in engine(folder).generate([prompt] * 2, fixed)]
    assert same[0] == same[1]


def test_a_step_that_fails_while_the_next_one_is_ahead(tiny):
    """The step in flight fails after the step behind it was launched, and that step had seated a new
    request: the failed step's requests end with the error, the new request starts over and still gets
    the plain implementation's tokens (its cached tokens of the dropped step are not trusted)."""
    cfg, folder, weights = tiny
    llm = engine(folder, max_seqs=2)
    prompts = [random_ids(cfg, n, 110 + n) for n in (4, 6, 5)]
    a = llm.add_request(prompts[0], SamplingParams(max_new_tokens=2))
    b = llm.add_request(prompts[1], SamplingParams(max_new_tokens=10))
    c = llm.add_request(prompts[2], SamplingParams(max_new_tokens=6))
    real = llm._to_host
    calls = {"n": 0}

    def flaky(chosen):
        fetch = real(chosen)
        calls["n"] += 1
        if calls["n"] != 3:
            return fetch

        def broken():
            # by now the step behind this one is launched, and it has seated c
            assert llm._ahead is not None and c in [p.request.request_id for p in llm._ahead[0].portions]
            raise RuntimeError("injected failure while fetching")
        return broken

    llm._to_host = flaky
    while llm.has_work():
        llm.run_step()
    assert calls["n"] > 3
    outs = {r: llm.take_output(r) for r in (a, b, c)}
    assert outs[a].finish_reason == "length" and outs[a].token_ids == plain_greedy(weights, cfg, prompts[0], 2)
    assert outs[b].finish_reason == "error" and "injected" in outs[b].error
    assert outs[c].finish_reason == "length" and outs[c].token_ids == plain_greedy(weights, cfg, prompts[2], 6)
    assert not llm._outputs
    llm.cache.check()
    assert llm.cache.free_pages() == [64, 64] and llm.cache.slots.num_free == llm.cache.num_slots


def test_step_stats_and_forgotten_records(tiny):
    cfg, folder, _ = tiny
    llm = engine(folder, step_stats=1000, token_budget=6)
    for _ in llm.stream([random_ids(cfg, 9, 1), random_ids(cfg, 3, 2)], SamplingParams(max_new_tokens=4)):
        pass
    assert not llm._outputs                                        # stream hands nothing on and keeps nothing
    summary = llm.stats.summary()
    assert set(summary) == {"decode", "prefill"}
    assert summary["prefill"]["tokens"] > summary["prefill"]["rows"] and summary["decode"]["tokens"] == summary["decode"]["rows"]
    assert all(row["host"] >= row["launch"] > 0 for row in summary.values())
    assert "device" not in summary["decode"]                       # no GPU here: host parts only
    assert "host=" in llm.stats.format()


def test_nothing_is_kept_of_a_step_launched_for_nothing(tiny):
    """The only request stops at an end-of-sequence token while the step after is already launched: the loop
    ends without another turn, and the engine lets go of that step's plan and logits all the same."""
    cfg, folder, weights = tiny
    prompt = random_ids(cfg, 9, 5)
    stop = plain_greedy(weights, cfg, prompt, 6)[4]
    llm = engine(folder)
    (out,) = llm.generate([prompt], SamplingParams(max_new_tokens=12, eos_id=stop))
    assert out.finish_reason == "stop" and llm.steps_ahead > 0
    assert llm._ahead is None
    emitted = list(llm.stream([prompt], SamplingParams(max_new_tokens=12, eos_id=stop)))
    assert emitted[-1].finished and llm._ahead is None
    llm.add_request(prompt, SamplingParams(max_new_tokens=12))
    for _ in range(3):
        llm.run_step()
    assert llm._ahead is not None
    llm.close()
    assert llm._ahead is None


def test_tokens_are_the_plain_draws_from_the_logits_they_were_drawn_from(tiny):
    """The check in two halves that the bfloat16 runs on the GPU use, here on the test double: the logits each
    token was drawn from are the oracle's for the tokens the engine saw, and each token is the plain draw from
    those logits; also for requests that gave way and recomputed."""
    from engine_util import check_generation_in_two_halves, run_and_keep_logits

    cfg, folder, weights = tiny
    prompts = [random_ids(cfg, n, 90 + n) for n in (5, 11, 17, 8)]
    params = [SamplingParams(max_new_tokens=10, temperature=0.7 if i % 2 else 0.0, seed=40 + i) for i in range(4)]
    for options in ({}, {"num_blocks": 8}):
        llm = engine(folder, **options)
        outs, kept = run_and_keep_logits(llm, prompts, params)
        assert (sum(o.preemptions for o in outs) > 0) == bool(options)
        for prompt, sp, out in zip(prompts, params, outs):
            check_generation_in_two_halves(weights, cfg, prompt, out.token_ids, kept[out.request_id], torch.float32,
                                           sp.temperature, sp.seed)
    # the check notices a wrong token
    with pytest.raises(AssertionError):
        wrong = list(outs[0].token_ids)
        wrong[3] = (wrong[3] + 1) % cfg["vocab_size"]
        check_generation_in_two_halves(weights, cfg, prompts[0], wrong, kept[outs[0].request_id], torch.float32, 0.0, 40)
