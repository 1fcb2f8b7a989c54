"""Generation through the entry point on the GPU against the plain implementation, token by token:
the two correctness workloads with greedy and temperature requests mixed in one batch, with and
without captured steps and steps planned ahead; a pool so tight that requests give way and recompute;
a cancellation and an arrival while a step is ahead (worker/tests/test_batched_engine.py:85-144).
And the other way round: a corrupted cache must fail the comparison, in float32 and under the wider
bfloat16 bound (benchmarks/correctness/test_hf_parity.py:108-127)."""

import pytest
import torch

import plain_qwen2 as plain
from distie_amd import LLM, SamplingParams
from distie_amd.engine.batch import StepEntry
from engine_util import (build_runner, check_generation, check_generation_in_two_halves, check_logits, make_model_dir,
                         random_ids, run_and_keep_logits)

pytestmark = pytest.mark.gpu


def plain_greedy(weights, cfg, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain.forward(weights, cfg, ids, torch.float64)[-1].argmax()))
    return ids[len(prompt):]


# (configuration, page size, prompt lengths, new tokens, token budget): the two tiny workloads
WORKLOADS = {
    "A": (plain.TINY_A, 4, (5, 11, 17), 8, 2048),
    "B": (plain.TINY_B, 8, (1, 9, 23, 40), 12, 7),
}


@pytest.mark.parametrize("name", sorted(WORKLOADS))
@pytest.mark.parametrize("graphs,lookahead", [(False, False), (False, True), (True, True)])
def test_greedy_and_temperature_mixed_in_one_batch(tmp_path, name, graphs, lookahead):
    cfg, block, lengths, new, budget = WORKLOADS[name]
    folder, weights = make_model_dir(tmp_path, cfg, seed=41)
    prompts = [random_ids(cfg, n, 200 + n) for n in lengths]
    params = [SamplingParams(max_new_tokens=new, temperature=0.7 if i % 2 == 0 else 0.0, seed=100 + i)
              for i in range(len(prompts))]
    llm = LLM(folder, dtype="fp32", block_size=block, num_blocks=48, token_budget=budget, use_graphs=graphs,
              lookahead=lookahead)
    outs = llm.generate(prompts, params)
    near = 0
    for prompt, sp, out in zip(prompts, params, outs):
        assert len(out.token_ids) == new and out.finish_reason == "length"
        near += check_generation(weights, cfg, prompt, out.token_ids, sp.temperature, sp.seed, tol=1e-4)
    assert near <= 1                  # a draw at an interval's very edge may fall either way; that is rare
    assert (llm.steps_ahead > 0) == lookahead
    if graphs:
        assert llm.runner.graphs.captured and llm.runner.graphs.failures == 0
        # the steps that hold a portion of a prompt are short enough to replay graphs as well
        assert llm.runner.graphs.captured_mixed and llm.runner.graphs.mixed_replays > 0
    llm.cache.check()
    assert all(f == 48 for f in llm.cache.free_pages())


@pytest.mark.parametrize("name", ["A", "B"])
def test_the_two_tiny_workloads_at_their_named_sizes_and_spread(tmp_path, name):
    """The two tiny workloads exactly as they are named for this engine: Tiny B with a feed-forward width of 256
    and a vocabulary of 320 (the other tests give it 250 and 323, which end inside a tile), weights and biases
    drawn from N(0, 0.02) and norm weights of one (the other tests spread the weights further and move the norms,
    so that a fault shows in the logits; here the logits of a row lie close together, so the check has two halves:
    the row every token was drawn from is the oracle's within the float32 bound, and the token is the plain draw
    from that row)."""
    cfg, block, lengths, new, budget = WORKLOADS[name]
    if name == "B":
        cfg = dict(cfg, intermediate_size=256, vocab_size=320)
    weights = plain.random_weights(cfg, seed=91, std=0.02, norm_jitter=0.0)
    folder = tmp_path / "model"
    plain.write_model_dir(folder, cfg, weights)
    prompts = [random_ids(cfg, n, 700 + n) for n in lengths]
    params = [SamplingParams(max_new_tokens=new, temperature=0.7 if name == "B" and i % 2 == 0 else 0.0, seed=300 + i)
              for i in range(len(prompts))]
    llm = LLM(folder, dtype="fp32", block_size=block, num_blocks=48, token_budget=budget)
    outs, kept = run_and_keep_logits(llm, prompts, params)
    for prompt, sp, out in zip(prompts, params, outs):
        assert len(out.token_ids) == new and out.finish_reason == "length"
        check_generation_in_two_halves(weights, cfg, prompt, out.token_ids, kept[out.request_id], torch.float32,
                                       sp.temperature, sp.seed)
    llm.cache.check()
    assert all(f == 48 for f in llm.cache.free_pages())


BF16_WORKLOADS = {
    "B": (plain.TINY_B, 8, (1, 9, 23, 40), 12, 7),
    "C": (plain.TINY_C, 16, (3, 30, 70, 18, 44), 20, 33),
}


@pytest.mark.parametrize("name", sorted(BF16_WORKLOADS))
@pytest.mark.parametrize("graphs,lookahead,pages", [(False, False, 48), (True, True, 48), (True, True, None)])
def test_bfloat16_generation_through_the_scheduler(tmp_path, name, graphs, lookahead, pages):
    """The serving precision through the whole loop: greedy and temperature requests in one batch, prompts in
    portions, captured steps launched ahead, and (pages=None) a pool so tight that requests give way and
    recompute. bfloat16 logits lie too far from the oracle's to judge a draw by the oracle's logits, so the
    check has two halves: the logits each token was drawn from are the oracle's for the tokens the engine saw,
    within the bfloat16 bounds, and each token is the plain draw from the engine's own logits, exactly."""
    cfg, block, lengths, new, budget = BF16_WORKLOADS[name]
    folder, weights = make_model_dir(tmp_path, cfg, seed=45, dtype=torch.bfloat16)
    prompts = [random_ids(cfg, n, 300 + n) for n in lengths]
    params = [SamplingParams(max_new_tokens=new, temperature=0.7 if i % 2 == 0 else 0.0, seed=200 + i)
              for i in range(len(prompts))]
    tight = pages is None
    if tight:
        # every request is seated (by the pages of what is known of it then), and they cannot all grow to their
        # length: B's draw 30 tokens each on 11 pages of 8, C's 20 each on 11 pages of 16
        pages, new = 11, {"B": 30, "C": 20}[name]
        params = [SamplingParams(max_new_tokens=new, temperature=p.temperature, seed=p.seed) for p in params]
    llm = LLM(folder, dtype="bf16", block_size=block, num_blocks=pages, token_budget=budget, use_graphs=graphs,
              lookahead=lookahead)
    outs, kept = run_and_keep_logits(llm, prompts, params)
    for prompt, sp, out in zip(prompts, params, outs):
        assert len(out.token_ids) == new and out.finish_reason == "length"
        check_generation_in_two_halves(weights, cfg, prompt, out.token_ids, kept[out.request_id], torch.bfloat16,
                                       sp.temperature, sp.seed)
    assert (sum(o.preemptions for o in outs) > 0) == tight
    assert (llm.steps_ahead > 0) == lookahead
    if graphs:
        assert llm.runner.graphs.captured and llm.runner.graphs.failures == 0
        assert llm.runner.graphs.captured_mixed and llm.runner.graphs.mixed_replays > 0
    llm.cache.check()
    assert all(f == pages for f in llm.cache.free_pages()) and llm.cache.slots.num_free == llm.cache.num_slots


def test_a_tight_pool_makes_requests_give_way_and_changes_nothing(tmp_path):
    cfg = plain.TINY_B
    folder, weights = make_model_dir(tmp_path, cfg, seed=42)
    prompts = [random_ids(cfg, n, 50 + n) for n in (5, 11, 17, 8)]
    params = [SamplingParams(max_new_tokens=10, temperature=0.7 if i == 2 else 0.0, seed=7) for i in range(4)]
    for options in ({}, {"use_graphs": False, "lookahead": False}):
        tight = LLM(folder, dtype="fp32", block_size=8, num_blocks=8, **options)    # 8 pages for up to 4 x 27 tokens
        outs = tight.generate(prompts, params)
        assert sum(o.preemptions for o in outs) > 0
        for prompt, sp, out in zip(prompts, params, outs):
            assert check_generation(weights, cfg, prompt, out.token_ids, sp.temperature, sp.seed, tol=1e-4) == 0
        tight.cache.check()
        assert tight.cache.free_pages() == [8, 8] and tight.cache.slots.num_free == tight.cache.num_slots


def test_abort_and_arrival_while_a_step_is_ahead(tmp_path):
    cfg = plain.TINY_B
    folder, weights = make_model_dir(tmp_path, cfg, seed=43)
    llm = LLM(folder, dtype="fp32", block_size=8, num_blocks=64)
    first, second, late = random_ids(cfg, 6, 1), random_ids(cfg, 4, 2), random_ids(cfg, 5, 3)
    a = llm.add_request(first, SamplingParams(max_new_tokens=30))
    b = llm.add_request(second, SamplingParams(max_new_tokens=8))
    for _ in range(3):
        llm.run_step()
    assert llm._ahead is not None            # a step is in flight beyond the tokens the host has seen
    llm.abort(a)
    c = llm.add_request(late, SamplingParams(max_new_tokens=6))
    while llm.has_work():
        llm.run_step()
    assert llm.take_output(a).finish_reason == "abort"
    assert llm.take_output(b).token_ids == plain_greedy(weights, cfg, second, 8)
    assert llm.take_output(c).token_ids == plain_greedy(weights, cfg, late, 6)
    llm.cache.check()
    assert llm.cache.free_pages() == [64, 64] and llm.cache.slots.num_free == llm.cache.num_slots


def test_a_failing_step_on_the_gpu_reaches_its_requests_and_frees(tmp_path):
    cfg = plain.TINY_A
    folder, weights = make_model_dir(tmp_path, cfg, seed=44)
    llm = LLM(folder, dtype="fp32", block_size=4, num_blocks=32, use_graphs=False)
    prompt = random_ids(cfg, 4, 7)
    real = llm.ops.paged_attention
    calls = {"n": 0}

    def flaky(*args, **kwargs):
        calls["n"] += 1
        if calls["n"] == 5:
            raise RuntimeError("injected failure before a launch")     # raised on the host: no kernel is harmed
        return real(*args, **kwargs)

    llm.ops.paged_attention = flaky
    out = llm.generate([prompt], SamplingParams(max_new_tokens=5))[0]
    assert out.finish_reason == "error" and "injected" in out.error
    llm.ops.paged_attention = real
    assert llm.cache.free_pages() == [32]
    assert llm.generate([prompt], SamplingParams(max_new_tokens=5))[0].token_ids == plain_greedy(weights, cfg, prompt, 5)


@pytest.mark.parametrize("name,block", [("A", 4), ("B", 8), ("C", 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_a_corrupted_cache_fails_the_comparison(tmp_path, name, block, dtype):
    """The bounds of `check_logits` are not so wide that a wrong key passes: one cached key of one
    layer set to zero after the prompt, or the last two entries of the request's block table of one group
    exchanged (the last page is partly filled, so the tokens that follow land on the wrong page and keys
    of the page before are read at the wrong places), must make it raise; the untouched run passes."""
    cfg = {"A": plain.TINY_A, "B": plain.TINY_B, "C": plain.TINY_C}[name]
    from distie_amd.kernels.hip_ops import HipOps

    ops = HipOps("cuda:0")
    folder, weights = make_model_dir(tmp_path, cfg, seed=11, dtype=dtype)
    ids = random_ids(cfg, 80, 3)
    prompt = 60 // block * block + block // 2      # the last page of the prompt is half full

    def run(damage):
        runner = build_runner(folder, ops, dtype, block_size=block)
        out = [runner.step([StepEntry("a", ids[:prompt], list(range(prompt)))])]
        damage(runner)
        for t in range(prompt, len(ids)):
            out.append(runner.step([StepEntry("a", [ids[t]], [0])]))
        return torch.cat(out).float().cpu()

    def zero_key(group, position):
        def damage(runner):
            page = runner.cache.request("a").tables[group][position // block]
            assert page >= 0
            runner.cache.groups[group].tensors["k"][0, page, :, position % block, :] = 0
        return damage

    def exchange_last_two(group):
        def damage(runner):
            table = runner.cache.request("a").tables[group]
            assert len(table) >= 2 and table[-1] >= 0 and table[-2] >= 0       # both held: no page out of bounds
            table[-1], table[-2] = table[-2], table[-1]
            slot = runner.cache.request("a").slot
            for i in (len(table) - 1, len(table) - 2):          # ... and on the device, where the kernels read them
                runner.cache._note(runner.cache.groups[group], slot, i, table[i])
        return damage

    check_logits(run(lambda runner: None), weights, cfg, ids, dtype)
    groups = len(build_runner(folder, ops, dtype, block_size=block).cache.groups)
    for group in range(groups):
        for damage in (zero_key(group, prompt - 2), exchange_last_two(group)):
            with pytest.raises(AssertionError):
                check_logits(run(damage), weights, cfg, ids, dtype)
                pytest.fail(f"group {group}: {damage.__qualname__} went unnoticed", pytrace=False)
