"""Helpers shared by the tests: model folders in a temporary place, an engine on the CPU
test double or on the GPU, and replays of one request under different ways of cutting."""

from __future__ import annotations

import torch

import plain_qwen2 as plain
from distie_amd.cache import CacheManager
from distie_amd.config import load_model_config
from distie_amd.engine.batch import StepEntry
from distie_amd.engine.model import Model
from distie_amd.engine.runner import ModelRunner
from distie_amd.weights import load_into


# Spread of the random weights for each tiny configuration: large enough that logits are far
# from uniform (the top probability is 20 to 50 times the uniform one), small enough that the
# float32 rounding of the plain implementation itself stays near 1e-5.
STD = {64: 0.2, 96: 0.15, 240: 0.1}
FP32_TOL = 1e-4   # the bound the reference holds for tiny models (worker/tests/test_qwen2.py:89-93)


def oracle(weights, cfg, ids):
    """Logits of the plain implementation in float64, as float32."""
    return plain.forward(weights, cfg, ids, torch.float64).float()


def make_model_dir(tmp_path, cfg, seed=0, std=None, norm_jitter=0.2, dtype=torch.float32, name="model"):
    std = STD.get(cfg["hidden_size"], 0.1) if std is None else std
    weights = plain.random_weights(cfg, seed, std=std, norm_jitter=norm_jitter, dtype=dtype)
    folder = tmp_path / name
    plain.write_model_dir(folder, cfg, weights)
    return folder, weights


def build_runner(model_dir, ops, dtype=torch.float32, block_size=4, num_blocks=64, num_slots=8,
                 max_model_len=None):
    config = load_model_config(model_dir)
    model = Model(config.model_spec())
    load_into(model, model_dir, ops.device, dtype)
    cache = CacheManager(model.cache_requirements(), block_size, num_blocks, num_slots,
                         device=ops.device, dtype=dtype)
    return ModelRunner(model, cache, ops, dtype, max_model_len)


def replay_whole(runner, rid, ids):
    logits = runner.step([StepEntry(rid, list(ids), list(range(len(ids))))])
    runner.finish(rid)
    return logits.float().cpu()


def replay_cut(runner, rid, ids, cuts):
    """Feed `ids` in portions of the sizes `cuts` (the rest one token at a time)."""
    out = []
    at = 0
    sizes = list(cuts)
    while at < len(ids):
        n = sizes.pop(0) if sizes else 1
        n = min(n, len(ids) - at)
        out.append(runner.step([StepEntry(rid, list(ids[at:at + n]), list(range(n)))]))
        at += n
    runner.finish(rid)
    return torch.cat(out).float().cpu()


def random_ids(cfg, n, seed):
    return torch.randint(0, cfg["vocab_size"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def check_logits(got, weights, cfg, ids, dtype, folder=None):
    """float32: within FP32_TOL of the float64 oracle.

    bfloat16: rounding activations to 8 bits moves the logits of these tiny models by 2 to 3 % of
    the largest logit at the worst place and by 0.4 % in the root mean square (measured with the
    test double, which rounds where the engine rounds; two runs that differ only in the order of
    float32 sums drift apart by as much, because one flipped rounding flips others downstream).
    The bounds are about twice that: 1/16 at the worst place and 1/64 in the root mean square. A
    wrong key, page or position moves logits by far more, and the float32 runs of the same code
    hold the tight bound."""
    want = oracle(weights, cfg, ids)
    diff = got - want
    err = diff.abs().max().item()
    scale = want.abs().max().item()
    if dtype == torch.float32:
        assert err < FP32_TOL, f"max error {err} vs oracle"
        return
    rms = diff.pow(2).mean().sqrt().item()
    assert err < scale / 16, f"max error {err} vs oracle, largest logit {scale}"
    assert rms < scale / 64, f"rms error {rms} vs oracle, largest logit {scale}"
    # The reference judges half precision by the share of positions whose largest logit is the same token as
    # the oracle's, at least 0.98 on real checkpoints (benchmarks/correctness/metrics.py:16-22, 62-69). With
    # random weights the two largest logits of a position lie 0.26-0.43 apart in the median where the rounding
    # moves a logit by up to 0.16, and the share measured on these models is 0.97-0.99 (whole sequences of 100
    # tokens, two seeds each): so a position whose winner is clear (ahead by more than twice the largest error
    # met) must agree, every one, and the share over all positions must stay near what was measured.
    if got.shape[0] >= 8:
        same = got.argmax(-1) == want.argmax(-1)
        top2 = want.topk(2, -1).values
        clear = (top2[:, 0] - top2[:, 1]) > 2 * err
        assert bool(same[clear].all()), "a position with a clear winner has another token on top"
        share = same.float().mean().item()
        assert share >= 0.9, f"top-1 agreement {share}"


def plain_uniform(seed, counter):
    """The uniform number of a request's `counter`-th draw, written out independently of the product's
    `uniform_of`: the state seed * G + counter * C + K goes through the output function of splitmix64
    (xor-shift 30, multiply, xor-shift 27, multiply, xor-shift 31); the top 24 bits are the number."""
    import numpy as np

    with np.errstate(over="ignore"):
        u = np.uint64
        z = u(seed & (2 ** 64 - 1)) * u(0x9E3779B97F4A7C15) + u(counter & (2 ** 64 - 1)) * u(0xD1B54A32D192ED03) \
            + u(0x94D049BB133111EB)
        z = (z ^ (z >> u(30))) * u(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> u(27))) * u(0x94D049BB133111EB)
        z = z ^ (z >> u(31))
    return float(int(z) >> 40) / float(1 << 24)


def check_generation(weights, cfg, prompt, token_ids, temperature=0.0, seed=0, tol=1e-4):
    """Every produced token is the plain implementation's choice given the tokens before it: the
    argmax of its float64 logits, or for a temperature the first index whose cumulative softmax weight
    exceeds the request's `n`-th uniform number. The engine's float32 logits differ from the oracle's
    by up to `tol`, so a draw within that distance of an interval's end may land in the neighbouring
    interval, and of two logits within `tol` either may win. -> how many tokens were such near misses."""
    ids = list(prompt)
    near = 0
    for n, token in enumerate(token_ids):
        logits = plain.forward(weights, cfg, ids, torch.float64)[-1]
        if temperature <= 0:
            best = int(logits.argmax())
            if token != best:
                assert logits[token] >= logits[best] - tol, f"token {n}: {token} is not the greedy pick {best}"
                near += 1
        else:
            w = torch.exp((logits - logits.max()) / temperature)
            c = torch.cumsum(w, 0) / w.sum()
            u = plain_uniform(seed, n)
            want = int((c > u).nonzero()[0])
            if token != want:
                below = float(c[token - 1]) if token else 0.0
                slack = 4 * tol / temperature
                assert w[token] > 0 and below - slack <= u <= float(c[token]) + slack, \
                    f"token {n}: {token} drawn, the plain draw is {want} (u = {u})"
                near += 1
        ids.append(int(token))
    return near


def run_and_keep_logits(llm, prompts, params):
    """`LLM.generate`, keeping the logits every token was drawn from: -> (outputs, {request: [(position, row)]})."""
    kept = {}
    seen = {}
    sample = llm.sampler.sample_device
    complete = llm.scheduler.complete

    def spy_sample(logits, *args):
        seen["logits"] = logits.clone()             # queued behind the step, ahead of whatever overwrites its buffer
        return sample(logits, *args)

    def spy_complete(plan, drawn):
        rows = [p for p in plan.portions if p.samples]
        for i, portion in enumerate(rows):
            kept.setdefault(portion.request.request_id, []).append((portion.end - 1, seen["logits"][i]))
        return complete(plan, drawn)

    llm.sampler.sample_device = spy_sample
    llm.scheduler.complete = spy_complete
    try:
        outs = llm.generate(prompts, params)
    finally:
        llm.sampler.sample_device = sample
        llm.scheduler.complete = complete
    return outs, kept


def check_generation_in_two_halves(weights, cfg, prompt, token_ids, rows, dtype, temperature=0.0, seed=0):
    """For a precision whose logits are too far from the oracle's to judge a draw by them: (1) the logits the
    engine drew from (`rows`: [(position, float32 row)], in the order of the tokens) are the oracle's for the
    tokens the engine saw, within the bounds of `check_logits`; (2) every token is the plain draw from the
    engine's own row: its argmax (lowest index among equals), or the first index whose cumulative softmax
    weight exceeds the request's n-th uniform number. A request that gave way and recomputed has drawn some
    tokens twice; the rows of the last time count."""
    ids = list(prompt) + list(token_ids[:-1])
    last = {}
    for position, row in rows:
        last[position] = row
    positions = list(range(len(prompt) - 1, len(ids)))
    assert sorted(last) == positions, "a token was drawn from a row at another place"
    got = torch.stack([last[p] for p in positions]).float().cpu()
    want = oracle(weights, cfg, ids)[positions]
    diff = got - want
    scale = want.abs().max().item()
    if dtype == torch.float32:
        assert diff.abs().max().item() < FP32_TOL
    else:
        assert diff.abs().max().item() < scale / 16 and diff.pow(2).mean().sqrt().item() < scale / 64
    for n, token in enumerate(token_ids):
        row = got[n].double()
        if temperature <= 0:
            assert token == int(row.argmax()), f"token {n}: {token} is not the largest of the engine's own logits"
            continue
        w = torch.exp((row - row.max()) / temperature)
        c = torch.cumsum(w, 0) / w.sum()
        u = plain_uniform(seed, n)
        pick = int((c > u).nonzero()[0])
        if token != pick:          # float32 sums of the kernel against float64 here: only at an interval's very edge
            below = float(c[token - 1]) if token else 0.0
            assert below - 1e-5 <= u <= float(c[token]) + 1e-5, f"token {n}: {token} drawn, the plain draw is {pick}"
