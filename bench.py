"""Decode and prefill throughput of Qwen2-shaped models with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape 1.5b|7b|32b] [--serve] [--dtype bf16|fp32]

Without options: the Qwen2.5-1.5B shape. A step is one decode step of the whole engine (schedule,
metadata, captured forward, sampling, completion) at batch 8, each request with a 2,048-token context
behind it. One JSON line on standard output: `value` = decoded tokens a second, plus `prefill` (one prompt,
the median of five runs), `roofline` (bytes the decode step has to read / its time, against 8 TB/s) and
`points` (batch 1 and batch 64).

`--shape 7b`, `--shape 32b`: the same measurements at the layer sizes of Qwen2.5-7B and Qwen2.5-32B; the
32B run has a context and a prompt of 8,192 tokens (run in portions of the token budget, as the engine
serves it), points at batch 1 and 32, and a cache that takes the card's memory up to `--gpu-mem-fraction`.

`--serve`: 64 requests at once, prompt lengths uniform in [128, 2048] and output lengths uniform in
[32, 256], served by the engine's loop with a token budget of 2,048: `value` = output tokens a second, with
the time to the first token and the time per output token after it, defined as the reference's load
generator defines them (benchmarks/load/stats.py:29-34, 67-86).

Random weights N(0, 0.02), seeded uniform token ids.
"""

import argparse
import json
import statistics
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

COMMON = {
    "architectures": ["Qwen2ForCausalLM"], "head_dim": 128, "rope_theta": 1000000.0,
    "use_sliding_window": False, "hidden_act": "silu",
}
# layer sizes of the published configurations; context, prompt and batches of the workloads measured on them
SHAPES = {
    "1.5b": dict(model="Qwen2.5-1.5B", num_hidden_layers=28, hidden_size=1536, num_attention_heads=12,
                 num_key_value_heads=2, intermediate_size=8960, vocab_size=151936, rms_norm_eps=1e-6,
                 tie_word_embeddings=True, max_position_embeddings=4096, context=2048, prefill=2048,
                 points=(1, 64)),
    "7b": dict(model="Qwen2.5-7B", num_hidden_layers=28, hidden_size=3584, num_attention_heads=28,
               num_key_value_heads=4, intermediate_size=18944, vocab_size=152064, rms_norm_eps=1e-6,
               tie_word_embeddings=False, max_position_embeddings=8192, context=2048, prefill=2048,
               points=(1, 64)),
    "32b": dict(model="Qwen2.5-32B", num_hidden_layers=64, hidden_size=5120, num_attention_heads=40,
                num_key_value_heads=8, intermediate_size=27648, vocab_size=152064, rms_norm_eps=1e-5,
                tie_word_embeddings=False, max_position_embeddings=16384, context=8192, prefill=8192,
                points=(1, 32)),
}
WORKLOAD_KEYS = ("model", "context", "prefill", "points")
BLOCK_SIZE = 16
TOKEN_BUDGET = 2048
PREFILL_REPEATS = 5
SERVE = dict(requests=64, prompt=(128, 2048), output=(32, 256))


def prompts(batch, length, vocab, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(batch)]


def linear_params(c):
    q = c["num_attention_heads"] * c["head_dim"]
    kv = c["num_key_value_heads"] * c["head_dim"]
    per_layer = c["hidden_size"] * (q + 2 * kv) + q * c["hidden_size"] + 3 * c["hidden_size"] * c["intermediate_size"]
    return per_layer * c["num_hidden_layers"], c["vocab_size"] * c["hidden_size"]


def early_tokens(batch, context):
    """Tokens a request may decode while the prompts of the others are run, a portion a step."""
    return batch * -(-context // TOKEN_BUDGET) + batch + 8


def check_logits(logits, rows, what):
    """A line is printed only for a model that computes: the logits of the last step are numbers, differ along
    the vocabulary and from request to request (random prompts), and are of the size a model with these
    weights gives (not zeros, not overflow)."""
    import torch

    assert logits is not None and logits.shape[0] >= rows, f"{what}: no logits for {rows} rows"
    logits = logits[:rows].float()
    assert bool(torch.isfinite(logits).all()), f"{what}: logits are not finite"
    spread = logits.std(dim=1)
    assert bool((spread > 1e-3).all()) and bool((spread < 1e3).all()), f"{what}: logits are constant or blown up"
    if rows > 1:
        assert bool((logits[1:] - logits[:1]).abs().amax(dim=1).gt(1e-3).all()), f"{what}: every request has the same logits"


def decode_run(llm, batch, context, steps, warmup, vocab, seed):
    """-> (seconds per step, mean context over the timed steps)"""
    import torch

    from distie_amd import SamplingParams

    # requests admitted early decode while later prompts are still prefilled: leave room for that
    params = SamplingParams(max_new_tokens=warmup + steps + early_tokens(batch, context), ignore_eos=True)
    ids = [llm.add_request(p, params) for p in prompts(batch, context, vocab, seed)]
    seqs = [llm.scheduler.request(i) for i in ids]
    while any(len(s.output_ids) == 0 for s in seqs):      # prefill, in portions under the token budget
        llm.run_step()
    for _ in range(warmup):
        llm.run_step()
    torch.cuda.synchronize()
    before = [s.num_tokens for s in seqs]
    t0 = time.perf_counter()
    for _ in range(steps):
        llm.run_step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert all(s.num_tokens == b + steps for s, b in zip(seqs, before)), "a timed step did not decode every request"
    check_logits(llm.last_logits, batch, f"decode at batch {batch}")
    picked = {s.output_ids[-1] for s in seqs} | {t for s in seqs[:1] for t in s.output_ids[-steps:]}
    assert len(picked) > 1, "every decoded token is the same"
    # keys a decode step reads for a request: everything cached before it, plus its own token
    mean_ctx = sum(before) / len(before) + (steps - 1) / 2.0
    for i in ids:
        llm.abort(i)
    while llm.has_work():
        llm.run_step()
    for i in ids:
        llm.take_output(i)
    return elapsed / steps, mean_ctx


def prefill_run(llm, tokens, portion, vocab, repeats=PREFILL_REPEATS):
    """Median seconds for one prompt of `tokens` tokens, run in portions of at most `portion`; the logits of
    the last token are asked for, as a prompt's last portion does."""
    import torch

    from distie_amd import StepEntry

    times = []
    for r in range(repeats + 1):
        ids = prompts(1, tokens, vocab, 100 + r)[0]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for begin in range(0, tokens, portion):
            part = ids[begin:begin + portion]
            logits = llm.step([StepEntry(f"prefill-{r}", part, [len(part) - 1] if begin + portion >= tokens else [])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        llm.finish(f"prefill-{r}")
        check_logits(logits, 1, "prefill")
        if r > 0:                                          # the first run warms up
            times.append(dt)
    return statistics.median(times)


def serve_run(llm, vocab, seed):
    """All requests arrive at once; the engine's loop runs until the last one ends."""
    import torch

    from distie_amd import SamplingParams
    from distie_amd.engine.stats import distribution_ms

    g = torch.Generator().manual_seed(seed)
    n = SERVE["requests"]
    prompt_lens = torch.randint(SERVE["prompt"][0], SERVE["prompt"][1] + 1, (n,), generator=g).tolist()
    output_lens = torch.randint(SERVE["output"][0], SERVE["output"][1] + 1, (n,), generator=g).tolist()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ids = [llm.add_request(torch.randint(0, vocab, (p,), generator=g).tolist(),
                           SamplingParams(max_new_tokens=o, ignore_eos=True))
           for p, o in zip(prompt_lens, output_lens)]
    steps = 0
    while llm.has_work():
        llm.run_step()
        steps += 1
    torch.cuda.synchronize()
    duration = time.perf_counter() - t0
    outs = [llm.take_output(i) for i in ids]
    assert all(o.finished and o.finish_reason == "length" and len(o.token_ids) == want
               for o, want in zip(outs, output_lens)), "a request did not run to its length"
    ttft = [o.time_to_first_token_ms / 1e3 for o in outs]
    # mean time per output token after the first (stats.py:29-34)
    tpot = [(o.total_latency_ms - o.time_to_first_token_ms) / 1e3 / (len(o.token_ids) - 1) for o in outs
            if len(o.token_ids) > 1]
    return {
        "duration_s": duration, "steps": steps, "prompt_tokens": sum(prompt_lens), "output_tokens": sum(output_lens),
        "preemptions": sum(o.preemptions for o in outs),
        "ttft_ms": distribution_ms(ttft), "tpot_ms": distribution_ms(tpot),
        "e2e_latency_ms": distribution_ms([o.total_latency_ms / 1e3 for o in outs]),
    }


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=256)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--shape", default="1.5b", choices=sorted(SHAPES))
    parser.add_argument("--serve", action="store_true", help="the 64-request serving workload instead of fixed batches")
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=None,
                        help="tokens behind every request when decoding starts (the shape's own: 2,048 or 8,192)")
    parser.add_argument("--prefill", type=int, default=None,
                        help="tokens of the timed prompt (the shape's own: 2,048 or 8,192), run in portions of the token budget")
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    parser.add_argument("--no-points", action="store_true", help="skip the other batch sizes")
    parser.add_argument("--no-tune", action="store_true",
                        help="leave the choice of the library's product kernels (prefill) to the library's defaults")
    parser.add_argument("--step-stats", action="store_true",
                        help="with --serve: add the mean time of a step on the host and on the device, by kind of step")
    parser.add_argument("--gpu-mem-fraction", type=float, default=None,
                        help="size the cache from free memory (the default for --shape 32b and --serve: 0.9)")
    parser.add_argument("--packed-weights", default=None, metavar="ROLES",
                        help="packed copies only for these products (qkv,attn_out,gate_up,down,head); 'none' for no copies")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not supported (this engine has no multi-GPU path)")
        return 2

    import torch

    from distie_amd import LLM

    preset = SHAPES[args.shape]
    shape = dict(COMMON, **{k: v for k, v in preset.items() if k not in WORKLOAD_KEYS})
    layers = shape["num_hidden_layers"]
    layers_run = args.layers or layers
    shape["num_hidden_layers"] = layers_run
    context, prefill_tokens = args.context or preset["context"], args.prefill or preset["prefill"]
    points_at = () if args.no_points or args.serve else preset["points"]
    max_batch = SERVE["requests"] if args.serve else max((args.batch,) + tuple(points_at))
    tokens_per_request = context + args.warmup + args.steps + early_tokens(max_batch, context)
    if args.serve:
        tokens_per_request = SERVE["prompt"][1] + SERVE["output"][1]
    shape["max_position_embeddings"] = max(shape["max_position_embeddings"], tokens_per_request, prefill_tokens)
    fraction = args.gpu_mem_fraction
    if fraction is None and (args.shape == "32b" or args.serve):
        fraction = 0.9
    pages = None if fraction is not None else max(max_batch * -(-tokens_per_request // BLOCK_SIZE),
                                                  -(-prefill_tokens // BLOCK_SIZE)) + 8
    packed = True
    if args.packed_weights is not None:
        packed = False if args.packed_weights == "none" else tuple(r for r in args.packed_weights.split(",") if r)
    llm = LLM(config=shape, random_weights=True, seed=0, dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=pages,
              gpu_mem_fraction=fraction, max_seqs=max_batch, token_budget=TOKEN_BUDGET, use_graphs=True,
              packed_weights=packed, tune_products=not args.no_tune, step_stats=10 ** 9 if args.step_stats else 0)
    vocab = shape["vocab_size"]
    elem = 2 if args.dtype == "bf16" else 4
    body, head = linear_params(shape)
    config = {
        "model": f"{preset['model']}-shaped, random weights N(0,0.02)", "layers": layers,
        "layers_run": layers_run, "hidden": shape["hidden_size"], "heads": shape["num_attention_heads"],
        "kv_heads": shape["num_key_value_heads"], "head_dim": shape["head_dim"],
        "intermediate": shape["intermediate_size"], "vocab": vocab, "tied_head": shape["tie_word_embeddings"],
        "global_batch": args.batch, "seq_len": context, "context_limit": shape["max_position_embeddings"],
        "block_size": BLOCK_SIZE, "cache_pages": llm.cache.num_blocks, "token_budget": TOKEN_BUDGET,
        "prefill_tokens": prefill_tokens, "captured_decode": True, "tuned_products": not args.no_tune,
        "parallelism": "single GPU",
    }

    if args.serve:
        served = serve_run(llm, vocab, seed=7)             # the first pass captures the graphs and warms the library
        if llm.stats is not None:
            llm.stats.flush()                              # forget the first pass
        served = serve_run(llm, vocab, seed=7)
        config.update({"global_batch": SERVE["requests"], "seq_len": "prompts U[128,2048], outputs U[32,256]",
                       "prefill_tokens": served["prompt_tokens"]})
        line = {
            "metric": f"output tok/s serving 64 requests at once ({preset['model']} shape)",
            "value": round(served["output_tokens"] / served["duration_s"], 1), "unit": "tok/s", "n_gpus": 1,
            "steps": served["steps"], "warmup": 0,
            "ms_per_step": round(served["duration_s"] * 1e3 / served["steps"], 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic", "config": config,
            "serve": {
                "duration_s": round(served["duration_s"], 4), "requests": SERVE["requests"],
                "request_throughput": round(SERVE["requests"] / served["duration_s"], 2),
                "output_tokens": served["output_tokens"], "prompt_tokens": served["prompt_tokens"],
                "total_tok_s": round((served["output_tokens"] + served["prompt_tokens"]) / served["duration_s"], 1),
                "preemptions": served["preemptions"],
                "ttft_ms": {k: round(v, 2) for k, v in served["ttft_ms"].items()},
                "tpot_ms": {k: round(v, 3) for k, v in served["tpot_ms"].items()},
                "e2e_latency_ms": {k: round(v, 1) for k, v in served["e2e_latency_ms"].items()},
            },
        }
        if llm.stats is not None:
            llm.stats._read(keep=0)
            line["serve"]["step_ms"] = {kind: {k: round(v, 3) for k, v in row.items()}
                                        for kind, row in llm.stats.summary().items()}
        print(json.dumps(line), flush=True)
        return 0

    t_prefill = prefill_run(llm, prefill_tokens, TOKEN_BUDGET, vocab)
    T = prefill_tokens
    flops = 2.0 * T * body + 2.0 * head + 2.0 * T * T * shape["num_attention_heads"] * shape["head_dim"] * layers_run
    prefill = {"value": round(T / t_prefill, 1), "tokens": T, "ms": round(t_prefill * 1e3, 3),
               "frac": round(flops / t_prefill / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}

    step_s, mean_ctx = decode_run(llm, args.batch, context, args.steps, args.warmup, vocab, seed=1)
    kv_per_token = 2 * shape["num_key_value_heads"] * shape["head_dim"] * layers_run * elem
    weight_bytes = (body + head) * elem
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_per_token
    achieved = step_bytes / step_s / 1e9
    points = {}
    for b in points_at:
        s, _ = decode_run(llm, b, context, min(args.steps, 128), min(args.warmup, 8), vocab, seed=2 + b)
        points[f"decode_b{b}"] = round(b / s, 1)

    line = {
        "metric": f"decode tok/s at batch {args.batch} after a {context:,}-token prompt ({preset['model']} shape)",
        "value": round(args.batch / step_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": config,
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
