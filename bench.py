"""Decode and prefill throughput of the Qwen2.5-1.5B-shaped model on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole engine (schedule, metadata, captured forward, sampling,
completion) at batch 8, each request with a 2,048-token context behind it. One JSON line on
standard output: `value` = decoded tokens a second, plus `prefill` (one 2,048-token prompt),
`roofline` (bytes the decode step has to read / its time, against 8 TB/s) and `points`
(batch 1 and batch 64). Random weights N(0, 0.02), seeded uniform token ids.
"""

import argparse
import json
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

# the layer sizes of Qwen2.5-1.5B, the configuration the headline figures are quoted on
SHAPE = {
    "architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 28, "hidden_size": 1536,
    "num_attention_heads": 12, "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 8960,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
    "use_sliding_window": False, "max_position_embeddings": 4096, "hidden_act": "silu",
}
CONTEXT = 2048
PREFILL_TOKENS = 2048
BLOCK_SIZE = 16
TOKEN_BUDGET = 2048


def prompts(batch, length, vocab, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(batch)]


def linear_params(c):
    q = c["num_attention_heads"] * c["head_dim"]
    kv = c["num_key_value_heads"] * c["head_dim"]
    per_layer = c["hidden_size"] * (q + 2 * kv) + q * c["hidden_size"] + 3 * c["hidden_size"] * c["intermediate_size"]
    return per_layer * c["num_hidden_layers"], c["vocab_size"] * c["hidden_size"]


def decode_run(llm, batch, steps, warmup, vocab, seed):
    """-> (seconds per step, mean context over the timed steps)"""
    import torch

    from distie_amd import SamplingParams

    # requests admitted early decode while later prompts are still prefilled: leave room for that
    params = SamplingParams(max_new_tokens=warmup + steps + 2 * batch + 8, ignore_eos=True)
    ids = [llm.add_request(p, params) for p in prompts(batch, CONTEXT, vocab, seed)]
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
    # keys a decode step reads for a request: everything cached before it, plus its own token
    mean_ctx = sum(before) / len(before) + (steps - 1) / 2.0
    for i in ids:
        llm.abort(i)
    while llm.has_work():
        llm.run_step()
    return elapsed / steps, mean_ctx


def prefill_run(llm, vocab, repeats=3):
    import torch

    from distie_amd import StepEntry

    best = None
    for r in range(repeats + 1):
        ids = prompts(1, PREFILL_TOKENS, vocab, 100 + r)[0]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = llm.step([StepEntry(f"prefill-{r}", ids, [PREFILL_TOKENS - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        llm.finish(f"prefill-{r}")
        if r > 0:                                          # the first run warms up
            best = dt if best is None else min(best, dt)
    return best


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=256)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    parser.add_argument("--no-points", action="store_true", help="skip batch 1 and batch 64")
    parser.add_argument("--no-tune", action="store_true",
                        help="leave the choice of the library's product kernels (prefill) to the library's defaults")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not supported (this engine has no multi-GPU path)")
        return 2

    import torch

    from distie_amd import LLM

    shape = dict(SHAPE)
    layers_run = args.layers or shape["num_hidden_layers"]
    shape["num_hidden_layers"] = layers_run
    shape["max_position_embeddings"] = max(shape["max_position_embeddings"], CONTEXT + args.warmup + args.steps + 2 * 64 + 8)
    max_batch = 64 if not args.no_points else args.batch
    tokens_per_request = CONTEXT + args.warmup + args.steps + 2 * max_batch + 8
    pages = max_batch * -(-tokens_per_request // BLOCK_SIZE) + 8
    llm = LLM(config=shape, random_weights=True, seed=0, dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=pages,
              max_seqs=max_batch, token_budget=TOKEN_BUDGET, use_graphs=True, tune_products=not args.no_tune)
    vocab = shape["vocab_size"]
    elem = 2 if args.dtype == "bf16" else 4

    t_prefill = prefill_run(llm, vocab)
    body, head = linear_params(shape)
    T = PREFILL_TOKENS
    flops = 2.0 * T * body + 2.0 * head + 2.0 * T * T * shape["num_attention_heads"] * shape["head_dim"] * layers_run
    prefill = {"value": round(T / t_prefill, 1), "tokens": T, "ms": round(t_prefill * 1e3, 3),
               "frac": round(flops / t_prefill / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}

    step_s, mean_ctx = decode_run(llm, args.batch, args.steps, args.warmup, vocab, seed=1)
    kv_per_token = 2 * shape["num_key_value_heads"] * shape["head_dim"] * layers_run * elem
    weight_bytes = (body + head) * elem
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_per_token
    achieved = step_bytes / step_s / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):
            s, _ = decode_run(llm, b, min(args.steps, 128), min(args.warmup, 8), vocab, seed=2 + b)
            points[f"decode_b{b}"] = round(b / s, 1)

    line = {
        "metric": "decode tok/s at batch 8 after a 2,048-token prompt (Qwen2.5-1.5B shape)",
        "value": round(args.batch / step_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {
            "model": "Qwen2.5-1.5B-shaped, random weights N(0,0.02)", "layers": SHAPE["num_hidden_layers"],
            "layers_run": layers_run, "hidden": shape["hidden_size"], "heads": shape["num_attention_heads"],
            "kv_heads": shape["num_key_value_heads"], "head_dim": shape["head_dim"],
            "intermediate": shape["intermediate_size"], "vocab": vocab, "tied_head": True,
            "global_batch": args.batch, "seq_len": CONTEXT, "context_limit": shape["max_position_embeddings"],
            "block_size": BLOCK_SIZE, "token_budget": TOKEN_BUDGET, "prefill_tokens": PREFILL_TOKENS,
            "captured_decode": True, "tuned_products": not args.no_tune, "parallelism": "single GPU",
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
