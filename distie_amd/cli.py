"""Command line: `python -m distie_amd.cli generate|replay|random-model ...`.

The reference has no generation command (its entry is a gRPC server:
worker/src/worker/main.py:11-23); option names follow its scripts and environment
variables where it has them: --model, --device, --dtype {auto,fp32,bf16}, --max-new-tokens,
--num-blocks, --out (benchmarks/correctness/hf_parity.py:168-182), WORKER_MAX_SEQS,
WORKER_TOKEN_BUDGET, WORKER_NUM_BLOCKS, WORKER_DECODE_GRAPHS, WORKER_STEP_STATS
(worker/src/inference/torch_engine.py:212-226) as --max-seqs, --token-budget,
--num-blocks, --no-decode-graphs, --step-stats; the variables themselves are read too.
Prompts are token ids: a tokenizer is not part of this engine.
"""

from __future__ import annotations

import argparse
import json
import logging
import sys
from pathlib import Path


def _engine_options(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("--model", help="folder with config.json and model.safetensors")
    parser.add_argument("--device", default="cuda:0")
    parser.add_argument("--dtype", default="auto", choices=["auto", "fp32", "bf16", "float32", "bfloat16"])
    parser.add_argument("--random-weights", action="store_true", help="ignore the folder's weights; draw them from --seed")
    parser.add_argument("--config-json", type=Path, help="a config.json to build a random-weights model from")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--block-size", type=int, default=None)
    parser.add_argument("--num-blocks", type=int, default=None)
    parser.add_argument("--max-seqs", type=int, default=None)
    parser.add_argument("--token-budget", type=int, default=None)
    parser.add_argument("--no-decode-graphs", action="store_true")
    parser.add_argument("--graph-buckets", default=None, metavar="SIZES",
                        help="batch sizes that get a captured decode step, comma-separated (default: 1,2,4,8, then "
                             "every multiple of 8 up to --max-seqs)")
    parser.add_argument("--graph-tokens", type=int, default=None, metavar="N",
                        help="steps that hold a portion of a prompt replay a captured step too if they bring at most "
                             "N tokens (default 96; 0: only decode steps are captured)")
    parser.add_argument("--step-stats", type=int, default=None, help="log a time breakdown every N steps")
    parser.add_argument("--no-packed-weights", action="store_true",
                        help="no second copy of the weights in the matrix cores' order (half the weight memory, "
                             "slower decode)")
    parser.add_argument("--packed-weights", default=None, metavar="ROLES",
                        help="packed copies only for the products the model's parts name so, comma-separated "
                             "(this architecture's parts name qkv, attn_out, gate_up, down, head)")
    parser.add_argument("--gpu-mem-fraction", type=float, default=None,
                        help="without --num-blocks: pages of the cache until this share of the card's memory is in use")
    parser.add_argument("--tune-products", action="store_true",
                        help="at start, let the library time its kernels for the products of a full portion and of 65 to 192 rows "
                             "(more with a larger --max-seqs)")


def _build(args):
    from . import LLM
    from .config import EngineConfig

    engine = EngineConfig.from_env(
        dtype=args.dtype, block_size=args.block_size, num_blocks=args.num_blocks, max_seqs=args.max_seqs,
        token_budget=args.token_budget, use_graphs=False if args.no_decode_graphs else None,
        graph_buckets=tuple(int(b) for b in args.graph_buckets.split(",") if b) if args.graph_buckets else None,
        graph_tokens=args.graph_tokens, step_stats=args.step_stats, seed=args.seed, packed_weights=False if args.no_packed_weights else (
            tuple(r for r in args.packed_weights.split(",") if r) if args.packed_weights else None),
        gpu_mem_fraction=args.gpu_mem_fraction,
        tune_products=True if args.tune_products else None)
    config = json.loads(args.config_json.read_text()) if args.config_json else None
    if args.model is None and config is None:
        raise SystemExit("give --model DIR, or --config-json FILE with --random-weights")
    return LLM(args.model, config=config, random_weights=args.random_weights or args.model is None,
               seed=args.seed, device=args.device, engine=engine)


def _prompts(args) -> list:
    prompts = []
    for text in args.prompt_ids or []:
        prompts.append([int(t) for t in text.replace(",", " ").split()])
    if args.prompts:
        data = json.loads(args.prompts.read_text())
        for item in data:
            if not isinstance(item, list) or not all(isinstance(t, int) for t in item):
                raise SystemExit("--prompts must hold a JSON list of lists of token ids")
            prompts.append(item)
    if not prompts:
        raise SystemExit("give --prompt-ids '1 2 3' (may repeat) or --prompts FILE")
    return prompts


def cmd_generate(args) -> int:
    from .sampling import SamplingParams

    llm = _build(args)
    params = SamplingParams(max_new_tokens=args.max_new_tokens, temperature=args.temperature, seed=args.seed,
                            ignore_eos=args.ignore_eos)
    outputs = llm.generate(_prompts(args), params)
    report = [{"request_id": o.request_id, "prompt_tokens": len(o.prompt_token_ids), "token_ids": o.token_ids,
               "finish_reason": o.finish_reason, "time_to_first_token_ms": round(o.time_to_first_token_ms, 3),
               "total_latency_ms": round(o.total_latency_ms, 3), "preemptions": o.preemptions} for o in outputs]
    text = json.dumps(report, indent=1)
    if args.out:
        args.out.write_text(text)
    print(text)
    return 0


def cmd_random_model(args) -> int:
    from .config import config_from_dict
    from .weights import write_random_model

    config = config_from_dict(json.loads(args.config_json.read_text()))
    dtype = {"fp32": "float32", "bf16": "bfloat16"}.get(args.dtype, args.dtype)
    path = write_random_model(config, args.out, args.seed, dtype, std=args.std)
    print(path)
    return 0


def cmd_replay(args) -> int:
    import runpy

    script = Path(__file__).resolve().parents[1] / "bin" / "trace_run"
    sys.argv = [str(script)] + args.rest
    runpy.run_path(str(script), run_name="__main__")
    return 0


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="distie_amd", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--log-level", default="WARNING")
    sub = parser.add_subparsers(dest="command", required=True)
    gen = sub.add_parser("generate", help="generate tokens for prompts given as token ids")
    _engine_options(gen)
    gen.add_argument("--prompt-ids", action="append", help="token ids, separated by spaces or commas")
    gen.add_argument("--prompts", type=Path, help="JSON file: a list of lists of token ids")
    gen.add_argument("--max-new-tokens", type=int, default=16)
    gen.add_argument("--temperature", type=float, default=0.0)
    gen.add_argument("--ignore-eos", action="store_true")
    gen.add_argument("--out", type=Path, help="write the JSON report here")
    gen.set_defaults(run=cmd_generate)
    rnd = sub.add_parser("random-model", help="write a model folder with random weights")
    rnd.add_argument("--config-json", type=Path, required=True)
    rnd.add_argument("--out", type=Path, required=True)
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--dtype", default="float32", choices=["float32", "bfloat16", "fp32", "bf16"])
    rnd.add_argument("--std", type=float, default=0.02)
    rnd.set_defaults(run=cmd_random_model)
    rep = sub.add_parser("replay", help="bin/trace_run: feed given tokens step by step, write logits")
    rep.add_argument("rest", nargs=argparse.REMAINDER)
    rep.set_defaults(run=cmd_replay)
    args = parser.parse_args(argv)
    logging.basicConfig(level=getattr(logging, args.log_level.upper(), logging.WARNING),
                        format="%(asctime)s %(name)s %(levelname)s %(message)s")
    return args.run(args)


if __name__ == "__main__":
    sys.exit(main())
