"""Configurations and traces drawn at random, through `LLM.step` against the plain implementation: head sizes
from 16 to 256 (one that is no multiple of 16), one to four kv heads with one to eight query heads each,
widths and vocabularies that are no multiple of 8, one to three layers, windows that begin at any layer, pages
of 4 to 64 tokens, with and without captured steps; up to four live requests in portions of 2 to 150 tokens
beside single tokens, requests that sit a step out, want no row, their last, or a few anywhere, on so few pages
that they are used again. The two tiny configurations and the sizes at the kernels' edges are stated elsewhere
(tests/test_engine_gpu.py); this draws what nobody thought of stating."""

import random

import pytest
import torch

import plain_qwen2 as plain
from distie_amd import LLM, StepEntry
from engine_util import make_model_dir

pytestmark = pytest.mark.gpu


def drawn_config(rng):
    while True:
        head_dim = rng.choice([16, 32, 40, 48, 64, 80, 96, 112, 128, 256])
        kv_heads = rng.choice([1, 1, 2, 3, 4])
        heads = kv_heads * rng.choice([1, 2, 3, 5, 6, 7, 8])
        if heads * head_dim <= 1536:
            break
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": rng.randint(1, 3),
           "hidden_size": heads * head_dim, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
           "head_dim": head_dim, "intermediate_size": rng.choice([8, 24, 100, 172, 250, 333, 512]),
           "vocab_size": rng.choice([9, 77, 256, 323, 1000, 4097]), "rope_theta": rng.choice([10000.0, 1e6, 500.0]),
           "rms_norm_eps": rng.choice([1e-6, 1e-5, 1e-3]), "tie_word_embeddings": rng.random() < 0.5,
           "max_position_embeddings": 512, "hidden_act": "silu"}
    if rng.random() < 0.5:
        cfg.update(use_sliding_window=True, sliding_window=rng.choice([5, 17, 40, 64, 100]),
                   max_window_layers=rng.randint(0, cfg["num_hidden_layers"]))
    return cfg


@pytest.mark.parametrize("case", range(24))
def test_a_drawn_configuration_and_trace(tmp_path, case):
    rng = random.Random(1000 + case)
    cfg = drawn_config(rng)
    # bfloat16 at a width of a few dozen is noise at single positions (the same rows whole and token by token,
    # measured); the serving precision is drawn only where the width carries it
    dtype = rng.choice(["fp32", "bf16"]) if cfg["hidden_size"] >= 128 else "fp32"
    block = rng.choice([4, 8, 16, 16, 32, 64])
    lengths = [rng.randint(2, 200) for _ in range(5)]
    act = torch.float32 if dtype == "fp32" else torch.bfloat16
    print(f"case {case}: {dtype}, pages of {block}, {cfg}, lengths {lengths}", flush=True)
    folder, weights = make_model_dir(tmp_path, cfg, seed=case, std=min(0.3, 2.0 / cfg["hidden_size"] ** 0.5), dtype=act)
    pages = 2 * (-(-max(lengths) // block)) + 3
    llm = LLM(folder, dtype=dtype, block_size=block, num_blocks=pages, max_seqs=4, graph_tokens=rng.choice([0, 48]),
              use_graphs=rng.random() < 0.7, lookahead=False, max_model_len=512)
    waiting = [(f"r{i}", torch.randint(0, cfg["vocab_size"], (n,),
                                       generator=torch.Generator().manual_seed(case * 10 + i)).tolist())
               for i, n in enumerate(lengths)]
    live, at, rows = {}, {}, {}
    while waiting or live:
        while waiting and len(live) < 4 and \
                sum(-(-len(ids) // block) for ids in live.values()) + -(-len(waiting[0][1]) // block) <= pages:
            rid, ids = waiting.pop(0)
            live[rid], at[rid], rows[rid] = ids, 0, []
        entries, budget = [], rng.choice([48, 200, 400])
        for rid, ids in live.items():
            if rng.random() < 0.15 or budget < 2:
                continue                                                # sits this step out
            if at[rid] > 0 and rng.random() < 0.5:
                n = 1
            else:
                n = min(len(ids) - at[rid], budget, rng.choice((2, 3, 5, 8, 13, 20, 64, 150)))
            k = rng.random()
            want = [] if k < 0.2 else ([n - 1] if k < 0.6 else sorted(rng.sample(range(n), min(n, rng.randint(1, 4)))))
            entries.append((rid, n, want))
            budget -= n
        if not entries:
            continue
        entries.sort(key=lambda e: e[1] != 1)
        out = llm.step([StepEntry(rid, live[rid][at[rid]:at[rid] + n], want) for rid, n, want in entries])
        logits = out.float().cpu() if out is not None else torch.zeros(0, cfg["vocab_size"])
        row = 0
        for rid, n, want in entries:
            for w in want:
                rows[rid].append((at[rid] + w, logits[row]))
                row += 1
            at[rid] += n
        assert row == logits.shape[0]
        for rid in [r for r in live if at[r] == len(live[r])]:
            ids = live.pop(rid)
            llm.finish(rid)
            if not rows[rid]:
                continue
            want = plain.forward(weights, cfg, ids, torch.float64).float()
            diff = torch.stack([r for _, r in rows[rid]]) - want[[p for p, _ in rows[rid]]]
            scale = want.abs().max().item()
            if dtype == "fp32":
                assert diff.abs().max().item() < 1e-4 * max(1.0, scale), (rid, diff.abs().max().item(), scale)
            else:
                assert diff.abs().max().item() < scale / 16, (rid, diff.abs().max().item(), scale)
                assert diff.pow(2).mean().sqrt().item() < scale / 64, rid
    llm.cache.check()
    assert all(f == pages for f in llm.cache.free_pages()) and llm.cache.slots.num_free == llm.cache.num_slots
    llm.close()
