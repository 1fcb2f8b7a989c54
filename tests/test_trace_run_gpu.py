"""bin/trace_run as a user drives it: a subprocess, steps on standard input, logits in files;
and greedy generation through the entry point and the command line."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen2 as plain
from engine_util import check_logits, make_model_dir, oracle, random_ids

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]


class Replay:
    def __init__(self, model, dtype, out, max_tokens):
        self.out = Path(out)
        self.proc = subprocess.Popen(
            [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model), "--dtype", dtype,
             "--out", str(out), "--max-tokens", str(max_tokens)],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.step = 0
        self.rows = {}          # step -> what its sidecar says of the rows of its logits

    def run(self, entries, end=()):
        record = {"step": self.step, "entries": entries, "end": list(end)}
        self.proc.stdin.write(json.dumps(record) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline().strip()
        assert line == f"done {self.step}", line
        path = self.out / f"{self.step}.f32"
        self.step += 1
        wanted = sum(len(e["want"]) for e in entries)
        if not wanted:
            assert not path.exists()
            return None
        data = np.fromfile(path, dtype="<f4")
        self.rows[self.step - 1] = json.loads((self.out / f"{self.step - 1}.json").read_text())
        return torch.from_numpy(data.reshape(wanted, -1))

    def close(self):
        self.proc.stdin.close()
        assert self.proc.wait(timeout=60) == 0
        # the index of the whole run repeats the sidecars
        index = json.loads((self.out / "index.json").read_text())
        assert index["steps"] == {str(step): side["rows"] for step, side in self.rows.items()}
        assert all(side["vocab"] == index["vocab"] and side["step"] == step for step, side in self.rows.items())


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16"), ("C", "bfloat16")])
def test_replay_mixed_trace(tmp_path, name, dtype):
    cfg = {"A": plain.TINY_A, "B": plain.TINY_B, "C": plain.TINY_C}[name]
    tdtype = getattr(torch, dtype)
    folder, weights = make_model_dir(tmp_path, cfg, seed=31, dtype=tdtype)
    lengths = {"p": 100, "q": 64, "r": 37, "s": 90, "t": 50}
    reqs = {r: random_ids(cfg, n, 40 + n) for r, n in lengths.items()}
    # four live at most: the largest four, each rounded up to 64
    max_tokens = sum(-(-n // 64) * 64 for n in sorted(lengths.values())[-4:])
    replay = Replay(folder, dtype, tmp_path / "out", max_tokens)
    got = {r: [] for r in reqs}
    at = {r: 0 for r in reqs}
    waiting, live = list(reqs), []
    gen = torch.Generator().manual_seed(9)
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries = []
        for r in live:
            left = len(reqs[r]) - at[r]
            n = 1 if left <= 32 else min(left - 32, int(torch.randint(2, 30, (1,), generator=gen)))
            want = list(range(n)) if r != "q" else [n - 1]
            entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + n], "want": want})
        logits = replay.run(entries, end=[e["id"] for e in entries if at[e["id"]] + len(e["tokens"]) == len(reqs[e["id"]])])
        # the index names (request, position) of every row, in the order of the entries and of `want`
        assert replay.rows[replay.step - 1]["rows"] == [[e["id"], at[e["id"]] + w] for e in entries for w in e["want"]]
        assert replay.rows[replay.step - 1]["vocab"] == cfg["vocab_size"]
        row = 0
        for e in entries:
            r, n = e["id"], len(e["tokens"])
            got[r].append((at[r], e["want"], logits[row:row + len(e["want"])]))
            row += len(e["want"])
            at[r] += n
        live = [r for r in live if at[r] < len(reqs[r])]
    replay.close()
    for r, pieces in got.items():
        want_all = oracle(weights, cfg, reqs[r])
        rows = [begin + w for begin, want, _ in pieces for w in want]
        stacked = torch.cat([l for _, _, l in pieces])
        # compare at the rows that were asked for
        diff = (stacked - want_all[rows]).abs().max().item()
        scale = want_all.abs().max().item()
        assert diff < (1e-4 if dtype == "float32" else scale / 16), (r, diff)


def test_replay_step_without_wanted_rows_and_a_pause(tmp_path):
    cfg = plain.TINY_A
    folder, weights = make_model_dir(tmp_path, cfg, seed=32)
    ids = random_ids(cfg, 20, 1)
    other = random_ids(cfg, 6, 2)
    replay = Replay(folder, "float32", tmp_path / "out", 128)
    assert replay.run([{"id": "a", "tokens": ids[:7], "want": []}]) is None
    replay.run([{"id": "b", "tokens": other, "want": [5]}], end=["b"])          # a sits out
    logits = replay.run([{"id": "a", "tokens": ids[7:], "want": [0, 12]}], end=["a"])
    want = oracle(weights, cfg, ids)
    assert (logits - want[[7, 19]]).abs().max() < 1e-4
    assert replay.rows[2]["rows"] == [["a", 7], ["a", 19]] and 0 not in replay.rows
    # a name that was given back names a new request; a request may be ended by a step it sits out
    replay.run([{"id": "a", "tokens": other[:4], "want": []}, {"id": "c", "tokens": ids[:3], "want": []}])
    again = replay.run([{"id": "a", "tokens": other[4:], "want": [1]}], end=["c"])
    assert (again - oracle(weights, cfg, other)[[5]]).abs().max() < 1e-4
    last = replay.run([{"id": "c", "tokens": other, "want": [5]}], end=["a", "c"])
    assert (last - oracle(weights, cfg, other)[[5]]).abs().max() < 1e-4
    replay.close()


def test_generation_through_the_entry_point_and_the_command_line(tmp_path):
    from distie_amd import LLM, SamplingParams

    cfg = plain.TINY_B
    folder, weights = make_model_dir(tmp_path, cfg, seed=33)
    prompts = [random_ids(cfg, n, 60 + n) for n in (1, 9, 23, 40)]

    def greedy(prompt, n):
        ids = list(prompt)
        for _ in range(n):
            ids.append(int(oracle(weights, cfg, ids)[-1].argmax()))
        return ids[len(prompt):]

    want = [greedy(p, 12) for p in prompts]
    for graphs in (False, True):
        llm = LLM(folder, dtype="fp32", block_size=8, num_blocks=32, token_budget=7, use_graphs=graphs)
        outs = llm.generate(prompts, SamplingParams(max_new_tokens=12))
        assert [o.token_ids for o in outs] == want, f"graphs={graphs}"
        llm.cache.check()
    (tmp_path / "prompts.json").write_text(json.dumps(prompts))
    done = subprocess.run(
        [sys.executable, "-m", "distie_amd.cli", "generate", "--model", str(folder), "--dtype", "fp32",
         "--prompts", str(tmp_path / "prompts.json"), "--max-new-tokens", "12", "--block-size", "8",
         "--num-blocks", "32", "--token-budget", "7", "--out", str(tmp_path / "report.json")],
        cwd=str(ROOT), capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stderr
    report = json.loads((tmp_path / "report.json").read_text())
    assert [r["token_ids"] for r in report] == want


def test_tuned_library_products(tmp_path):
    """`tune_products`: the engine starts with one full portion while the library's candidate kernels are
    timed for the large products, and with steps of 96, 128, 160 and 192 rows for the products of large decode
    batches and short portions; afterwards new shapes take the choice of their class of 32 rows if one of its
    shapes was timed, else the library's first. Results stay within the bounds, with whatever kernels were picked."""
    from distie_amd import LLM
    from distie_amd.engine.batch import StepEntry
    from engine_util import check_logits

    cfg = plain.TINY_C
    folder, weights = make_model_dir(tmp_path, cfg, seed=5, dtype=torch.bfloat16)
    llm = LLM(folder, dtype="bf16", block_size=16, num_blocks=40, token_budget=400, tune_products=True,
              packed_weights=False)                 # without packed copies 400 rows are the library's
    made, timed = llm.ops.library_plans()
    assert timed >= 1 and not llm.ops._tuning       # the full portion's products were timed, and tuning is off again
    assert llm.ops.library_timed_rows == 192 and not llm.ops.captured
    for n, seed in ((160, 6), (150, 7), (96, 8)):   # a timed shape, another of its class, a timed shape
        ids = random_ids(cfg, n, seed)
        logits = llm.step([StepEntry("c", ids, list(range(n)))]).float().cpu()
        llm.finish("c")
        check_logits(logits, weights, cfg, ids, torch.bfloat16, folder)
    assert llm.ops.library_plans()[1] == timed
    ids = random_ids(cfg, 300, 4)
    logits = llm.step([StepEntry("a", ids, list(range(len(ids))))]).float().cpu()
    llm.finish("a")
    assert llm.ops.library_plans()[1] == timed      # another number of rows: not timed
    check_logits(logits, weights, cfg, ids, torch.bfloat16, folder)
    ids = random_ids(cfg, 400, 5)
    logits = llm.step([StepEntry("b", ids, list(range(len(ids))))]).float().cpu()
    llm.finish("b")
    check_logits(logits, weights, cfg, ids, torch.bfloat16, folder)     # the timed shapes
    llm.cache.check()


def test_captured_steps_per_class_of_context_length(tmp_path, monkeypatch):
    """A captured decode step is made for a longest context (decode attention cuts the keys into runs by
    it), so a bucket holds one graph per class of length; contexts that grow through several classes,
    alone and three at a time, give the logits of the whole sequences."""
    from distie_amd import LLM
    from distie_amd.engine.batch import StepEntry
    from distie_amd.parts.attention import Attention
    from engine_util import check_logits

    monkeypatch.setattr(Attention, "FIRST_CONTEXT", 32)
    cfg = plain.TINY_C
    folder, weights = make_model_dir(tmp_path, cfg, seed=8, dtype=torch.bfloat16)
    llm = LLM(folder, dtype="bf16", block_size=16, num_blocks=40, max_seqs=4)
    assert [llm.model.capture_context(n, 256) for n in (1, 33, 49, 97, 200)] == [32, 48, 64, 128, 256]
    seqs = {name: random_ids(cfg, n, 17 + n) for name, n in (("a", 150), ("b", 70), ("c", 101))}
    got = {name: [] for name in seqs}
    starts = {"a": 20, "b": 1, "c": 40}
    for name, ids in seqs.items():                 # the first tokens as a portion, uncaptured
        n = starts[name]
        got[name].append(llm.step([StepEntry(name, ids[:n], list(range(n)))]).float().cpu())
    at = dict(starts)
    while any(at[name] < len(ids) for name, ids in seqs.items()):
        live = [name for name, ids in seqs.items() if at[name] < len(ids)]
        logits = llm.step([StepEntry(name, [seqs[name][at[name]]], [0]) for name in live]).float().cpu()
        for row, name in enumerate(live):
            got[name].append(logits[row:row + 1])
            at[name] += 1
    made = llm.runner.graphs.captured_contexts
    assert {size for size, _ in made} == {1, 2, 4} and len({limit for _, limit in made}) >= 5, made
    for name, ids in seqs.items():
        llm.finish(name)
        check_logits(torch.cat(got[name]), weights, cfg, ids, torch.bfloat16, folder)
    llm.cache.check()


def test_engines_made_and_dropped_one_after_the_other(tmp_path):
    """Every engine captures its decode steps anew while the remains of the one before (pinned buffers,
    graphs) wait for the garbage collector: their destructors must not run inside a capture."""
    from distie_amd import LLM, SamplingParams

    cfg = plain.TINY_A
    folder, weights = make_model_dir(tmp_path, cfg, seed=3)
    prompts = [random_ids(cfg, n, 80 + n) for n in (3, 11, 6)]
    first = None
    for _ in range(8):
        llm = LLM(folder, dtype="fp32", block_size=16, num_blocks=24, max_seqs=4)
        outs = [o.token_ids for o in llm.generate(prompts, SamplingParams(max_new_tokens=10))]
        assert llm.runner.graphs.captured and llm.steps_ahead > 0
        first = first or outs
        assert outs == first
        llm.circular = llm            # a cycle: only the garbage collector can free this engine
