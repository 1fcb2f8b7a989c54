"""The engine on the GPU against the plain implementation: whole requests, decoding,
portions of changing size, mixed batches with page reuse; float32 and bfloat16."""

import pytest
import torch

import plain_qwen2 as plain
from distie_amd.engine.batch import StepEntry
from engine_util import build_runner, check_logits, make_model_dir, random_ids, replay_cut, replay_whole

pytestmark = pytest.mark.gpu

CONFIGS = {"A": (plain.TINY_A, 4), "B": (plain.TINY_B, 8), "C": (plain.TINY_C, 16)}
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from distie_amd.kernels.hip_ops import HipOps

    return HipOps("cuda:0")


@pytest.fixture(scope="module", params=[(c, d) for c in sorted(CONFIGS) for d in DTYPES])
def setup(request, tmp_path_factory):
    name, dtype_name = request.param
    cfg, block = CONFIGS[name]
    dtype = DTYPES[dtype_name]
    # the file holds what the engine keeps: bfloat16 weights for the bfloat16 run
    folder, weights = make_model_dir(tmp_path_factory.mktemp(f"m{name}{dtype_name}"), cfg, seed=11, dtype=dtype)
    return cfg, block, folder, weights, dtype


def test_whole(setup, ops):
    cfg, block, folder, weights, dtype = setup
    runner = build_runner(folder, ops, dtype, block_size=block)
    ids = random_ids(cfg, 100, 1)
    check_logits(replay_whole(runner, "a", ids), weights, cfg, ids, dtype, folder)
    # the first tokens of a sequence
    check_logits(replay_whole(runner, "b", ids[:3]), weights, cfg, ids[:3], dtype, folder)
    check_logits(replay_whole(runner, "c", ids[:1]), weights, cfg, ids[:1], dtype, folder)
    runner.cache.check()


def test_prompt_then_last_32_one_by_one(setup, ops):
    cfg, block, folder, weights, dtype = setup
    runner = build_runner(folder, ops, dtype, block_size=block)
    ids = random_ids(cfg, 120, 2)
    check_logits(replay_cut(runner, "a", ids, [88]), weights, cfg, ids, dtype, folder)


@pytest.mark.parametrize("packed", [False, ("qkv", "down"), ("gate_up", "attn_out", "head")],
                         ids=["none", "qkv+down", "gate_up+attn_out+head"])
def test_without_packed_weights(setup, packed):
    """The products on the stored layout (no second copy of the weights), rotation and activation as
    kernels of their own, for every weight or for some: the same requests, the same bounds."""
    from distie_amd.kernels.hip_ops import HipOps

    cfg, block, folder, weights, dtype = setup
    plain_ops = HipOps("cuda:0", packed_weights=packed)
    runner = build_runner(folder, plain_ops, dtype, block_size=block)
    ids = random_ids(cfg, 120, 2)
    check_logits(replay_cut(runner, "a", ids, [40, 20, 17, 11]), weights, cfg, ids, dtype, folder)
    copies = ("_distie_packed", "_distie_gated", "_distie_rotary")
    has = lambda t: any(hasattr(t, name) for name in copies)
    wanted = set(packed or ())
    by_role = {"qkv": [b.mixer.qkv_weight for b in runner.model.blocks],
               "attn_out": [b.mixer.out_weight for b in runner.model.blocks],
               "gate_up": [b.feed_forward.gate_up_weight for b in runner.model.blocks],
               "down": [b.feed_forward.down_weight for b in runner.model.blocks],
               "head": [runner.model.head]}
    for role, tensors in by_role.items():
        # bfloat16 weights with rows of whole 16-byte pieces get the copy where it is asked for; others never
        for t in tensors:
            assert has(t) == (role in wanted and dtype == torch.bfloat16 and t.shape[1] % 8 == 0), role


@pytest.mark.parametrize("cuts", [[2, 3, 5, 7, 2, 11, 4, 33, 2, 2, 19], [64, 2, 2, 2, 30], [1, 1, 2, 70, 9]])
def test_portions(setup, ops, cuts):
    cfg, block, folder, weights, dtype = setup
    runner = build_runner(folder, ops, dtype, block_size=block)
    ids = random_ids(cfg, 110, 3)
    check_logits(replay_cut(runner, "a", ids, cuts), weights, cfg, ids, dtype, folder)


def test_mixed_with_page_reuse(setup, ops):
    cfg, block, folder, weights, dtype = setup
    lengths = [90, 120, 45, 101, 64, 77, 33]
    pages = sum(-(-n // block) for n in sorted(lengths)[-4:])
    runner = build_runner(folder, ops, dtype, block_size=block, num_blocks=pages, num_slots=4)
    # poison the cache: stale contents must never be read
    for group in runner.cache.groups:
        for slab in group.tensors.values():
            slab.fill_(float("nan"))
    reqs = {f"r{i}": random_ids(cfg, n, 10 + i) for i, n in enumerate(lengths)}
    got = {r: [] for r in reqs}
    at = {r: 0 for r in reqs}
    waiting, live = list(reqs), []
    gen = torch.Generator().manual_seed(5)
    step = 0
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries = []
        for r in live:
            left = len(reqs[r]) - at[r]
            n = 1 if left <= 32 else min(left - 32, int(torch.randint(2, 40, (1,), generator=gen)))
            if step % 4 == 3 and r == live[0] and len(live) > 1:
                continue
            entries.append(StepEntry(r, reqs[r][at[r]:at[r] + n], list(range(n))))
        logits = runner.step(entries)
        row = 0
        for e in entries:
            n = len(e.tokens)
            got[e.request_id].append(logits[row:row + n].float().cpu())
            row += n
            at[e.request_id] += n
        for r in list(live):
            if at[r] == len(reqs[r]):
                runner.finish(r)
                live.remove(r)
        runner.cache.check()
        step += 1
    for r in reqs:
        check_logits(torch.cat(got[r]), weights, cfg, reqs[r], dtype, folder)
    assert all(f == pages for f in runner.cache.free_pages())


def test_long_decoding(setup, ops):
    cfg, block, folder, weights, dtype = setup
    n = min(cfg["max_position_embeddings"], 250)
    runner = build_runner(folder, ops, dtype, block_size=block, num_blocks=-(-n // block))
    ids = random_ids(cfg, n, 4)
    check_logits(replay_cut(runner, "a", ids, [5]), weights, cfg, ids, dtype, folder)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_long_context_in_portions_then_decoding(tmp_path, ops, dtype_name):
    """2,300 tokens: portions whose walks over the keys are cut in parts (from 1,024 keys on), a window
    layer whose pages are given back on the way, then single tokens over many runs of keys."""
    dtype = DTYPES[dtype_name]
    cfg = dict(plain.TINY_C, max_position_embeddings=4096, sliding_window=700)
    folder, weights = make_model_dir(tmp_path, cfg, seed=13, dtype=dtype)
    runner = build_runner(folder, ops, dtype, block_size=16, num_blocks=160, max_model_len=4096)
    ids = random_ids(cfg, 2310, 6)
    got = replay_cut(runner, "a", ids, [1500, 700, 100, 2])
    check_logits(got, weights, cfg, ids, dtype, folder)
    runner.cache.check()
    free = runner.cache.free_pages()
    assert free[0] == 160 and free[1] == 160


def test_a_file_in_32_bit_under_a_bfloat16_engine(tmp_path, ops):
    """Tensors that the file keeps in 32-bit stay so: the products then run on the float32 kernel with
    bfloat16 activations, without packed copies and without the fused epilogues."""
    cfg, block = CONFIGS["C"]
    folder, weights = make_model_dir(tmp_path, cfg, seed=17, dtype=torch.float32)
    runner = build_runner(folder, ops, torch.bfloat16, block_size=block)
    assert runner.model.blocks[0].mixer.qkv_weight.dtype == torch.float32
    assert not hasattr(runner.model.blocks[0].mixer.qkv_weight, "_distie_rotary")
    ids = random_ids(cfg, 90, 8)
    check_logits(replay_cut(runner, "a", ids, [50, 20, 3]), weights, cfg, ids, torch.bfloat16, folder)


LAYER_SIZES = {
    "1.5b": dict(hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                 vocab_size=151936, tie_word_embeddings=True),
    "7b": dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944,
               vocab_size=152064, tie_word_embeddings=False),
}


@pytest.mark.timeout(600)
@pytest.mark.parametrize("shape", sorted(LAYER_SIZES))
def test_layer_sizes_of_the_models_the_benchmark_runs(tmp_path, ops, shape):
    """Two layers with the sizes the benchmark runs: width 1,536, 12 heads over 2 kv heads of 128, feed-forward
    8,960, vocabulary 151,936, tied head; and width 3,584, 28 heads over 4 kv heads (seven to a kv head),
    feed-forward 18,944, vocabulary 152,064, a head of its own. Sizes the tiny configurations do not reach
    (products cut along 8,960 and 18,944, rows of the head beyond 2^17, head size 128). One file in bfloat16
    serves both engines, since the float32 engine keeps every tensor in 32-bit whatever the file holds."""
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "head_dim": 128,
           "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 4096, "hidden_act": "silu",
           **LAYER_SIZES[shape]}
    folder, weights = make_model_dir(tmp_path, cfg, seed=19, std=0.03 if shape == "1.5b" else 0.02, dtype=torch.bfloat16)
    seqs = {"a": random_ids(cfg, 120, 1), "b": random_ids(cfg, 45, 2)}
    on_device = {k: v.to("cuda", torch.float64) for k, v in weights.items()}
    want = {name: plain.forward(on_device, cfg, ids, torch.float64).float().cpu() for name, ids in seqs.items()}
    del on_device
    for dtype in (torch.float32, torch.bfloat16):
        runner = build_runner(folder, ops, dtype, block_size=16, num_blocks=24, max_model_len=4096)
        got = {name: [] for name in seqs}
        # a whole, then: a portion of a beside all of b; the rest of a in a portion of 70 and single tokens,
        # the first of them beside b's last token
        whole = replay_whole(runner, "w", seqs["a"])
        steps = [[("a", 0, 40), ("b", 0, 44)], [("a", 40, 110)], [("a", 110, 111), ("b", 44, 45)]] + \
                [[("a", at, at + 1)] for at in range(111, 120)]
        for step in steps:
            logits = runner.step([StepEntry(r, seqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in step]).float().cpu()
            at = 0
            for r, lo, hi in step:
                got[r].append(logits[at:at + hi - lo])
                at += hi - lo
        for name in seqs:
            runner.finish(name)
        runner.cache.check()
        for name, rows in [("a", whole)] + [(n, torch.cat(g)) for n, g in got.items()]:
            diff = rows - want[name]
            scale = want[name].abs().max().item()
            if dtype == torch.float32:
                assert diff.abs().max().item() < 1e-4 * max(1.0, scale), (name, diff.abs().max().item(), scale)
            else:
                assert diff.abs().max().item() < scale / 16 and diff.pow(2).mean().sqrt().item() < scale / 64, name


ODD_SIZES = [
    dict(hidden_size=120, num_attention_heads=3, num_key_value_heads=1, head_dim=40, intermediate_size=96, vocab_size=77),
    dict(hidden_size=48, num_attention_heads=3, num_key_value_heads=1, head_dim=16, intermediate_size=100, vocab_size=1001),
    dict(hidden_size=336, num_attention_heads=7, num_key_value_heads=1, head_dim=48, intermediate_size=250, vocab_size=333,
         layer_types=["sliding_attention", "full_attention"], sliding_window=40),
    dict(hidden_size=1056, num_attention_heads=66, num_key_value_heads=1, head_dim=16, intermediate_size=64, vocab_size=130),
    dict(hidden_size=1024, num_attention_heads=4, num_key_value_heads=2, head_dim=256, intermediate_size=36, vocab_size=9,
         tie_word_embeddings=False),
]


@pytest.mark.parametrize("sizes", ODD_SIZES, ids=lambda s: f"{s['num_attention_heads']}x{s['head_dim']}")
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_odd_sizes(tmp_path, ops, sizes, dtype_name):
    """Sizes at the edges of what the kernels take: a feed-forward width and a vocabulary that are no multiple
    of 8, seven and 66 query heads on one kv head (more than the decode kernel's columns), head sizes 16 and
    256 and one that is no multiple of 16 (40: attention then runs on the wave-per-token kernel in both
    precisions), a vocabulary of nine."""
    dtype = DTYPES[dtype_name]
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "rope_theta": 10000.0,
           "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 512, "hidden_act": "silu", **sizes}
    folder, weights = make_model_dir(tmp_path, cfg, seed=23, std=min(0.3, 2.0 / cfg["hidden_size"] ** 0.5), dtype=dtype)
    runner = build_runner(folder, ops, dtype, block_size=16, num_blocks=24, max_model_len=512)
    ids = random_ids(cfg, 150, 9)
    check_logits(replay_whole(runner, "a", ids), weights, cfg, ids, dtype, folder)
    check_logits(replay_cut(runner, "b", ids, [70, 3, 40, 2, 17]), weights, cfg, ids, dtype, folder)
    runner.cache.check()
