"""Configuration, registry, weight files and their errors."""

import json

import pytest
import torch

import plain_qwen2 as plain
from distie_amd.config import (ConfigError, EngineConfig, Qwen2Config, config_from_dict, known_architectures,
                               load_model_config, register_architecture)
from distie_amd.engine.model import Model
from distie_amd.weights import (SafetensorsFile, WeightsError, kept_dtype, load_into, write_random_model,
                                write_safetensors)
from engine_util import make_model_dir


def test_qwen2_config_reads_every_key():
    c = config_from_dict(plain.TINY_B)
    assert isinstance(c, Qwen2Config)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (3, 96, 3, 1, 32)
    assert (c.intermediate_size, c.vocab_size, c.rope_theta, c.rms_norm_eps) == (250, 323, 1e6, 1e-5)
    assert c.tie_word_embeddings is False and c.max_position_embeddings == 256
    assert c.layer_windows == (None, 8, 8)
    assert c.num_key_value_groups == 3
    a = config_from_dict(plain.TINY_A)
    assert a.head_dim == 16 and a.layer_windows == (None, None) and a.tie_word_embeddings
    assert config_from_dict(plain.TINY_C).layer_windows == (20, None)
    # rope_parameters wins over rope_theta (worker/src/inference/qwen2/model.py:413-419)
    assert config_from_dict(dict(plain.TINY_A, rope_parameters={"rope_theta": 5.0})).rope_theta == 5.0


@pytest.mark.parametrize("change,message", [
    ({"num_key_value_heads": 3}, "multiple of num_key_value_heads"),
    ({"hidden_size": 70}, "hidden_size must equal"),
    ({"hidden_size": 12, "num_attention_heads": 4, "num_key_value_heads": 2}, "even"),
    ({"hidden_act": "gelu"}, "silu"),
    ({"rope_parameters": {"rope_type": "yarn"}}, "RoPE type"),
    ({"num_hidden_layers": 0}, ">= 1"),
    ({"layer_types": ["full_attention", "chunked_attention"]}, "unknown layer type"),
    ({"layer_types": ["full_attention"]}, "entries"),
    ({"vocab_size": None}, "required key 'vocab_size'"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"max_position_embeddings": None}, "max_position_embeddings"),
])
def test_config_errors(change, message):
    with pytest.raises(ConfigError, match=message):
        config_from_dict(dict(plain.TINY_A, **change))


def test_registry():
    assert "Qwen2ForCausalLM" in known_architectures()
    with pytest.raises(ConfigError, match="unknown architecture 'LlamaForCausalLM'.*Qwen2ForCausalLM"):
        config_from_dict(dict(plain.TINY_A, architectures=["LlamaForCausalLM"]))
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in plain.TINY_A.items() if k != "architectures"})
    with pytest.raises(TypeError):
        register_architecture("X", object)


def test_model_spec_has_no_size_in_code():
    spec = config_from_dict(plain.TINY_B).model_spec()
    assert [l.parts["mixer"].params["window"] for l in spec.layers] == [None, 8, 8]
    assert spec.layers[0].parts["mixer"].params["scale"] == 32 ** -0.5
    assert spec.layers[2].parts["mixer"].prefix == "model.layers.2.self_attn."
    assert [c.layer for c in spec.order] == [0, 1, 2]
    names = Model.declare(spec)
    assert set(names) == set(plain.tensor_shapes(plain.TINY_B))
    assert {n: tuple(s.shape) for n, s in names.items()} == plain.tensor_shapes(plain.TINY_B)


def test_engine_config():
    assert EngineConfig(dtype="bf16").dtype == "bfloat16"
    assert EngineConfig(dtype="auto").dtype == "bfloat16"
    assert EngineConfig(dtype="fp32", max_cache_tokens=130, block_size=16).pages() == 9
    with pytest.raises(ValueError):
        EngineConfig(dtype="fp16")
    with pytest.raises(ValueError):
        EngineConfig(token_budget=0)


def test_cache_sized_from_the_cards_memory():
    """Pages until the given share of the card is in use: the free memory minus what must stay free, in
    pages, less the one page that the cache keeps beyond the pool."""
    gib = 2 ** 30
    config = EngineConfig(gpu_mem_fraction=0.75)
    assert config.pages(page_bytes=gib, free_bytes=60 * gib, total_bytes=100 * gib) == 60 - 25 - 1
    assert EngineConfig(gpu_mem_fraction=1.0).pages(page_bytes=3 * gib, free_bytes=10 * gib, total_bytes=64 * gib) == 2
    assert EngineConfig(gpu_mem_fraction=0.5, num_blocks=7).pages() == 7          # a given size wins
    with pytest.raises(ValueError, match="no room"):
        config.pages(page_bytes=gib, free_bytes=25 * gib, total_bytes=100 * gib)
    with pytest.raises(ValueError, match="needs the card"):
        config.pages()
    for bad in (0.0, 1.5, -1.0):
        with pytest.raises(ValueError):
            EngineConfig(gpu_mem_fraction=bad)
    assert EngineConfig(packed_weights=["qkv", "head"]).packed_weights == ("qkv", "head")


def test_latency_distribution_matches_numpy():
    import numpy as np

    from distie_amd.engine.stats import distribution_ms

    values = torch.rand(37, generator=torch.Generator().manual_seed(3)).double().numpy()
    got = distribution_ms(values)
    for key, q in (("p50", 50), ("p90", 90), ("p99", 99)):
        assert abs(got[key] - np.percentile(values * 1e3, q)) < 1e-9
    assert abs(got["mean"] - values.mean() * 1e3) < 1e-9 and got["max"] == values.max() * 1e3
    assert distribution_ms([0.25]) == {"mean": 250.0, "p50": 250.0, "p90": 250.0, "p99": 250.0, "max": 250.0}
    assert distribution_ms([]) == {}


def test_safetensors_round_trip_matches_the_library(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int64).view(2, 3)}
    write_safetensors(tmp_path / "ours.safetensors", [(n, t.dtype, tuple(t.shape)) for n, t in tensors.items()],
                      iter(tensors.items()), {"k": "v"})
    theirs = load_file(str(tmp_path / "ours.safetensors"))
    for n, t in tensors.items():
        assert torch.equal(theirs[n], t)
    save_file(tensors, str(tmp_path / "theirs.safetensors"))
    f = SafetensorsFile(tmp_path / "theirs.safetensors")
    assert {n: s for n, (d, s) in f.index.items()} == {"a": (3, 5), "b": (7,), "c": (2, 3)}
    for n, t in tensors.items():
        assert torch.equal(f.read(n), t)
    f.close()


def test_kept_precision():
    bf, f32 = torch.bfloat16, torch.float32
    assert kept_dtype(bf, bf) == bf and kept_dtype(torch.float16, bf) == bf
    assert kept_dtype(f32, bf) == f32          # a tensor stored in 32-bit stays so
    assert kept_dtype(bf, f32) == f32 and kept_dtype(torch.float64, f32) == f32
    assert kept_dtype(torch.int64, bf) == torch.int32


def test_mixed_file_keeps_each_tensors_precision(tmp_path):
    cfg = plain.TINY_A
    weights = plain.random_weights(cfg, 1, dtype=torch.bfloat16)
    for name in weights:
        if name.endswith("norm.weight"):
            weights[name] = weights[name].float()
    plain.write_model_dir(tmp_path / "m", cfg, weights)
    model = Model(load_model_config(tmp_path / "m").model_spec())
    load_into(model, tmp_path / "m", "cpu", torch.bfloat16)
    assert model.embedding.dtype == torch.bfloat16
    assert model.blocks[0].mixer_norm.weight.dtype == torch.float32
    assert model.blocks[0].mixer.qkv_weight.dtype == torch.bfloat16
    assert model.head is model.embedding       # tied: one buffer (worker/tests/test_qwen2.py:52-58)


def test_weight_errors_list_everything(tmp_path):
    cfg = plain.TINY_B
    weights = plain.random_weights(cfg, 1)
    del weights["model.layers.1.mlp.up_proj.weight"]
    del weights["lm_head.weight"]
    weights["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(5)
    weights["model.layers.7.extra.weight"] = torch.zeros(2)
    plain.write_model_dir(tmp_path / "m", cfg, weights)
    model = Model(load_model_config(tmp_path / "m").model_spec())
    with pytest.raises(WeightsError) as info:
        load_into(model, tmp_path / "m", "cpu", torch.float32)
    err = info.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "lm_head.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert err.wrong_shape == [("model.layers.0.self_attn.q_proj.bias", (5,), (96,))]
    text = str(err)
    for piece in ("missing (2)", "unexpected (1)", "wrong shape (1)", "is [5], want [96]"):
        assert piece in text


def test_tied_head_ignores_a_copy_in_the_file(tmp_path):
    cfg = plain.TINY_A
    weights = plain.random_weights(cfg, 1)
    weights["lm_head.weight"] = weights["model.embed_tokens.weight"].clone()
    plain.write_model_dir(tmp_path / "m", cfg, weights)
    model = Model(load_model_config(tmp_path / "m").model_spec())
    load_into(model, tmp_path / "m", "cpu", torch.float32)
    assert model.head is model.embedding


def test_random_weights_mode_writes_a_model_folder(tmp_path):
    config = config_from_dict(plain.TINY_B)
    a = write_random_model(config, tmp_path / "a", seed=3, dtype="float32")
    b = write_random_model(config, tmp_path / "b", seed=3, dtype="bfloat16")
    c = write_random_model(config, tmp_path / "c", seed=4, dtype="float32")
    wa, wb, wc = plain.read_weights(a), plain.read_weights(b), plain.read_weights(c)
    assert {n: tuple(t.shape) for n, t in wa.items()} == plain.tensor_shapes(plain.TINY_B)
    assert all(torch.equal(wa[n].to(torch.bfloat16), wb[n]) for n in wa)    # same numbers in every precision
    assert not torch.equal(wa["lm_head.weight"], wc["lm_head.weight"])
    assert torch.equal(wa["model.norm.weight"], torch.ones(96))
    assert abs(wa["model.embed_tokens.weight"].std().item() - 0.02) < 0.002
    assert abs(wa["model.layers.0.self_attn.q_proj.bias"].std().item() - 0.02) < 0.006
    again = load_model_config(a)
    assert again == config
    assert json.loads((b / "config.json").read_text())["torch_dtype"] == "bfloat16"
    # the plain implementation reads the folder too
    logits = plain.forward(wa, plain.read_config(a), [1, 2, 3])
    assert logits.shape == (3, 323)


def _write_sharded(folder, cfg, weights, pieces=3):
    """A folder whose tensors are spread over several files, named by `model.safetensors.index.json`."""
    from safetensors.torch import save_file

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    names = list(weights)
    weight_map = {}
    for i in range(pieces):
        file = f"model-{i + 1:05d}-of-{pieces:05d}.safetensors"
        mine = names[i::pieces]                       # interleaved: a layer's tensors lie in different files
        save_file({n: weights[n].contiguous() for n in mine}, str(folder / file))
        weight_map.update({n: file for n in mine})
    (folder / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}))


def test_sharded_folder_loads_as_the_single_file_does(tmp_path):
    cfg = plain.TINY_B
    weights = plain.random_weights(cfg, 3, std=0.1)
    plain.write_model_dir(tmp_path / "one", cfg, weights)
    _write_sharded(tmp_path / "many", cfg, weights)
    single, sharded = (Model(load_model_config(tmp_path / name).model_spec()) for name in ("one", "many"))
    load_into(single, tmp_path / "one", "cpu", torch.float32)
    load_into(sharded, tmp_path / "many", "cpu", torch.float32)
    assert torch.equal(single.embedding, sharded.embedding) and torch.equal(single.head, sharded.head)
    for a, b in zip(single.blocks, sharded.blocks):
        assert torch.equal(a.mixer.qkv_weight, b.mixer.qkv_weight) and torch.equal(a.mixer.qkv_bias_t, b.mixer.qkv_bias_t)
        assert torch.equal(a.feed_forward.gate_up_weight, b.feed_forward.gate_up_weight)
        assert torch.equal(a.feed_forward_norm.weight, b.feed_forward_norm.weight)
    # a tensor that the index names but no file holds, and one that no file of the index holds at all
    broken = dict(weights)
    del broken["model.layers.2.mlp.down_proj.weight"]
    _write_sharded(tmp_path / "broken", cfg, broken)
    index = json.loads((tmp_path / "broken" / "model.safetensors.index.json").read_text())
    files = sorted(set(index["weight_map"].values()))
    holder = index["weight_map"]["model.norm.weight"]
    index["weight_map"]["model.norm.weight"] = [f for f in files if f != holder][0]
    (tmp_path / "broken" / "model.safetensors.index.json").write_text(json.dumps(index))
    model = Model(load_model_config(tmp_path / "broken").model_spec())
    with pytest.raises(WeightsError) as info:
        load_into(model, tmp_path / "broken", "cpu", torch.float32)
    assert set(info.value.missing) == {"model.layers.2.mlp.down_proj.weight", "model.norm.weight"}


def test_a_half_precision_file(tmp_path):
    """fp16 is not a precision of the engine: a bfloat16 engine keeps such tensors in bfloat16, a float32
    engine in float32, each converted from the stored values."""
    cfg = plain.TINY_A
    weights = plain.random_weights(cfg, 4, std=0.1, dtype=torch.float16)
    plain.write_model_dir(tmp_path / "m", cfg, weights)
    for engine_dtype in (torch.bfloat16, torch.float32):
        model = Model(load_model_config(tmp_path / "m").model_spec())
        load_into(model, tmp_path / "m", "cpu", engine_dtype)
        assert model.embedding.dtype == engine_dtype and model.blocks[1].feed_forward.down_weight.dtype == engine_dtype
        assert torch.equal(model.embedding, weights["model.embed_tokens.weight"].to(engine_dtype))
        assert torch.equal(model.blocks[1].feed_forward.down_weight,
                           weights["model.layers.1.mlp.down_proj.weight"].to(engine_dtype))


def test_random_values_are_a_function_of_seed_name_and_index():
    """The bits behind the random weights, written out again with numpy's unsigned integers: splitmix64 of
    base + index * golden ratio, top 16 bits an interval of the normal quantiles, next 24 a place in it."""
    import numpy as np

    from distie_amd.weights import random_init as ri

    base = ri.stream_base(7, "model.layers.0.mlp.down_proj.weight")
    with np.errstate(over="ignore"):
        u = np.uint64
        z = np.arange(5, 5 + 1000, dtype=np.uint64) * u(0x9E3779B97F4A7C15) + u(base)
        z = (z ^ (z >> u(30))) * u(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> u(27))) * u(0x94D049BB133111EB)
        z = z ^ (z >> u(31))
    got = ri.mixed_bits(base, 5, 1000, "cpu").numpy().view(np.uint64)
    assert np.array_equal(got, z)
    # a value is its interval's lower edge plus the place times the width, each rounded once
    values = ri.standard_normal(7, "model.layers.0.mlp.down_proj.weight", 1005, "cpu")[5:].numpy()
    lower, width = (t.numpy() for t in ri._tables("cpu"))
    interval = (z >> u(48)).astype(np.int64)
    place = ((z >> u(24)) & u(0xFFFFFF)).astype(np.float32) * np.float32(2.0 ** -24)
    assert np.array_equal(values, lower[interval] + (width[interval] * place).astype(np.float32))
    # chunks change nothing, names and seeds do
    old = ri.CPU_CHUNK
    try:
        ri.CPU_CHUNK = 97
        assert np.array_equal(ri.standard_normal(7, "model.layers.0.mlp.down_proj.weight", 1005, "cpu")[5:].numpy(), values)
    finally:
        ri.CPU_CHUNK = old
    assert not np.array_equal(ri.standard_normal(8, "model.layers.0.mlp.down_proj.weight", 1005, "cpu")[5:].numpy(), values)
    assert not np.array_equal(ri.standard_normal(7, "model.layers.1.mlp.down_proj.weight", 1005, "cpu")[5:].numpy(), values)


def test_random_values_are_normal():
    from distie_amd.weights import random_init as ri

    x = ri.standard_normal(1, "w", 2_000_000, "cpu").double()
    assert abs(x.mean().item()) < 3e-3
    assert abs(x.std().item() - 1.0) < 3e-3
    assert abs((x ** 3).mean().item()) < 1e-2                     # symmetric
    assert abs((x ** 4).mean().item() - 3.0) < 3e-2               # the normal's fourth moment
    assert abs((x.abs() > 1.959964).double().mean().item() - 0.05) < 1e-3
    assert x.abs().max().item() < 4.9 and x.abs().max().item() > 4.0
    # neighbours in a tensor are not correlated
    assert abs((x[1:] * x[:-1]).mean().item()) < 3e-3


def test_an_engine_with_random_weights_is_the_model_of_the_written_folder(tmp_path):
    """One generator: `LLM(config=..., random_weights=True, seed=s)` holds tensor for tensor what
    `write_random_model(config, dir, s)` writes, so the plain implementation reading the folder is the
    oracle of the engine that never saw it."""
    from distie_amd import LLM, StepEntry
    from torch_ops import TorchOps

    for cfg in (plain.TINY_A, plain.TINY_B):
        config = config_from_dict(cfg)
        folder = write_random_model(config, tmp_path / f"m{cfg['hidden_size']}", seed=11, dtype="float32", std=0.1)
        weights = plain.read_weights(folder)
        llm = LLM(config=config, random_weights=True, seed=11, weights_std=0.1, dtype="fp32", ops=TorchOps(), block_size=4, num_blocks=32)
        ids = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3]
        got = llm.step([StepEntry("a", ids, list(range(len(ids))))])
        want = plain.forward(weights, cfg, ids, torch.float64).float()
        assert (got - want).abs().max().item() < 1e-4
        from_folder = LLM(folder, dtype="fp32", ops=TorchOps(), block_size=4, num_blocks=32)
        assert torch.equal(from_folder.step([StepEntry("a", ids, list(range(len(ids))))]), got)
