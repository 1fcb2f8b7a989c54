"""Bucket sizes of captured decode steps (vectors of worker/tests/test_batch_decode.py:50-62)."""

import pytest

from distie_amd.engine.batch import StepEntry
from distie_amd.engine.graphs import DecodeGraphs, bucket_for, decode_buckets, token_buckets
from distie_amd.parts.attention import context_classes


def test_decode_buckets():
    assert decode_buckets(32) == (1, 2, 4, 8, 16, 24, 32)
    assert decode_buckets(64) == (1, 2, 4, 8, 16, 24, 32, 40, 48, 56, 64)
    assert decode_buckets(5) == (1, 2, 4, 5)
    assert decode_buckets(1) == (1,)
    with pytest.raises(ValueError):
        decode_buckets(0)


def test_chosen_buckets_replace_the_rule():
    assert decode_buckets(32, (8, 1, 8, 64)) == (1, 8)            # sorted, once each, none above the maximum
    assert decode_buckets(4, (16, 32)) == (4,)                      # nothing left: the maximum alone
    with pytest.raises(ValueError):
        decode_buckets(32, (0, 4))
    with pytest.raises(ValueError):
        decode_buckets(32, ())


def test_engine_config_holds_the_buckets():
    from distie_amd.config import EngineConfig

    assert EngineConfig().graph_buckets is None
    assert EngineConfig(graph_buckets=[16, 2, 2]).graph_buckets == (2, 16)
    with pytest.raises(ValueError):
        EngineConfig(graph_buckets=[0])


def test_engine_config_reads_the_graph_options_from_the_environment(monkeypatch):
    from distie_amd.config import EngineConfig

    monkeypatch.setenv("WORKER_GRAPH_BUCKETS", "4,1,32")
    monkeypatch.setenv("WORKER_GRAPH_TOKENS", "48")
    config = EngineConfig.from_env()
    assert config.graph_buckets == (1, 4, 32) and config.graph_tokens == 48
    assert EngineConfig.from_env(graph_tokens=0).graph_tokens == 0          # an option given wins, zero too
    with pytest.raises(ValueError):
        EngineConfig(graph_tokens=-1)


def test_bucket_for():
    buckets = decode_buckets(32)
    assert [bucket_for(buckets, n) for n in (1, 3, 8, 9, 17, 32)] == [1, 4, 8, 16, 24, 32]
    with pytest.raises(ValueError):
        bucket_for(buckets, 33)
    with pytest.raises(ValueError):
        bucket_for(buckets, 0)


def test_context_classes():
    assert context_classes(4096) == (1024, 1536, 2048, 3072, 4096)
    assert context_classes(700) == (700,)
    assert context_classes(1025) == (1024, 1025)
    assert context_classes(40, first=2) == (2, 3, 4, 6, 8, 12, 16, 24, 32, 40)
    classes = context_classes(32768)
    assert classes[0] == 1024 and classes[-1] == 32768
    assert all(b <= 1.5 * a for a, b in zip(classes, classes[1:]))
    with pytest.raises(ValueError):
        context_classes(0)


def test_token_buckets():
    assert token_buckets(96) == (16, 24, 32, 48, 64, 96)
    assert token_buckets(512) == (16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512)
    assert token_buckets(100) == (16, 24, 32, 48, 64, 96)
    assert token_buckets(10) == (10,) and token_buckets(1) == ()


def test_which_captured_step_takes_a_mixed_step():
    """(tokens, requests) of the bucket: the smallest token bucket that holds the step and leaves every padding
    request a token; a step is padded with at least one request unless it fills its token bucket exactly."""
    graphs = DecodeGraphs(None, 8, mixed_tokens=96)
    assert graphs.request_buckets == (1, 2, 4, 8, 9)
    entry = lambda n, want=None: StepEntry(object(), [1] * n, [n - 1] if want is None else want)
    pick = graphs._mixed_bucket
    assert pick([entry(5)]) == (16, 2)                      # 11 tokens of padding in one request
    assert pick([entry(16)]) == (16, 1)                     # fills the bucket: no padding
    assert pick([entry(15), entry(1)]) == (16, 2)
    assert pick([entry(14), entry(1), entry(1)]) == (24, 4) # 16 would need a request of padding without a token
    assert pick([entry(13), entry(1), entry(1)]) == (16, 4)
    assert pick([entry(40), entry(1)] + [entry(1)] * 6) == (48, 9)
    assert pick([entry(90), entry(7)]) is None              # more than the largest bucket
    assert pick([entry(5, want=[0])]) is None               # wants a row that is not its last
    assert pick([entry(5, want=[3, 4])]) is None
    assert pick([entry(5, want=[]), entry(3)]) == (16, 4)   # nothing wanted is fine
    assert DecodeGraphs(None, 8)._mixed_bucket([entry(5)]) is None      # switched off
    assert DecodeGraphs(None, 8).request_buckets == (1, 2, 4, 8, 9)
