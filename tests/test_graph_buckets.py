"""Bucket sizes of captured decode steps (vectors of worker/tests/test_batch_decode.py:50-62)."""

import pytest

from distie_amd.engine.graphs import bucket_for, decode_buckets
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
