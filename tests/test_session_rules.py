"""Rules of the session that need no GPU: the batch sizes and context bounds that captured
decode steps are made for."""
from edge_infer_amd.engine.session import batch_bucket, context_bound


def test_batch_buckets():
    """Powers of two up to 16, multiples of 8 up to 64, multiples of 32 beyond; a bucket is
    never below the live batch and never more than a third above it from 3 sequences on."""
    assert [batch_bucket(n) for n in (1, 2, 3, 4, 5, 8, 9, 16)] == [1, 2, 4, 4, 8, 8, 16, 16]
    assert [batch_bucket(n) for n in (17, 24, 25, 33, 48, 49, 64)] == [24, 24, 32, 40, 48, 56, 64]
    assert [batch_bucket(n) for n in (65, 96, 97, 200, 256)] == [96, 96, 128, 224, 256]
    for live in range(1, 257):
        bucket = batch_bucket(live)
        assert bucket >= live
        if live >= 3:
            assert bucket <= live * 4 // 3 + 1 or bucket - live < 32
    assert len({batch_bucket(n) for n in range(1, 257)}) == 5 + 6 + 6


def test_context_bounds():
    """256, 384, 512, 768, ...: at most a third above the context they serve, capped by the
    capacity."""
    assert [context_bound(n, 1 << 20) for n in (1, 256, 257, 385, 513, 769, 1025, 24577)] == \
        [256, 256, 384, 512, 768, 1024, 1536, 32768]
    for context in (300, 1000, 5000, 30000):
        bound = context_bound(context, 1 << 20)
        assert context <= bound <= context * 3 // 2
    assert context_bound(5000, 4096) == 4096 and context_bound(10, 64) == 64
