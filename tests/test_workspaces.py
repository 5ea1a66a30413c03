"""Scratch buffers that captured graphs may point at: an outgrown buffer stays allocated exactly
as long as a graph captured while it was current is still leased."""
import weakref

import torch

from minfer_amd.kernels import ops


def fresh(monkeypatch):
    for name, value in (("_workspaces", {}), ("_counters", {}), ("_retired", []), ("_leases", {})):
        monkeypatch.setattr(ops, name, value)


def test_outgrown_buffers_live_as_long_as_an_older_lease(monkeypatch):
    fresh(monkeypatch)
    a = ops.workspace("t", 100_000, "cpu")
    assert ops.workspace("t", 50_000, "cpu") is a              # large enough: the same buffer
    ref_a = weakref.ref(a)
    lease = ops.lease_graph()                                   # a graph was captured: it may hold a's address
    assert not lease.stale()
    b = ops.workspace("t", 100_001, "cpu")
    assert b is not a and b.numel() >= 200_000, "replaced by one at least twice as large"
    assert lease.stale()
    del a
    assert ref_a() is not None, "the outgrown buffer is kept for the leased graph"
    later = ops.lease_graph()                                   # captured after the replacement: holds b only
    ops.release_graph(lease)
    assert ref_a() is None, "nothing can address it any more"
    ref_b = weakref.ref(b)
    c = ops.workspace("t", b.numel() + 1, "cpu")
    del b
    assert ref_b() is not None and later.stale()
    ops.release_graph(later)
    ops.release_graph(later)                                    # twice is harmless
    assert ref_b() is None and not ops._retired and not ops._leases
    assert c.numel() >= 400_000


def test_without_leases_nothing_is_kept(monkeypatch):
    fresh(monkeypatch)
    a = ops.workspace("u", 70_000, "cpu")
    ref_a = weakref.ref(a)
    del a
    ops.workspace("u", 80_000, "cpu")
    assert ref_a() is None and not ops._retired
    counters = ops._zeroed_counters("c", 10, "cpu")
    assert counters.numel() >= 1024 and not counters.any()
    lease = ops.lease_graph()
    more = ops._zeroed_counters("c", 5000, "cpu")
    assert more is not counters and not more.any() and len(ops._retired) == 1
    old = torch.ones(3)
    ops.note_replaced_buffer(old)                               # a rotation table rebuilt longer
    assert len(ops._retired) == 2
    ops.release_graph(lease)
    assert not ops._retired


def test_session_reach_is_a_power_of_two():
    """Prompts of many lengths share few captured steps: the reach a decode session is made for is
    rounded up to a power of two (at least 256, at most the model's positions)."""
    from minfer_amd.engine.engine import Engine

    class Probe(Engine):
        def __init__(self):
            self.max_positions = 5000
            self._sessions = {}

    import minfer_amd.engine.decode as decode
    made = []

    class FakeSession:
        def __init__(self, engine, n, max_len, sampler, use_graph):
            made.append(max_len)

        def release(self):
            pass
    real = decode.DecodeSession
    decode.DecodeSession = FakeSession
    try:
        from collections import OrderedDict
        e = Probe()
        e._sessions = OrderedDict()

        class S:
            structure = ("greedy",)
        for want, reach in ((1, 256), (256, 256), (257, 512), (2176, 4096), (4097, 5000), (5000, 5000)):
            e.decode_session(2, want, S())
            assert made[-1] == reach, (want, made[-1])
        assert len(e._sessions) == 4                            # 256, 512, 4096, 5000
    finally:
        decode.DecodeSession = real
