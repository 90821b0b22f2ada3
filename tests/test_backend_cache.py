"""Host-side rules of the executable cache (no GPU): an executable that a captured graph replays is never released
under it, neither by eviction past `cacheLimit` nor by `clearCache()`.  The device is a recording stand-in; the logic
under test is `HipBackend._remember` / `clearCache` / `pin` / `unpin` and `GraphedProgram.launch`'s check."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "jax-js_amd"))

from jaxjs_hip import backend as B  # noqa: E402
from jaxjs_hip.kernelgen import KernelSource  # noqa: E402


class FakeDevice:
    def __init__(self):
        self.freed, self.unloaded, self.syncs, self.zeroed = [], [], 0, []

    def sync(self):
        self.syncs += 1

    def free(self, ptr):
        self.freed.append(ptr)

    def unload_module(self, m):
        self.unloaded.append(m)

    def h2d(self, ptr, data):
        self.zeroed.append((ptr, len(data)))


def make_backend(limit):
    be = B.HipBackend.__new__(B.HipBackend)
    be.dev = FakeDevice()
    from collections import OrderedDict
    be._exes = OrderedDict()
    be.cacheLimit = limit
    return be


def make_exe(i, zeroed=()):
    ks = KernelSource([""], [], [64, 16] if zeroed else [64], "map", {}, {}, zeroed_scratch=list(zeroed))
    scratch = [1000 + 2 * i, 1001 + 2 * i] if zeroed else [1000 + 2 * i]
    return B.Executable(("k", i), B._Prepared(ks, [], scratch, [2000 + i]))


def test_eviction_releases_the_oldest_unpinned_executable_and_never_a_pinned_one():
    be = make_backend(2)
    e0, e1, e2, e3 = (make_exe(i) for i in range(4))
    be._remember("k0", e0)
    be._remember("k1", e1)
    be.pin(e0)  # a graph replays e0
    be._remember("k2", e2)  # over the limit: e0 is the oldest but pinned, e1 goes
    assert not e0.data.released and e1.data.released and not e2.data.released
    assert be.dev.freed == [1002] and be.dev.unloaded == [2001]
    be._remember("k3", e3)  # e2 goes; e0 still stays
    assert not e0.data.released and e2.data.released and list(be._exes) == ["k0", "k3"]
    be.unpin(e0)
    be._remember("k4", make_exe(4))
    assert e0.data.released  # unpinned: now it is the oldest and is released


def test_clear_cache_keeps_pinned_executables_prepared():
    be = make_backend(10)
    e0, e1 = make_exe(0), make_exe(1)
    be._remember("k0", e0)
    be._remember("k1", e1)
    be.pin(e1)
    be.clearCache()
    assert e0.data.released and not e1.data.released and list(be._exes) == ["k1"]
    with pytest.raises(ValueError, match="pinned"):
        e1.data.release(be.dev)
    be.unpin(e1)
    be.clearCache()
    assert e1.data.released and not be._exes


def test_a_released_executable_cannot_be_pinned_and_a_graph_refuses_to_replay_one():
    from jaxjs_hip.graph import GraphedProgram

    be = make_backend(10)
    e0 = make_exe(0)
    be._remember("k0", e0)
    be.clearCache()
    with pytest.raises(ValueError, match="released"):
        be.pin(e0)

    launched = []

    class Dev(FakeDevice):
        def graph_launch(self, g):
            launched.append(g)

    g = GraphedProgram.__new__(GraphedProgram)
    g.backend, g._graph = make_backend(10), object()
    g.backend.dev = Dev()
    live, dead = make_exe(1), make_exe(2)
    g._exes = [live]
    g.launch()
    assert len(launched) == 1
    dead.data.released = True  # what a release behind the graph's back would leave
    g._exes = [live, dead]
    with pytest.raises(ValueError, match="released"):
        g.launch()
    assert len(launched) == 1


def test_counters_are_zeroed_again_after_a_failed_launch():
    be = make_backend(10)
    exe = make_exe(0, zeroed=[1])
    exe.data.rezero(be.dev)
    assert be.dev.zeroed == [(1001, 16)] and be.dev.syncs == 1
