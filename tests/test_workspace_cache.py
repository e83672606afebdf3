"""Host logic of the backward-workspace cache of oslo_amd.torch._C, without a GPU:
one workspace per (device, stream, op), handed out under the slot's lock for the
duration of one C call (so two host threads on one stream cannot interleave the
main and the finalize launch of their calls), and never touched while a stream
is being captured (a captured call gets a workspace of its own)."""
import threading

import torch

from oslo_amd.torch import _C


def make_cache(capturing=None):
    made = []

    def allocate(nbytes, index):
        t = torch.empty(nbytes, dtype=torch.uint8)
        made.append(t)
        return t

    state = {"capturing": False}
    cache = _C._WorkspaceCache(allocate, capturing or (lambda: state["capturing"]))
    return cache, made, state


def test_one_workspace_per_device_stream_and_op_grown_on_demand():
    cache, made, _ = make_cache()
    with cache.lease(0, 111, _C.OSLO_OP_LN_BWD, 1000) as ws:
        first = ws.tensor
        assert ws.nbytes == 1000 and first.numel() >= 1000
    with cache.lease(0, 111, _C.OSLO_OP_LN_BWD, 500) as ws:
        assert ws.tensor is first and ws.nbytes == 500        # reused
    with cache.lease(0, 111, _C.OSLO_OP_LN_BWD, 300000) as ws:
        assert ws.tensor is not first and ws.tensor.numel() >= 300000   # grown
        assert ws.tensor.numel() % (1 << 20) == 0
        grown = ws.tensor
    with cache.lease(0, 222, _C.OSLO_OP_LN_BWD, 1000) as ws:
        assert ws.tensor is not grown                            # another stream
    with cache.lease(1, 111, _C.OSLO_OP_LN_BWD, 1000) as ws:
        assert ws.tensor is not grown                            # another device
    with cache.lease(0, 111, _C.OSLO_OP_RMS_BWD, 1000) as ws:
        assert ws.tensor is not grown                            # another op
    assert len(cache.slots) == 4 and len(made) == 5
    # a call without a workspace takes no slot and no lock
    with _C._NO_WORKSPACE as ws:
        assert ws.tensor is None and ws.nbytes == 0
    with cache.lease(0, 111, _C.OSLO_OP_LN_BWD, 0) as ws:
        assert ws.tensor is None


def test_the_slot_is_locked_for_the_duration_of_the_call():
    cache, _, _ = make_cache()
    key = (0, 111, _C.OSLO_OP_LN_BWD)
    order = []
    inside = threading.Event()
    release = threading.Event()

    def first():
        with cache.lease(*key, 1000):
            order.append("first in")
            inside.set()
            release.wait(10)
            order.append("first out")

    def second():
        inside.wait(10)
        with cache.lease(*key, 1000):
            order.append("second in")

    def other_stream():
        inside.wait(10)
        with cache.lease(0, 222, _C.OSLO_OP_LN_BWD, 1000):
            order.append("other stream in")
        release.set()

    threads = [threading.Thread(target=f) for f in (first, second, other_stream)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(20)
    assert not any(t.is_alive() for t in threads)
    # the other stream's call went through while the first held its slot; the second
    # call on the same stream had to wait for the first to return
    assert order.index("other stream in") < order.index("first out") < order.index("second in")
    assert not cache.slots[key].lock.locked()


def test_an_exception_releases_the_slot():
    cache, _, _ = make_cache()
    key = (0, 111, _C.OSLO_OP_LN_BWD)
    try:
        with cache.lease(*key, 1000):
            raise RuntimeError("the C call failed")
    except RuntimeError:
        pass
    assert not cache.slots[key].lock.locked()

    def failing(nbytes, index):
        raise MemoryError("out of memory")

    bad = _C._WorkspaceCache(failing, lambda: False)
    try:
        with bad.lease(*key, 1000):
            pass
    except MemoryError:
        pass
    assert not bad.slots[key].lock.locked()


def test_a_captured_call_neither_reads_nor_writes_the_cache():
    cache, made, state = make_cache()
    key = (0, 111, _C.OSLO_OP_LN_BWD)
    with cache.lease(*key, 1000) as ws:
        cached = ws.tensor
    state["capturing"] = True
    with cache.lease(*key, 1000) as a:
        assert a.tensor is not cached and a.tensor.numel() == 1000
        assert not cache.slots[key].lock.locked()
        first = a.tensor
    with cache.lease(*key, 1000) as b:
        assert b.tensor is not first and b.tensor is not cached   # one per captured call
    with cache.lease(0, 333, _C.OSLO_OP_LN_BWD, 5000):
        pass
    assert (0, 333, _C.OSLO_OP_LN_BWD) not in cache.slots        # nothing cached under capture
    state["capturing"] = False
    with cache.lease(*key, 1000) as ws:
        assert ws.tensor is cached
