"""Pins the integer side of the oracle (version selection, 1F1B order) and the C
ring against brute force.  No GPU needed: the ring is host-side bookkeeping."""
import collections
import ctypes

import pytest

from oracle import stash_oracle as so
from pipedream_amd import _cabi


@pytest.mark.parametrize("warmup", range(0, 9))
def test_closed_form_matches_bruteforce(warmup):
    nv = warmup + 1
    for n in list(range(1, 20)) + [33, 64]:
        fwd, bwd, queue = so.simulate_versions(n, warmup, nv)
        for k in range(n):
            # k < warmup minibatches only exist if n > k
            assert fwd[k] == so.forward_version(k, min(warmup, n)) or n <= warmup
            assert bwd[k] == so.backward_version(k, min(warmup, n)) or n <= warmup
            # the invariant weight stashing exists for: backward sees the forward's weights
            assert fwd[k] == bwd[k]
        # with a single version the reference never rotates the deque (optimizer.py:156)
        assert queue == (so.ring_versions_after(n, nv) if nv > 1 else [0])


def test_truth_table_on_integers():
    """runtime/tests/backprop/sgd_with_stashing.py:68-70: three forwards at v0, then three
    [load_old, backward, load_new, step]; which backwards still see v0?"""
    for nv, truth in ((1, [False, False]), (2, [True, False]), (3, [True, True])):
        _, bwd, _ = so.simulate_versions(3, 3, nv)
        assert [bwd[1] == bwd[0], bwd[2] == bwd[0]] == truth


def test_one_f_one_b_invariants():
    for warmup in range(0, 6):
        for n in range(1, 30):
            ev = so.one_f_one_b(n, warmup)
            in_flight = 0
            next_b = 0
            for kind, k in ev:
                if kind == "F":
                    in_flight += 1
                else:
                    assert k == next_b  # FIFO
                    next_b += 1
                    in_flight -= 1
                assert 0 <= in_flight <= min(warmup, n) + 1
            assert in_flight == 0 and next_b == n


def test_warmup_depth_straight_pipeline():
    # runtime/runtime.py:170-175 for a straight 4-stage pipe -> 3,2,1,0 (stash depths 4,3,2,1)
    m = {0: [0], 1: [1], 2: [2], 3: [3]}
    assert [so.warmup_depth(s, m) for s in range(4)] == [3, 2, 1, 0]
    # replicated first stage: 2 replicas, then two single stages
    m = {0: [0, 1], 1: [2], 2: [3]}
    assert [so.warmup_depth(s, m) for s in range(3)] == [1, 1, 0]
    assert so.warmup_depth(1, m, {"0": 5, "1": 7, "2": 0}) == 7


def test_macrobatch_versions():
    # update every 2 minibatches, 2 versions (runtime/optimizer.py:36-52)
    fwd, bwd, queue = so.simulate_versions(8, 1, 2, update_interval=2)
    assert queue == [3, 4]
    assert [bwd[k] for k in range(8)] == [0, 0, 0, 0, 1, 1, 2, 2]  # hand-derived: queue[0] lags one real update


class _Ring(object):
    def __init__(self, nv):
        self.lib = _cabi.lib()
        self.h = ctypes.c_void_p()
        self.lib.pd_ring_create(ctypes.c_void_p(1 << 20), 4096, nv, ctypes.byref(self.h))
        self.nv = nv

    def entry(self, i):
        s, v = ctypes.c_int(), ctypes.c_int64()
        self.lib.pd_ring_entry(self.h, i, ctypes.byref(s), ctypes.byref(v))
        return s.value, v.value

    def push(self, version):
        s = ctypes.c_int()
        self.lib.pd_ring_push(self.h, version, ctypes.byref(s))
        return s.value

    def write_slot(self):
        s = ctypes.c_int()
        self.lib.pd_ring_write_slot(self.h, ctypes.byref(s))
        return s.value

    def close(self):
        self.lib.pd_ring_destroy(self.h)


@pytest.mark.parametrize("nv", [1, 2, 3, 4, 7])
def test_c_ring_is_a_deque(nv):
    ring = _Ring(nv)
    dq = collections.deque(maxlen=nv)
    storage = collections.deque(maxlen=nv)  # physical slot of each queue entry
    for s in range(nv):
        dq.append(0)
        storage.append(s)
    for step in range(1, 40):
        assert [ring.entry(i)[1] for i in range(nv)] == list(dq)
        assert [ring.entry(i)[0] for i in range(nv)] == list(storage)
        assert ring.entry(-1) == ring.entry(nv - 1)
        oldest = storage[0]
        assert ring.write_slot() == oldest
        assert ring.push(step) == oldest
        dq.append(step)
        storage.append(oldest)
    # slot addresses
    p = ctypes.c_void_p()
    ring.lib.pd_ring_slot_ptr(ring.h, nv - 1, ctypes.byref(p))
    assert p.value == (1 << 20) + 4096 * (nv - 1)
    ring.close()


def test_c_ring_argument_errors():
    lib = _cabi.lib()
    h = ctypes.c_void_p()
    with pytest.raises(_cabi.PipedreamAmdError):
        lib.pd_ring_create(ctypes.c_void_p(1 << 20), 4096, 0, ctypes.byref(h))
    with pytest.raises(_cabi.PipedreamAmdError):
        lib.pd_ring_create(ctypes.c_void_p((1 << 20) + 8), 4096, 2, ctypes.byref(h))
    with pytest.raises(_cabi.PipedreamAmdError):
        lib.pd_ring_create(ctypes.c_void_p(1 << 20), 100, 2, ctypes.byref(h))
    with pytest.raises(_cabi.PipedreamAmdError):
        lib.pd_ring_create(None, 4096, 2, ctypes.byref(h))
    ring = _Ring(3)
    with pytest.raises(_cabi.PipedreamAmdError) as ei:
        ring.entry(3)
    assert ei.value.code == -3 and "out of range" in str(ei.value)
    with pytest.raises(_cabi.PipedreamAmdError):
        ring.entry(-4)
    ring.close()


def test_lr_policies():
    # closed forms of main_with_runtime.py:545-557
    assert so.adjust_learning_rate(0.1, 0, 90, "step", 0, 100) == 0.1
    assert abs(so.adjust_learning_rate(0.1, 30, 90, "step", 0, 100) - 0.01) < 1e-15
    assert abs(so.adjust_learning_rate(0.1, 45, 90, "polynomial", 0, 100) - 0.025) < 1e-15
    assert abs(so.adjust_learning_rate(0.1, 90, 90, "exponential_decay", 0, 100) - 0.097) < 1e-15
    assert abs(so.adjust_learning_rate(0.1, 0, 90, "step", 49, 100, lr_warmup=True) - 0.01) < 1e-15
    with pytest.raises(NotImplementedError):
        so.adjust_learning_rate(0.1, 0, 90, "cosine", 0, 100)
