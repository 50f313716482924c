"""Host-side logic of the product library (no GPU): the request -> QP-piece split and the lane
monitor, checked against the hand vectors and, on random sequences, against the CPU oracle."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from fuselink_amd import _lib
from fuselink_amd import plugin as P
from tests import oracle_binding as ob

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat_vectors.json")))


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


@pytest.fixture()
def net():
    p = P.NetPlugin(8)
    p.lib.fl_monitor_reset()
    p.lib.fl_monitor_set_clock(0, 0)
    return p


@pytest.mark.parametrize("v", KAT["qp_split"])
def test_qp_split_vectors(lib, v):
    off = (C.c_int * v["nqps"])()
    ln = (C.c_int * v["nqps"])()
    assert lib.flh_qp_split(v["size"], v["nqps"], off, ln) == v["stride"]
    assert list(off) == v["off"] and list(ln) == v["len"]


def test_qp_split_matches_oracle_randomly(lib):
    rng = np.random.default_rng(0)
    for _ in range(2000):
        size, nqps = int(rng.integers(0, 1 << 24)), int(rng.integers(1, 33))
        off = (C.c_int * nqps)()
        ln = (C.c_int * nqps)()
        stride = lib.flh_qp_split(size, nqps, off, ln)
        assert (stride, list(off), list(ln)) == ob.qp_split(size, nqps)
    assert lib.flh_qp_split(10, 0, off, ln) < 0


def test_constants_and_struct_sizes(lib):
    assert lib.flh_constant(1) == 16 and lib.flh_constant(2) == 2 << 20 and lib.flh_constant(3) == 256
    assert lib.flh_constant(4) == C.sizeof(_lib.ChunkDesc) == ob.DESC_DTYPE.itemsize == 32
    assert lib.flh_constant(5) == C.sizeof(_lib.SchedState) == ob.STATE_DTYPE.itemsize
    assert lib.flh_constant(6) == C.sizeof(_lib.SchedHdr) == ob.HDR_DTYPE.itemsize
    assert lib.flh_constant(8) == C.sizeof(_lib.Windows) and lib.flh_constant(9) == C.sizeof(_lib.SchedParams)
    assert lib.flh_constant(0) % 128 == 0


@pytest.mark.parametrize("v", KAT["monitor_timeout"])
def test_monitor_timeout_vectors(net, v):
    L = net.lib
    L.fl_monitor_mark_active(3, 1, v["mark_at"])
    L.fl_monitor_mark_active(5, 0, v["mark_at"])
    L.fl_monitor_tick(v["tick_at"])
    tx = (C.c_int32 * 16)()
    rx = (C.c_int32 * 16)()
    L.fl_monitor_status(1, 16, tx)
    L.fl_monitor_status(0, 16, rx)
    assert tx[3] == v["status"] and rx[5] == v["status"]


@pytest.mark.parametrize("v", KAT["idle_pick"])
def test_idle_pick_vectors(net, v):
    L = net.lib
    is_tx = 1 if v["dir"] == "tx" else 0
    _load_status(L, is_tx, v["status"])
    assert L.fl_monitor_idle_pick(is_tx, v["group"], v["mask"], 0) == v["ret"]
    out = (C.c_int32 * 16)()
    L.fl_monitor_status(is_tx, 16, out)
    assert list(out) == v["after"]


def _load_status(L, is_tx, status):
    L.fl_monitor_reset()
    for i, st in enumerate(status):
        L.fl_monitor_set_entry(i, is_tx, st, 0)


def test_exact_borrow_takes_one_lane_and_release_gives_it_back(net):
    """The fixed borrow (exact = 1) marks only the first idle lane outside the group, and a release returns
    it at once instead of after the daemon's timeout; BUSY and IDLE entries are not touched by a release."""
    L = net.lib
    for is_tx in (1, 0):
        _load_status(L, is_tx, [0, 1, 0, 0] + [1] * 12)
        assert L.fl_monitor_idle_pick(is_tx, 0, 0xFFFF, 1) == 2        # lane 0 is the group's own, lane 1 is busy
        out = (C.c_int32 * 16)()
        L.fl_monitor_status(is_tx, 16, out)
        assert list(out)[:4] == [0, 1, 2, 0]
        assert L.fl_monitor_release(1, is_tx) == 0 and L.fl_monitor_release(3, is_tx) == 0
        assert L.fl_monitor_release(2, is_tx) == 1
        L.fl_monitor_status(is_tx, 16, out)
        assert list(out)[:4] == [0, 1, 0, 0]
    assert L.fl_monitor_release(16, 1) < 0


def test_monitor_random_sequences_match_oracle(net):
    """Random mark / tick / pick sequences: the product table and the oracle's stay identical."""
    L = net.lib
    O = ob.lib()
    rng = np.random.default_rng(1)
    for trial in range(30):
        L.fl_monitor_reset()
        m = ob.Monitor()
        O.fl_mon_init(C.byref(m))
        now = 1000
        for _ in range(200):
            op = int(rng.integers(0, 5))
            now += int(rng.integers(0, 120))
            lane, is_tx = int(rng.integers(0, 16)), int(rng.integers(0, 2))
            if op <= 1:
                L.fl_monitor_mark_active(lane, is_tx, now)
                (O.fl_mon_mark_tx if is_tx else O.fl_mon_mark_rx)(C.byref(m), lane, 0, now)
            elif op == 2:
                L.fl_monitor_tick(now)
                O.fl_mon_tick(C.byref(m), now)
            elif op == 3:
                group = int(rng.integers(0, 16))
                assert L.fl_monitor_idle_pick(1, group, -1, 0) == O.fl_mon_idle_pick_tx(C.byref(m), group)
            else:
                group, mask = int(rng.integers(0, 16)), int(rng.integers(0, 1 << 16))
                assert L.fl_monitor_idle_pick(0, group, mask, 0) == O.fl_mon_idle_pick_rx(C.byref(m), group, mask)
            tx = (C.c_int32 * 16)()
            rx = (C.c_int32 * 16)()
            L.fl_monitor_status(1, 16, tx)
            L.fl_monitor_status(0, 16, rx)
            assert list(tx) == list(m.tx_status) and list(rx) == list(m.rx_status)
        # credits read off the table
        st = (C.c_int32 * 16)()
        L.fl_monitor_status(1, 16, st)
        got = (C.c_uint32 * 16)()
        exp = (C.c_uint32 * 16)()
        L.fl_monitor_credits(8, 3, 4, got)
        O.fl_credits_from_status(st, 8, 3, 4, exp)
        assert list(got)[:8] == list(exp)[:8]
        # the two halves of the lane decision: the sender's mask off the send statuses, the receiver's row off the
        # receive statuses and a mask
        rx = (C.c_int32 * 16)()
        L.fl_monitor_status(0, 16, rx)
        mask = C.c_uint32()
        for own in (-1, 0, 5):
            assert L.fl_monitor_tx_mask(8, own, C.byref(mask)) == 0
            assert mask.value == O.fl_tx_usage_mask(st, 8, own)
            for m_ in (0xffffffff, mask.value, int(rng.integers(0, 1 << 8))):
                assert L.fl_monitor_rx_credits(8, own, 4, m_, got) == 0
                O.fl_rx_credits_from_status(rx, 8, own, 4, m_, exp)
                assert list(got)[:8] == list(exp)[:8]
    assert L.fl_monitor_tx_mask(0, 0, C.byref(mask)) < 0 and L.fl_monitor_rx_credits(17, 0, 4, 0, got) < 0


def test_exact_pick_borrows_only_one(net):
    L = net.lib
    L.fl_monitor_reset()
    assert L.fl_monitor_idle_pick(1, 0, -1, 1) == 1          # first idle NIC outside group 0
    st = (C.c_int32 * 16)()
    L.fl_monitor_status(1, 16, st)
    assert list(st) == [0, 2] + [0] * 14
