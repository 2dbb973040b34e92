"""Calibration kernels behind bench.py --calibrate-barrier: the device-wide barrier completes when its
workgroups are resident together, and gives up -- every wave still exits -- when the host makes the
bounded wait too short to succeed."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

WORDS = 32 * 18          # counters on lines of their own, the error word last
ERR = 32 * 17


def _run(hip, blocks, rounds, spin_limit, groups, counter0=0, error0=0):
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    init = np.zeros(WORDS, dtype=np.uint32)
    init[0], init[ERR] = counter0, error0
    words = HIPTensor.from_numpy(init.view(np.int32))
    hip.call("mh_grid_barrier_probe", None, words.data_ptr, words.data_ptr + ERR * 4, blocks, rounds, spin_limit, groups)
    memory.synchronize()
    return words.numpy().view(np.uint32)


@pytest.mark.parametrize("groups", [1, 8])
def test_grid_barrier_completes(hip, groups):
    blocks, rounds = 64, 50
    w = _run(hip, blocks, rounds, 1 << 16, groups)
    assert w[ERR] == 0
    assert w[0] == rounds * (blocks if groups == 1 else groups)
    if groups > 1:
        assert [int(w[32 * (1 + g)]) for g in range(groups)] == [rounds * blocks // groups] * groups


def test_grid_barrier_gives_up_and_exits(hip):
    # the host makes the wait impossible to satisfy: the counter starts 64 below its wrap-around, so after
    # the 64 arrivals of the only round it reads 0 < 64; every workgroup polls spin_limit times, sets the
    # error word and the launch returns
    w = _run(hip, 64, 1, 8, 1, counter0=2 ** 32 - 64)
    assert w[ERR] == 1 and w[0] == 0
    # and once the error word is set nobody waits: 50 rounds that could complete are left without arrivals
    w = _run(hip, 64, 50, 1 << 16, 1, error0=1)
    assert w[ERR] == 1


def test_grid_barrier_rejects_more_workgroups_than_fit(hip):
    from minit_amd.hip.tensor import HIPTensor
    words = HIPTensor.allocate((WORDS,), "int32")
    with pytest.raises(hip.HipError, match="resident"):
        hip.call("mh_grid_barrier_probe", None, words.data_ptr, words.data_ptr + ERR * 4, 100000, 1, 10, 1)
