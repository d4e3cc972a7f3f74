"""GPU parity of the entry point that allocates nothing: zk_fr_sum_static against zk_fr_sum (and python big
integers) through the C ABI, two calls in a row on one GPU, the second with a smaller input, so the second call sees the
first call's partials in the shared device array."""
import ctypes

import numpy as np
import pytest

from zkhelp import R_MOD, fr_array, fr_ints, mt_random_vec

pytestmark = pytest.mark.gpu

c_void_p, c_size_t = ctypes.c_void_p, ctypes.c_size_t


@pytest.fixture(scope="module")
def hip():
    from gpuhelp import Hip
    return Hip()


def both_sums(hip, A, d_out):
    n = A.shape[0]
    d_a = hip.upload(A) if n else hip.malloc(32)
    ref = np.zeros(8, dtype=np.uint32)
    hip.call("zk_fr_sum", ref, c_void_p(d_a), c_size_t(n), None)
    hip.call("zk_fr_sum_static", c_void_p(d_out), c_void_p(d_a), c_size_t(n), None)
    got = hip.download(d_out, (8,), np.uint32)
    hip.free(d_a)
    return got, ref


def test_sum_static_matches_sum_on_two_calls_in_a_row(hip):
    d_out = hip.malloc(32)
    edge = fr_array([R_MOD - 1, R_MOD - 2, 1, 0, R_MOD >> 1])
    # the first call fills all 2048 block partials; the later, smaller ones leave most of them stale
    for n, seed in (((1 << 20) + 3, 11), (70001, 12), (300, 13), (1, 14), (0, 15)):
        print("case zk_fr_sum_static n", n, "seed", seed, flush=True)
        A = np.concatenate([edge, mt_random_vec(np.random.RandomState(seed), n)])[:n] if n else np.zeros((0, 8), dtype=np.uint32)
        got, ref = both_sums(hip, A, d_out)
        assert (got == ref).all(), n
        assert fr_ints(got)[0] == sum(fr_ints(A)) % R_MOD, n
    hip.free(d_out)


def test_sum_static_allocates_nothing_and_rejects_oversize(hip):
    n = 1 << 18
    A = mt_random_vec(np.random.RandomState(21), n)
    d_a, d_out = hip.upload(A), hip.malloc(32)
    live0, cached0 = c_size_t(), c_size_t()
    hip.call("zk_pool_stats", ctypes.byref(live0), ctypes.byref(cached0))
    hip.call("zk_fr_sum_static", c_void_p(d_out), c_void_p(d_a), c_size_t(n), None)
    live1, cached1 = c_size_t(), c_size_t()
    hip.call("zk_pool_stats", ctypes.byref(live1), ctypes.byref(cached1))
    assert (live0.value, cached0.value) == (live1.value, cached1.value)
    assert fr_ints(hip.download(d_out, (8,), np.uint32))[0] == sum(fr_ints(A)) % R_MOD
    rc = hip.lib.zk_fr_sum_static(c_void_p(d_out), c_void_p(d_a), c_size_t(1 << 32), None)
    assert rc != 0 and b"ZK_FR_SUM_STATIC_MAX_N" in hip.lib.zk_last_error()
    hip.free(d_a)
    hip.free(d_out)
