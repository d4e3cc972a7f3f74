"""Pins the oracle's restatement of the deprecated sumchecks (inner product, Hadamard product, binary) and of the
window split against big-integer brute force: every round's three terms are recomputed from the folded tables, with the
factor R^-1 that the step kernels leave on each product, and the split against a numpy reshape. A dropped cross term, a
fold by the wrong challenge vector or an off-by-one in the remaining evaluation point fails one of these."""
import random

import numpy as np
import pytest

from zkhelp import R_MOD, fr_array, fr_ints, load_oracle, me_bruteforce, orc_check

RINV = pow(1 << 256, -1, R_MOD)   # the Montgomery radix of 8 x 32-bit limbs
RMONT = (1 << 256) % R_MOD


def rnd(rng, n):
    return [rng.randrange(R_MOD) for _ in range(n)]


def pairs(t):
    """(t[2g], t[2g+1]) with zeros beyond the end"""
    t = list(t) + [0] * (len(t) & 1)
    return t[0::2], t[1::2]


def fold(t, x):
    lo, hi = pairs(t)
    return [(a + x * (b - a)) % R_MOD for a, b in zip(lo, hi)]


@pytest.mark.parametrize("n", [2, 3, 5, 8, 13, 32, 37])
def test_inner_product_sumcheck_rounds(n):
    orc = load_oracle()
    rng = random.Random(100 + n)
    a, b = rnd(rng, n), rnd(rng, n)
    k = (n - 1).bit_length()
    u = rnd(rng, k)
    out = np.zeros((3 * k + 2, 8), np.uint32)
    orc_check(orc.orc_inner_product_sumcheck(fr_array(a), fr_array(b), n, fr_array(u), k, out))
    got = fr_ints(out)
    claim = sum(x * y for x, y in zip(a, b)) * RINV % R_MOD
    for r in range(k):
        a0, a1 = pairs(a)
        b0, b1 = pairs(b)
        s0 = sum(x * y for x, y in zip(a0, b0)) * RINV % R_MOD
        s1 = sum(x0 * (y1 - y0) + y0 * (x1 - x0) for x0, x1, y0, y1 in zip(a0, a1, b0, b1)) * RINV % R_MOD
        s2 = sum((x1 - x0) * (y1 - y0) for x0, x1, y0, y1 in zip(a0, a1, b0, b1)) * RINV % R_MOD
        assert got[3 * r:3 * r + 3] == [s0, s1, s2]
        assert (2 * s0 + s1 + s2) % R_MOD == claim            # p(0) + p(1) is the running claim
        claim = (s0 + s1 * u[r] + s2 * u[r] * u[r]) % R_MOD
        a, b = fold(a, u[r]), fold(b, u[r])
    assert got[3 * k:] == [a[0], b[0]]
    assert a[0] * b[0] * RINV % R_MOD == claim


@pytest.mark.parametrize("n", [2, 3, 5, 8, 13, 32, 37])
def test_hadamard_product_sumcheck_rounds(n):
    orc = load_oracle()
    rng = random.Random(200 + n)
    a, b = rnd(rng, n), rnd(rng, n)
    k = (n - 1).bit_length()
    u, v = rnd(rng, k), rnd(rng, k)
    out = np.zeros((3 * k + 2, 8), np.uint32)
    orc_check(orc.orc_hadamard_product_sumcheck(fr_array(a), fr_array(b), n, fr_array(u), fr_array(v), k, out))
    got = fr_ints(out)
    claim = me_bruteforce([x * y * RINV % R_MOD for x, y in zip(a, b)], u)
    for r in range(k):
        a0, a1 = pairs(a)
        b0, b1 = pairs(b)
        rest = u[r + 1:]
        at = lambda x: me_bruteforce([(x0 + x * (x1 - x0)) * (y0 + x * (y1 - y0)) * RINV % R_MOD
                                      for x0, x1, y0, y1 in zip(a0, a1, b0, b1)], rest)
        p0, p1, p2 = got[3 * r:3 * r + 3]
        for x in (0, 1, 2):
            assert (p0 + p1 * x + p2 * x * x) % R_MOD == at(x)
        # the running claim is the value at u_r, with the weight of the round's variable
        assert ((1 - u[r]) * at(0) + u[r] * at(1)) % R_MOD == claim
        claim = (p0 + p1 * v[r] + p2 * v[r] * v[r]) % R_MOD
        a, b = fold(a, v[r]), fold(b, v[r])
    assert got[3 * k:] == [a[0], b[0]]
    assert a[0] * b[0] * RINV % R_MOD == claim


@pytest.mark.parametrize("n", [2, 3, 5, 8, 13, 32, 37])
def test_binary_sumcheck_rounds(n):
    orc = load_oracle()
    rng = random.Random(300 + n)
    a = rnd(rng, n)
    k = (n - 1).bit_length()
    u, v = rnd(rng, k), rnd(rng, k)
    out = np.zeros((3 * k + 1, 8), np.uint32)
    orc_check(orc.orc_binary_sumcheck(fr_array(a), n, fr_array(u), fr_array(v), k, out))
    got = fr_ints(out)
    f = lambda z: (z * z * RINV - z) % R_MOD
    for r in range(k):
        a0, a1 = pairs(a)
        rest = u[r + 1:]
        p0, p1, p2 = got[3 * r:3 * r + 3]
        for x in (0, 1, 2):
            assert (p0 + p1 * x + p2 * x * x) % R_MOD == me_bruteforce([f(x0 + x * (x1 - x0)) for x0, x1 in zip(a0, a1)], rest)
        a = fold(a, v[r])
    assert got[3 * k:] == [a[0]]


def test_binary_sumcheck_of_a_bit_tensor_is_zero_on_the_cube():
    """Bits in Montgomery form (0 or R mod r) satisfy a*a*R^-1 = a: the first round's polynomial vanishes at 0 and 1."""
    orc = load_oracle()
    rng = random.Random(7)
    n, k = 16, 4
    a = [RMONT * rng.randrange(2) % R_MOD for _ in range(n)]
    u, v = rnd(rng, k), rnd(rng, k)
    out = np.zeros((3 * k + 1, 8), np.uint32)
    orc_check(orc.orc_binary_sumcheck(fr_array(a), n, fr_array(u), fr_array(v), k, out))
    p0, p1, p2 = fr_ints(out)[:3]
    assert p0 == 0 and (p1 + p2) % R_MOD == 0
    a[5] = 2 * RMONT % R_MOD
    orc_check(orc.orc_binary_sumcheck(fr_array(a), n, fr_array(u), fr_array(v), k, out))
    p0, p1, p2 = fr_ints(out)[:3]
    assert (p0, (p0 + p1 + p2) % R_MOD) != (0, 0)


def test_sumcheck_size_checks():
    orc = load_oracle()
    rng = random.Random(9)
    a = fr_array(rnd(rng, 4))
    out = np.zeros((16, 8), np.uint32)
    assert orc.orc_inner_product_sumcheck(a, a, 4, fr_array(rnd(rng, 3)), 3, out) != 0   # 4 <= 2^3 / 2
    assert orc.orc_inner_product_sumcheck(a, a, 4, fr_array(rnd(rng, 1)), 1, out) != 0   # 4 > 2^1
    assert orc.orc_binary_sumcheck(a, 4, fr_array(rnd(rng, 3)), fr_array(rnd(rng, 3)), 3, out) != 0


@pytest.mark.parametrize("n,w", [(8, 2), (8, 1), (12, 4), (13, 4), (10, 3), (7, 6), (9, 4)])
def test_split_against_reshape(n, w):
    orc = load_oracle()
    rng = random.Random(n * 31 + w)
    t = rnd(rng, n)
    nin = -(-n // w)
    nout = (nin + 1) // 2
    grid = np.zeros((2 * nout * w,), object)
    grid[:n] = t
    grid = grid.reshape(nout, 2, w)
    even, odd = np.zeros((nout * w, 8), np.uint32), np.zeros((nout * w, 8), np.uint32)
    orc_check(orc.orc_fr_split(fr_array(t), n, w, even, odd))
    assert fr_ints(even) == [int(x) for x in grid[:, 0, :].reshape(-1)]
    assert fr_ints(odd) == [int(x) for x in grid[:, 1, :].reshape(-1)]


def test_split_rejects_bad_windows():
    orc = load_oracle()
    t = fr_array([1, 2, 3, 4])
    e, o = np.zeros((8, 8), np.uint32), np.zeros((8, 8), np.uint32)
    assert orc.orc_fr_split(t, 4, 0, e, o) != 0
    assert orc.orc_fr_split(t, 4, 4, e, o) != 0
