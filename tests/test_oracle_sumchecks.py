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


# ---- multi_hadamard_sumchecks (proof.cu:191-241) and zkip_stacked (zkfc.cu:153-229) by brute force ------------------------------
def halves(t):
    """(t[g], t[g + n/2]) for the power-of-two length the tables are folded at, zeros beyond the end"""
    n2 = (1 << max(len(t) - 1, 0).bit_length()) >> 1
    t = list(t) + [0] * (2 * n2 - len(t))
    return t[:n2], t[n2:]


def fold_halves(t, x):
    lo, hi = halves(t)
    return [(a + x * (b - a)) % R_MOD for a, b in zip(lo, hi)]


def lagrange_eval(ys, x):
    """value at x of the polynomial through (0, ys[0]), (1, ys[1]), ..."""
    acc = 0
    for i, yi in enumerate(ys):
        num, den = 1, 1
        for j in range(len(ys)):
            if j != i:
                num = num * (x - j) % R_MOD
                den = den * (i - j) % R_MOD
        acc = (acc + yi * num * pow(den, -1, R_MOD)) % R_MOD
    return acc


@pytest.mark.parametrize("K,n", [(1, 8), (2, 16), (3, 8), (4, 4), (2, 2)])
def test_multi_hadamard_round_polynomials_bruteforce(K, n):
    """Round polynomial of degree K: p(x) = sum_i eq(u[:-1], i) prod_k (X_k[i] + x (X_k[i + n/2] - X_k[i])); the running
    claim is (1 - u_last) p(0) + u_last p(1), the next one p(v_last), the tables fold by v_last; the last claim is the
    product of the tables' evaluations at v."""
    orc = load_oracle()
    rng = random.Random(500 + 10 * K + n)
    Xs = [rnd(rng, n) for _ in range(K)]
    k = n.bit_length() - 1
    u, v = rnd(rng, k), rnd(rng, k)
    prod = [1] * n
    for X in Xs:
        prod = [p * x % R_MOD for p, x in zip(prod, X)]
    claim = me_bruteforce(prod, u)
    out = np.zeros((k * (K + 1), 8), np.uint32)
    fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_multi_hadamard(fr_array([claim]), np.concatenate([fr_array(X) for X in Xs]), K, n, fr_array(u), fr_array(v), k, out, fin))
    got = fr_ints(out)
    cur, uu, vv = [list(X) for X in Xs], list(u), list(v)
    for r in range(k):
        coefs = got[r * (K + 1):(r + 1) * (K + 1)]
        p = lambda x: sum(c * pow(x, e, R_MOD) for e, c in enumerate(coefs)) % R_MOD
        n2 = len(cur[0]) // 2

        def brute(x):
            vals = [1] * n2
            for X in cur:
                vals = [w * ((X[i] + x * (X[i + n2] - X[i])) % R_MOD) % R_MOD for i, w in enumerate(vals)]
            return me_bruteforce(vals, uu[:-1])
        for x in range(K + 2):
            assert p(x) == brute(x), (r, x)
        assert ((1 - uu[-1]) * p(0) + uu[-1] * p(1)) % R_MOD == claim
        claim = p(vv[-1])
        cur = [fold_halves(X, vv[-1]) for X in cur]
        uu, vv = uu[:-1], vv[:-1]
    assert fr_ints(fin)[0] == claim
    expect = 1
    for X in Xs:
        expect = expect * me_bruteforce(X, v) % R_MOD
    assert claim == expect
    # a claim that is not the product's evaluation is rejected in the first round
    assert orc.orc_multi_hadamard(fr_array([(claim + 1) % R_MOD]), np.concatenate([fr_array(X) for X in Xs]), K, n, fr_array(u), fr_array(v), k, out, fin) != 0


def brute_zkip_plain(claim, a, b, u):
    """zkip (zkfc.cu:94-151): halves (g, g + n/2), folded by u.back(); returns the round polynomials and the last claim"""
    polys = []
    a, b, u = list(a), list(b), list(u)
    while u:
        a0, a1 = halves(a)
        b0, b1 = halves(b)
        p = [sum(x * y for x, y in zip(a0, b0)) % R_MOD,
             sum(x0 * (y1 - y0) + y0 * (x1 - x0) for x0, x1, y0, y1 in zip(a0, a1, b0, b1)) % R_MOD,
             sum((x1 - x0) * (y1 - y0) for x0, x1, y0, y1 in zip(a0, a1, b0, b1)) % R_MOD]
        assert (2 * p[0] + p[1] + p[2]) % R_MOD == claim
        polys.append(p)
        x = u.pop()
        claim = (p[0] + p[1] * x + p[2] * x * x) % R_MOD
        a, b = fold_halves(a, x), fold_halves(b, x)
    return polys, claim


@pytest.mark.parametrize("N,D", [(4, 8), (3, 4), (5, 4), (2, 16), (8, 2), (1, 8)])
def test_zkip_stacked_round_polynomials_bruteforce(N, D):
    """Stacking rounds: p = [sum_n eq(uN[:-1], n) sum_d o_k[n][d]] over the halves (n, n + N_out) of the stacking axis,
    claim = (1 - uN_last) p(0) + uN_last p(1), next claim p(vN_last), rows folded by vN_last; then a plain zkip over D.
    The first claim is sum_n eq(uN, n) <A_n, B_n>."""
    orc = load_oracle()
    rng = random.Random(600 + 16 * N + D)
    A, B = rnd(rng, N * D), rnd(rng, N * D)
    kN, kD = (N - 1).bit_length(), (D - 1).bit_length()
    uN, vN, uD = rnd(rng, kN), rnd(rng, kN), rnd(rng, kD)
    rows = [sum(A[n * D + d] * B[n * D + d] for d in range(D)) % R_MOD for n in range(N)]
    claim = me_bruteforce(rows, uN)
    out = np.zeros(((kN + kD) * 3, 8), np.uint32)
    fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_zkip_stacked(fr_array([claim]), fr_array(A), fr_array(B), N, D, fr_array(uN) if kN else np.zeros((0, 8), np.uint32),
                                   fr_array(vN) if kN else np.zeros((0, 8), np.uint32), kN, fr_array(uD), kD, out, fin))
    got = fr_ints(out)
    a, b, n_cur = list(A), list(B), N
    uu, vv = list(uN), list(vN)
    for r in range(kN):
        n_out = (1 << (n_cur - 1).bit_length()) >> 1
        full = n_out * 2 * D
        ap, bp = a + [0] * (full - len(a)), b + [0] * (full - len(b))
        so = n_out * D
        o0 = [ap[g] * bp[g] % R_MOD for g in range(so)]
        o1 = [(ap[g] * (bp[g + so] - bp[g]) + (ap[g + so] - ap[g]) * bp[g]) % R_MOD for g in range(so)]
        o2 = [(ap[g + so] - ap[g]) * (bp[g + so] - bp[g]) % R_MOD for g in range(so)]
        p = [me_bruteforce([sum(o[n * D:(n + 1) * D]) % R_MOD for n in range(n_out)], uu[:-1]) for o in (o0, o1, o2)]
        assert got[3 * r:3 * r + 3] == p, r
        ev = lambda x: (p[0] + p[1] * x + p[2] * x * x) % R_MOD
        assert ((1 - uu[-1]) * ev(0) + uu[-1] * ev(1)) % R_MOD == claim
        claim = ev(vv[-1])
        a = [(ap[g] + vv[-1] * (ap[g + so] - ap[g])) % R_MOD for g in range(so)]
        b = [(bp[g] + vv[-1] * (bp[g + so] - bp[g])) % R_MOD for g in range(so)]
        n_cur, uu, vv = n_out, uu[:-1], vv[:-1]
    polys, last = brute_zkip_plain(claim, a, b, uD)
    for r, p in enumerate(polys):
        assert got[3 * (kN + r):3 * (kN + r) + 3] == p
    assert fr_ints(fin)[0] == last
    # the reduced rows at vN, then folded over D: the final claim is A(vN, uD) * B(vN, uD)
    Av = [me_bruteforce([A[n * D + d] for n in range(N)], vN) for d in range(D)]
    Bv = [me_bruteforce([B[n * D + d] for n in range(N)], vN) for d in range(D)]
    assert last == me_bruteforce(Av, uD) * me_bruteforce(Bv, uD) % R_MOD


def test_zkfc_stacked_claims_bruteforce():
    """zkFCStacked::prove (zkfc.cu:261-307) on 2 layers of 2 x 4 x 2: the claim is Y(u_num, u_batch, u_output) minus the
    bias term, the sumcheck is zkip_stacked over the rows reduced at u_batch / u_output, and the last claim equals
    X(v_num, u_batch, u_input) * W(v_num, u_input, u_output)."""
    from zkhelp import mt_random_vec, orc_transcript
    orc = load_oracle()
    rng = random.Random(71)
    num, batch, fin_, fout = 2, 2, 4, 2
    for with_bias in (False, True):
        X = [rng.randrange(-50, 50) % R_MOD for _ in range(num * batch * fin_)]
        Wt = [rng.randrange(-50, 50) % R_MOD for _ in range(num * fin_ * fout)]
        bias = [rng.randrange(-50, 50) % R_MOD for _ in range(num * fout)] if with_bias else None
        seed = 900 + with_bias
        orc.orc_seed(seed)
        orc.orc_transcript_clear()
        Y = np.zeros((num * batch * fout, 8), np.uint32)
        orc_check(orc.orc_zkfc_stacked(fr_array(X), fr_array(Wt), fr_array(bias) if with_bias else None, num, batch, fin_, fout, Y))
        Yi = fr_ints(Y)
        for l in range(num):
            for r in range(batch):
                for c in range(fout):
                    acc = sum(X[(l * batch + r) * fin_ + k] * Wt[(l * fin_ + k) * fout + c] for k in range(fin_)) + (bias[l * fout + c] if with_bias else 0)
                    assert Yi[(l * batch + r) * fout + c] == acc % R_MOD
        t = fr_ints(orc_transcript(orc))
        draws = fr_ints(mt_random_vec(np.random.RandomState(seed), 1 + 1 + 1 + 2 + 1))
        u_num, v_num, u_batch, u_input, u_output = draws[0:1], draws[1:2], draws[2:3], draws[3:5], draws[5:6]

        def me3(T, shape, us):
            """T[i0][i1][i2] evaluated at (us[0], us[1], us[2]), each axis LSB first"""
            d0, d1, d2 = shape
            acc = 0
            for i0 in range(d0):
                for i1 in range(d1):
                    row = [T[(i0 * d1 + i1) * d2 + i2] for i2 in range(d2)]
                    w = me_bruteforce([1 if j == i0 else 0 for j in range(d0)], us[0]) * me_bruteforce([1 if j == i1 else 0 for j in range(d1)], us[1])
                    acc = (acc + w * me_bruteforce(row, us[2])) % R_MOD
            return acc
        claim = me3(Yi, (num, batch, fout), (u_num, u_batch, u_output))
        if with_bias:
            ones_at = me_bruteforce([1] * batch, u_batch)
            b_at = me_bruteforce([me_bruteforce(bias[l * fout:(l + 1) * fout], u_output) for l in range(num)], u_num)
            claim = (claim - ones_at * b_at) % R_MOD
        assert t[0] == claim
        assert t[-1] == me3(X, (num, batch, fin_), (v_num, u_batch, u_input)) * me3(Wt, (num, fin_, fout), (v_num, u_input, u_output)) % R_MOD
        assert len(t) == 1 + 3 * (1 + 2) + 1


def test_rescaling_prove_transcript_is_the_claim_then_the_remainder_range_proof():
    """Rescaling::prove (rescaling.cu:41-79): draws u, v, (alpha, beta); records X(u) after checking X(u) = X_(u) sf + rem(u);
    the rest is tLookupRange::prove of the remainders in [-sf/2, sf/2), itself pinned by brute force elsewhere."""
    from zkhelp import mt_random_vec, orc_transcript
    orc = load_oracle()
    rng = random.Random(5)
    n, sf = 32, 8
    xs = [rng.randrange(-1000, 1000) for _ in range(n)]
    seed = 77
    orc.orc_seed(seed)
    orc.orc_transcript_clear()
    out = np.zeros((n, 8), np.uint32)
    orc_check(orc.orc_rescale_prove(fr_array([x % R_MOD for x in xs]), n, sf, out))
    t = fr_ints(orc_transcript(orc))
    q = [(x + sf // 2) // sf for x in xs]                     # floor: remainder x - q sf in [-sf/2, sf/2)
    rem = [x - qi * sf for x, qi in zip(xs, q)]
    assert all(-sf // 2 <= r < sf // 2 for r in rem)
    assert fr_ints(out) == [v % R_MOD for v in q]
    draws = fr_ints(mt_random_vec(np.random.RandomState(seed), 5 + 5 + 2))
    u, v, alpha, beta = draws[0:5], draws[5:10], draws[10], draws[11]
    assert t[0] == me_bruteforce([x % R_MOD for x in xs], u)
    assert t[0] == (me_bruteforce([v_ % R_MOD for v_ in q], u) * sf + me_bruteforce([r % R_MOD for r in rem], u)) % R_MOD
    orc.orc_transcript_clear()
    fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_range_prove(fr_array([r % R_MOD for r in rem]), n, -(sf // 2), sf, fr_array([alpha]), fr_array([beta]), fr_array(u), fr_array(v), fin))
    assert t[1:] == fr_ints(orc_transcript(orc))
