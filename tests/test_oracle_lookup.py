"""Pins the oracle's lookup / rescaling / softmax restatement (oracle/protocols.hpp) against big-int
re-derivations: numpy.bincount, A_i (S_i + beta) = 1, the LogUp identity, brute-force round polynomials
of the two-phase sumcheck on a tiny instance, exhaustive rescaling, and digit recombination."""
import math
import random

import numpy as np

from zkhelp import R_MOD, fr_array, fr_ints, load_oracle, me_bruteforce, mt_random_vec, orc_check, orc_transcript

INV2 = pow(2, -1, R_MOD)


def test_rescaling_exhaustive_small_range():
    orc = load_oracle()
    for sf in (16, 7):
        xs = list(range(-3 * sf // 2 - 3, 3 * sf // 2 + 4)) + [2 ** 40 + 5, -(2 ** 40) - 5]
        X = fr_array([x % R_MOD for x in xs])
        out, rem = np.zeros_like(X), np.zeros_like(X)
        orc_check(orc.orc_rescale(X, len(xs), sf, out, rem))
        q = [v if v < R_MOD // 2 else v - R_MOD for v in fr_ints(out)]
        r = [v if v < R_MOD // 2 else v - R_MOD for v in fr_ints(rem)]
        h = sf >> 1
        for x, qi, ri in zip(xs, q, r):
            assert x == qi * sf + ri and -h <= ri < sf - h, (x, qi, ri)
            assert ri == ((x + h) % sf) - h          # python's floor-mod is the kernel's adjusted C remainder


def test_relu_decomposition_exhaustive_small_range():
    """zkReLU's parts from python's floor division: x = q sf + rem with rem in [-h, sf - h); sign = [q >= 0], abs = |q|,
    result = max(q, 0); multiplicities of the remainders = bincount.  sign * abs - (1 - sign) * abs = q ties them."""
    orc = load_oracle()
    for sf in (16, 8):
        h = sf >> 1
        xs = list(range(-3 * sf - 3, 3 * sf + 4)) + [2 ** 40 + 5, -(2 ** 40) - 5]
        n = len(xs)
        X = fr_array([x % R_MOD for x in xs])
        res, sign, mag, rem = (np.zeros_like(X) for _ in range(4))
        m = np.zeros((sf, 8), np.uint32)
        orc_check(orc.orc_relu(X, n, sf, res, sign, mag, rem, m))
        signed = lambda a: [v if v < R_MOD // 2 else v - R_MOD for v in fr_ints(a)]
        q = [(x + h) // sf for x in xs]
        assert signed(rem) == [x - qi * sf for x, qi in zip(xs, q)]
        assert fr_ints(sign) == [int(qi >= 0) for qi in q]
        assert fr_ints(mag) == [abs(qi) for qi in q]
        assert fr_ints(res) == [max(qi, 0) for qi in q]
        assert fr_ints(m) == list(np.bincount(np.array(signed(rem)) + h, minlength=sf))
        assert all(s * a - (1 - s) * a == qi for s, a, qi in zip(fr_ints(sign), fr_ints(mag), q))


def test_range_prep_is_bincount_and_inverse_identity():
    orc = load_oracle()
    rng = random.Random(51)
    low, length, D = -5, 11, 64
    vals = [rng.randrange(low, low + length) for _ in range(D)]
    m = np.zeros((16, 8), np.uint32)
    orc_check(orc.orc_range_prep(fr_array([v % R_MOD for v in vals]), D, low, length, m))
    assert fr_ints(m) == list(np.bincount(np.array(vals) - low, minlength=16))
    beta = rng.randrange(R_MOD)
    S = [rng.randrange(R_MOD) for _ in range(10)] + [(-beta) % R_MOD]
    A = np.zeros((len(S), 8), np.uint32)
    orc_check(orc.orc_lookup_inv(fr_array(S), len(S), fr_array([beta]), A))
    for a, s in zip(fr_ints(A), S):
        assert a * (s + beta) % R_MOD == (1 if (s + beta) % R_MOD else 0)


def brute_lookup(S, T, m, alpha, beta, u, v):
    """tLookup::prove by the protocol's definition, with multilinear evaluations done by brute force"""
    D, N = len(S), len(T)
    inv = lambda x: pow(x, -1, R_MOD)
    A = [inv((s + beta) % R_MOD) for s in S]
    B = [inv((t + beta) % R_MOD) for t in T]
    assert sum(A) % R_MOD == sum(mk * bk for mk, bk in zip(m, B)) % R_MOD       # LogUp identity
    k, n1 = len(u), (D // N).bit_length() - 1
    v1, v2 = v[:n1], v[n1:]
    C = (alpha * alpha - sum(mk * bk for mk, bk in zip(m, B))) % R_MOD
    a_sq, claim, ratio = alpha * alpha % R_MOD, (alpha + alpha * alpha) % R_MOD, N * inv(D) % R_MOD
    polys = []
    u = list(u)

    def eq_poly(w):
        return [(1 - w) % R_MOD, (2 * w - 1) % R_MOD]

    def pmul(p, q):
        out = [0] * (len(p) + len(q) - 1)
        for i, a in enumerate(p):
            for j, b in enumerate(q):
                out[i + j] = (out[i + j] + a * b) % R_MOD
        return out

    def padd(p, q, sign=1):
        n = max(len(p), len(q))
        return [((p[i] if i < len(p) else 0) + sign * (q[i] if i < len(q) else 0)) % R_MOD for i in range(n)]

    def ev(p, x):
        return sum(c * pow(x, i, R_MOD) for i, c in enumerate(p)) % R_MOD

    def terms(X, Y, coef):
        h = len(X) // 2
        t0 = [coef * X[i] * ((Y[i] + beta) % R_MOD) % R_MOD for i in range(h)]
        t1 = [coef * ((X[i + h] - X[i]) * (Y[i] + beta) + X[i] * (Y[i + h] - Y[i])) % R_MOD for i in range(h)]
        t2 = [coef * (X[i + h] - X[i]) * (Y[i + h] - Y[i]) % R_MOD for i in range(h)]
        return [me_bruteforce(t, u[:-1]) for t in (t0, t1, t2)]

    fold = lambda X, w: [(X[i] + w * (X[i + len(X) // 2] - X[i])) % R_MOD for i in range(len(X) // 2)]
    for w in reversed(v1):
        h = len(A) // 2
        p0 = pmul(terms(A, S, alpha), eq_poly(u[-1]))
        p1 = [sum(A[:h]) % R_MOD, (sum(A[h:]) - sum(A[:h])) % R_MOD]
        p = padd(padd(p0, p1), [C * INV2 % R_MOD])
        assert (ev(p, 0) + ev(p, 1)) % R_MOD == claim
        polys.append(p)
        claim = ev(p, w)
        e = (2 * u[-1] * w - u[-1] - w + 1) % R_MOD
        alpha, C = alpha * e % R_MOD, C * INV2 % R_MOD
        A, S, u = fold(A, w), fold(S, w), u[:-1]
    for w in reversed(v2):
        h = len(A) // 2
        p0 = padd(terms(A, S, alpha), terms(B, T, ratio * a_sq % R_MOD))
        p1 = [sum(A[:h]) % R_MOD, (sum(A[h:]) - sum(A[:h])) % R_MOD]
        p2 = [sum(m[i] * B[i] for i in range(h)) % R_MOD,
              sum((m[i + h] - m[i]) * B[i] + m[i] * (B[i + h] - B[i]) for i in range(h)) % R_MOD,
              sum((m[i + h] - m[i]) * (B[i + h] - B[i]) for i in range(h)) % R_MOD]
        p = padd(padd(pmul(eq_poly(u[-1]), p0), p1), [c * ratio % R_MOD for c in p2], -1)
        assert (ev(p, 0) + ev(p, 1)) % R_MOD == claim
        polys.append(p)
        claim = ev(p, w)
        e = (2 * u[-1] * w - u[-1] - w + 1) % R_MOD
        alpha, a_sq = alpha * e % R_MOD, a_sq * e % R_MOD
        A, S, B, T, m, u = fold(A, w), fold(S, w), fold(B, w), fold(T, w), fold(m, w), u[:-1]
    return polys, claim


def test_lookup_prove_bruteforce_D16_N4():
    orc = load_oracle()
    rng = random.Random(52)
    low, length, D = 3, 4, 16
    vals = [rng.randrange(low, low + length) for _ in range(D)]
    alpha, beta = rng.randrange(R_MOD), rng.randrange(R_MOD)
    u, v = [rng.randrange(R_MOD) for _ in range(4)], [rng.randrange(R_MOD) for _ in range(4)]
    orc.orc_transcript_clear()
    fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_range_prove(fr_array(vals), D, low, length, fr_array([alpha]), fr_array([beta]), fr_array(u), fr_array(v), fin))
    t = fr_ints(orc_transcript(orc))
    T = [low + i for i in range(4)]
    m = list(np.bincount(np.array(vals) - low, minlength=4))
    polys, claim = brute_lookup(vals, T, [int(x) for x in m], alpha, beta, u, v)
    flat = [c for p in polys for c in p]
    assert t[:-1] == flat and t[-1] == claim == fr_ints(fin)[0]


def test_mapping_lookup_bruteforce_with_padding():
    orc = load_oracle()
    rng = random.Random(53)
    low, length, D = -2, 4, 6            # D is not a power of two: padded with table[0] / mapped[0]
    mv = [rng.randrange(1000) for _ in range(length)]
    vals = [rng.randrange(low, low + length) for _ in range(D)]
    r, alpha, beta = (rng.randrange(R_MOD) for _ in range(3))
    u, v = [rng.randrange(R_MOD) for _ in range(3)], [rng.randrange(R_MOD) for _ in range(3)]
    orc.orc_transcript_clear()
    y, m, fin = np.zeros((D, 8), np.uint32), np.zeros((4, 8), np.uint32), np.zeros(8, np.uint32)
    orc_check(orc.orc_mapping(fr_array([x % R_MOD for x in vals]), D, low, length, fr_array(mv), fr_array([r]), fr_array([alpha]), fr_array([beta]),
                              fr_array(u), fr_array(v), y, m, fin))
    assert fr_ints(y) == [mv[x - low] for x in vals]
    cnt = [int(c) for c in np.bincount(np.array(vals) - low, minlength=4)]
    assert fr_ints(m) == cnt
    cnt[0] += 2
    Sp = [(x + r * mv[x - low]) % R_MOD for x in vals] + [(low + r * mv[0]) % R_MOD] * 2
    Tc = [(low + i + r * mv[i]) % R_MOD for i in range(4)]
    polys, claim = brute_lookup(Sp, Tc, cnt, alpha, beta, u, v)
    t = fr_ints(orc_transcript(orc))
    assert t[:-1] == [c for p in polys for c in p] and t[-1] == claim == fr_ints(fin)[0]


def test_detmath_accuracy_against_python_libm():
    orc = load_oracle()
    rng = random.Random(54)
    xs = np.array([0.0, 1e-7, -1e-7, 1.0, -1.0, 700.0, -700.0] + [rng.uniform(-700, 700) for _ in range(20000)])
    out = np.zeros_like(xs)
    orc.orc_detmath(0, xs, out, len(xs))
    for x, y in zip(xs, out):
        assert abs(y - math.exp(x)) <= 4e-16 * math.exp(x)
    ys = np.array([1.0, 2.0, 2048.0, 0.5, 1e-300, 1e300] + [math.exp(rng.uniform(-700, 700)) for _ in range(20000)])
    orc.orc_detmath(1, ys, out, len(ys))
    for x, y in zip(ys, out):
        assert abs(y - math.log(x)) <= 4e-16 * max(abs(math.log(x)), 1e-3), (x, y)


def test_softmax_integer_structure():
    orc = load_oracle()
    rng = np.random.default_rng(55)
    m, n, d = 16, 16, 16
    bs = np.array([16, 16, 16], np.uint32)
    sf = 256
    thetas = np.array([float(1 << 10), float(1 << 12)])
    X = rng.integers(-200, 200, (m, n))
    Xf = fr_array([int(x) % R_MOD for x in X.reshape(-1)])
    Y, shift = np.zeros((m * n, 8), np.uint32), np.zeros((m, 8), np.uint32)
    orc_check(orc.orc_softmax(Xf, m, n, d, bs, 3, 1, 0, sf, thetas, 2, Y, shift, 0))
    s = sf * math.sqrt(d)
    sh = fr_ints(shift)
    for r in range(m):
        want = s * math.log(sum(math.exp(x / s) for x in X[r]))
        assert abs(sh[r] - want) <= 0.5 + 1e-6                 # the rounded shift
    # Y = prod_{k >= L} tbl_k[digit_k] with tbl_k[j] = floor(exp(ln theta - B_k j / s) + 0.5)
    Yi = fr_ints(Y)
    B = [1, 16, 256]
    for r in range(m):
        for c in range(n):
            t = sh[r] - int(X[r, c])
            assert 0 <= t < 4096
            digs = [t % 16, (t // 16) % 16, t // 256]
            assert sum(dg * b for dg, b in zip(digs, B)) == t   # digit recombination (zksoftmax.cu:207-218)
            want = 1
            for kk in (1, 2):
                tv = math.exp(math.log(thetas[kk - 1]) - B[kk] / s * digs[kk]) + 0.5
                assert abs(tv - round(tv)) > 1e-6               # no table entry of this instance sits on a rounding boundary
                want *= int(tv)
            assert Yi[r * n + c] == want
    # full proof runs (every in-prover identity holds) with seeded challenges
    orc.orc_seed(7)
    orc.orc_transcript_clear()
    orc_check(orc.orc_softmax(Xf, m, n, d, bs, 3, 1, 0, sf, thetas, 2, Y, shift, 1))
    assert len(orc_transcript(orc)) > 20


def _fr_signed(a):
    return [v if v < R_MOD // 2 else v - R_MOD for v in fr_ints(a)]


def test_attention_forward_is_per_head_softmax_attention_and_both_proofs_run():
    """zkattn_compute against numpy integer matrix products around the (separately pinned) row softmax: scores = Q_h K_h^T
    per head of the head-major stacks, out = Y_h V_h; then zkAttn::prove (one head) and zkAttnStacked::prove run through
    all their in-prover identities (inner-product rounds, out = Y V at the drawn point, scores = Q K^T at the softmax's
    point): a transposed operand or a wrong split of the challenge vectors fails one of them."""
    orc = load_oracle()
    bs = np.array([16, 16, 16], np.uint32)
    thetas = np.array([float(1 << 10), float(1 << 12)])
    for num, stacked, m, n, d in [(1, 0, 16, 16, 16), (4, 1, 8, 16, 16), (2, 1, 4, 8, 4)]:
        rng = np.random.default_rng(num * 100 + m)
        qmax = 3 if d == 16 else 6
        Qi, Ki, Vi = (rng.integers(-qmax, qmax + 1, (num, r, d)) for r in (m, n, n))
        Q, K, V = (fr_array([int(x) % R_MOD for x in a.reshape(-1)]) for a in (Qi, Ki, Vi))
        out, fin = np.zeros((num * m * d, 8), np.uint32), np.zeros(8, np.uint32)
        orc.orc_seed(3)
        orc.orc_transcript_clear()
        orc_check(orc.orc_attn(Q, K, V, num, m, n, d, stacked, bs, 3, 1, 0, 16, 16, thetas, 2, out, fin))
        assert len(orc_transcript(orc)) > 30
        # the softmax of the stacked scores through the entry point that test_softmax_integer_structure pins
        X = np.einsum("hik,hjk->hij", Qi, Ki)
        Xf = fr_array([int(x) % R_MOD for x in X.reshape(-1)])
        Y, shift = np.zeros((num * m * n, 8), np.uint32), np.zeros((num * m, 8), np.uint32)
        orc_check(orc.orc_softmax(Xf, num * m, n, d, bs, 3, 1, 0, 256, thetas, 2, Y, shift, 0))
        Yi = np.array(fr_ints(Y), dtype=object).reshape(num, m, n)
        want = [[[sum(int(Yi[h][i][j]) * int(Vi[h][j][k]) for j in range(n)) for k in range(d)] for i in range(m)] for h in range(num)]
        assert _fr_signed(out) == [v for h in want for row in h for v in row]
