"""Pins the oracle's G1-tensor and commitment restatement (oracle/protocols.hpp) with textbook affine
arithmetic in python big ints: naive sum_j [s_j]G_j, linearity, and the opening's round invariant."""
import random

import numpy as np

from zkhelp import (G1_X, G1_Y, R_MOD, affine_to_jac, ec_add, ec_mul, ec_neg, fr_array, fr_ints, jac_to_affine, load_oracle,
                    me_bruteforce, mt_random_vec, orc_check)

G = (G1_X, G1_Y)


def gens_from_seed(orc, seed, n):
    orc.orc_seed(seed)
    g = np.zeros((n, 36), np.uint32)
    orc_check(orc.orc_commitment_random(n, g))
    return g


def test_generators_are_seeded_multiples_of_G():
    orc = load_oracle()
    g = gens_from_seed(orc, 77, 4)
    s = fr_ints(mt_random_vec(np.random.RandomState(77), 4))
    assert [jac_to_affine(r) for r in g] == [ec_mul(k, G) for k in s]


def test_commit_int_is_naive_msm_and_linear():
    orc = load_oracle()
    rng = random.Random(41)
    n, m = 4, 3
    g = gens_from_seed(orc, 5, n)
    pts = [jac_to_affine(r) for r in g]
    t = [rng.randrange(-2 ** 15, 2 ** 15) for _ in range(m * n)]
    t[1] = 0
    t[2] = -(2 ** 31) + 1
    com = np.zeros((m, 36), np.uint32)
    orc_check(orc.orc_commit_int(g, n, fr_array([x % R_MOD for x in t]), m * n, com))
    exp = []
    for r in range(m):
        acc = None
        for j in range(n):
            acc = ec_add(acc, ec_mul(t[r * n + j], pts[j]))
        exp.append(acc)
    assert [jac_to_affine(r) for r in com] == exp
    # linearity: com(a) + com(b) = com(a+b)
    a = [rng.randrange(-1000, 1000) for _ in range(n)]
    b = [rng.randrange(-1000, 1000) for _ in range(n)]
    ca, cb, cab = (np.zeros((1, 36), np.uint32) for _ in range(3))
    orc_check(orc.orc_commit_int(g, n, fr_array([x % R_MOD for x in a]), n, ca))
    orc_check(orc.orc_commit_int(g, n, fr_array([x % R_MOD for x in b]), n, cb))
    orc_check(orc.orc_commit_int(g, n, fr_array([(x + y) % R_MOD for x, y in zip(a, b)]), n, cab))
    assert ec_add(jac_to_affine(ca[0]), jac_to_affine(cb[0])) == jac_to_affine(cab[0])
    # full-width commit agrees on small scalars
    cf = np.zeros((1, 36), np.uint32)
    orc_check(orc.orc_commit(g, n, fr_array([x % R_MOD for x in a]), n, cf))
    assert jac_to_affine(cf[0]) == jac_to_affine(ca[0])


def test_open_returns_multilinear_evaluation_and_round_invariant():
    orc = load_oracle()
    rng = random.Random(42)
    n, m = 4, 2          # 4 generators, 2 committed rows
    g = gens_from_seed(orc, 6, n)
    pts = [jac_to_affine(r) for r in g]
    t = [rng.randrange(R_MOD) for _ in range(m * n)]
    u = [rng.randrange(R_MOD) for _ in range(3)]     # 2 bits for the generator index, 1 for the row
    proof = np.zeros((3 * 2 + 1, 36), np.uint32)
    val = np.zeros(8, np.uint32)
    orc_check(orc.orc_open(g, n, fr_array(t), m * n, m, fr_array(u), 3, proof, val))
    assert fr_ints(val) == [me_bruteforce(t, u)]
    # round 0 of me_open on the row-folded vector s: T = sum [s_i] g_i, T0 = sum_pairs [s_2i] g_2i+1, T1 = sum_pairs [s_2i+1] g_2i
    s = [(t[j] + u[2] * (t[n + j] - t[j])) % R_MOD for j in range(n)]
    T = None
    for j in range(n):
        T = ec_add(T, ec_mul(s[j], pts[j]))
    T0 = ec_add(ec_mul(s[0], pts[1]), ec_mul(s[2], pts[3]))
    T1 = ec_add(ec_mul(s[1], pts[0]), ec_mul(s[3], pts[2]))
    assert [jac_to_affine(p) for p in proof[:3]] == [T, T0, T1]
    # folded generators g' = g1 + [u](g0 - g1), scalars s' = s0 + u (s1 - s0); round 1 sums over the single pair
    g2 = [ec_add(pts[2 * i + 1], ec_mul(u[0], ec_add(pts[2 * i], ec_neg(pts[2 * i + 1])))) for i in range(2)]
    s2 = [(s[2 * i] + u[0] * (s[2 * i + 1] - s[2 * i])) % R_MOD for i in range(2)]
    assert jac_to_affine(proof[3]) == ec_add(ec_mul(s2[0], g2[0]), ec_mul(s2[1], g2[1]))
    assert jac_to_affine(proof[4]) == ec_mul(s2[0], g2[1])
    assert jac_to_affine(proof[5]) == ec_mul(s2[1], g2[0])
    assert jac_to_affine(proof[6]) == ec_add(g2[1], ec_mul(u[1], ec_add(g2[0], ec_neg(g2[1]))))


def test_g1_me_matches_textbook():
    orc = load_oracle()
    rng = random.Random(43)
    g = gens_from_seed(orc, 8, 3)
    pts = [jac_to_affine(r) for r in g]
    u = [rng.randrange(R_MOD) for _ in range(2)]
    out = np.zeros(36, np.uint32)
    orc_check(orc.orc_g1_me(g, 3, fr_array(u), 2, out))
    # the reference multiplies by unmont(u) = u / R (g1-tensor.cu:491)
    rinv = pow(1 << 256, -1, R_MOD)
    x = [v * rinv % R_MOD for v in u]
    lvl = [ec_add(pts[0], ec_mul(x[0], ec_add(pts[1], ec_neg(pts[0])))), ec_add(pts[2], ec_neg(ec_mul(x[0], pts[2])))]
    exp = ec_add(lvl[0], ec_mul(x[1], ec_add(lvl[1], ec_neg(lvl[0]))))
    assert jac_to_affine(out) == exp
