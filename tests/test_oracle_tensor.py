"""Pins the oracle's tensor- and protocol-level restatement (oracle/tensor.hpp) against what the
mathematics fixes: brute-force multilinear extensions, integer matmul mod r, sumcheck invariants.
A transposed operand, a wrong fold order or a dropped Montgomery correction fails one of these."""
import random

import numpy as np
import pytest

from zkhelp import R_MOD, fr_array, fr_ints, load_oracle, me_bruteforce, orc_check, orc_transcript


def rnd(rng, n):
    return [rng.randrange(R_MOD) for _ in range(n)]


def test_sum_and_me_against_bruteforce():
    orc = load_oracle()
    rng = random.Random(21)
    for n in (1, 2, 5, 8, 13, 16, 37):
        t = rnd(rng, n)
        k = max(0, (n - 1).bit_length())
        u = rnd(rng, k)
        out = np.zeros(8, np.uint32)
        orc_check(orc.orc_fr_sum(fr_array(t), n, out))
        assert fr_ints(out) == [sum(t) % R_MOD]
        orc_check(orc.orc_fr_me(fr_array(t), n, fr_array(u) if k else np.zeros((0, 8), np.uint32), k, out))
        assert fr_ints(out) == [me_bruteforce(t, u)]
    # Boolean points return the table entries
    t = rnd(rng, 8)
    for i in range(8):
        u = [(i >> j) & 1 for j in range(3)]
        out = np.zeros(8, np.uint32)
        orc_check(orc.orc_fr_me(fr_array(t), 8, fr_array(u), 3, out))
        assert fr_ints(out) == [t[i]]


def me_axis(t, shape, axis, u):
    """brute-force fold of one axis of a row-major tensor (zero-extended), returns flat list"""
    other = int(np.prod(shape[:axis])) if axis else 1
    cur = shape[axis]
    win = int(np.prod(shape[axis + 1:])) if axis + 1 < len(shape) else 1
    out = []
    for o in range(other):
        for w in range(win):
            col = [t[(o * cur + c) * win + w] for c in range(cur)]
            out.append(me_bruteforce(col, u))
    # layout [other][1][win]
    res = [0] * (other * win)
    i = 0
    for o in range(other):
        for w in range(win):
            res[o * win + w] = out[i]
            i += 1
    return res


@pytest.mark.parametrize("other,cur,win", [(1, 8, 1), (3, 4, 5), (2, 5, 3), (4, 11, 1), (1, 6, 7)])
def test_partial_me_against_bruteforce(other, cur, win):
    orc = load_oracle()
    rng = random.Random(22)
    n = other * cur * win
    t = rnd(rng, n)
    k = (cur - 1).bit_length()
    u = rnd(rng, k)
    out = np.zeros((n, 8), np.uint32)
    out_n = np.zeros(1, np.int64)
    orc_check(orc.orc_fr_partial_me(fr_array(t), n, fr_array(u), k, cur, win, out, out_n))
    assert out_n[0] == other * win
    assert fr_ints(out[:other * win]) == me_axis(t, (other, cur, win), 1, u)


def test_window_fold_equals_axis_fold_and_zero_extends():
    orc = load_oracle()
    rng = random.Random(23)
    for nwin, win, extra in ((8, 4, 0), (5, 3, 0), (4, 4, 2)):
        n = nwin * win + extra
        t = rnd(rng, n)
        tot = nwin + (1 if extra else 0)
        k = (tot - 1).bit_length()
        u = rnd(rng, k)
        out = np.zeros((n + 2 * win, 8), np.uint32)
        out_n = np.zeros(1, np.int64)
        orc_check(orc.orc_fr_partial_me_window(fr_array(t), n, fr_array(u), k, win, out, out_n))
        padded = t + [0] * (tot * win - n)
        assert out_n[0] == win
        assert fr_ints(out[:win]) == me_axis(padded, (1, tot, win), 1, u)


def test_multi_dim_me_is_the_full_extension():
    orc = load_oracle()
    rng = random.Random(24)
    B, O = 4, 8
    t = rnd(rng, B * O)
    ub, uo = rnd(rng, 2), rnd(rng, 3)
    us = fr_array(ub + uo)
    out = np.zeros(8, np.uint32)
    orc_check(orc.orc_fr_multi_dim_me(fr_array(t), B * O, us, np.array([2, 3], np.uint32), np.array([B, O], np.uint32), 2, out))
    # flat index = b*O + o: low 3 bits <-> u_out, next 2 <-> u_batch
    assert fr_ints(out) == [me_bruteforce(t, uo + ub)]


def test_pad_transpose_matmul():
    orc = load_oracle()
    rng = random.Random(25)
    t = rnd(rng, 3 * 5)
    out = np.zeros((64, 8), np.uint32)
    out_n = np.zeros(1, np.int64)
    pv = fr_array([7])
    orc_check(orc.orc_fr_pad(fr_array(t), 15, np.array([3, 5], np.uint32), 2, pv, out, out_n))
    assert out_n[0] == 4 * 8
    exp = []
    for r in range(4):
        for c in range(8):
            exp.append(t[r * 5 + c] if (r < 3 and c < 5) else 7)
    assert fr_ints(out[:32]) == exp
    tr = np.zeros((15, 8), np.uint32)
    orc_check(orc.orc_fr_transpose(fr_array(t), 3, 5, tr))
    assert fr_ints(tr) == [t[r * 5 + c] for c in range(5) for r in range(3)]
    M, N, P = 3, 4, 5
    A = [rng.randrange(-1000, 1000) for _ in range(M * N)]
    Bm = [rng.randrange(-1000, 1000) for _ in range(N * P)]
    C = np.zeros((M * P, 8), np.uint32)
    orc_check(orc.orc_fr_matmul(fr_array([x % R_MOD for x in A]), fr_array([x % R_MOD for x in Bm]), M, N, P, C))
    exp = [sum(A[i * N + k] * Bm[k * P + j] for k in range(N)) % R_MOD for i in range(M) for j in range(P)]
    assert fr_ints(C) == exp
    # generic residues too
    A2, B2 = rnd(rng, M * N), rnd(rng, N * P)
    orc_check(orc.orc_fr_matmul(fr_array(A2), fr_array(B2), M, N, P, C))
    assert fr_ints(C) == [sum(A2[i * N + k] * B2[k * P + j] for k in range(N)) % R_MOD for i in range(M) for j in range(P)]


def brute_zkip(a, b, u):
    """round polynomials of the MSB-first inner-product sumcheck by direct summation"""
    polys, claim = [], sum(x * y for x, y in zip(a, b)) % R_MOD
    k = len(u)
    a, b = a + [0] * ((1 << k) - len(a)), b + [0] * ((1 << k) - len(b))
    for r in range(k):
        h = len(a) // 2
        v = u[k - 1 - r]
        c0 = sum(a[i] * b[i] for i in range(h)) % R_MOD
        c1 = sum(a[i] * (b[i + h] - b[i]) + b[i] * (a[i + h] - a[i]) for i in range(h)) % R_MOD
        c2 = sum((a[i + h] - a[i]) * (b[i + h] - b[i]) for i in range(h)) % R_MOD
        polys.append([c0, c1, c2])
        assert (2 * c0 + c1 + c2) % R_MOD == claim          # p(0) + p(1) == claim
        claim = (c0 + c1 * v + c2 * v * v) % R_MOD
        a = [(a[i] + v * (a[i + h] - a[i])) % R_MOD for i in range(h)]
        b = [(b[i] + v * (b[i + h] - b[i])) % R_MOD for i in range(h)]
    return polys, claim, a[0], b[0]


@pytest.mark.parametrize("n", [2, 8, 11, 64])
def test_zkip_round_polynomials_bruteforce(n):
    orc = load_oracle()
    rng = random.Random(26)
    a, b = rnd(rng, n), rnd(rng, n)
    k = (n - 1).bit_length()
    u = rnd(rng, k)
    claim = sum(x * y for x, y in zip(a, b)) % R_MOD
    proof = np.zeros((k, 3, 8), np.uint32)
    fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_zkip(fr_array([claim]), fr_array(a), fr_array(b), n, fr_array(u), k, proof, fin))
    polys, final, af, bf = brute_zkip(a, b, u)
    assert [fr_ints(p) for p in proof] == polys
    assert fr_ints(fin) == [final] == [af * bf % R_MOD]
    assert af == me_bruteforce(a, u) and bf == me_bruteforce(b, u)


def test_zkfc_scenario_claims():
    """zkFC::prove on the toy shape: Y(u_b,u_o) = sum_k X(u_b,k) W(k,u_o) and the final opening identity."""
    orc = load_oracle()
    rng = np.random.default_rng(27)
    B, I, O = 4, 8, 4
    X = np.round(rng.normal(0, 0.02, (B, I)) * 65536).astype(np.int32)
    W = np.round(rng.normal(0, 0.02, (I, O)) * 65536).astype(np.int32)
    orc.orc_seed(99)
    orc.orc_transcript_clear()
    Y = np.zeros((B * O, 8), np.uint32)
    cw = np.zeros(8, np.uint32)
    orc_check(orc.orc_zkfc(X, W, B, I, O, Y, cw))
    t = fr_ints(orc_transcript(orc))
    Yi = (X.astype(object) @ W.astype(object)).reshape(-1)
    assert fr_ints(Y) == [int(v) % R_MOD for v in Yi]
    # replay the challenge stream independently
    from zkhelp import mt_random_vec
    rs = np.random.RandomState(99)
    ub, ui, uo = (fr_ints(mt_random_vec(rs, k)) for k in (2, 3, 2))
    Xl = [int(v) % R_MOD for v in X.reshape(-1)]
    Wl = [int(v) % R_MOD for v in W.reshape(-1)]
    Yl = [int(v) % R_MOD for v in Yi]
    claim = me_bruteforce(Yl, uo + ub)
    assert t[0] == claim
    polys = [t[1 + 3 * r: 4 + 3 * r] for r in range(3)]
    final, claim_X, claim_W = t[10], t[11], t[12]
    assert claim_X == me_bruteforce(Xl, ui + ub)
    assert claim_W == me_bruteforce(Wl, uo + ui) == fr_ints(cw)[0]
    assert final == claim_X * claim_W % R_MOD
    cur = claim
    for r, (c0, c1, c2) in enumerate(polys):
        assert (2 * c0 + c1 + c2) % R_MOD == cur
        v = ui[2 - r]
        cur = (c0 + c1 * v + c2 * v * v) % R_MOD
    assert cur == final
