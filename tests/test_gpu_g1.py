"""GPU parity: G1 tensor kernels, Pedersen commitment (fixed-base windowed MSM) and its opening, compared
with the CPU oracle as group elements (both sides normalised to z = ONE, which makes them byte-equal)."""
import random

import numpy as np
import pytest

from zkhelp import (G1_X, G1_Y, P_MOD, R_MOD, affine_to_jac, ec_add, ec_mul, fr_array, fr_ints, jac_to_affine, load_oracle,
                    mt_random_vec, orc_check)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pv():
    from gpuhelp import Prover
    return Prover()


@pytest.fixture(scope="module")
def orc():
    return load_oracle()


def norm(orc, pts):
    pts = np.ascontiguousarray(pts, dtype=np.uint32).reshape(-1, 36)
    out = np.zeros_like(pts)
    orc_check(orc.orc_g1_op(3, pts, pts, out, pts.shape[0]))
    return out


def oracle_gens(orc, seed, n):
    orc.orc_seed(seed)
    g = np.zeros((n, 36), np.uint32)
    orc_check(orc.orc_commitment_random(n, g))
    return g


def test_generators_match_oracle_stream(pv, orc):
    pv.seed(321)
    g = pv.commitment_random(8)
    exp = oracle_gens(orc, 321, 8)
    assert (norm(orc, g.host()) == norm(orc, exp)).all()
    assert jac_to_affine(g.host()[0]) == ec_mul(fr_ints(mt_random_vec(np.random.RandomState(321), 1))[0], (G1_X, G1_Y))


def test_elementwise_and_special_cases(pv, orc):
    gens = oracle_gens(orc, 11, 16)
    inf = np.zeros(36, np.uint32)
    A = gens.copy()
    B = gens[::-1].copy()
    B[0] = A[0]                      # equal points -> doubling branch
    neg = np.zeros_like(A[:1])
    orc_check(orc.orc_g1_op(4, A[1:2].copy(), A[1:2].copy(), neg, 1))
    B[1] = neg[0]                    # opposite points -> infinity
    A[2] = inf                       # infinity + Q
    B[3] = inf                       # P + infinity
    hA, hB = pv.g1_from_host(A), pv.g1_from_host(B)
    exp = np.zeros_like(A)
    orc_check(orc.orc_g1_op(0, A, B, exp, 16))
    got = pv.g1_binop(0, hA, hB).host()
    assert (norm(orc, got) == norm(orc, exp)).all()
    assert not norm(orc, got)[1].any()          # canonical infinity = all-zero limbs
    # subtraction and negation
    nb = np.zeros_like(B)
    orc_check(orc.orc_g1_op(4, B, B, nb, 16))
    orc_check(orc.orc_g1_op(0, A, nb, exp, 16))
    assert (norm(orc, pv.g1_binop(1, hA, hB).host()) == norm(orc, exp)).all()
    assert (norm(orc, pv.g1_binop(2, hB).host()) == norm(orc, nb)).all()
    # device-side normalisation equals the oracle's
    assert (pv.g1_binop(3, hA).host() == norm(orc, A)).all()
    # broadcast add / mixed add of one point
    P = gens[5]
    Pb = np.tile(P, (16, 1))
    orc_check(orc.orc_g1_op(0, A, Pb, exp, 16))
    assert (norm(orc, pv.g1_pointop(0, hA, P).host()) == norm(orc, exp)).all()
    Pn = norm(orc, P)[0]
    assert (norm(orc, pv.g1_pointop(2, hA, Pn).host()) == norm(orc, exp)).all()


def test_affine_tensor_ops(pv, orc, tmp_path):
    """G1TensorAffine against the Jacobian arithmetic of the oracle: mixed additions and subtractions (also in place,
    with an equal point -> doubling, an opposite point -> infinity and an infinite left operand), negation, the
    conversion, the file round trip and the element read."""
    n = 70                                         # more than one workgroup
    gens = oracle_gens(orc, 12, n)
    A = gens.copy()
    B = norm(orc, gens[::-1].copy())
    B[0] = norm(orc, A[:1])[0]                     # equal
    neg = np.zeros_like(A[:1])
    orc_check(orc.orc_g1_op(4, A[1:2].copy(), A[1:2].copy(), neg, 1))
    B[1] = norm(orc, neg)[0]                       # opposite
    A[2] = np.zeros(36, np.uint32)                 # infinity + Q
    aff = np.ascontiguousarray(B[:, :24])
    hA = pv.g1_from_host(A)
    exp, nb = np.zeros_like(A), np.zeros_like(B)
    orc_check(orc.orc_g1_op(2, A, B, exp, n))
    for op in (0, 2):
        got = norm(orc, pv.g1_affineop(op, hA, aff).host())
        assert (got == norm(orc, exp)).all() and not got[1].any()
    orc_check(orc.orc_g1_op(4, B, B, nb, n))
    orc_check(orc.orc_g1_op(2, A, nb, exp, n))
    for op in (1, 3):
        assert (norm(orc, pv.g1_affineop(op, hA, aff).host()) == norm(orc, exp)).all()
    assert (pv.g1_affineop(4, hA, aff).host() == B).all()                          # z = one in Montgomery form
    assert (pv.g1_affineop(5, hA, aff).host() == norm(orc, nb)).all()
    assert (pv.g1_affineop(6, hA, aff, str(tmp_path / "aff.bin")).host() == B).all()
    assert (tmp_path / "aff.bin").stat().st_size == n * 96
    assert (pv.g1_affineop(7, hA, aff).host() == B[-1:]).all()
    with pytest.raises(RuntimeError):
        pv.g1_affineop(0, hA, aff[:5])


def test_scalar_mul_sum_rowsum_me(pv, orc):
    gens = oracle_gens(orc, 12, 8)
    rng = random.Random(3)
    ks = [0, 1, 2, R_MOD - 1, 2 ** 31 - 1] + [rng.randrange(R_MOD) for _ in range(19)]   # 24 = 3 x 8 scalars, broadcast over the generators
    S = fr_array(ks)
    exp = np.zeros((24, 36), np.uint32)
    orc_check(orc.orc_g1_mul(gens, 8, S, exp, 24, 0))
    hG, hS = pv.g1_from_host(gens), pv.from_fr(S)
    got = pv.g1_scalar_mul(hG, hS)
    assert (norm(orc, got.host()) == norm(orc, exp)).all()
    tot = np.zeros(36, np.uint32)
    orc_check(orc.orc_g1_sum(exp, 24, tot))
    assert (norm(orc, pv.g1_sum(got)) == norm(orc, tot)).all()
    rows = np.zeros((3, 36), np.uint32)
    for r in range(3):
        orc_check(orc.orc_g1_sum(exp[8 * r:8 * r + 8].copy(), 8, rows[r]))
    assert (norm(orc, pv.g1_rowwise_sum(got, 3, 8).host()) == norm(orc, rows)).all()
    u = mt_random_vec(np.random.RandomState(4), 3)
    me = np.zeros(36, np.uint32)
    orc_check(orc.orc_g1_me(gens, 8, u, 3, me))
    assert (norm(orc, pv.g1_me(hG, u)) == norm(orc, me)).all()
    # larger sum exercising the segmented reduction
    big = np.tile(gens, (200, 1))[:1500]
    orc_check(orc.orc_g1_sum(big, 1500, tot))
    assert (norm(orc, pv.g1_sum(pv.g1_from_host(big))) == norm(orc, tot)).all()


@pytest.mark.parametrize("m,n,lim", [(1, 1, 100), (3, 4, 2 ** 15), (16, 64, 2 ** 14), (5, 64, 2 ** 31 - 1), (300, 32, 2 ** 13)])
def test_commit_int_matches_oracle(pv, orc, m, n, lim):
    print("case", m, n, lim, flush=True)
    gens = oracle_gens(orc, 13 + n, n)
    rng = np.random.default_rng(m * n)
    t = rng.integers(-lim, lim, m * n, endpoint=True).astype(np.int64)
    t[0] = 0
    if m * n > 2:
        t[1], t[2] = lim, -lim
    T = fr_array([int(x) % R_MOD for x in t])
    exp = np.zeros((m, 36), np.uint32)
    orc_check(orc.orc_commit_int(gens, n, T, m * n, exp))
    got = pv.commit_int(pv.g1_from_host(gens), pv.from_fr(T)).host()
    assert (norm(orc, got) == norm(orc, exp)).all()


def test_commit_int_rejects_non_integer_scalars_and_is_linear(pv, orc):
    gens = oracle_gens(orc, 14, 8)
    hG = pv.g1_from_host(gens)
    bad = fr_array([R_MOD >> 1] * 8)
    with pytest.raises(RuntimeError, match="int32"):
        pv.commit_int(hG, pv.from_fr(bad))
    rng = np.random.default_rng(9)
    a, b = rng.integers(-1000, 1000, 8), rng.integers(-1000, 1000, 8)
    ca = jac_to_affine(pv.commit_int(hG, pv.from_i32(a)).host()[0])
    cb = jac_to_affine(pv.commit_int(hG, pv.from_i32(b)).host()[0])
    cab = jac_to_affine(pv.commit_int(hG, pv.from_i32(a + b)).host()[0])
    assert ec_add(ca, cb) == cab
    # the general-scalar commit agrees with commit_int on integers
    assert jac_to_affine(pv.commit(hG, pv.from_i32(a)).host()[0]) == ca


# 300 x 1: raw small integers, whose negative embeddings share their high bytes (one bucket receives whole chunks);
# 4500 x 2: more than one chunk of the bucket kernel and odd sizes in several rounds; 20000 x 2: two halving rounds
# (the second takes T from the first round's points) before the batched rest; 70000 x 1: four halving rounds, so T of
# rounds 1..3 are combinations of up to seven earlier points, with an odd size (4375 pairs + 1) on the way
# 9001 x 1: an odd size in the first halving round, whose T is the sum over pairs with one element left alone
@pytest.mark.parametrize("n,m", [(4, 2), (8, 1), (16, 4), (5, 3), (1, 2), (300, 1), (4500, 2), (9001, 1), (20000, 2), (70000, 1)])
def test_open_value_and_g1_transcript(pv, orc, n, m):
    gens = oracle_gens(orc, 15 + n, n)
    rng = np.random.default_rng(n * m)
    t = rng.integers(-2 ** 15, 2 ** 15, m * n).astype(np.int64)
    T = fr_array([int(x) % R_MOD for x in t])
    k = (n - 1).bit_length() + (m - 1).bit_length()
    u = mt_random_vec(np.random.RandomState(16), k)
    exp_proof = np.zeros((3 * (n - 1).bit_length() + 1, 36), np.uint32)
    exp_val = np.zeros(8, np.uint32)
    # rows are padded to a power of two exactly as verifyWeightClaim pads the weight
    mp = 1 << (m - 1).bit_length()
    Tp = np.concatenate([T, np.zeros(((mp - m) * n, 8), np.uint32)])
    orc_check(orc.orc_open(gens, n, Tp, mp * n, mp, u, k, exp_proof, exp_val))
    hG, hT = pv.g1_from_host(gens), pv.from_fr(Tp)
    com = pv.commit_int(hG, hT)
    val, proof = pv.open(hG, hT, com, u)
    assert (val == exp_val).all()
    assert proof.shape == exp_proof.shape
    assert (norm(orc, proof) == norm(orc, exp_proof)).all()


@pytest.mark.parametrize("n,val", [(300, 70000), (5000, -3), (5000, 0)])
def test_open_with_equal_scalars(pv, orc, n, val):
    """Every scalar in the same bucket of every window (norm weights share their high bytes; here all bytes): the
    bucket sums must not depend on how the elements spread over the buckets."""
    gens = oracle_gens(orc, 40 + n, n)
    T = fr_array([val % R_MOD] * n)
    k = (n - 1).bit_length()
    u = mt_random_vec(np.random.RandomState(17), k)
    exp_proof = np.zeros((3 * k + 1, 36), np.uint32)
    exp_val = np.zeros(8, np.uint32)
    orc_check(orc.orc_open(gens, n, T, n, 1, u, k, exp_proof, exp_val))
    hG, hT = pv.g1_from_host(gens), pv.from_fr(T)
    com = pv.commit_int(hG, hT)
    val_got, proof = pv.open(hG, hT, com, u)
    assert (val_got == exp_val).all()
    assert (norm(orc, proof) == norm(orc, exp_proof)).all()


def test_open_with_equal_opposite_and_infinite_generators_in_the_first_round(pv, orc):
    """More generators than the batched rest takes, so the first round halves them on the device: pairs of equal
    generators (their sum is a doubling), of opposite ones (their sum is infinity), with an infinite member, and an
    infinite pair, in the pair sums that give T, in the fold and in the bucket sums."""
    n = 8200
    gens = oracle_gens(orc, 77, n)
    neg = np.zeros((1, 36), np.uint32)
    gens[1] = gens[0]
    orc_check(orc.orc_g1_op(4, gens[2:3].copy(), gens[2:3].copy(), neg, 1))
    gens[3] = neg[0]
    gens[5] = 0
    gens[6] = 0
    gens[7] = 0
    gens[8] = 0
    T = mt_random_vec(np.random.RandomState(3), n)
    k = (n - 1).bit_length()
    u = mt_random_vec(np.random.RandomState(18), k)
    exp_proof = np.zeros((3 * k + 1, 36), np.uint32)
    exp_val = np.zeros(8, np.uint32)
    orc_check(orc.orc_open(gens, n, T, n, 1, u, k, exp_proof, exp_val))
    hG, hT = pv.g1_from_host(gens), pv.from_fr(T)
    com = pv.g1_from_host(np.zeros((1, 36), np.uint32))
    val_got, proof = pv.open(hG, hT, com, u)
    assert (val_got == exp_val).all()
    assert (norm(orc, proof) == norm(orc, exp_proof)).all()


def test_open_begin_end_matches_open_through_the_c_abi(orc):
    """zk_g1_open_begin/_end (openings on the library's own streams, several in flight, results fetched in another
    order) deliver exactly what zk_g1_open delivers: the proof points are normalised, so even the bytes agree."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    cases = []
    for n, seed in ((37, 3), (9000, 4), (1, 5)):
        gens = oracle_gens(orc, 60 + n, n)
        S = mt_random_vec(np.random.RandomState(seed), n)
        k = max(1, (n - 1).bit_length())
        u = mt_random_vec(np.random.RandomState(seed + 10), k)
        dG, dS = hip.upload(gens), hip.upload(S)
        proof = np.zeros((3 * k + 1, 36), np.uint32)
        val = np.zeros(8, np.uint32)
        hip.call("zk_g1_open", proof, val, c_void_p(dS), c_void_p(dG), c_size_t(n), u, c_int(k), None)
        cases.append((n, k, u, dG, dS, proof, val))
    handles = []
    for n, k, u, dG, dS, _, _ in cases:
        h = c_void_p()
        hip.call("zk_g1_open_begin", ctypes.byref(h), c_void_p(dS), c_void_p(dG), c_size_t(n), u, c_int(k), None)
        handles.append(h)
    for (n, k, u, dG, dS, proof, val), h in reversed(list(zip(cases, handles))):
        p2 = np.zeros_like(proof)
        v2 = np.zeros(8, np.uint32)
        hip.call("zk_g1_open_end", h, p2, v2)
        assert (v2 == val).all(), n
        assert (p2 == proof).all(), n
    for _, _, _, dG, dS, _, _ in cases:
        hip.free(dG)
        hip.free(dS)


def test_open_batch_over_prepared_generators_matches_single_openings(orc):
    """zk_g1_open_begin_batch (openings of one size as ONE job: every round's kernels launched once for all of them) over
    generators prepared with zk_g1_open_prepare delivers, opening by opening, the bytes of zk_g1_open.  Sizes on both
    sides of the batched last rounds, a ragged one (odd halves: its first two rounds run on the prepared tables), special
    generators (equal, opposite, infinite, also among the second round's prepared points) in one member of the batch,
    and zk_g1_open_begin_prepared alone."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    for n, count in ((9001, 3), (600, 2), (4096, 8), (2049, 2)):
        k = (n - 1).bit_length()
        npts = 3 * k + 1
        gens, dG, dS, us, preps = [], [], [], [], []
        exp_p = np.zeros((count, npts, 36), np.uint32)
        exp_v = np.zeros((count, 8), np.uint32)
        for i in range(count):
            g = oracle_gens(orc, 300 + 7 * i + n, n)
            if i == 1 and n > 20:
                neg = np.zeros((1, 36), np.uint32)
                g[1] = g[0]
                orc_check(orc.orc_g1_op(4, g[2:3].copy(), g[2:3].copy(), neg, 1))
                g[3] = neg[0]
                g[6] = 0
                g[7] = 0
                g[9] = 0
                # special among the points of the second round's tables (pairs of pairs g_4j .. g_4j+3): equal odd members
                # (their difference is infinity), equal pair differences (infinity again), opposite odd members (a doubling)
                g[15] = g[13]
                g[18] = g[16]
                g[19] = g[17]
                orc_check(orc.orc_g1_op(4, g[21:22].copy(), g[21:22].copy(), neg, 1))
                g[23] = neg[0]
            S = mt_random_vec(np.random.RandomState(50 + i), n)
            u = mt_random_vec(np.random.RandomState(70 + i), k)
            gens.append(g); us.append(u)
            dG.append(hip.upload(g)); dS.append(hip.upload(S))
            print(f"open n={n} item={i}: zk_g1_open", flush=True)
            hip.call("zk_g1_open", exp_p[i], exp_v[i], c_void_p(dS[i]), c_void_p(dG[i]), c_size_t(n), u, c_int(k), None)
            pr = c_void_p()
            print(f"open n={n} item={i}: zk_g1_open_prepare", flush=True)
            hip.call("zk_g1_open_prepare", ctypes.byref(pr), c_void_p(dG[i]), c_size_t(n), None)
            preps.append(pr)
        h = c_void_p()
        sc = (c_void_p * count)(*[c_void_p(x) for x in dS])
        pp = (c_void_p * count)(*preps)
        uall = np.ascontiguousarray(np.concatenate(us), dtype=np.uint32)
        print(f"open n={n}: zk_g1_open_begin_batch of {count}", flush=True)
        hip.call("zk_g1_open_begin_batch", ctypes.byref(h), c_int(count), sc, pp, uall, c_int(k), None)
        got_p = np.zeros_like(exp_p)
        got_v = np.zeros_like(exp_v)
        hip.call("zk_g1_open_end_batch", h, got_p, got_v)
        assert (got_v == exp_v).all(), n
        assert (got_p == exp_p).all(), n
        # one prepared opening on its own
        h1 = c_void_p()
        print(f"open n={n}: zk_g1_open_begin_prepared", flush=True)
        hip.call("zk_g1_open_begin_prepared", ctypes.byref(h1), c_void_p(dS[0]), preps[0], us[0], c_int(k), None)
        p1 = np.zeros((npts, 36), np.uint32)
        v1 = np.zeros(8, np.uint32)
        hip.call("zk_g1_open_end", h1, p1, v1)
        assert (v1 == exp_v[0]).all() and (p1 == exp_p[0]).all(), n
        for pr in preps:
            hip.call("zk_g1_open_prepared_free", pr)
        for x in dG + dS:
            hip.free(x)


def test_open_batch_with_row_commitments_delivers_the_points_of_the_plain_opening(pv):
    """zk_g1_open_begin_batch_rows takes the first round's T from the tensors' row commitments (sum_r eq(u_rows, r) C_r)
    instead of summing over all generators: for commitments made by commit_int of the same tensors every point of the
    proof, T of the first round included, equals zk_g1_open's on the row-folded vector.  One tensor with a number of
    rows that is no power of two, one with a single row (no row challenge), more generators than the batched last
    rounds take; and with another tensor's commitments only the T of the halving rounds change."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    pv.lib.zkp_g1_devptr.restype = ctypes.c_void_p
    n = 5000
    k = (n - 1).bit_length()
    npts = 3 * k + 1
    pv.seed(77)
    gens = pv.commitment_random(n)
    dG = pv.lib.zkp_g1_devptr(c_void_p(gens.h))
    prep = c_void_p()
    hip.call("zk_g1_open_prepare", ctypes.byref(prep), c_void_p(dG), c_size_t(n), None)
    rng = np.random.default_rng(5)
    keep, folded, coms, urows, us = [], [], [], [], []
    exp_p = np.zeros((2, npts, 36), np.uint32)
    exp_v = np.zeros((2, 8), np.uint32)
    for i, nrows in enumerate((5, 1)):
        W = pv.from_i32(rng.integers(-30000, 30000, nrows * n).astype(np.int32))
        com = pv.commit_int(gens, W)
        assert com.size == nrows
        kr = (nrows - 1).bit_length()
        ur = mt_random_vec(np.random.RandomState(40 + i), max(kr, 1))[:kr]
        f = pv.partial_me_window(W, ur, n) if kr else W
        assert f.size == n
        u = mt_random_vec(np.random.RandomState(60 + i), k)
        print(f"rows={nrows}: zk_g1_open", flush=True)
        hip.call("zk_g1_open", exp_p[i], exp_v[i], c_void_p(f.devptr), c_void_p(dG), c_size_t(n), u, c_int(k), None)
        keep += [W, com, f]
        folded.append(f); coms.append(com); urows.append(np.ascontiguousarray(ur, dtype=np.uint32)); us.append(u)

    def run(com_order):
        h = c_void_p()
        sc = (c_void_p * 2)(*[c_void_p(f.devptr) for f in folded])
        pp = (c_void_p * 2)(prep, prep)
        rows = (c_void_p * 2)(*[c_void_p(pv.lib.zkp_g1_devptr(c_void_p(coms[j].h))) for j in com_order])
        nr = np.array([coms[j].size for j in com_order], np.uint32)
        ur = (c_void_p * 2)(*[c_void_p(urows[j].ctypes.data if urows[j].size else None) for j in com_order])
        kr = np.array([urows[j].shape[0] for j in com_order], np.int32)
        uall = np.ascontiguousarray(np.concatenate(us), dtype=np.uint32)
        print(f"zk_g1_open_begin_batch_rows, commitments {com_order}", flush=True)
        hip.call("zk_g1_open_begin_batch_rows", ctypes.byref(h), c_int(2), sc, pp, uall, c_int(k), rows, nr, ur, kr, c_int(0), None)
        got_p = np.zeros_like(exp_p)
        got_v = np.zeros_like(exp_v)
        hip.call("zk_g1_open_end_batch", h, got_p, got_v)
        return got_p, got_v

    got_p, got_v = run((0, 1))
    assert (got_v == exp_v).all()
    assert (got_p == exp_p).all()
    # the statement "these are the tensor's row commitments" is the caller's: with the other tensor's, T of the first round
    # is what those commitments give, and with it T of the later halving rounds, which follow from the earlier rounds' points
    # (5000 -> 2500 -> 1250 -> 625 generators, then the batched last rounds, which sum over the generators); T0, T1 of
    # every round, the folded generator and the value do not depend on them
    got_p, got_v = run((1, 0))
    assert (got_v == exp_v).all()
    same = np.ones(npts, bool)
    same[[0, 3, 6]] = False
    assert (got_p[:, same] == exp_p[:, same]).all()
    for i in range(2):
        assert not (got_p[i, 0] == exp_p[i, 0]).all() and not (got_p[i, 3] == exp_p[i, 3]).all() and not (got_p[i, 6] == exp_p[i, 6]).all()
    hip.call("zk_g1_open_prepared_free", prep)


@pytest.mark.parametrize("n,R,tables", [(8192, 2, 2), (16384, 3, 3), (32768, 3, 3)])
def test_open_batch_with_cross_commitments_needs_no_sum_over_the_generators(pv, orc, n, R, tables):
    """With the cross commitments of its first R rounds -- commitments of every 2nd / 4th / 8th column of the tensor's rows
    under every 2nd / 4th / 8th generator, made here with commit_int on slices -- zk_g1_open_begin_batch_rows forms T, T0 and
    T1 of those rounds from rows x patterns points: of the three halvings of 8192 generators before the batched last rounds
    only the third sums over its generators.  With three rounds of them and the tables of zk_g1_open_prepare_tables(.., 3) the
    three rounds are one fold (16384 generators: that fold, one ordinary round and the batched last rounds; 32768: two ordinary
    rounds behind it).  Every point of the proof equals zk_g1_open's on the row-folded vector, and at 16384 generators also the
    oracle's own opening of the padded tensor (Commitment::open, commitment.cu:133-141: row fold, then me_open), point by
    point after normalisation, so the batched path is compared with the reference's algorithm directly."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    pv.lib.zkp_g1_devptr.restype = ctypes.c_void_p
    k = (n - 1).bit_length()
    npts = 3 * k + 1
    pv.seed(78)
    gens = pv.commitment_random(n)
    gens_host = gens.host()
    dG = pv.lib.zkp_g1_devptr(c_void_p(gens.h))
    prep = c_void_p()
    hip.call("zk_g1_open_prepare_tables", ctypes.byref(prep), c_void_p(dG), c_size_t(n), c_int(tables), None)
    rng = np.random.default_rng(6)
    keep, folded, cross, urows, us = [], [], [], [], []
    exp_p = np.zeros((2, npts, 36), np.uint32)
    exp_v = np.zeros((2, 8), np.uint32)
    for i, nrows in enumerate((3, 4)):
        Wi = rng.integers(-30000, 30000, (nrows, n)).astype(np.int32)
        W = pv.from_i32(Wi.ravel())
        pats = [pv.commit_int(gens, W).host()]
        for q in range(R):
            half, L = 1 << q, 2 << q
            for side in (0, 1):
                for a in range(half):
                    for b in range(half):
                        s_off, g_off = (half if side else 0) + a, (0 if side else half) + b
                        sub_g = pv.g1_from_host(np.ascontiguousarray(gens_host[g_off::L]))
                        sub_w = pv.from_i32(np.ascontiguousarray(Wi[:, s_off::L]).ravel())
                        pats.append(pv.commit_int(sub_g, sub_w).host())
        assert len(pats) == 1 + 2 * (4 ** R - 1) // 3 and all(x.shape == (nrows, 36) for x in pats)
        cross.append(hip.upload(np.ascontiguousarray(np.concatenate(pats))))
        kr = (nrows - 1).bit_length()
        ur = mt_random_vec(np.random.RandomState(45 + i), kr)
        f = pv.partial_me_window(W, ur, n)
        u = mt_random_vec(np.random.RandomState(65 + i), k)
        print(f"rows={nrows}: zk_g1_open", flush=True)
        hip.call("zk_g1_open", exp_p[i], exp_v[i], c_void_p(f.devptr), c_void_p(dG), c_size_t(n), u, c_int(k), None)
        keep += [W, f]
        folded.append(f); urows.append(np.ascontiguousarray(ur, dtype=np.uint32)); us.append(u)
        if n == 16384:
            rows_p = 1 << kr
            Tp = np.zeros((rows_p * n, 8), np.uint32)
            Tp[:nrows * n] = fr_array([int(x) % R_MOD for x in Wi.ravel()])
            o_p, o_v = np.zeros((npts, 36), np.uint32), np.zeros(8, np.uint32)
            print(f"rows={nrows}: oracle opening over {n} generators", flush=True)
            orc_check(orc.orc_open(np.ascontiguousarray(gens_host), n, Tp, rows_p * n, rows_p, np.ascontiguousarray(np.concatenate([u, ur]), dtype=np.uint32), k + kr, o_p, o_v))
            assert (o_v == exp_v[i]).all()
            assert (norm(orc, o_p) == exp_p[i]).all()          # the product delivers its points normalised
    for cr in (R, 1):
        h = c_void_p()
        sc = (c_void_p * 2)(*[c_void_p(f.devptr) for f in folded])
        pp = (c_void_p * 2)(prep, prep)
        rows = (c_void_p * 2)(*[c_void_p(x) for x in cross])
        nr = np.array([3, 4], np.uint32)
        ur = (c_void_p * 2)(*[c_void_p(x.ctypes.data) for x in urows])
        kr = np.array([x.shape[0] for x in urows], np.int32)
        uall = np.ascontiguousarray(np.concatenate(us), dtype=np.uint32)
        print(f"zk_g1_open_begin_batch_rows with {cr} rounds of cross commitments", flush=True)
        hip.call("zk_g1_open_begin_batch_rows", ctypes.byref(h), c_int(2), sc, pp, uall, c_int(k), rows, nr, ur, kr, c_int(cr), None)
        got_p = np.zeros_like(exp_p)
        got_v = np.zeros_like(exp_v)
        hip.call("zk_g1_open_end_batch", h, got_p, got_v)
        assert (got_v == exp_v).all(), cr
        assert (got_p == exp_p).all(), cr
    hip.call("zk_g1_open_prepared_free", prep)
    for x in cross:
        hip.free(x)


def test_fixed_base_multiplication_equals_the_generic_one_and_big_integer_arithmetic(orc):
    """zk_g1_fixed_base_mul (what Commitment::random runs on) against zk_g1_scalar_mul on the same base and, for the
    small cases, against affine big-integer arithmetic: digits at the signed-window boundaries (127, 128, 129, bytes of
    0x80 and 0xff that carry all the way up), zero, r - 1 and integers above r up to 2^256 - 1; a second base replaces the
    table kept on the device and the first base builds it again."""
    from gpuhelp import Hip, c_void_p, c_size_t
    hip = Hip()
    edge = [0, 1, 2, 127, 128, 129, 255, 256, 0x8080, 0x80 << 248, (1 << 255) - 1, R_MOD - 1, R_MOD, R_MOD + 5,
            (1 << 256) - 1, int("80" * 32, 16), int("7f" * 32, 16), int("81" * 32, 16), 1 << 255]
    S = np.concatenate([fr_array(edge), mt_random_vec(np.random.RandomState(77), 300)])
    n = S.shape[0]
    G = affine_to_jac((G1_X, G1_Y))
    other = oracle_gens(orc, 91, 1)[0]
    dS, dF, dM, dB = hip.upload(S), hip.malloc(144 * n), hip.malloc(144 * n), hip.malloc(144)
    for base in (G, other, G):
        base = np.ascontiguousarray(base, dtype=np.uint32)
        hip.call("zk_memcpy_h2d", c_void_p(dB), base, c_size_t(144), None)
        hip.call("zk_g1_fixed_base_mul", c_void_p(dF), base, c_void_p(dS), c_size_t(n), None)
        hip.call("zk_g1_scalar_mul", c_void_p(dM), c_void_p(dB), c_void_p(dS), c_size_t(1), c_size_t(n), None)
        fixed, generic = hip.download(dF, (n, 36), np.uint32), hip.download(dM, (n, 36), np.uint32)
        assert (norm(orc, fixed) == norm(orc, generic)).all()
        assert not norm(orc, fixed)[0].any()                     # [0] B is the point at infinity
    for i in (1, 3, 4, 5, 11, 14):
        assert jac_to_affine(fixed[i]) == ec_mul(edge[i] % R_MOD, (G1_X, G1_Y)), i
    for p in (dS, dF, dM, dB):
        hip.free(p)


def test_config3_full_size_commitment_and_opening_pass_the_verifier(pv, orc):
    """A 11008 x 4096 fixed-point weight (scale 2^16, N(0, 0.02)) over 4096 generators, far beyond what the oracle can
    follow: the 11008 commitments and the opening at a random point are checked the way a verifier would, in big-integer
    affine arithmetic.  The first T of the opening is the commitments' own multilinear extension at the row challenges
    (this ties commit_int to the opening), every round satisfies T' = u(1-u) T + (1-u)^2 T0 + u^2 T1, the last one
    against [value] g_final, and the value is the tensor's multilinear extension computed apart from the opening."""
    m, n = 11008, 4096
    rng = np.random.default_rng(2024)
    W = np.round(rng.normal(0, 0.02, m * n) * 65536).astype(np.int32)
    pv.seed(33)
    hG = pv.commitment_random(n)
    hW = pv.from_i32(W)
    com = pv.commit_int(hG, hW)
    assert com.size == m
    k_in, k_out = 12, 14
    u = mt_random_vec(np.random.RandomState(34), k_in + k_out)
    val, proof = pv.open(hG, hW, com, u)
    assert proof.shape[0] == 3 * k_in + 1
    ui = fr_ints(u)
    # value = W(u_out, u_in), rows by the last 14 challenges
    assert (pv.multi_dim_me(hW, [u[k_in:], u[:k_in]], (m, n)) == val).all()
    # T of the first round = sum_rows eq(u_out, row) com_row; G1TensorJacobian::operator()(u) reads its challenges as u / R
    u_me = fr_array([x * (1 << 256) % R_MOD for x in ui[k_in:]])
    pts = [jac_to_affine(p) for p in proof]
    assert pts[0] == jac_to_affine(pv.g1_me(com, u_me))
    for r in range(k_in):
        x = ui[r]
        T, T0, T1 = pts[3 * r:3 * r + 3]
        nxt = ec_add(ec_add(ec_mul(x * (1 - x) % R_MOD, T), ec_mul((1 - x) * (1 - x) % R_MOD, T0)), ec_mul(x * x % R_MOD, T1))
        expect = pts[3 * r + 3] if r + 1 < k_in else ec_mul(fr_ints(val)[0], pts[3 * k_in])
        assert nxt == expect, r
    # linearity of the commitment on a few rows: com(a) + com(b) = com(a + b)
    rows = [0, 1, 5503, 11007]
    A = np.concatenate([W[r * n:(r + 1) * n] for r in rows])
    B = np.concatenate([W[((r + 7) % m) * n:((r + 7) % m + 1) * n] for r in rows])
    ca, cb, cab = (pv.commit_int(hG, pv.from_i32(x)).host() for x in (A, B, A + B))
    exp = np.zeros_like(ca)
    orc_check(orc.orc_g1_op(0, ca, cb, exp, len(rows)))
    assert (norm(orc, cab) == norm(orc, exp)).all()
    assert (norm(orc, ca) == norm(orc, com.host()[rows])).all()
