"""Pins the CPU oracle's field and curve arithmetic (oracle/ff.hpp).

Three independent anchors, so that a dropped term, wrong sign, wrong limb order or missing
Montgomery factor fails at least one of them:
  * python big-int closed forms ((a*b*R^-1) mod r, pow(a,-1,r), textbook affine curve law);
  * constants the reference itself holds (ONE, R2, P_sub_2, TWO_INV, generator hex comments);
  * the reference's bls12-381.cu compiled as host C++ (oracle/_ref/libzkref.so), bit for bit,
    when that library is present (it can only be built where /root/reference exists).
"""
import random

import numpy as np
import pytest

from zkhelp import (FP_R, FR_R, G1_X, G1_Y, P_MOD, R_MOD, affine_to_jac, ec_add, ec_mul, ec_neg, fp_array, fp_ints,
                    fr_array, fr_ints, from_limbs, jac_to_affine, load_oracle, load_ref, mt_random_vec, orc_check, to_limbs)

# limb tables as held by the reference (bls12-381.cu:3-11,595; tlookup.cu:179-180; g1-tensor.cuh:28-60)
REF_FR_ONE = [4294967294, 1, 215042, 1485092858, 3971764213, 2576109551, 2898593135, 405057881]
REF_FR_P = [1, 4294967295, 4294859774, 1404937218, 161601541, 859428872, 698187080, 1944954707]
REF_FR_R2 = [4092763245, 3382307216, 2274516003, 728559051, 1918122383, 97719446, 2673475345, 122214873]
REF_FR_P_SUB_2 = [4294967295, 4294967294, 4294859774, 1404937218, 161601541, 859428872, 698187080, 1944954707]
REF_TWO_INV = [2147483649, 2147483647, 2147429887, 2849952257, 80800770, 429714436, 2496577188, 972477353]
REF_TWO_INV_HEX = 0x39F6D3A994CEBEA4199CEC0404D0EC02A9DED2017FFF2DFF7FFFFFFF80000001
REF_FP_ONE = [196605, 1980301312, 3289120770, 3958636555, 1405573306, 1598593111, 1884444485, 2010011731, 2723605613, 1543969431, 4202751123, 368467651]
REF_FP_P = [4294945451, 3120496639, 2975072255, 514588670, 4138792484, 1731252896, 4085584575, 1685539716, 1129032919, 1260103606, 964683418, 436277738]
REF_FP_R2 = [473175878, 4108263220, 164693233, 175564454, 1284880085, 2380613484, 2476573632, 1743489193, 3038352685, 2591637125, 2462770090, 295210981]
REF_GX_MONT_HEX = 0x120177419E0BFB75EDCE6ECC21DBF440F0AE6ACDF3D0E747154F95C7143BA1C17817FC679976FFF55CB38790FD530C16
REF_GY_MONT_HEX = 0x0BBC3EFC5008A26A0E1C8C3FAD0059C051AC582950405194DD595F13570725CE8C22631A7918FD8EBAAC93D50CE72271

EDGE_FR = [0, 1, 2, R_MOD - 1, R_MOD - 2, FR_R, FR_R * FR_R % R_MOD, (1 << 32) - 1, ((1 << 32) - 1) << 32,
           (1944954706 << 224) | ((1 << 224) - 1), (1 << 254), R_MOD >> 1, (R_MOD + 1) >> 1]


def rand_fr(rng, n):
    return EDGE_FR + [rng.randrange(R_MOD) for _ in range(n)]


def test_reference_constants_are_the_standard_ones():
    assert from_limbs(REF_FR_P) == R_MOD
    assert from_limbs(REF_FR_ONE) == FR_R
    assert from_limbs(REF_FR_R2) == FR_R * FR_R % R_MOD
    assert from_limbs(REF_FR_P_SUB_2) == R_MOD - 2
    assert from_limbs(REF_TWO_INV) == pow(2, -1, R_MOD) == REF_TWO_INV_HEX
    assert (-pow(R_MOD, -1, 1 << 32)) % (1 << 32) == 4294967295
    assert from_limbs(REF_FP_P) == P_MOD
    assert from_limbs(REF_FP_ONE) == FP_R
    assert from_limbs(REF_FP_R2) == FP_R * FP_R % P_MOD
    assert (-pow(P_MOD, -1, 1 << 32)) % (1 << 32) == 4294770685
    assert G1_X * FP_R % P_MOD == REF_GX_MONT_HEX
    assert G1_Y * FP_R % P_MOD == REF_GY_MONT_HEX
    assert (G1_Y * G1_Y - G1_X ** 3 - 4) % P_MOD == 0
    assert ec_mul(R_MOD, (G1_X, G1_Y)) is None


def test_oracle_constants_match_reference_tables():
    orc = load_oracle()
    g = np.zeros(36, dtype=np.uint32)
    orc.orc_g1_generator(g)
    assert jac_to_affine(g) == (G1_X, G1_Y)
    one = fr_array([1])
    out = np.zeros_like(one)
    orc_check(orc.orc_fr_op(4, one, one, out, 1))  # mont(1) = ONE
    assert list(out[0]) == REF_FR_ONE
    orc_check(orc.orc_fr_op(4, fr_array([FR_R]), one, out, 1))  # mont(R) = R2
    assert list(out[0]) == REF_FR_R2
    orc_check(orc.orc_fr_op(8, fr_array([2]), one, out, 1))  # 1/2 in standard form = TWO_INV
    assert list(out[0]) == REF_TWO_INV


def test_fr_ops_against_bigint():
    orc = load_oracle()
    rng = random.Random(1)
    a = rand_fr(rng, 300)
    b = list(reversed(rand_fr(rng, 300)))
    A, B = fr_array(a), fr_array(b)
    out = np.zeros_like(A)
    n = len(a)
    rinv = pow(FR_R, -1, R_MOD)
    closed = {
        0: lambda x, y: (x + y) % R_MOD,
        1: lambda x, y: (x - y) % R_MOD,
        2: lambda x, y: x * y * rinv % R_MOD,
        3: lambda x, y: 2 * x % R_MOD,
        4: lambda x, y: x * FR_R % R_MOD,
        5: lambda x, y: x * rinv % R_MOD,
        7: lambda x, y: x * y % R_MOD,
        9: lambda x, y: (-x) % R_MOD,
    }
    for op, f in closed.items():
        orc_check(orc.orc_fr_op(op, A, B, out, n))
        assert fr_ints(out) == [f(x, y) for x, y in zip(a, b)], f"fr op {op}"
    # inverses (0 maps to 0, as 0^(r-2) does in the reference)
    orc_check(orc.orc_fr_op(8, A, B, out, n))
    assert fr_ints(out) == [pow(x, -1, R_MOD) if x else 0 for x in a]
    orc_check(orc.orc_fr_op(6, A, B, out, n))  # Montgomery in/out: (xR)^-1 R ... input x = yR -> y^-1 R
    assert fr_ints(out) == [pow(x * rinv % R_MOD, -1, R_MOD) * FR_R % R_MOD if x else 0 for x in a]


def test_fp_ops_against_bigint():
    orc = load_oracle()
    rng = random.Random(2)
    edge = [0, 1, 2, P_MOD - 1, P_MOD - 2, FP_R, (1 << 380), (436277737 << 352) | ((1 << 352) - 1)]
    a = edge + [rng.randrange(P_MOD) for _ in range(200)]
    b = list(reversed(a))
    A, B = fp_array(a), fp_array(b)
    out = np.zeros_like(A)
    rinv = pow(FP_R, -1, P_MOD)
    closed = {
        0: lambda x, y: (x + y) % P_MOD,
        1: lambda x, y: (x - y) % P_MOD,
        2: lambda x, y: x * y * rinv % P_MOD,
        3: lambda x, y: 2 * x % P_MOD,
        4: lambda x, y: x * FP_R % P_MOD,
        5: lambda x, y: x * rinv % P_MOD,
    }
    for op, f in closed.items():
        orc_check(orc.orc_fp_op(op, A, B, out, len(a)))
        assert fp_ints(out) == [f(x, y) for x, y in zip(a, b)], f"fp op {op}"
    orc_check(orc.orc_fp_op(6, A, B, out, len(a)))
    assert fp_ints(out) == [pow(x * rinv % P_MOD, -1, P_MOD) * FP_R % P_MOD if x else 0 for x in a]


def _rand_points(rng, n):
    G = (G1_X, G1_Y)
    ks = [rng.randrange(1, R_MOD) for _ in range(n)]
    return ks, [ec_mul(k, G) for k in ks]


def _randomize_z(rng, P):
    """same group element, random Jacobian representative"""
    if P is None:
        z = 0
        return np.array(to_limbs(rng.randrange(P_MOD), 12) + to_limbs(rng.randrange(P_MOD), 12) + to_limbs(0, 12), dtype=np.uint32)
    z = rng.randrange(1, P_MOD)
    x = P[0] * z * z % P_MOD
    y = P[1] * z * z * z % P_MOD
    return np.array(to_limbs(x * FP_R % P_MOD, 12) + to_limbs(y * FP_R % P_MOD, 12) + to_limbs(z * FP_R % P_MOD, 12), dtype=np.uint32)


def test_g1_ops_against_textbook_affine():
    orc = load_oracle()
    rng = random.Random(3)
    _, pts = _rand_points(rng, 12)
    cases = []
    for i in range(0, 12, 2):
        cases.append((pts[i], pts[i + 1]))
    cases += [(pts[0], pts[0]), (pts[1], ec_neg(pts[1])), (None, pts[2]), (pts[3], None), (None, None)]
    A = np.stack([_randomize_z(rng, p) for p, _ in cases])
    B = np.stack([_randomize_z(rng, q) for _, q in cases])
    out = np.zeros_like(A)
    orc_check(orc.orc_g1_op(0, A, B, out, len(cases)))
    assert [jac_to_affine(r) for r in out] == [ec_add(p, q) for p, q in cases]
    orc_check(orc.orc_g1_op(1, A, B, out, len(cases)))
    assert [jac_to_affine(r) for r in out] == [ec_add(p, p) for p, _ in cases]
    # mixed add takes b in affine form (z = ONE)
    Baff = np.stack([affine_to_jac(q) for _, q in cases if q is not None])
    Asel = np.stack([a for a, (_, q) in zip(A, cases) if q is not None])
    out2 = np.zeros_like(Asel)
    orc_check(orc.orc_g1_op(2, Asel, Baff, out2, len(Asel)))
    assert [jac_to_affine(r) for r in out2] == [ec_add(p, q) for p, q in cases if q is not None]
    # normalisation: canonical z = ONE, infinity = all zero
    orc_check(orc.orc_g1_op(3, A, B, out, len(cases)))
    for row, (p, _) in zip(out, cases):
        if p is None:
            assert not row.any()
        else:
            assert from_limbs(row[24:]) == FP_R and jac_to_affine(row) == p
    orc_check(orc.orc_g1_op(4, A, B, out, len(cases)))
    assert [jac_to_affine(r) for r in out] == [ec_neg(p) for p, _ in cases]


def test_g1_scalar_mul_against_textbook():
    orc = load_oracle()
    rng = random.Random(4)
    G = (G1_X, G1_Y)
    ks = [1, 2, 3, 2 ** 31 - 1, R_MOD - 1, 0] + [rng.randrange(R_MOD) for _ in range(6)]
    g = affine_to_jac(G).reshape(1, 36)
    out = np.zeros((len(ks), 36), dtype=np.uint32)
    orc_check(orc.orc_g1_mul(g, 1, fr_array(ks), out, len(ks), 0))
    assert [jac_to_affine(r) for r in out] == [ec_mul(k, G) for k in ks]
    # int32 walk: scalars are embedded ints, negatives as r-|x|
    xs = [0, 1, -1, 2 ** 15, -(2 ** 15), 2 ** 31 - 1, -(2 ** 31) + 1, 12345, -54321]
    out = np.zeros((len(xs), 36), dtype=np.uint32)
    orc_check(orc.orc_g1_mul(g, 1, fr_array([x % R_MOD for x in xs]), out, len(xs), 1))
    assert [jac_to_affine(r) for r in out] == [ec_mul(x, G) for x in xs]


def test_int_embedding_roundtrip():
    orc = load_oracle()
    xs = np.array([0, 1, -1, 2 ** 15, -(2 ** 15), 2 ** 31 - 1, -(2 ** 31) + 1], dtype=np.int32)
    fr = np.zeros((len(xs), 8), dtype=np.uint32)
    orc.orc_fr_from_i32(xs, fr, len(xs))
    assert fr_ints(fr) == [int(x) % R_MOD for x in xs]
    back = np.zeros_like(xs)
    orc.orc_fr_to_i32(fr, back, len(xs))
    assert (back == xs).all()
    ls = np.array([0, 1, -1, 2 ** 40, -(2 ** 40), 2 ** 63 - 1, -(2 ** 63) + 1], dtype=np.int64)
    fr = np.zeros((len(ls), 8), dtype=np.uint32)
    orc.orc_fr_from_i64(ls, fr, len(ls))
    assert fr_ints(fr) == [int(x) % R_MOD for x in ls]
    back = np.zeros_like(ls)
    orc.orc_fr_to_i64(fr, back, len(ls))
    assert (back == ls).all()
    fl = np.array([0.0, 0.49999, 0.5, -0.5, 1.5, -1.5, 0.02, -0.02], dtype=np.float64)
    orc.orc_fr_from_f64(fl, 1 << 16, fr := np.zeros((len(fl), 8), dtype=np.uint32), len(fl))
    exp = [int(np.floor(abs(x) * 65536 + 0.5)) * (1 if x >= 0 else -1) for x in fl]
    assert fr_ints(fr) == [e % R_MOD for e in exp]


def test_seeded_challenge_stream_is_mt19937():
    # std::mt19937 known answer: the 10000th output of the default seed 5489 is 4123659995
    rs = np.random.RandomState(5489)
    raw = rs._bit_generator.random_raw(10000)
    assert int(raw[-1]) == 4123659995
    orc = load_oracle()
    orc.orc_seed(5489)
    got = np.zeros((1250, 8), dtype=np.uint32)
    orc.orc_random_vec(got, 1250)
    exp = raw.astype(np.uint64).reshape(1250, 8)
    exp[:, 7] %= 1944954707
    assert (got == exp.astype(np.uint32)).all()
    assert (got == mt_random_vec(np.random.RandomState(5489), 1250)).all()
    assert all(v < R_MOD for v in fr_ints(got))


@pytest.mark.skipif(load_ref() is None, reason="oracle/_ref/libzkref.so not built (needs /root/reference)")
def test_oracle_bit_equal_to_compiled_reference():
    orc, ref = load_oracle(), load_ref()
    rng = random.Random(5)
    a = rand_fr(rng, 2000)
    b = list(reversed(rand_fr(rng, 2000)))
    A, B = fr_array(a), fr_array(b)
    o1, o2 = np.zeros_like(A), np.zeros_like(A)
    for op in range(6):
        orc_check(orc.orc_fr_op(op, A, B, o1, len(a)))
        ref.ref_fr_op(op, A, B, o2, len(a))
        assert (o1 == o2).all(), f"fr op {op}"
    orc_check(orc.orc_fr_op(6, A[:64], B, o1, 64))
    ref.ref_fr_op(6, A[:64], B, o2, 64)
    assert (o1[:64] == o2[:64]).all()
    fa = [rng.randrange(P_MOD) for _ in range(1000)] + [0, 1, P_MOD - 1]
    FA, FB = fp_array(fa), fp_array(list(reversed(fa)))
    p1, p2 = np.zeros_like(FA), np.zeros_like(FA)
    for op in range(6):
        orc_check(orc.orc_fp_op(op, FA, FB, p1, len(fa)))
        ref.ref_fp_op(op, FA, FB, p2, len(fa))
        assert (p1 == p2).all(), f"fp op {op}"
    # G1 formulas: identical Jacobian triples, including the special cases
    _, pts = _rand_points(rng, 8)
    cases = [(pts[i], pts[i + 1]) for i in range(0, 8, 2)] + [(pts[0], pts[0]), (pts[1], ec_neg(pts[1])), (None, pts[2]), (pts[3], None)]
    GA = np.stack([_randomize_z(rng, p) if p else affine_to_jac(None) for p, _ in cases])
    GB = np.stack([_randomize_z(rng, q) if q else affine_to_jac(None) for _, q in cases])
    g1, g2 = np.zeros_like(GA), np.zeros_like(GA)
    for op in range(2):
        orc_check(orc.orc_g1_op(op, GA, GB, g1, len(cases)))
        ref.ref_g1_op(op, GA, GB, g2, len(cases))
        assert (g1 == g2).all(), f"g1 op {op}"
    GBaff = np.stack([affine_to_jac(q if q else pts[5]) for _, q in cases])
    orc_check(orc.orc_g1_op(2, GA, GBaff, g1, len(cases)))
    ref.ref_g1_op(2, GA, GBaff, g2, len(cases))
    assert (g1 == g2).all()
    fr4, fp4, psub = np.zeros((4, 8), np.uint32), np.zeros((4, 12), np.uint32), np.zeros(8, np.uint32)
    ref.ref_constants(fr4, fp4, psub)
    assert list(fr4[0]) == REF_FR_ONE and list(fr4[1]) == REF_FR_P and list(fr4[2]) == REF_FR_R2
    assert list(fp4[0]) == REF_FP_ONE and list(fp4[1]) == REF_FP_P and list(fp4[2]) == REF_FP_R2
    assert list(psub) == REF_FR_P_SUB_2
