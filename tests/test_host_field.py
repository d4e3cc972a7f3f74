"""The product's own limb arithmetic (zkllm-ccs2024_amd/csrc/field.hpp -- one source for the GPU kernels
and the prover's host-side scalar work), run on the CPU through the class-layer library and compared
with python big-int closed forms and with the oracle.  No GPU needed."""
import random

import numpy as np

from gpuhelp import _np_ptr, pkg
from zkhelp import FP_R, FR_R, P_MOD, R_MOD, fp_array, fp_ints, fr_array, fr_ints, load_oracle, orc_check

import ctypes


def _lib():
    return pkg.load_prover()


def test_host_fr_ops_match_bigint_and_oracle():
    lib, orc = _lib(), load_oracle()
    rng = random.Random(11)
    edge = [0, 1, 2, R_MOD - 1, R_MOD - 2, FR_R, (1 << 32) - 1, 1 << 254, (1944954706 << 224) | ((1 << 224) - 1)]
    a = edge + [rng.randrange(R_MOD) for _ in range(500)]
    b = list(reversed(a))
    A, B = fr_array(a), fr_array(b)
    got, exp = np.zeros_like(A), np.zeros_like(A)
    rinv = pow(FR_R, -1, R_MOD)
    closed = {0: lambda x, y: (x + y) % R_MOD, 1: lambda x, y: (x - y) % R_MOD, 2: lambda x, y: x * y * rinv % R_MOD,
              3: lambda x, y: 2 * x % R_MOD, 4: lambda x, y: x * FR_R % R_MOD, 5: lambda x, y: x * rinv % R_MOD,
              7: lambda x, y: x * y % R_MOD, 8: lambda x, y: pow(x, -1, R_MOD) if x else 0, 9: lambda x, y: (-x) % R_MOD}
    for op, f in closed.items():
        assert lib.zkp_host_fr_op(ctypes.c_int(op), _np_ptr(A), _np_ptr(B), _np_ptr(got), ctypes.c_long(len(a))) == 0
        assert fr_ints(got) == [f(x, y) for x, y in zip(a, b)], f"host fr op {op}"
        orc_check(orc.orc_fr_op(op, A, B, exp, len(a)))
        assert (got == exp).all(), f"host fr op {op} vs oracle"
    # Montgomery inverse (binary algorithm in the product, exponentiation in the oracle): x = aR -> a^-1 R = x^-1 R^2
    inv_in = a + [1 << k for k in range(0, 255, 7)] + [R_MOD - (1 << k) for k in range(0, 254, 9)] + [(1 << 254) + 1, 3, R_MOD // 2, R_MOD // 2 + 1]
    IA = fr_array(inv_in)
    got, exp = np.zeros_like(IA), np.zeros_like(IA)
    assert lib.zkp_host_fr_op(ctypes.c_int(6), _np_ptr(IA), _np_ptr(IA), _np_ptr(got), ctypes.c_long(len(inv_in))) == 0
    assert fr_ints(got) == [pow(x, -1, R_MOD) * FR_R * FR_R % R_MOD if x else 0 for x in inv_in]
    orc_check(orc.orc_fr_op(6, IA, IA, exp, 64))
    assert (got[:64] == exp[:64]).all()


def test_29_bit_limb_products_match_bigint():
    """fr29_mul (a b 2^-261 mod r) and fr29_mul_small (a k 2^-58 mod r for a small integer k: the first lookup round of a plain
    table, whose queries differ by small integers) of the sumcheck kernels, run on the CPU, against big integers: edge operands,
    random ones, and k at 0, 1, the 32-bit extremes and the routine's own limit; fr29_from_small (a signed integer as a residue)."""
    lib = _lib()
    rng = random.Random(29)
    edge = [0, 1, 2, R_MOD - 1, R_MOD - 2, (1 << 29) - 1, 1 << 29, (1 << 232) - 1, 1 << 232, 1 << 254]
    a = edge + [rng.randrange(R_MOD) for _ in range(600)]
    b = list(reversed(a))
    ks = [0, 1, 2, (1 << 29) - 1, 1 << 29, (1 << 32) - 1, 1 << 32, (1 << 33) - 1, (1 << 58) - 1, 12345678901]
    k = [ks[i % len(ks)] if i < 3 * len(ks) else rng.randrange(1 << rng.choice([8, 16, 31, 32, 33, 58])) for i in range(len(a))]
    A, B, K = fr_array(a), fr_array(b), np.array(k, dtype=np.uint64)
    got = np.zeros_like(A)
    lib.zkp_host_fr29_op.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long]
    assert lib.zkp_host_fr29_op(0, _np_ptr(A), _np_ptr(B), K.ctypes.data, _np_ptr(got), len(a)) == 0
    i261 = pow(1 << 261, -1, R_MOD)
    assert fr_ints(got) == [x * y * i261 % R_MOD for x, y in zip(a, b)]
    assert lib.zkp_host_fr29_op(1, _np_ptr(A), _np_ptr(B), K.ctypes.data, _np_ptr(got), len(a)) == 0
    i58 = pow(1 << 58, -1, R_MOD)
    assert fr_ints(got) == [x * kk * i58 % R_MOD for x, kk in zip(a, k)]
    signed = [0, 1, -1, 2 ** 31 - 1, -2 ** 31, 2 ** 29, -2 ** 29, 2 ** 29 - 1, -(2 ** 29 - 1), 2 ** 58 - 1, -(2 ** 58 - 1)] + [rng.randrange(-2 ** 57, 2 ** 57) for _ in range(200)]
    Ks = np.array(signed, dtype=np.int64)
    got = np.zeros((len(signed), 8), np.uint32)
    assert lib.zkp_host_fr29_op(2, _np_ptr(A), _np_ptr(B), Ks.ctypes.data, _np_ptr(got), len(signed)) == 0
    assert fr_ints(got) == [v % R_MOD for v in signed]


def test_unreduced_sums_of_products_reduce_to_the_sum_of_montgomery_products():
    """wide_mac / wide_redc (the sumcheck rounds' accumulator: products added as 512-bit integers, one reduction at the end)
    against big integers: sum a_i b_i / R mod r for operands below r, for arbitrary 256-bit operands (the accumulator does
    not ask for reduced inputs), for the extremes, and for sums long enough to reach the seventeenth limb."""
    lib = _lib()
    rng = random.Random(21)
    rinv = pow(FR_R, -1, R_MOD)
    top = (1 << 256) - 1
    cases = [([0], [0]), ([1], [1]), ([R_MOD - 1], [R_MOD - 1]), ([top], [top]), ([top] * 70000, [top] * 70000),
             ([rng.randrange(R_MOD) for _ in range(300)], [rng.randrange(R_MOD) for _ in range(300)]),
             ([rng.randrange(1 << 256) for _ in range(1000)], [rng.randrange(1 << 256) for _ in range(1000)])]
    for a, b in cases:
        A = np.array([[(x >> (32 * k)) & 0xFFFFFFFF for k in range(8)] for x in a], dtype=np.uint32)
        B = np.array([[(x >> (32 * k)) & 0xFFFFFFFF for k in range(8)] for x in b], dtype=np.uint32)
        got = np.zeros((1, 8), dtype=np.uint32)
        assert lib.zkp_host_fr_wide_dot(_np_ptr(A), _np_ptr(B), _np_ptr(got), ctypes.c_long(len(a))) == 0
        assert fr_ints(got)[0] == sum(x * y for x, y in zip(a, b)) * rinv % R_MOD


def test_host_fp_ops_match_bigint_and_oracle():
    lib, orc = _lib(), load_oracle()
    rng = random.Random(12)
    a = [0, 1, P_MOD - 1, FP_R, 1 << 380] + [rng.randrange(P_MOD) for _ in range(300)]
    b = list(reversed(a))
    A, B = fp_array(a), fp_array(b)
    got, exp = np.zeros_like(A), np.zeros_like(A)
    rinv = pow(FP_R, -1, P_MOD)
    closed = {0: lambda x, y: (x + y) % P_MOD, 1: lambda x, y: (x - y) % P_MOD, 2: lambda x, y: x * y * rinv % P_MOD,
              3: lambda x, y: 2 * x % P_MOD, 4: lambda x, y: x * FP_R % P_MOD, 5: lambda x, y: x * rinv % P_MOD}
    for op, f in closed.items():
        assert lib.zkp_host_fp_op(ctypes.c_int(op), _np_ptr(A), _np_ptr(B), _np_ptr(got), ctypes.c_long(len(a))) == 0
        assert fp_ints(got) == [f(x, y) for x, y in zip(a, b)], f"host fp op {op}"
        orc_check(orc.orc_fp_op(op, A, B, exp, len(a)))
        assert (got == exp).all()
    inv_in = a + [1 << k for k in range(0, 381, 11)] + [P_MOD - (1 << k) for k in range(0, 380, 13)] + [3, P_MOD // 2, P_MOD // 2 + 1]
    IA = fp_array(inv_in)
    got, exp = np.zeros_like(IA), np.zeros_like(IA)
    assert lib.zkp_host_fp_op(ctypes.c_int(6), _np_ptr(IA), _np_ptr(IA), _np_ptr(got), ctypes.c_long(len(inv_in))) == 0
    assert fp_ints(got) == [pow(x, -1, P_MOD) * FP_R * FP_R % P_MOD if x else 0 for x in inv_in]
    orc_check(orc.orc_fp_op(6, IA, IA, exp, 32))
    assert (got[:32] == exp[:32]).all()


def test_host_polynomial_eval_matches_horner():
    lib = _lib()
    rng = random.Random(13)
    coefs = [rng.randrange(R_MOD) for _ in range(5)]
    x = rng.randrange(R_MOD)
    out = np.zeros(8, np.uint32)
    C, X = fr_array(coefs), fr_array([x])
    assert lib.zkp_poly_eval(_np_ptr(C), ctypes.c_int(5), _np_ptr(X), _np_ptr(out)) == 0
    assert fr_ints(out) == [sum(c * pow(x, i, R_MOD) for i, c in enumerate(coefs)) % R_MOD]
