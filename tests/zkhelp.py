"""Shared helpers for the test-suite: big-int field/curve arithmetic (independent of every C
implementation), limb packing, and ctypes loaders for the oracle, the compiled reference and
the product libraries."""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# BLS12-381 (standard constants; cross-checked against the reference's limb tables in
# tests/test_oracle_field.py)
R_MOD = 0x73EDA753299D7D483339D80809A1D80553BDA402FFFE5BFEFFFFFFFF00000001
P_MOD = 0x1A0111EA397FE69A4B1BA7B6434BACD764774B84F38512BF6730D2A0F6B0F6241EABFFFEB153FFFFB9FEFFFFFFFFAAAB
FR_R = (1 << 256) % R_MOD
FP_R = (1 << 384) % P_MOD
G1_X = 0x17F1D3A73197D7942695638C4FA9AC0FC3688C4F9774B905A14E3A3F171BAC586C55E83FF97A1AEFFB3AF00ADB22C6BB
G1_Y = 0x08B3F481E3AAA0F1A09E30ED741D8AE4FCF5E095D5D00AF600DB18CB2C04B3EDD03CC744A2888AE40CAA232946C5E7E1


def to_limbs(x, n):
    return [(x >> (32 * i)) & 0xFFFFFFFF for i in range(n)]


def from_limbs(a):
    return sum(int(v) << (32 * i) for i, v in enumerate(a))


def fr_array(vals):
    """list of python ints -> (n, 8) uint32"""
    return np.array([to_limbs(v % (1 << 256), 8) for v in vals], dtype=np.uint32).reshape(-1, 8)


def fr_ints(arr):
    arr = np.asarray(arr, dtype=np.uint32).reshape(-1, 8)
    return [from_limbs(row) for row in arr]


def fr_signed(fr):
    """(n, 8) uint32 field elements of magnitude below 2^63 -> list of python ints in (-r/2, r/2)"""
    fr = np.asarray(fr, dtype=np.uint32).reshape(-1, 8)
    lo = fr[:, 0].astype(np.uint64) | (fr[:, 1].astype(np.uint64) << np.uint64(32))
    neg = fr[:, 7] != 0
    r_lo = np.uint64(R_MOD & ((1 << 64) - 1))
    mag = np.where(neg, r_lo - lo, lo)                       # wraps mod 2^64, which is the low half of r - x
    small = np.where(neg, (fr[:, 2:] == fr_array([R_MOD - 1])[0, 2:]).all(axis=1), (fr[:, 2:] == 0).all(axis=1))
    if not small.all():
        return [x - R_MOD if x > R_MOD // 2 else x for x in fr_ints(fr)]
    return [int(v) for v in np.where(neg, -mag.astype(np.int64), mag.astype(np.int64))]


def fp_array(vals):
    return np.array([to_limbs(v, 12) for v in vals], dtype=np.uint32).reshape(-1, 12)


def fp_ints(arr):
    arr = np.asarray(arr, dtype=np.uint32).reshape(-1, 12)
    return [from_limbs(row) for row in arr]


def int_to_fr(x):
    return x % R_MOD


# ---- textbook affine arithmetic on y^2 = x^3 + 4 over F_p (None = infinity) -------------------
def ec_add(P, Q):
    if P is None:
        return Q
    if Q is None:
        return P
    x1, y1 = P
    x2, y2 = Q
    if x1 == x2:
        if (y1 + y2) % P_MOD == 0:
            return None
        lam = 3 * x1 * x1 * pow(2 * y1, -1, P_MOD) % P_MOD
    else:
        lam = (y2 - y1) * pow(x2 - x1, -1, P_MOD) % P_MOD
    x3 = (lam * lam - x1 - x2) % P_MOD
    return (x3, (lam * (x1 - x3) - y1) % P_MOD)


def ec_neg(P):
    return None if P is None else (P[0], (-P[1]) % P_MOD)


def ec_mul(k, P):
    if k < 0:
        return ec_mul(-k, ec_neg(P))
    R = None
    while k:
        if k & 1:
            R = ec_add(R, P)
        P = ec_add(P, P)
        k >>= 1
    return R


def jac_to_affine(row):
    """36 u32 limbs (x,y,z Montgomery) -> affine (x,y) standard ints or None"""
    row = np.asarray(row, dtype=np.uint32).reshape(36)
    rinv = pow(FP_R, -1, P_MOD)
    x, y, z = (from_limbs(row[12 * i:12 * i + 12]) * rinv % P_MOD for i in range(3))
    if z == 0:
        return None
    zi = pow(z, -1, P_MOD)
    return (x * zi * zi % P_MOD, y * zi * zi * zi % P_MOD)


def affine_to_jac(P):
    """affine std ints -> 36 u32 limbs, z = ONE (Montgomery)"""
    if P is None:
        return np.array(to_limbs(0, 12) + to_limbs(FP_R, 12) + to_limbs(0, 12), dtype=np.uint32)
    return np.array(to_limbs(P[0] * FP_R % P_MOD, 12) + to_limbs(P[1] * FP_R % P_MOD, 12) + to_limbs(FP_R, 12), dtype=np.uint32)


# ---- multilinear extension by brute force -------------------------------------------------------
def me_bruteforce(t, u):
    """sum_i t_i prod_j (u_j if bit_j(i) else 1-u_j), zero-extended to 2^len(u)"""
    acc = 0
    for i, ti in enumerate(t):
        w = 1
        for j, uj in enumerate(u):
            w = w * (uj if (i >> j) & 1 else (1 - uj)) % R_MOD
        acc = (acc + ti * w) % R_MOD
    return acc


def mt_random_vec(rs, n):
    """The reference's random_vec draw rule on a numpy RandomState (init_genrand seeding == std::mt19937)."""
    raw = rs._bit_generator.random_raw(8 * n).astype(np.uint64).reshape(n, 8)
    raw[:, 7] %= 1944954707
    return raw.astype(np.uint32)


# ---- ctypes loaders ----------------------------------------------------------------------------------
def _ptr(a):
    if a is None:
        return None
    if isinstance(a, np.ndarray):
        assert a.flags["C_CONTIGUOUS"]
        return ctypes.c_void_p(a.ctypes.data)
    return a


class Lib:
    """Thin ctypes wrapper: numpy arrays are passed as raw pointers, ints as c_long/c_int per call site."""

    def __init__(self, path):
        self.path = path
        self.dll = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)

    def __getattr__(self, name):
        fn = getattr(self.dll, name)

        def call(*args):
            conv = []
            for a in args:
                if isinstance(a, np.ndarray) or a is None:
                    conv.append(_ptr(a))
                elif isinstance(a, (bool, int, np.integer)):
                    conv.append(ctypes.c_int64(int(a)))
                elif isinstance(a, float):
                    conv.append(ctypes.c_double(a))
                else:
                    conv.append(a)
            return fn(*conv)

        call.raw = fn
        return call


_cache = {}


def load_oracle():
    if "orc" not in _cache:
        path = os.path.join(ROOT, "oracle", "liboracle.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/liboracle.so missing: run `make -C oracle` (or __graft_entry__.build())")
        lib = Lib(path)
        lib.dll.orc_last_error.restype = ctypes.c_char_p
        lib.dll.orc_transcript_size.restype = ctypes.c_long
        lib.dll.orc_g1_count_equal.restype = ctypes.c_long
        _cache["orc"] = lib
    return _cache["orc"]


def load_ref():
    """The reference's own bls12-381.cu compiled as host C++ (only present where it could be built)."""
    path = os.path.join(ROOT, "oracle", "_ref", "libzkref.so")
    if not os.path.exists(path):
        return None
    if "ref" not in _cache:
        _cache["ref"] = Lib(path)
    return _cache["ref"]


def orc_check(rc):
    if rc != 0:
        raise RuntimeError(load_oracle().dll.orc_last_error().decode())


def orc_transcript(orc):
    n = orc.dll.orc_transcript_size()
    out = np.zeros((n, 8), dtype=np.uint32)
    if n:
        orc.orc_transcript_get(out)
    return out
