"""GPU parity: FrTensor kernels, folds, matmul, inner-product sumcheck and zkFC::prove, through the
C ABI / class layer, bit-exact against the CPU oracle on the same seeded inputs."""
import ctypes
import random

import numpy as np
import pytest

from zkhelp import FR_R, R_MOD, fr_array, fr_ints, load_oracle, me_bruteforce, mt_random_vec, orc_check, orc_transcript

pytestmark = pytest.mark.gpu

EDGE = [0, 1, 2, R_MOD - 1, R_MOD - 2, FR_R, FR_R * FR_R % R_MOD, (1 << 32) - 1, ((1 << 32) - 1) << 32,
        (1944954706 << 224) | ((1 << 224) - 1), 1 << 254, R_MOD >> 1]


@pytest.fixture(scope="module")
def hip():
    from gpuhelp import Hip
    return Hip()


@pytest.fixture(scope="module")
def pv():
    from gpuhelp import Prover
    return Prover()


@pytest.fixture(scope="module")
def orc():
    return load_oracle()


def seeded(n, seed):
    """n field elements from the seeded challenge generator (plus the edge set in front)"""
    raw = mt_random_vec(np.random.RandomState(seed), n)
    return np.concatenate([fr_array(EDGE), raw])


def test_elementwise_ops_bit_exact(hip, orc):
    n = 1 << 16
    A, B = seeded(n, 1), seeded(n, 2)[::-1].copy()
    N = A.shape[0]
    exp = np.zeros_like(A)
    for name, op in (("zk_fr_add", 0), ("zk_fr_sub", 1), ("zk_fr_montmul", 2), ("zk_fr_mul", 7)):
        print("case", name, flush=True)
        got = hip.fr_binary(name, A, B)
        orc_check(orc.orc_fr_op(op, A, B, exp, N))
        assert (got == exp).all(), name
    for name, op in (("zk_fr_neg", 9), ("zk_fr_mont", 4), ("zk_fr_unmont", 5)):
        print("case", name, flush=True)
        got = hip.fr_unary(name, A)
        orc_check(orc.orc_fr_op(op, A, A, exp, N))
        assert (got == exp).all(), name
    s = fr_array([R_MOD - 12345])[0]
    S = np.tile(s, (N, 1))
    for name, op in (("zk_fr_add_s", 0), ("zk_fr_sub_s", 1), ("zk_fr_mul_s", 7)):
        print("case", name, flush=True)
        got = hip.fr_scalar(name, A, s)
        orc_check(orc.orc_fr_op(op, A, S, exp, N))
        assert (got == exp).all(), name


def test_empty_and_single_element(hip, pv):
    empty = np.zeros((0, 8), np.uint32)
    assert hip.fr_binary("zk_fr_add", empty, empty).shape == (0, 8)
    one = fr_array([5])
    assert fr_ints(hip.fr_binary("zk_fr_mul", one, fr_array([7]))) == [35]
    h = pv.from_fr(one)
    assert fr_ints(pv.sum(h)) == [5]
    assert fr_ints(pv.me(h, np.zeros((0, 8), np.uint32))) == [5]


def test_conversions(hip, pv, orc):
    xs = np.array([0, 1, -1, 2 ** 15, -(2 ** 15), 2 ** 31 - 1, -(2 ** 31) + 1] + list(np.random.default_rng(3).integers(-2 ** 31 + 1, 2 ** 31 - 1, 1000)), dtype=np.int32)
    h = pv.from_i32(xs)
    assert fr_ints(h.host()) == [int(x) % R_MOD for x in xs]
    ls = np.array([0, 1, -1, 2 ** 40, -(2 ** 40), 2 ** 62, -(2 ** 62)] + list(np.random.default_rng(4).integers(-2 ** 62, 2 ** 62, 1000)), dtype=np.int64)
    hl = pv.from_i64(ls)
    assert fr_ints(hl.host()) == [int(x) % R_MOD for x in ls]
    # back to integers through the C ABI
    from gpuhelp import c_void_p, c_size_t
    d = hip.malloc(4 * len(xs))
    hip.call("zk_fr_to_i32", c_void_p(d), c_void_p(h.devptr), c_size_t(len(xs)), None)
    assert (hip.download(d, (len(xs),), np.int32) == xs).all()
    hip.free(d)
    d = hip.malloc(8 * len(ls))
    hip.call("zk_fr_to_i64", c_void_p(d), c_void_p(hl.devptr), c_size_t(len(ls)), None)
    assert (hip.download(d, (len(ls),), np.int64) == ls).all()
    hip.free(d)
    fl = np.random.default_rng(5).normal(0, 0.02, 4096)
    fl[:6] = [0.0, 0.5 / 65536, -0.5 / 65536, 1.5 / 65536, -1.5 / 65536, 0.49999 / 65536]
    exp = np.zeros((len(fl), 8), np.uint32)
    orc.orc_fr_from_f64(fl, 1 << 16, exp, len(fl))
    assert (pv.from_f64(fl, 1 << 16).host() == exp).all()
    f32 = fl.astype(np.float32)
    orc.orc_fr_from_f32(f32, 1 << 16, exp, len(fl))
    assert (pv.from_f32(f32, 1 << 16).host() == exp).all()


@pytest.mark.parametrize("n", [1, 2, 3, 255, 256, 257, 1000, 1024, 1025, 4096, 50000, (1 << 20) + 3])
def test_sum_and_me(pv, orc, n):
    print("case n", n, flush=True)
    A = mt_random_vec(np.random.RandomState(100 + n % 97), n)
    h = pv.from_fr(A)
    exp = np.zeros(8, np.uint32)
    orc_check(orc.orc_fr_sum(A, n, exp))
    assert (pv.sum(h) == exp).all()
    k = max(0, (n - 1).bit_length())
    u = mt_random_vec(np.random.RandomState(7), k)
    orc_check(orc.orc_fr_me(A, n, u, k, exp))
    assert (pv.me(h, u) == exp).all()


def test_me_boolean_points_and_bruteforce(pv):
    rng = random.Random(5)
    t = [rng.randrange(R_MOD) for _ in range(13)]
    h = pv.from_fr(fr_array(t))
    u = [rng.randrange(R_MOD) for _ in range(4)]
    assert fr_ints(pv.me(h, fr_array(u))) == [me_bruteforce(t, u)]
    for i in (0, 5, 12, 15):
        pt = [(i >> j) & 1 for j in range(4)]
        assert fr_ints(pv.me(h, fr_array(pt))) == [t[i] if i < 13 else 0]


# (64, 4, 33), (16, 8, 40): thousands of four-term groups that share one Montgomery reduction, whose value before the final
# subtractions reaches 2.8 r (about one group in fifteen passes 2 r)
@pytest.mark.parametrize("other,cur,win", [(1, 8, 1), (3, 4, 5), (2, 5, 3), (4, 11, 1), (1, 6, 7), (7, 43, 1), (1, 16, 64), (5, 1000, 3), (1, 2048, 33), (64, 4096, 1),
                                           (64, 4, 33), (16, 8, 40)])
def test_partial_me(pv, orc, other, cur, win):
    print("case", other, cur, win, flush=True)
    n = other * cur * win
    A = mt_random_vec(np.random.RandomState(cur), n)
    k = (cur - 1).bit_length()
    u = mt_random_vec(np.random.RandomState(8), k)
    exp = np.zeros((n, 8), np.uint32)
    out_n = np.zeros(1, np.int64)
    orc_check(orc.orc_fr_partial_me(A, n, u, k, cur, win, exp, out_n))
    got = pv.partial_me(pv.from_fr(A), u, cur, win).host()
    assert got.shape[0] == out_n[0] == other * win
    assert (got == exp[:out_n[0]]).all()
    # fewer levels than bits: the axis is only partly folded
    if k >= 2:
        kk = k - 1
        # legal only when 2^(kk-1) < cur <= 2^kk fails -> use the raw step count via a sub-axis
        sub = 1 << kk
        if cur >= sub:
            A2 = A[: other * sub * win].copy()
            orc_check(orc.orc_fr_partial_me(A2, other * sub * win, u[:kk].copy(), kk, sub, win, exp, out_n))
            got = pv.partial_me(pv.from_fr(A2), u[:kk].copy(), sub, win).host()
            assert (got == exp[:out_n[0]]).all()


@pytest.mark.parametrize("n,win,k", [(32, 4, 3), (15, 3, 3), (18, 4, 3), (4096 * 16, 4096, 4), (11008 * 8, 8, 14)])
def test_window_fold(pv, orc, n, win, k):
    A = mt_random_vec(np.random.RandomState(n % 1000), n)
    u = mt_random_vec(np.random.RandomState(9), k)
    exp = np.zeros((n + 2 * win, 8), np.uint32)
    out_n = np.zeros(1, np.int64)
    orc_check(orc.orc_fr_partial_me_window(A, n, u, k, win, exp, out_n))
    got = pv.partial_me_window(pv.from_fr(A), u, win).host()
    assert got.shape[0] == out_n[0]
    assert (got == exp[:out_n[0]]).all()


def test_multi_dim_me(pv, orc):
    for shape in ((4, 8), (16, 64), (3, 5, 7), (2048, 33)):
        n = int(np.prod(shape))
        A = mt_random_vec(np.random.RandomState(n % 991), n)
        us = [mt_random_vec(np.random.RandomState(10 + i), max(0, (d - 1).bit_length())) for i, d in enumerate(shape)]
        cat = np.ascontiguousarray(np.concatenate(us))
        lens = np.array([u.shape[0] for u in us], np.uint32)
        exp = np.zeros(8, np.uint32)
        orc_check(orc.orc_fr_multi_dim_me(A, n, cat, lens, np.array(shape, np.uint32), len(shape), exp))
        assert (pv.multi_dim_me(pv.from_fr(A), us, shape) == exp).all(), shape


def test_pad_and_transpose(pv, orc):
    for shape in ((3, 5), (11, 43), (1, 7), (16, 16), (5, 3, 6)):
        n = int(np.prod(shape))
        A = mt_random_vec(np.random.RandomState(n), n)
        padv = fr_array([R_MOD - 3])[0]
        exp = np.zeros((n * 8 + 64, 8), np.uint32)
        out_n = np.zeros(1, np.int64)
        orc_check(orc.orc_fr_pad(A, n, np.array(shape, np.uint32), len(shape), padv, exp, out_n))
        got = pv.pad(pv.from_fr(A), shape, padv).host()
        assert got.shape[0] == out_n[0] and (got == exp[:out_n[0]]).all(), shape
    for M, N in ((3, 5), (32, 32), (33, 65), (1, 100), (100, 1), (257, 130)):
        A = mt_random_vec(np.random.RandomState(M * N), M * N)
        exp = np.zeros_like(A)
        orc_check(orc.orc_fr_transpose(A, M, N, exp))
        assert (pv.transpose(pv.from_fr(A), M, N).host() == exp).all(), (M, N)


@pytest.mark.parametrize("n,w", [(8, 2), (8, 1), (13, 4), (10, 3), (7, 6), (4096 * 9 + 5, 4096), (100003, 7)])
def test_split_into_even_and_odd_windows(pv, orc, n, w):
    A = mt_random_vec(np.random.RandomState(n % 997), n)
    out_n = ((-(-n // w) + 1) // 2) * w
    e_exp, o_exp = np.zeros((out_n, 8), np.uint32), np.zeros((out_n, 8), np.uint32)
    orc_check(orc.orc_fr_split(A, n, w, e_exp, o_exp))
    even, odd = pv.split(pv.from_fr(A), w)
    assert (even.host() == e_exp).all() and (odd.host() == o_exp).all()


def test_split_rejects_bad_windows(pv):
    t = pv.from_fr(mt_random_vec(np.random.RandomState(1), 4))
    for w in (0, 4, 9):
        with pytest.raises(RuntimeError, match="Invalid window size"):
            pv.split(t, w)


@pytest.mark.parametrize("M,N,P", [(1, 1, 1), (3, 4, 5), (16, 64, 64), (17, 9, 33), (40, 100, 24)])
def test_matmul_generic_matches_oracle(pv, orc, M, N, P):
    print("case", M, N, P, flush=True)
    A = mt_random_vec(np.random.RandomState(M), M * N)
    B = mt_random_vec(np.random.RandomState(P + 50), N * P)
    exp = np.zeros((M * P, 8), np.uint32)
    orc_check(orc.orc_fr_matmul(A, B, M, N, P, exp))
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(1))
    got = pv.matmul(pv.from_fr(A), pv.from_fr(B), M, N, P).host()
    assert pv.lib.zkp_last_matmul_path() == 1
    assert (got == exp).all()
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    got = pv.matmul(pv.from_fr(A), pv.from_fr(B), M, N, P).host()   # full-width residues: the bound check must refuse the integer path
    assert pv.lib.zkp_last_matmul_path() == 1 and (got == exp).all()


def test_matmul_small_integer_path_equals_generic(pv):
    rng = np.random.default_rng(31)
    M, N, P = 70, 130, 50
    A = np.round(rng.normal(0, 1, (M, N)) * 65536).astype(np.int32)
    B = np.round(rng.normal(0, 0.02, (N, P)) * 65536).astype(np.int32)
    exp = [int(v) % R_MOD for v in (A.astype(object) @ B.astype(object)).reshape(-1)]
    for mode, path in ((0, 2), (1, 1)):
        pv.lib.zkp_set_matmul_mode(ctypes.c_int(mode))
        got = pv.matmul(pv.from_i32(A), pv.from_i32(B), M, N, P).host()
        assert pv.lib.zkp_last_matmul_path() == path
        assert fr_ints(got) == exp
    # int64-range operands (softmax outputs are ~2^40): still exact, or falls back when the bound fails
    A64 = rng.integers(-2 ** 40, 2 ** 40, (8, 16)).astype(np.int64)
    B64 = rng.integers(-2 ** 15, 2 ** 15, (16, 8)).astype(np.int64)
    exp = [int(v) % R_MOD for v in (A64.astype(object) @ B64.astype(object)).reshape(-1)]
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    got = pv.matmul(pv.from_i64(A64), pv.from_i64(B64), 8, 16, 8).host()
    assert pv.lib.zkp_last_matmul_path() == 2 and fr_ints(got) == exp
    # several tiles of the wide-by-narrow kernel (left operand split at 31 bits), ragged edges, negative values on both sides
    Aw = rng.integers(-2 ** 40, 2 ** 40, (130, 300)).astype(np.int64)
    Bn = rng.integers(-2 ** 12, 2 ** 12, (300, 70)).astype(np.int64)
    Aw[0, :4] = [2 ** 31, -(2 ** 31), 2 ** 31 - 1, -(2 ** 31) - 1]
    expw = [int(v) % R_MOD for v in (Aw.astype(object) @ Bn.astype(object)).reshape(-1)]
    got = pv.matmul(pv.from_i64(Aw), pv.from_i64(Bn), 130, 300, 70).host()
    assert pv.lib.zkp_last_matmul_path() == 2 and fr_ints(got) == expw
    # narrow left, wide right: the 64-bit kernel
    An = rng.integers(-2 ** 20, 2 ** 20, (8, 16)).astype(np.int64)
    Bw = rng.integers(-2 ** 33, 2 ** 33, (16, 8)).astype(np.int64)
    expn = [int(v) % R_MOD for v in (An.astype(object) @ Bw.astype(object)).reshape(-1)]
    got = pv.matmul(pv.from_i64(An), pv.from_i64(Bw), 8, 16, 8).host()
    assert pv.lib.zkp_last_matmul_path() == 2 and fr_ints(got) == expn
    A64 = rng.integers(-2 ** 50, 2 ** 50, (8, 16)).astype(np.int64)
    exp = [int(v) % R_MOD for v in (A64.astype(object) @ B64.astype(object)).reshape(-1)]
    got = pv.matmul(pv.from_i64(A64), pv.from_i64(B64), 8, 16, 8).host()
    assert pv.lib.zkp_last_matmul_path() == 1 and fr_ints(got) == exp
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))


@pytest.mark.parametrize("n", [2, 3, 8, 11, 64, 1000, 4096, 8192, 8193, 40000, 1 << 17])
def test_zkip_matches_oracle(pv, orc, n):
    print("case n", n, flush=True)
    a = mt_random_vec(np.random.RandomState(n % 89), n)
    b = mt_random_vec(np.random.RandomState(n % 83 + 200), n)
    k = (n - 1).bit_length()
    u = mt_random_vec(np.random.RandomState(12), k)
    claim = np.zeros(8, np.uint32)
    ha, hb = pv.from_fr(a), pv.from_fr(b)
    # the claim is <a,b>
    orc_check(orc.orc_fr_op(7, a, b, prod := np.zeros_like(a), n))
    orc_check(orc.orc_fr_sum(prod, n, claim))
    exp_proof = np.zeros((k, 3, 8), np.uint32)
    exp_fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_zkip(claim, a, b, n, u, k, exp_proof, exp_fin))
    proof, fin = pv.zkip(claim, ha, hb, u)
    assert (proof == exp_proof).all() and (fin == exp_fin).all()
    # a wrong claim is rejected exactly like the reference does
    bad = claim.copy()
    bad[0] ^= 1
    with pytest.raises(RuntimeError, match="claim != p"):
        pv.zkip(bad, ha, hb, u)


@pytest.mark.parametrize("B,I,O,mode", [(16, 64, 64, 1), (16, 64, 64, 0), (5, 24, 10, 1), (64, 256, 128, 0)])
def test_zkfc_forward_and_proof_transcript(pv, orc, B, I, O, mode):
    rng = np.random.default_rng(B * I + O)
    X = np.round(rng.normal(0, 0.02, (B, I)) * 65536).astype(np.int32)
    W = np.round(rng.normal(0, 0.02, (I, O)) * 65536).astype(np.int32)
    got_Y, got_t = pv.zkfc_scenario(X, W, seed=4242, matmul_mode=mode)
    orc.orc_seed(4242)
    orc.orc_transcript_clear()
    exp_Y = np.zeros((B * O, 8), np.uint32)
    orc_check(orc.orc_zkfc(X, W, B, I, O, exp_Y, np.zeros(8, np.uint32)))
    exp_t = orc_transcript(orc)
    assert (got_Y == exp_Y).all()
    assert got_t.shape == exp_t.shape and (got_t == exp_t).all()
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))


def test_zkfc_proof_with_an_input_axis_that_needs_rounds_of_their_own(pv, orc):
    """An input axis of 11008 (the 7B down projection's; 14 index bits): the inner-product sumcheck runs one round as launches of
    its own before the single-workgroup kernel takes the other thirteen, all queued ahead by zkFC::prove_begin.  Transcript
    and output are the oracle's."""
    B, I, O = 4, 11008, 8
    rng = np.random.default_rng(77)
    X = np.round(rng.normal(0, 0.02, (B, I)) * 65536).astype(np.int32)
    W = np.round(rng.normal(0, 0.02, (I, O)) * 65536).astype(np.int32)
    got_Y, got_t = pv.zkfc_scenario(X, W, seed=777, matmul_mode=0)
    orc.orc_seed(777)
    orc.orc_transcript_clear()
    exp_Y = np.zeros((B * O, 8), np.uint32)
    orc_check(orc.orc_zkfc(X, W, B, I, O, exp_Y, np.zeros(8, np.uint32)))
    exp_t = orc_transcript(orc)
    assert (got_Y == exp_Y).all()
    assert got_t.shape == exp_t.shape and (got_t == exp_t).all()


def test_deferred_results_arrive_in_call_order_with_the_values_of_the_immediate_calls(hip):
    """zk_defer_begin / _end / _wait: evaluations and inner-product rounds queued without waiting deliver, in call order, what the
    same calls return when each waits for itself; the host outputs of the deferred calls are left alone."""
    rng = np.random.default_rng(31)
    n, k = 5000, 13
    a = hip.upload(fr_array([int(x) % R_MOD for x in rng.integers(-2 ** 40, 2 ** 40, n)]))
    b = hip.upload(mt_random_vec(np.random.RandomState(32), n))
    u = mt_random_vec(np.random.RandomState(33), k)
    n2 = 20000
    c = hip.upload(mt_random_vec(np.random.RandomState(34), n2))
    d = hip.upload(mt_random_vec(np.random.RandomState(35), n2))

    def calls(out):
        hip.call("zk_fr_me", out[0], ctypes.c_void_p(a), ctypes.c_size_t(n), u, ctypes.c_int(k), None)
        hip.call("zk_ip_round", out[1], ctypes.c_void_p(c), ctypes.c_void_p(d), ctypes.c_size_t(n2), ctypes.c_size_t(16384), None)
        hip.call("zk_ip_sumcheck_small", out[2], out[3], ctypes.c_void_p(a), ctypes.c_void_p(b), ctypes.c_uint32(n), u, ctypes.c_int(k), None)
        hip.call("zk_fr_me", out[4], ctypes.c_void_p(b), ctypes.c_size_t(n), u, ctypes.c_int(k), None)

    shapes = [(1, 8), (3, 8), (3 * k, 8), (2, 8), (1, 8)]
    want = [np.zeros(sh, np.uint32) for sh in shapes]
    calls(want)
    assert all(w.any() for w in want)
    batch = ctypes.c_void_p()
    hip.call("zk_defer_begin", ctypes.byref(batch))
    untouched = [np.full(sh, 0xA5A5A5A5, np.uint32) for sh in shapes]
    calls(untouched)
    hip.call("zk_defer_end", batch, None)
    got = np.zeros((64, 8), np.uint32)
    cnt = ctypes.c_size_t()
    hip.call("zk_defer_wait", batch, got, ctypes.c_size_t(64), ctypes.byref(cnt))
    hip.call("zk_defer_free", batch)
    # call order: evaluation, round (three sums), small sumcheck (3k polynomials' values, then the two folded values), evaluation
    flat = np.concatenate([want[0], want[1], want[2], want[3], want[4]])
    assert cnt.value == flat.shape[0] and (got[:cnt.value] == flat).all()
    assert (untouched[0] == 0xA5A5A5A5).all() and (untouched[1] == 0xA5A5A5A5).all() and (untouched[4] == 0xA5A5A5A5).all()
    # a second batch on the same thread after the first was released, and immediate calls work again in between
    again = [np.zeros(sh, np.uint32) for sh in shapes]
    calls(again)
    assert all((x == y).all() for x, y in zip(again, want))
    for p in (a, b, c, d):
        hip.free(p)


def test_row_sums_of_squares_in_double_follow_a_plain_loop():
    """zk_row_sumsq_f64 must round exactly as `for j: acc += (x[j] / scale) ** 2` does: Python floats are IEEE doubles and
    every operation involved is exactly rounded, so the device result is compared bit for bit."""
    from gpuhelp import Hip, c_void_p
    hip = Hip()
    rng = np.random.default_rng(77)
    rows, cols, scale = 7, 333, 65536.0
    x = rng.integers(-(1 << 22), 1 << 22, (rows, cols))
    x[0, :3] = [0, -1, (1 << 40) + 12345]
    X = fr_array([int(v) % R_MOD for v in x.reshape(-1)])
    dX = hip.upload(X)
    dout = hip.malloc(8 * rows)
    hip.call("zk_row_sumsq_f64", c_void_p(dout), c_void_p(dX), ctypes.c_uint32(rows), ctypes.c_uint32(cols), ctypes.c_double(scale), None)
    got = hip.download(dout, (rows,), np.float64)
    exp = np.zeros(rows, np.float64)
    for r in range(rows):
        acc = 0.0
        for j in range(cols):
            t = float(int(x[r, j])) / scale
            acc += t * t
        exp[r] = acc
    assert (got.view(np.uint64) == exp.view(np.uint64)).all()
    hip.free(dX)
    hip.free(dout)


def test_matmul_int8_plane_path_equals_generic_at_projection_size(pv):
    """1024 x 4096 x 1024 (2^32 multiply-accumulates): the small-integer product goes to the matrix cores as balanced
    base-256 digit planes.  Checked against the generic Montgomery kernel on the whole output and against big-int dot
    products on sampled entries; the operands hold the values around every digit carry."""
    rng = np.random.default_rng(5)
    M, N, P = 1024, 4096, 1024
    A = rng.integers(-(1 << 19), 1 << 19, (M, N)).astype(np.int64)
    B = rng.integers(-(1 << 13), 1 << 13, (N, P)).astype(np.int64)
    edge = np.array([0, 1, -1, 127, 128, -128, -129, 255, 256, -255, -256, 32767, 32768, -32768, -32769, 65535, 65536, -65536, -65537, (1 << 19) - 1, -(1 << 19)])
    A[0, :edge.size] = edge
    A[1:1 + edge.size, 0] = edge
    B[:12, 0] = edge[:12]
    B[0, :15] = edge[:15] // 8
    hA, hB = pv.from_i64(A), pv.from_i64(B)
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    got = pv.matmul(hA, hB, M, N, P).host()
    assert pv.lib.zkp_last_matmul_path() == 2
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(1))
    ref = pv.matmul(hA, hB, M, N, P).host()
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    assert (got == ref).all()
    Ao, Bo = A.astype(object), B.astype(object)
    for (i, j) in [(0, 0), (1, 0), (5, 0), (0, 3)] + [(int(rng.integers(M)), int(rng.integers(P))) for _ in range(40)]:
        want = int(sum(Ao[i, :] * Bo[:, j])) % R_MOD
        assert fr_ints(got[i * P + j].reshape(1, 8))[0] == want


def test_matmul_int8_plane_path_on_ragged_stacks_and_wide_operands(pv):
    """The matrix-core path (digit planes, k_gemm_i8_planes) forced onto small stacks whose sizes are no multiples of its
    tiles (rows, columns and the contraction all ragged; a single row; a contraction shorter than one tile), with a left
    operand of up to 2^38 (five planes) and a right operand of up to 2^33 (five planes), which go pair by pair, and with one to three
    planes a side, which take every pair in one pass: every entry against big integers."""
    import os
    rng = np.random.default_rng(91)
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    old = os.environ.get("ZKLLM_MATMUL_PLANES")
    os.environ["ZKLLM_MATMUL_PLANES"] = "1"
    try:
        for num, M, N, P, (alo, ahi), (blo, bhi) in [(3, 70, 130, 50, (-2 ** 17, 2 ** 17), (-2 ** 10, 2 ** 10)),
                                                     (2, 200, 1000, 150, (-2 ** 38, 2 ** 38), (-2 ** 12, 2 ** 12)),
                                                     (1, 33, 5, 257, (-2 ** 20, 2 ** 20), (-2 ** 33, 2 ** 33)),
                                                     (4, 129, 257, 32, (-128, 128), (-129, 129)),
                                                     (2, 64, 128, 64, (-127, 128), (-127, 128)),
                                                     (1, 100, 300, 90, (-2 ** 22, 2 ** 22), (-2 ** 22, 2 ** 22))]:
            A = rng.integers(alo, ahi, (num, M, N)).astype(np.int64)
            B = rng.integers(blo, bhi, (num, N, P)).astype(np.int64)
            A[0, 0, :3] = [alo, ahi - 1, 0]
            B[0, :3, 0] = [bhi - 1, blo, 0]
            got = pv.matmul_stack(pv.from_i64(A), pv.from_i64(B), num, M, N, P).host()
            assert pv.lib.zkp_last_matmul_path() == 2
            want = [int(v) % R_MOD for i in range(num) for v in (A[i].astype(object) @ B[i].astype(object)).reshape(-1)]
            assert fr_ints(got) == want, (num, M, N, P)
    finally:
        if old is None:
            del os.environ["ZKLLM_MATMUL_PLANES"]
        else:
            os.environ["ZKLLM_MATMUL_PLANES"] = old


def test_matmul_with_a_kept_right_operand_and_layers_over_views(pv):
    """A weight kept as the right operand of matrix products (FrTensor::keep_as_matmul_rhs: largest magnitude and digit planes
    computed once, zk_fr_matmul_rhs_prepare / zk_fr_matmul_rhs) gives the products of the plain path, on the matrix-core path and
    on the others; what was kept is dropped when the weight is modified in place; a zkFC over a view of the weight
    (FrTensor::view) computes with the weight's own elements and leaves them alive."""
    import os
    rng = np.random.default_rng(17)
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    old = os.environ.get("ZKLLM_MATMUL_PLANES")
    try:
        for planes, (M, N, P), (wlo, whi) in [("1", (70, 130, 50), (-2 ** 13, 2 ** 13)), ("1", (33, 257, 64), (-2 ** 33, 2 ** 33)),
                                               ("0", (40, 100, 24), (-2 ** 13, 2 ** 13))]:
            os.environ["ZKLLM_MATMUL_PLANES"] = planes
            W = rng.integers(wlo, whi, (N, P)).astype(np.int64)
            D = rng.integers(-50, 50, (N, P)).astype(np.int64)
            hW, hD = pv.from_i64(W), pv.from_i64(D)
            pv.keep_as_matmul_rhs(hW)
            for rep in range(3):                      # first product prepares, the others reuse
                X = rng.integers(-2 ** 17, 2 ** 17, (M, N)).astype(np.int64)
                got = pv.matmul(pv.from_i64(X), hW, M, N, P).host()
                assert pv.lib.zkp_last_matmul_path() == 2
                assert fr_ints(got) == [int(v) % R_MOD for v in (X.astype(object) @ W.astype(object)).reshape(-1)], (planes, rep)
            got = pv.fc_forward_over_view(hW, pv.from_i64(X), N, P).host()
            assert fr_ints(got) == [int(v) % R_MOD for v in (X.astype(object) @ W.astype(object)).reshape(-1)]
            # a left operand that keeps an int32 form is read from it (zk_fr_matmul_rhs_ints), extremes included: same product
            Xi = rng.integers(-2 ** 31, 2 ** 31, (M, N)).astype(np.int64) if whi <= 2 ** 13 else X.copy()
            Xi[0, :3] = [-2 ** 31, 2 ** 31 - 1, 0]
            hXi = pv.from_i64(Xi)
            pv.keep_for_folds(hXi)
            assert pv.folds_from_ints(hXi) == 1
            got = pv.matmul(hXi, hW, M, N, P).host()
            assert fr_ints(got) == [int(v) % R_MOD for v in (Xi.astype(object) @ W.astype(object)).reshape(-1)], planes
            pv.add_inplace(hW, hD)                    # the weight changes: nothing stale may be used
            W2 = W + D
            got = pv.matmul(pv.from_i64(X), hW, M, N, P).host()
            assert fr_ints(got) == [int(v) % R_MOD for v in (X.astype(object) @ W2.astype(object)).reshape(-1)]
            assert fr_ints(hW.host()) == [int(v) % R_MOD for v in W2.reshape(-1)]
        # a right operand of full-width residues: kept, and the generic path still runs
        Af = mt_random_vec(np.random.RandomState(5), 9 * 20)
        Bf = mt_random_vec(np.random.RandomState(6), 20 * 7)
        hB = pv.from_fr(Bf)
        pv.keep_as_matmul_rhs(hB)
        for rep in range(2):
            got = pv.matmul(pv.from_fr(Af), hB, 9, 20, 7).host()
            assert pv.lib.zkp_last_matmul_path() == 1
            Ai, Bi = np.array(fr_ints(Af), dtype=object).reshape(9, 20), np.array(fr_ints(Bf), dtype=object).reshape(20, 7)
            assert fr_ints(got) == [int(v) % R_MOD for v in (Ai @ Bi).reshape(-1)]
    finally:
        if old is None:
            os.environ.pop("ZKLLM_MATMUL_PLANES", None)
        else:
            os.environ["ZKLLM_MATMUL_PLANES"] = old


@pytest.mark.parametrize("other,cur,win", [(1, 128, 4096), (3, 100, 64), (37, 1000, 1), (16, 4096, 1), (9, 11008, 1), (5, 63, 1), (2, 2, 8), (1, 512, 1024), (6, 7, 5),
                                           (1, 70000, 1)])
def test_folds_of_a_tensor_kept_for_folds_read_its_int32_form_and_give_the_same_elements(pv, orc, other, cur, win):
    """A tensor of 32-bit integers kept for folds (FrTensor::keep_for_folds -> zk_fr_fold_prepare / zk_fr_fold_axis_prepared:
    unreduced ten-limb sums of entry x integer products, one reduction per output) folds to the elements the oracle's
    level-by-level fold gives, for the row folds of the openings (long windows), the column folds of zkFC::prove (window 1:
    one wave per four rows), ragged axes and the extreme integers; a change in place drops the kept form; a tensor with an
    element outside 32 bits keeps none and folds as before."""
    print("case", other, cur, win, flush=True)
    rng = np.random.default_rng(cur * 31 + win)
    n = other * cur * win
    W = rng.integers(-2 ** 31, 2 ** 31, n).astype(np.int64)
    W[0], W[1 % n], W[2 % n] = -2 ** 31, 2 ** 31 - 1, 0
    if n > 8:
        W[n - 1], W[n - 2] = -2 ** 31, -2 ** 31        # the largest magnitude side by side
    k = (cur - 1).bit_length()
    u = mt_random_vec(np.random.RandomState(18), k)
    A = fr_array([int(v) % R_MOD for v in W])
    exp = np.zeros((n, 8), np.uint32)
    out_n = np.zeros(1, np.int64)
    orc_check(orc.orc_fr_partial_me(A, n, u, k, cur, win, exp, out_n))
    h = pv.from_i64(W)
    pv.keep_for_folds(h)
    assert pv.folds_from_ints(h) == 1
    for rep in range(2):
        got = pv.partial_me(h, u, cur, win).host()
        assert got.shape[0] == out_n[0] == other * win
        assert (got == exp[:out_n[0]]).all(), rep
    if other == 1:          # the deprecated window form (the fold at the head of an opening) takes the same path
        got = pv.partial_me_window(h, u, win).host()
        assert (got == exp[:out_n[0]]).all()
    # the tensor changes in place: nothing stale may be read, and the new elements are examined again
    D = rng.integers(-5, 5, n).astype(np.int64)
    D[0], D[1 % n] = 1, 0
    if n > 8:
        D[n - 1], D[n - 2] = 0, 3
    pv.add_inplace(h, pv.from_i64(D))
    W2 = W + D
    A2 = fr_array([int(v) % R_MOD for v in W2])
    orc_check(orc.orc_fr_partial_me(A2, n, u, k, cur, win, exp, out_n))
    got = pv.partial_me(h, u, cur, win).host()
    assert (got == exp[:out_n[0]]).all()
    assert pv.folds_from_ints(h) == 1
    # one element of 33 bits: no int32 form is kept, the fold is the plain one
    W3 = W2.copy()
    W3[n // 2] = 2 ** 31
    h3 = pv.from_i64(W3)
    pv.keep_for_folds(h3)
    assert pv.folds_from_ints(h3) == 0
    A3 = fr_array([int(v) % R_MOD for v in W3])
    orc_check(orc.orc_fr_partial_me(A3, n, u, k, cur, win, exp, out_n))
    got = pv.partial_me(h3, u, cur, win).host()
    assert (got == exp[:out_n[0]]).all()


def test_stacks_of_matrices_transpose_and_multiply_like_their_members(pv):
    """zk_fr_matmul_batched / zk_fr_transpose_batched on every path of the dispatcher (both operands in 31 bits, wide left
    operand, wide right operand, full-width residues): each product of the stack against big-int arithmetic."""
    rng = np.random.default_rng(77)
    num, M, N, P = 3, 70, 130, 50
    cases = [((-2 ** 17, 2 ** 17), (-2 ** 10, 2 ** 10), 2), ((-2 ** 40, 2 ** 40), (-2 ** 12, 2 ** 12), 2), ((-2 ** 20, 2 ** 20), (-2 ** 33, 2 ** 33), 2)]
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    for (alo, ahi), (blo, bhi), path in cases:
        A = rng.integers(alo, ahi, (num, M, N)).astype(np.int64)
        B = rng.integers(blo, bhi, (num, N, P)).astype(np.int64)
        got = pv.matmul_stack(pv.from_i64(A), pv.from_i64(B), num, M, N, P).host()
        assert pv.lib.zkp_last_matmul_path() == path
        want = [int(v) % R_MOD for i in range(num) for v in (A[i].astype(object) @ B[i].astype(object)).reshape(-1)]
        assert fr_ints(got) == want
    Af = mt_random_vec(np.random.RandomState(1), num * 9 * 20)
    Bf = mt_random_vec(np.random.RandomState(2), num * 20 * 7)
    got = pv.matmul_stack(pv.from_fr(Af), pv.from_fr(Bf), num, 9, 20, 7).host()
    assert pv.lib.zkp_last_matmul_path() == 1
    Ai, Bi = np.array(fr_ints(Af), dtype=object).reshape(num, 9, 20), np.array(fr_ints(Bf), dtype=object).reshape(num, 20, 7)
    assert fr_ints(got) == [int(v) % R_MOD for i in range(num) for v in (Ai[i] @ Bi[i]).reshape(-1)]
    T = rng.integers(-2 ** 40, 2 ** 40, (5, 37, 70)).astype(np.int64)
    got = pv.transpose_stack(pv.from_i64(T), 5, 37, 70).host()
    assert fr_ints(got) == [int(v) % R_MOD for v in T.transpose(0, 2, 1).reshape(-1)]
    # the leading two axes swapped in one pass (zk_fr_swap_axes: tokens x heads x k to heads x tokens x k and back)
    for A, B, C in ((5, 37, 70), (16, 2, 16), (1, 9, 3), (33, 1, 7)):
        T3 = rng.integers(-2 ** 40, 2 ** 40, (A, B, C)).astype(np.int64)
        hT3 = pv.from_i64(T3)
        got = pv.swap_axes(hT3, A, B, C)
        assert fr_ints(got.host()) == [int(v) % R_MOD for v in T3.transpose(1, 0, 2).reshape(-1)], (A, B, C)
        assert (pv.swap_axes(got, B, A, C).host() == hT3.host()).all()


@pytest.mark.parametrize("num,M,N,P,abits,bbits,ybits", [(3, 70, 130, 50, 16, 16, 17), (2, 33, 65, 128, 31, 31, 17), (1, 128, 256, 64, 8, 9, 12), (2, 20, 40, 9, 31, 31, 40),
                                                          (1, 64, 64, 64, 16, 15, 280)])
def test_a_product_of_two_int32_tensors_multiplies_and_folds_without_being_written(pv, orc, num, M, N, P, abits, bbits, ybits):
    """zk_fr_matmul_batched_prod / zk_fr_fold_axis_prod (the softmax output as the product of its two segments' table values,
    zksoftmax.cu:160-166, then Y x V and the fold of Y over its rows, zksoftmax.cu:315-336 in stacked form): the same elements as
    the product written out first, on every path of the dispatcher (narrow and wide products, wide and full-width right operand)
    and with the extreme integers in both factors."""
    print("case", num, M, N, P, abits, bbits, ybits, flush=True)
    rng = np.random.default_rng(num * 1000 + M + abits)
    A = rng.integers(-2 ** abits, 2 ** abits, (num, M, N)).astype(np.int64)
    B = rng.integers(-2 ** bbits, 2 ** bbits, (num, M, N)).astype(np.int64)
    if abits == 31:
        A[0, 0, :4], B[0, 0, :4] = [-2 ** 31, -2 ** 31, 2 ** 31 - 1, 2 ** 31 - 1], [-2 ** 31, 2 ** 31 - 1, -2 ** 31, 2 ** 31 - 1]
        A[-1, -1, -1], B[-1, -1, -1] = -2 ** 31, -2 ** 31
    A, B = np.clip(A, -2 ** 31, 2 ** 31 - 1), np.clip(B, -2 ** 31, 2 ** 31 - 1)
    if ybits > 64:
        Yf = mt_random_vec(np.random.RandomState(5), num * N * P)
        hY = pv.from_fr(Yf)
        Yi = np.array(fr_ints(Yf), dtype=object).reshape(num, N, P)
    else:
        Y64 = rng.integers(-2 ** ybits, 2 ** ybits, (num, N, P)).astype(np.int64)
        hY = pv.from_i64(Y64)
        Yi = Y64.astype(object)
    hA, hB = pv.from_i64(A), pv.from_i64(B)
    pv.keep_for_folds(hA)
    pv.keep_for_folds(hB)
    assert pv.folds_from_ints(hA) == 1 and pv.folds_from_ints(hB) == 1
    prod = A.astype(object) * B.astype(object)
    pv.lib.zkp_set_matmul_mode(ctypes.c_int(0))
    got = pv.matmul_stack_prod(hA, hB, hY, num, M, N, P).host()
    want = [int(v) % R_MOD for i in range(num) for v in (prod[i] @ Yi[i]).reshape(-1)]
    assert fr_ints(got) == want, pv.lib.zkp_last_matmul_path()
    # the fold over the rows of each matrix (cur = M, window = N, other = num) against the oracle's fold of the written product
    k = max((M - 1).bit_length(), 1)
    u = mt_random_vec(np.random.RandomState(19), k)
    n = num * M * N
    Pf = fr_array([int(v) % R_MOD for v in prod.reshape(-1)])
    exp = np.zeros((n, 8), np.uint32)
    out_n = np.zeros(1, np.int64)
    orc_check(orc.orc_fr_partial_me(Pf, n, u, k, M, N, exp, out_n))
    for rep in range(2):
        got = pv.partial_me_prod(hA, hB, u, M, N).host()
        assert got.shape[0] == out_n[0] == num * N
        assert (got == exp[:out_n[0]]).all(), rep
    # a factor without an int32 form is refused
    hC = pv.from_i64(A)
    with pytest.raises(RuntimeError):
        pv.partial_me_prod(hA, hC, u, M, N)


def test_products_written_as_64_bit_integers(monkeypatch):
    """zk_fr_matmul_batched_i64 / _bt (the attention scores Q K^T for the pass that shifts and decomposes them): the matrix-core
    path's products as int64 against numpy, the right operand given either way round; a product the path does not take (operands
    of full width, or too few multiply-adds for it) reports 0 and writes nothing."""
    from gpuhelp import Hip, c_void_p, c_uint, c_int
    hip = Hip()
    rng = np.random.default_rng(64)
    num, M, N, P = 3, 70, 24, 90
    A = rng.integers(-2 ** 17, 2 ** 17, (num, M, N)).astype(np.int64)
    B = rng.integers(-2 ** 17, 2 ** 17, (num, N, P)).astype(np.int64)
    A[0, 0, :2], B[0, :2, 0] = [2 ** 17 - 1, -2 ** 17], [-2 ** 17, 2 ** 17 - 1]
    want = np.stack([A[i] @ B[i] for i in range(num)])
    dA = hip.upload(fr_array([int(v) % R_MOD for v in A.reshape(-1)]))
    dB = hip.upload(fr_array([int(v) % R_MOD for v in B.reshape(-1)]))
    dBt = hip.upload(fr_array([int(v) % R_MOD for v in B.transpose(0, 2, 1).reshape(-1)]))
    dC = hip.malloc(8 * num * M * P)
    taken = ctypes.c_int(-1)
    monkeypatch.setenv("ZKLLM_MATMUL_PLANES", "1")
    for name, b in (("zk_fr_matmul_batched_i64", dB), ("zk_fr_matmul_batched_i64_bt", dBt)):
        hip.lib.zk_memset(c_void_p(dC), c_int(0x5A), ctypes.c_size_t(8 * num * M * P), None)
        hip.call(name, c_void_p(dC), c_void_p(dA), c_void_p(b), c_uint(num), c_uint(M), c_uint(N), c_uint(P), ctypes.byref(taken), None)
        assert taken.value == 1, name
        assert (hip.download(dC, (num, M, P), np.int64) == want).all(), name
    # below the threshold of the matrix-core path: not taken, nothing written
    monkeypatch.setenv("ZKLLM_MATMUL_PLANES", "40")
    hip.lib.zk_memset(c_void_p(dC), c_int(0x5A), ctypes.c_size_t(8 * num * M * P), None)
    hip.call("zk_fr_matmul_batched_i64", c_void_p(dC), c_void_p(dA), c_void_p(dB), c_uint(num), c_uint(M), c_uint(N), c_uint(P), ctypes.byref(taken), None)
    assert taken.value == 0
    assert (hip.download(dC, (num * M * P,), np.uint64) == 0x5A5A5A5A5A5A5A5A).all()
    # a left operand of full-width residues: no small-integer bound, not taken
    monkeypatch.setenv("ZKLLM_MATMUL_PLANES", "1")
    dAf = hip.upload(mt_random_vec(np.random.RandomState(3), num * M * N))
    hip.call("zk_fr_matmul_batched_i64_bt", c_void_p(dC), c_void_p(dAf), c_void_p(dBt), c_uint(num), c_uint(M), c_uint(N), c_uint(P), ctypes.byref(taken), None)
    assert taken.value == 0
    # a null operand is an argument error, not a launch
    with pytest.raises(RuntimeError, match="null operand"):
        hip.call("zk_fr_matmul_batched_i64", c_void_p(dC), None, c_void_p(dB), c_uint(num), c_uint(M), c_uint(N), c_uint(P), ctypes.byref(taken), None)
    for p in (dA, dB, dBt, dC, dAf):
        hip.free(p)


def test_config2_full_size_fully_connected_proof_passes_the_verifier(pv):
    """X 2048 x 4096 times W 4096 x 4096 (fixed point, scale 2^16, N(0, 0.02)), beyond what the oracle can follow: rows
    of the product are compared with int64 arithmetic, and the proof transcript under a seeded stream is checked as a
    verifier would in big integers: the claim is Y at (u_batch, u_output), each of the 12 rounds satisfies p(0) + p(1) =
    claim and hands on p(v), and the last claim is X(u_batch, u_input) * W(u_input, u_output), both recomputed from the
    full tensors apart from the proof."""
    B, I, O = 2048, 4096, 4096
    rng = np.random.default_rng(20242)
    X = np.round(rng.normal(0, 0.02, (B, I)) * 65536).astype(np.int32)
    W = np.round(rng.normal(0, 0.02, (I, O)) * 65536).astype(np.int32)
    hX, hW = pv.from_i32(X), pv.from_i32(W)
    hY = pv.matmul(hX, hW, B, I, O)
    Y = hY.host()
    for r in (0, 777, 2047):
        exp = X[r].astype(np.int64) @ W.astype(np.int64)
        assert fr_ints(Y[r * O:(r + 1) * O]) == [int(v) % R_MOD for v in exp], r
    del Y
    seed = 909
    pv.seed(seed)
    pv.transcript_begin()
    pv.zkfc_prove(hX, hW, hY, I, O)
    pv.lib.zkp_transcript_end()
    t = fr_ints(pv.transcript())
    rs = np.random.RandomState(seed)
    u_b, u_i, u_o = mt_random_vec(rs, 11), mt_random_vec(rs, 12), mt_random_vec(rs, 12)
    assert len(t) == 1 + 3 * 12 + 3
    claim = t[0]
    assert [claim] == fr_ints(pv.multi_dim_me(hY, [u_b, u_o], (B, O)))
    vi = fr_ints(u_i)
    for r in range(12):
        c0, c1, c2 = t[1 + 3 * r:4 + 3 * r]
        assert (2 * c0 + c1 + c2) % R_MOD == claim, r
        v = vi[11 - r]                                   # the rounds consume u_input from the back
        claim = (c0 + c1 * v + c2 * v * v) % R_MOD
    final, cX, cW = t[37:40]
    assert final == claim and cX * cW % R_MOD == final
    assert [cX] == fr_ints(pv.multi_dim_me(hX, [u_b, u_i], (B, I)))
    assert [cW] == fr_ints(pv.multi_dim_me(hW, [u_i, u_o], (I, O)))


# ---- .bin files (fr-tensor.cu:181-248, ioutils.cu:3-45) ---------------------------------------------------------------------
def ref_scalar_to_int(x, bits):
    """scalar_to_int / scalar_to_long (fr-tensor.cu:922-945): the value when it is a non-negative number below 2^(bits-1),
    else minus the low word of r - x, which scalar_to_uint / scalar_to_ulong read as 0 when r - x does not fit the word"""
    top = 1 << bits
    if x < (top >> 1):
        return x
    n = (R_MOD - x) % R_MOD
    u = n if n < top else 0
    v = (-u) % top
    return v - top if v >= (top >> 1) else v


def test_fr_bin_files_round_trip_and_conversions(pv, tmp_path):
    rng = np.random.default_rng(3)
    # int32 files: from_int_bin embeds negatives as r - |x|; save_int gives the same bytes back
    a32 = np.concatenate([np.array([0, 1, -1, 2**31 - 1, -2**31, 65536, -65536], dtype=np.int32), rng.integers(-2**31, 2**31, 1000).astype(np.int32)])
    a32.tofile(tmp_path / "a32.bin")
    t = pv.from_file(tmp_path / "a32.bin", 1)
    assert fr_ints(t.host()) == [int(v) % R_MOD for v in a32]
    pv.save(t, tmp_path / "a32_back.bin", 1)
    assert (tmp_path / "a32_back.bin").read_bytes() == (tmp_path / "a32.bin").read_bytes()
    # int64 files: every byte of the file is read (the reference's from_long_bin copies only the first half of the buffer to
    # the device, fr-tensor.cu:243-244, and converts whatever the second half of its allocation holds)
    a64 = np.concatenate([np.array([0, 1, -1, 2**63 - 1, -2**63 + 1, 2**40, -2**40], dtype=np.int64), rng.integers(-2**62, 2**62, 1000)])
    a64.tofile(tmp_path / "a64.bin")
    t64 = pv.from_file(tmp_path / "a64.bin", 2)
    assert t64.size == a64.size and fr_ints(t64.host()) == [int(v) % R_MOD for v in a64]
    pv.save(t64, tmp_path / "a64_back.bin", 2)
    assert (tmp_path / "a64_back.bin").read_bytes() == (tmp_path / "a64.bin").read_bytes()
    # raw field elements: 32 bytes each, standard form, as they lie in device memory
    raw = seeded(500, 9)
    h = pv.from_fr(raw)
    pv.save(h, tmp_path / "raw.bin", 0)
    assert (tmp_path / "raw.bin").read_bytes() == raw.tobytes()
    assert (pv.from_file(tmp_path / "raw.bin", 0).host() == raw).all()
    # values outside the integer types: what scalar_to_int / scalar_to_long give
    odd = [2**31, 2**31 + 5, 2**32 + 7, R_MOD - 2**31, R_MOD - 2**31 - 5, R_MOD - 2**32 - 9, R_MOD - 1, 2**63, 2**64 + 3, R_MOD - 2**63, R_MOD - 2**64 - 1, R_MOD >> 1]
    ho = pv.from_fr(fr_array(odd))
    pv.save(ho, tmp_path / "odd32.bin", 1)
    pv.save(ho, tmp_path / "odd64.bin", 2)
    assert list(np.fromfile(tmp_path / "odd32.bin", dtype=np.int32)) == [ref_scalar_to_int(x, 32) for x in odd]
    assert list(np.fromfile(tmp_path / "odd64.bin", dtype=np.int64)) == [ref_scalar_to_int(x, 64) for x in odd]
    # an int32 file read as int64 halves the element count (sizes come from the file length alone)
    assert pv.from_file(tmp_path / "a32.bin", 2).size == a32.size // 2
    with pytest.raises(RuntimeError):
        pv.from_file(tmp_path / "missing.bin", 1)


# ---- the allocator across streams and host threads ---------------------------------------------------------------------------------
def _hip_streams(n):
    rt = ctypes.CDLL("libamdhip64.so")
    out = []
    for _ in range(n):
        s = ctypes.c_void_p()
        assert rt.hipStreamCreateWithFlags(ctypes.byref(s), ctypes.c_uint(1)) == 0      # non-blocking, default priority
        out.append(s)
    return rt, out


def test_scratch_blocks_reused_on_another_stream_wait_for_their_last_user(hip):
    """Two matrix products of one shape on two streams back to back: the second call gets the scratch blocks that the first
    call has just given back while its kernels are still queued, and must not overwrite them early."""
    rt, (sA, sB) = _hip_streams(2)
    M, N, P = 2048, 1024, 2048
    rng = np.random.default_rng(12)
    mats = [rng.integers(-2000, 2000, size=(M, N)), rng.integers(-2000, 2000, size=(N, P)), rng.integers(-2000, 2000, size=(M, N)), rng.integers(-2000, 2000, size=(N, P))]
    dev = []
    for m in mats:
        d_i = hip.upload(m.astype(np.int64))
        d_f = hip.malloc(32 * m.size)
        hip.call("zk_fr_from_i64", ctypes.c_void_p(d_f), ctypes.c_void_p(d_i), ctypes.c_size_t(m.size), None)
        hip.free(d_i)
        dev.append(d_f)
    hip.sync()
    C = [hip.malloc(32 * M * P) for _ in range(2)]
    path = ctypes.c_int(0)
    # entries below 2000 and 1024 terms: every sum stays below 2^53, so the float64 product is exact
    want = [(mats[0].astype(np.float64) @ mats[1].astype(np.float64)).astype(np.int64).reshape(-1), (mats[2].astype(np.float64) @ mats[3].astype(np.float64)).astype(np.int64).reshape(-1)]
    for rep in range(3):
        print("case two streams rep", rep, flush=True)
        hip.call("zk_fr_matmul", ctypes.c_void_p(C[0]), ctypes.c_void_p(dev[0]), ctypes.c_void_p(dev[1]), ctypes.c_uint32(M), ctypes.c_uint32(N), ctypes.c_uint32(P), ctypes.c_int(2), ctypes.byref(path), sA)
        hip.call("zk_fr_matmul", ctypes.c_void_p(C[1]), ctypes.c_void_p(dev[2]), ctypes.c_void_p(dev[3]), ctypes.c_uint32(M), ctypes.c_uint32(N), ctypes.c_uint32(P), ctypes.c_int(2), ctypes.byref(path), sB)
        assert rt.hipStreamSynchronize(sA) == 0 and rt.hipStreamSynchronize(sB) == 0
        for c, exp in zip(C, want):
            got = hip.download(c, (M * P, 8), np.uint32)
            lo = got[:, 0].astype(np.uint64) | (got[:, 1].astype(np.uint64) << np.uint64(32))
            neg = got[:, 7] != 0
            val = np.where(neg, -((np.uint64(R_MOD & (2**64 - 1)) - lo).astype(np.int64)), lo.astype(np.int64))
            assert (val == exp).all()
    for p in dev + C:
        hip.free(p)
    assert rt.hipStreamDestroy(sA) == 0 and rt.hipStreamDestroy(sB) == 0


def test_two_host_threads_reduce_on_two_streams(hip):
    """results come back through a pinned buffer per host thread"""
    import threading
    rt, streams = _hip_streams(2)
    data = [seeded(1 << 18, 50 + i) for i in range(2)]
    want = [sum(fr_ints(d)) % R_MOD for d in data]
    dev = [hip.upload(d) for d in data]
    bad = []

    def work(i):
        out = np.zeros(8, np.uint32)
        for _ in range(200):
            rc = hip.lib.zk_fr_sum(ctypes.c_void_p(out.ctypes.data), ctypes.c_void_p(dev[i]), ctypes.c_size_t(data[i].shape[0]), streams[i])
            if rc != 0 or fr_ints(out.reshape(1, 8))[0] != want[i]:
                bad.append((i, rc))
                return
    th = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    assert not bad
    for p in dev:
        hip.free(p)
    for s in streams:
        assert rt.hipStreamDestroy(s) == 0
