"""GPU parity: multiplicities, batch inversion, the two-phase lookup sumcheck, range / mapping tables,
rescaling, multi-Hadamard sumcheck, stacked inner-product sumcheck and zkSoftmax -- bit-exact against the oracle."""
import numpy as np
import pytest
from ctypes import c_uint64 as c_u64

from zkhelp import R_MOD, fr_array, fr_ints, load_oracle, mt_random_vec, orc_check, orc_transcript

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pv():
    from gpuhelp import Prover
    return Prover()


@pytest.fixture(scope="module")
def orc():
    return load_oracle()


def ch(seed, n):
    return mt_random_vec(np.random.RandomState(seed), n)


@pytest.mark.parametrize("n,sf", [(1, 16), (1000, 16), (4096, 1 << 16), (70000, 1 << 20), (5000, 1000), (300, 3), (70000, 65537), (100, 1), (100, 2)])
def test_rescale(pv, orc, n, sf):
    rng = np.random.default_rng(n)
    x = rng.integers(-(1 << 40), 1 << 40, n)
    x[: min(n, 6)] = [0, sf // 2, -(sf // 2), sf // 2 - 1, -(sf // 2) - 1, 3 * sf][: min(n, 6)]
    X = fr_array([int(v) % R_MOD for v in x])
    e_out, e_rem = np.zeros_like(X), np.zeros_like(X)
    orc_check(orc.orc_rescale(X, n, sf, e_out, e_rem))
    out, rem = pv.rescale(pv.from_fr(X), sf)
    assert (out.host() == e_out).all() and (rem.host() == e_rem).all()


@pytest.mark.parametrize("n,sf", [(1, 16), (1000, 16), (70000, 1 << 16)])
def test_relu_decomposition(pv, orc, n, sf):
    rng = np.random.default_rng(n + 1)
    x = rng.integers(-(1 << 40), 1 << 40, n)
    x[: min(n, 7)] = [0, sf // 2, -(sf // 2), sf // 2 - 1, -(sf // 2) - 1, 3 * sf, -3 * sf][: min(n, 7)]
    X = fr_array([int(v) % R_MOD for v in x])
    e = [np.zeros_like(X) for _ in range(4)]
    e_m = np.zeros((sf, 8), np.uint32)
    orc_check(orc.orc_relu(X, n, sf, *e, e_m))
    out, parts = pv.relu(pv.from_fr(X), sf)
    assert (out.host() == e[0]).all()
    for got, want in zip(parts, e[1:] + [e_m]):
        assert (got.host() == want).all()


@pytest.mark.parametrize("D,low,length", [(64, -5, 11), (5000, -8, 16), (1 << 16, -(1 << 15), 1 << 16), (300000, 0, 1 << 18), (100000, 0, 3)])
def test_multiplicities(pv, D, low, length):
    rng = np.random.default_rng(D)
    vals = rng.integers(low, low + length, D)
    vals[: D // 3] = low + length // 2               # a long run of equal values (wave aggregation path)
    # queries that keep an int32 form are counted from it, positions formed by the counting passes (zk_lookup_hist_i32)
    hk = pv.from_i64(vals)
    pv.keep_for_folds(hk)
    assert pv.folds_from_ints(hk) == 1
    mk = pv.range_prep(hk, low, length).host()
    m = pv.range_prep(pv.from_i64(vals), low, length).host()
    assert (mk == m).all()
    size = 1 << max(0, (length - 1).bit_length())
    assert fr_ints(m) == [int(c) for c in np.bincount(vals - low, minlength=size)]


@pytest.mark.parametrize("D,low,length,skew", [((1 << 21) + 12345, -5, (1 << 18) + 777, 3), (1500000, 0, 1 << 20, 1), ((1 << 20) + 1, -9, 1 << 22, 0)])
def test_multiplicities_of_many_queries_into_a_large_table(pv, D, low, length, skew):
    """Above 2^20 queries and 16384 bins the counts come from the partitioned path (scatter by high bits, LDS counts per
    partition): ragged sizes, a table that is no power of two, a third of the queries equal, all queries equal."""
    rng = np.random.default_rng(D)
    vals = rng.integers(low, low + length, D)
    if skew == 3:
        vals[: D // 3] = low + length // 2
    elif skew == 1:
        vals[:] = low + 4097
    m = pv.range_prep(pv.from_i64(vals), low, length).host()
    want = np.bincount(vals - low, minlength=m.shape[0]).astype(np.uint32)
    assert (m[:, 0] == want).all() and not m[:, 1:].any()
    hk = pv.from_i64(vals)          # the same from the queries' int32 form
    pv.keep_for_folds(hk)
    mk = pv.range_prep(hk, low, length).host()
    assert (mk[:, 0] == want).all() and not mk[:, 1:].any()


def test_lookup_out_of_range_is_an_error(pv):
    with pytest.raises(RuntimeError, match="outside the table"):
        pv.range_prep(pv.from_i64(np.array([0, 1, 99])), 0, 8)
    for bad in (8, -1, 6):          # from the int32 form too; 6: inside the padded table of 8, outside the range of 6
        h = pv.from_i64(np.array([0, 1, bad] + [2] * 5000))
        pv.keep_for_folds(h)
        with pytest.raises(RuntimeError, match="outside the table"):
            pv.range_prep(h, 0, 6)


def test_range_lookup_rejects_values_in_the_padding_gap(pv):
    """A range of 6 values is kept in a table of 8 whose last two entries repeat low + 5: a query of low + 6 or low + 7 has
    room in the padded table but is outside the range, and must be refused like any other stray value."""
    low, length = -3, 6
    good = [-3, 2, 0, 1, -1, 2, 2, -3]
    mv = pv.from_fr(ch(31, length))
    pv.range_prep(pv.from_fr(fr_array([v % R_MOD for v in good])), low, length)
    pv.mapping(pv.from_fr(fr_array([v % R_MOD for v in good])), low, length, mv)
    for bad in (3, 4, 5, -4):
        vals = list(good)
        vals[5] = bad
        S = pv.from_fr(fr_array([v % R_MOD for v in vals]))
        with pytest.raises(RuntimeError, match="outside the table"):
            pv.range_prep(S, low, length)
        with pytest.raises(RuntimeError, match="outside the table"):
            pv.mapping(S, low, length, mv)


@pytest.mark.parametrize("n", [1, 7, 4096, 4097, 50000])
def test_batch_inverse(pv, orc, n):
    S = ch(n, n)
    beta = ch(5, 1)[0]
    if n >= 7:
        S[3] = fr_array([(-fr_ints(beta.reshape(1, 8))[0]) % R_MOD])[0]     # S + beta == 0 -> output 0
    exp = np.zeros_like(S)
    orc_check(orc.orc_lookup_inv(S, n, beta, exp))
    got = pv.batch_inv(pv.from_fr(S), beta).host()
    assert (got == exp).all()
    if n >= 7:
        assert not got[3].any()


def test_batch_inverse_at_full_size_inverts(pv):
    """2^24 + 5 values: the products of the workgroups are themselves too many for one step, so the scheme nests twice.
    Checked by what an inverse is: out * (in + beta) == 1 everywhere (0 where in + beta == 0)."""
    n = (1 << 24) + 5
    rng = np.random.default_rng(24)
    S = np.zeros((n, 8), np.uint32)
    S[:, :7] = rng.integers(0, 1 << 32, (n, 7), dtype=np.uint64).astype(np.uint32)     # below 2^224: standard-form residues
    beta = ch(6, 1)[0]
    hole = n - 3
    S[hole] = fr_array([(-fr_ints(beta.reshape(1, 8))[0]) % R_MOD])[0]
    hS = pv.from_fr(S)
    inv = pv.batch_inv(hS, beta)
    prod = pv.binop(2, inv, pv.scalarop(0, hS, beta)).host()
    expect = np.zeros((n, 8), np.uint32)
    expect[:, 0] = 1
    expect[hole, 0] = 0
    assert (prod == expect).all()


@pytest.mark.parametrize("D,low,length", [(16, 3, 4), (4, 0, 4), (256, -8, 16), (4096, -32, 64), (1 << 15, -(1 << 9), 1 << 10)])
def test_range_lookup_proof_transcript(pv, orc, D, low, length):
    rng = np.random.default_rng(D + length)
    vals = rng.integers(low, low + length, D)
    S = fr_array([int(v) % R_MOD for v in vals])
    k = (D - 1).bit_length()
    alpha, beta, u, v = ch(1, 1)[0], ch(2, 1)[0], ch(3, k), ch(4, k)
    orc.orc_transcript_clear()
    e_fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_range_prove(S, D, low, length, alpha, beta, u, v, e_fin))
    e_t = orc_transcript(orc)
    pv.transcript_begin()
    fin = pv.range_prove(pv.from_fr(S), low, length, alpha, beta, u, v)
    pv.lib.zkp_transcript_end()
    assert (fin == e_fin).all()
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()


@pytest.mark.parametrize("D,low,length", [(6, -2, 4), (64, -8, 16), (1000, -16, 32), (1 << 17, -16, 32)])
def test_mapping_lookup(pv, orc, D, low, length):
    rng = np.random.default_rng(D)
    vals = rng.integers(low, low + length, D)
    mv = ch(6, length)
    S = fr_array([int(v) % R_MOD for v in vals])
    k = (D - 1).bit_length()
    r, alpha, beta, u, v = ch(7, 1)[0], ch(8, 1)[0], ch(9, 1)[0], ch(10, k), ch(11, k)
    size = 1 << (length - 1).bit_length()
    e_y, e_m, e_fin = np.zeros((D, 8), np.uint32), np.zeros((size, 8), np.uint32), np.zeros(8, np.uint32)
    orc.orc_transcript_clear()
    orc_check(orc.orc_mapping(S, D, low, length, mv, r, alpha, beta, u, v, e_y, e_m, e_fin))
    e_t = orc_transcript(orc)
    pv.transcript_begin()
    y, m, fin = pv.mapping(pv.from_fr(S), low, length, pv.from_fr(mv), r, alpha, beta, u, v)
    pv.lib.zkp_transcript_end()
    assert (y.host() == e_y).all() and (m.host() == e_m).all() and (fin == e_fin).all()
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()


@pytest.mark.parametrize("lazy", [0, 1])
@pytest.mark.parametrize("n,sf,bits,fits", [(5000, 1 << 8, 30, True), (1 << 17, 1 << 8, 38, True), (1 << 17, 1 << 8, 41, False), (70000, 1 << 16, 36, True)])
def test_rescaling_that_gives_its_output_an_int32_form(pv, orc, n, sf, bits, fits, lazy):
    """Rescaling::rescale(X, true): output and proof transcript are the oracle's; the output keeps an int32 form exactly when
    every rescaled value fits 32 bits (41-bit inputs over 2^8 do not); the remainders' int32 form serves the proof either way
    (70000 and 5000 elements: padded; 2^17: read from the int32 form alone).  lazy (Rescaling::out_ints_lazy): whether the
    values fit is read from the device at the first use of the form, not by the rescaling; same results, and a fold of the
    output afterwards (from the int32 form when it was kept) is the oracle's."""
    x = np.random.default_rng(n + bits).integers(-(1 << bits), 1 << bits, n)
    x[0], x[1] = (1 << bits) - 1, -(1 << bits)
    X = fr_array([int(v) % R_MOD for v in x])
    orc.orc_seed(77)
    orc.orc_transcript_clear()
    e_out = np.zeros_like(X)
    orc_check(orc.orc_rescale_prove(X, n, sf, e_out))
    e_t = orc_transcript(orc)
    pv.seed(77)
    pv.transcript_begin()
    pv.lib.zkp_rescale_set_lazy(lazy)
    try:
        out = pv.rescale_ints_prove(pv.from_fr(X), sf)
    finally:
        pv.lib.zkp_rescale_set_lazy(0)
    pv.lib.zkp_transcript_end()
    assert (out.host() == e_out).all()
    assert pv.folds_from_ints(out) == (1 if fits else 0)
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()
    k = (n - 1).bit_length()
    u = mt_random_vec(np.random.RandomState(5), k)
    exp, out_n = np.zeros((n, 8), np.uint32), np.zeros(1, np.int64)
    orc_check(orc.orc_fr_partial_me(e_out, n, u, k, n, 1, exp, out_n))
    got = pv.partial_me(out, u, n, 1).host()
    assert got.shape[0] == out_n[0] == 1 and (got == exp[:1]).all()


@pytest.mark.parametrize("D,low,length", [(1000, -16, 32), (100000, -16, 32), (1 << 17, -20, 40), (1 << 18, -20, 40), (300000, -16, 32)])
def test_mapping_lookup_with_int32_forms(pv, orc, D, low, length):
    """tLookupRangeMapping with integer mapped values over queries that keep an int32 form: outputs, multiplicities and the
    proof's transcript are the oracle's.  1000 queries: padded in both forms, the small job reads the field elements; 100000:
    padded to 2^17 in the int32 form only (the job reads nothing else); 2^17: no padding; 2^18 and 300000 (padded to 2^19): the
    job's first two rounds run as one pass (k_lookup_first2_29)."""
    rng = np.random.default_rng(D + 1)
    vals = rng.integers(low, low + length, D)
    mvi = rng.integers(-2 ** 31, 2 ** 31, length).astype(np.int64)
    mvi[0], mvi[1] = -2 ** 31, 2 ** 31 - 1
    mv = fr_array([int(v) % R_MOD for v in mvi])
    S = fr_array([int(v) % R_MOD for v in vals])
    k = (D - 1).bit_length()
    r, alpha, beta, u, v = ch(7, 1)[0], ch(8, 1)[0], ch(9, 1)[0], ch(10, k), ch(11, k)
    size = 1 << (length - 1).bit_length()
    e_y, e_m, e_fin = np.zeros((D, 8), np.uint32), np.zeros((size, 8), np.uint32), np.zeros(8, np.uint32)
    orc.orc_transcript_clear()
    orc_check(orc.orc_mapping(S, D, low, length, mv, r, alpha, beta, u, v, e_y, e_m, e_fin))
    e_t = orc_transcript(orc)
    hS = pv.from_i64(vals.astype(np.int64))
    pv.keep_for_folds(hS)
    assert pv.folds_from_ints(hS) == 1
    pv.transcript_begin()
    y, m, fin = pv.mapping(hS, low, length, pv.from_fr(mv), r, alpha, beta, u, v)
    pv.lib.zkp_transcript_end()
    assert pv.folds_from_ints(y) == 1
    assert (y.host() == e_y).all() and (m.host() == e_m).all() and (fin == e_fin).all()
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()


@pytest.mark.parametrize("D,low,length", [(1 << 17, -(1 << 9), 1 << 10), (1 << 18, -(1 << 7), 1 << 8), (1 << 19, -(1 << 15), 1 << 16)])
def test_range_lookup_over_an_int32_form_against_the_oracle(pv, orc, D, low, length):
    """tLookupRange::prove over queries that keep an int32 form, at sizes where the job reads that form alone: 2^17 queries -- the
    first round on its own --, 2^18 and 2^19 -- the first two rounds in one pass.  Transcript and final claim are the oracle's."""
    rng = np.random.default_rng(D + length)
    vals = rng.integers(low, low + length, D)
    vals[:4] = [low, low + length - 1, low, low + length - 1]
    S = fr_array([int(v) % R_MOD for v in vals])
    k = (D - 1).bit_length()
    alpha, beta, u, v = ch(1, 1)[0], ch(2, 1)[0], ch(3, k), ch(4, k)
    orc.orc_transcript_clear()
    e_fin = np.zeros(8, np.uint32)
    orc_check(orc.orc_range_prove(S, D, low, length, alpha, beta, u, v, e_fin))
    e_t = orc_transcript(orc)
    hS = pv.from_i64(vals.astype(np.int64))
    pv.keep_for_folds(hS)
    assert pv.folds_from_ints(hS) == 1
    pv.transcript_begin()
    fin = pv.range_prove(hS, low, length, alpha, beta, u, v)
    pv.lib.zkp_transcript_end()
    assert (fin == e_fin).all()
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()


@pytest.mark.parametrize("n,sf", [(1 << 17, 1 << 8), (100000, 1 << 10), (1 << 18, 1 << 16)])
def test_rescaling_whose_remainders_exist_as_int32_only(pv, orc, n, sf):
    """Rescaling::lean: at these sizes the remainders' range proof reads their int32 form alone, so their field elements are never
    written (the pool is poisoned first); outputs and transcript are the oracle's.  100000: the proof pads that form to 2^17."""
    x = np.random.default_rng(n + sf).integers(-(1 << 40), 1 << 40, n)
    X = fr_array([int(v) % R_MOD for v in x])
    orc.orc_seed(98)
    orc.orc_transcript_clear()
    e_out = np.zeros_like(X)
    orc_check(orc.orc_rescale_prove(X, n, sf, e_out))
    e_t = orc_transcript(orc)
    junk = [pv.from_fr(ch(5, n)) for _ in range(3)]
    del junk
    pv.lib.zkp_rescale_set_lean(1)
    try:
        pv.seed(98)
        pv.transcript_begin()
        out = pv.rescale_prove(pv.from_fr(X), sf)
        pv.lib.zkp_transcript_end()
    finally:
        pv.lib.zkp_rescale_set_lean(0)
    assert (out.host() == e_out).all()
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()


def test_rescaling_prove_seeded_transcript(pv, orc, monkeypatch):
    """The proof's first entry, X(u), is formed from X_(u) and rem(u) (X = sf X_ + rem element by element); the oracle evaluates X
    itself, and so does the prover in the runs with ZKLLM_CHECK_CLAIMS=1, which throw if the two differ."""
    for n, sf, check in ((256, 16, False), (5000, 1 << 8, False), (256, 16, True), (70000, 1 << 8, True)):
        monkeypatch.delenv("ZKLLM_CHECK_CLAIMS", raising=False)
        if check:
            monkeypatch.setenv("ZKLLM_CHECK_CLAIMS", "1")
        x = np.random.default_rng(n).integers(-(1 << 30), 1 << 30, n)
        X = fr_array([int(v) % R_MOD for v in x])
        orc.orc_seed(99)
        orc.orc_transcript_clear()
        e_out = np.zeros_like(X)
        orc_check(orc.orc_rescale_prove(X, n, sf, e_out))
        e_t = orc_transcript(orc)
        pv.seed(99)
        pv.transcript_begin()
        out = pv.rescale_prove(pv.from_fr(X), sf)
        pv.lib.zkp_transcript_end()
        assert (out.host() == e_out).all()
        t = pv.transcript()
        assert t.shape == e_t.shape and (t == e_t).all()


@pytest.mark.parametrize("nX,n", [(1, 8), (1, 2048), (2, 16), (2, 4096), (2, 1 << 18), (3, 64), (3, 2048), (4, 32), (4, 2048)])
def test_multi_hadamard(pv, orc, nX, n):
    Xs = [ch(20 + i, n) for i in range(nX)]
    k = (n - 1).bit_length()
    u, v = ch(30, k), ch(31, k)
    prod = Xs[0].copy()
    tmp = np.zeros_like(prod)
    for x in Xs[1:]:
        orc_check(orc.orc_fr_op(7, prod, x, tmp, n))
        prod = tmp.copy()
    claim = np.zeros(8, np.uint32)
    orc_check(orc.orc_fr_me(prod, n, u, k, claim))
    e_proof, e_fin = np.zeros((k * (nX + 1), 8), np.uint32), np.zeros(8, np.uint32)
    orc_check(orc.orc_multi_hadamard(claim, np.ascontiguousarray(np.concatenate(Xs)), nX, n, u, v, k, e_proof, e_fin))
    proof, fin = pv.multi_hadamard(claim, [pv.from_fr(x) for x in Xs], u, v)
    assert (proof == e_proof).all() and (fin == e_fin).all()


@pytest.mark.parametrize("special", [1, 0])
def test_multi_hadamard_with_evaluation_challenges_of_one_and_zero(pv, orc, special):
    """The rounds of a sumcheck job read the first eq table's prefix and their weighted sums are multiplied by
    prod 1 / (1 - u_top) when they are collected; a challenge equal to 1 has no such constant (the job then writes every
    round's table), one equal to 0 makes half of the table zero.  Both against the oracle, 2^16 elements (the large-round
    kernels, the short rounds and the last-rounds kernel all take part)."""
    n, nX = 1 << 16, 2
    Xs = [ch(120 + i, n) for i in range(nX)]
    k = (n - 1).bit_length()
    u, v = ch(130, k), ch(131, k)
    for i in (3, k - 2, k - 1):
        u[i] = fr_array([special])[0]
    prod = np.zeros_like(Xs[0])
    orc_check(orc.orc_fr_op(7, Xs[0], Xs[1], prod, n))
    claim = np.zeros(8, np.uint32)
    orc_check(orc.orc_fr_me(prod, n, u, k, claim))
    e_proof, e_fin = np.zeros((k * (nX + 1), 8), np.uint32), np.zeros(8, np.uint32)
    orc_check(orc.orc_multi_hadamard(claim, np.ascontiguousarray(np.concatenate(Xs)), nX, n, u, v, k, e_proof, e_fin))
    proof, fin = pv.multi_hadamard(claim, [pv.from_fr(x) for x in Xs], u, v)
    assert (proof == e_proof).all() and (fin == e_fin).all()


@pytest.mark.parametrize("n,kept", [(4096, (True, True)), (1 << 17, (True, True)), (1 << 17, (True, False)), (1 << 15, (False, True))])
def test_multi_hadamard_of_two_tensors_that_keep_an_int32_form(pv, orc, n, kept):
    """Two tensors of 32-bit integers, the extremes included, kept for folds: the job's first round reads their int32 forms
    (k_hadamard_round2_ints: exact 64-bit products weighted into unreduced twelve-limb sums) and the proof is the oracle's;
    with only one of them kept the plain round runs."""
    rng = np.random.default_rng(n + 7 * kept[0] + 3 * kept[1])
    Ws = [rng.integers(-2 ** 31, 2 ** 31, n).astype(np.int64) for _ in range(2)]
    half = n // 2
    for W in Ws:
        W[0], W[half] = -2 ** 31, 2 ** 31 - 1                  # the widest difference of a pair, both signs
        W[1], W[1 + half] = 2 ** 31 - 1, -2 ** 31
        W[2], W[2 + half] = -2 ** 31, -2 ** 31
        W[3] = 0
    Xs = [fr_array([int(v) % R_MOD for v in W]) for W in Ws]
    k = (n - 1).bit_length()
    u, v = ch(32, k), ch(33, k)
    prod = np.zeros_like(Xs[0])
    orc_check(orc.orc_fr_op(7, Xs[0], Xs[1], prod, n))
    claim = np.zeros(8, np.uint32)
    orc_check(orc.orc_fr_me(prod, n, u, k, claim))
    e_proof, e_fin = np.zeros((k * 3, 8), np.uint32), np.zeros(8, np.uint32)
    orc_check(orc.orc_multi_hadamard(claim, np.ascontiguousarray(np.concatenate(Xs)), 2, n, u, v, k, e_proof, e_fin))
    hs = [pv.from_i64(W) for W in Ws]
    for h, kp in zip(hs, kept):
        if kp:
            pv.keep_for_folds(h)
            assert pv.folds_from_ints(h) == 1
    proof, fin = pv.multi_hadamard(claim, hs, u, v)
    assert (proof == e_proof).all() and (fin == e_fin).all()


# 70001: several workgroups per round and odd lengths on the way down (70001, 35001, 17501, 8751, 4376, ...)
@pytest.mark.parametrize("n", [2, 3, 5, 64, 1000, 70001])
def test_deprecated_hadamard_product_sumcheck(pv, orc, n):
    a, b = ch(40, n), ch(41, n)
    k = (n - 1).bit_length()
    u, v = ch(42, k), ch(43, k)
    exp = np.zeros((3 * k + 2, 8), np.uint32)
    orc_check(orc.orc_hadamard_product_sumcheck(a, b, n, u, v, k, exp))
    got = pv.hadamard_product_sumcheck(pv.from_fr(a), pv.from_fr(b), u, v)
    assert (got == exp).all()


@pytest.mark.parametrize("n", [2, 3, 5, 64, 1000, 70001])
def test_deprecated_inner_product_sumcheck(pv, orc, n):
    a, b = ch(44, n), ch(45, n)
    k = (n - 1).bit_length()
    u = ch(46, k)
    exp = np.zeros((3 * k + 2, 8), np.uint32)
    orc_check(orc.orc_inner_product_sumcheck(a, b, n, u, k, exp))
    got = pv.inner_product_sumcheck(pv.from_fr(a), pv.from_fr(b), u)
    assert (got == exp).all()


@pytest.mark.parametrize("n", [2, 3, 5, 64, 1000, 70001])
def test_deprecated_binary_sumcheck(pv, orc, n):
    a = ch(47, n)
    k = (n - 1).bit_length()
    u, v = ch(48, k), ch(49, k)
    exp = np.zeros((3 * k + 1, 8), np.uint32)
    orc_check(orc.orc_binary_sumcheck(a, n, u, v, k, exp))
    got = pv.binary_sumcheck(pv.from_fr(a), u, v)
    assert (got == exp).all()


def test_deprecated_sumchecks_reject_sizes_out_of_range(pv):
    a = pv.from_fr(ch(47, 4))
    with pytest.raises(RuntimeError, match="Incompatible dimensions"):
        pv.inner_product_sumcheck(a, a, ch(46, 3))
    with pytest.raises(RuntimeError, match="Incompatible dimensions"):
        pv.inner_product_sumcheck(a, pv.from_fr(ch(47, 3)), ch(46, 2))
    with pytest.raises(RuntimeError, match="Incompatible dimensions"):
        pv.binary_sumcheck(a, ch(46, 1), ch(48, 1))


@pytest.mark.parametrize("N,D", [(2, 4), (4, 16), (3, 8), (32, 128)])
def test_zkip_stacked(pv, orc, N, D):
    A, B = ch(50, N * D), ch(51, N * D)
    kN, kD = (N - 1).bit_length(), (D - 1).bit_length()
    uN, vN, uD = ch(52, kN), ch(53, kN), ch(54, kD)
    # claim = sum_n eq(uN, n) <A_n, B_n>
    per = np.zeros((N, 8), np.uint32)
    tmp = np.zeros((D, 8), np.uint32)
    for i in range(N):
        orc_check(orc.orc_fr_op(7, A[i * D:(i + 1) * D].copy(), B[i * D:(i + 1) * D].copy(), tmp, D))
        orc_check(orc.orc_fr_sum(tmp, D, per[i]))
    claim = np.zeros(8, np.uint32)
    orc_check(orc.orc_fr_me(per, N, uN, kN, claim))
    e_proof, e_fin = np.zeros((kN + kD, 3, 8), np.uint32), np.zeros(8, np.uint32)
    orc_check(orc.orc_zkip_stacked(claim, A, B, N, D, uN, vN, kN, uD, kD, e_proof, e_fin))
    proof, fin = pv.zkip_stacked(claim, pv.from_fr(A), pv.from_fr(B), N, D, uN, vN, uD)
    assert (proof == e_proof).all() and (fin == e_fin).all()


@pytest.mark.parametrize("m,n,d,bs,sf,lim", [(16, 16, 16, [16, 16, 16], 256, 200), (64, 64, 32, [1 << 4, 1 << 6, 1 << 6], 1 << 10, 4000), (7, 64, 8, [1 << 3, 1 << 6, 1 << 6], 1 << 9, 1000)])
def test_softmax_compute_and_prove(pv, orc, m, n, d, bs, sf, lim):
    rng = np.random.default_rng(m * n)
    X = rng.integers(-lim, lim, (m, n))
    Xf = fr_array([int(x) % R_MOD for x in X.reshape(-1)])
    thetas = np.array([float(1 << 10), float(1 << 12)])
    bsa = np.array(bs, np.uint32)
    prove = ((m * n) & (m * n - 1)) == 0
    e_Y, e_shift = np.zeros((m * n, 8), np.uint32), np.zeros((m, 8), np.uint32)
    orc.orc_seed(5)
    orc.orc_transcript_clear()
    orc_check(orc.orc_softmax(Xf, m, n, d, bsa, 3, 1, 0, sf, thetas, 2, e_Y, e_shift, 1 if prove else 0))
    e_t = orc_transcript(orc)
    pv.seed(5)
    pv.transcript_begin()
    Y, shift = pv.softmax(pv.from_fr(Xf), m, n, d, bsa, 1, 0, sf, thetas, prove)
    pv.lib.zkp_transcript_end()
    assert (shift.host() == e_shift).all()
    assert (Y.host() == e_Y).all()
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()


@pytest.mark.parametrize("num,stacked,m,n,d", [(1, 0, 16, 16, 16), (1, 1, 16, 16, 16), (4, 1, 16, 16, 16), (2, 1, 8, 32, 4), (2, 1, 256, 256, 4), (2, 2, 256, 256, 4),
                                               (4, 2, 16, 16, 16), (2, 1, 8, 16, 8)])
def test_attention_forward_and_proof(pv, orc, monkeypatch, num, stacked, m, n, d):
    """zkAttn (one head) and zkAttnStacked (head-major stacks): forward pass, transcript and returned claim.  stacked == 2:
    zkSoftmax::lean_forward -- at 2 x 256 x 256 scores the lookup and Hadamard jobs read int32 forms alone, so the digit planes
    and the mapped values exist in that form only and the shifted scores are never written (at 4 x 16 x 16 nothing is large
    enough for that and the switch changes nothing)."""
    rng = np.random.default_rng(num * 1000 + m + n + d)
    qmax = 3 if d == 16 else 6
    Q, K, V = (fr_array([int(x) % R_MOD for x in rng.integers(-qmax, qmax + 1, num * r * d)]) for r in (m, n, n))
    bs = np.array([16, 16, 16], np.uint32)
    thetas = np.array([float(1 << 10), float(1 << 12)])
    e_out, e_fin = np.zeros((num * m * d, 8), np.uint32), np.zeros(8, np.uint32)
    orc.orc_seed(11)
    orc.orc_transcript_clear()
    orc_check(orc.orc_attn(Q, K, V, num, m, n, d, 1 if stacked else 0, bs, 3, 1, 0, c_u64(16), c_u64(16), thetas, 2, e_out, e_fin))
    e_t = orc_transcript(orc)
    # The stacked proof takes the scores' value at the softmax's point from the folded Q and K instead of reading the scores;
    # the second run (ZKLLM_CHECK_CLAIMS=1) evaluates the scores as well and throws if the two differ.
    # The third run of the lean variant lowers the matrix-core threshold so that the scores are written as 64-bit integers only
    # (zk_fr_matmul_batched_i64 -> zk_softmax_shift_decompose_i64; sm_in stays unwritten).
    # The fourth run writes the softmax's output as a tensor (ZKLLM_SOFTMAX_PRODUCT=0) instead of leaving it the product of its
    # two factors: the same bytes either way.
    for check in ((False, True, "i64", "written") if stacked == 2 else (False, True) if stacked else (False,)):
        monkeypatch.delenv("ZKLLM_CHECK_CLAIMS", raising=False)
        monkeypatch.delenv("ZKLLM_MATMUL_PLANES", raising=False)
        monkeypatch.delenv("ZKLLM_SOFTMAX_PRODUCT", raising=False)
        monkeypatch.delenv("ZKLLM_SCORES_I64", raising=False)
        if check == "written":
            monkeypatch.setenv("ZKLLM_SOFTMAX_PRODUCT", "0")
        if check is True:
            monkeypatch.setenv("ZKLLM_CHECK_CLAIMS", "1")
        if check == "i64":
            monkeypatch.setenv("ZKLLM_MATMUL_PLANES", "1")
        pv.seed(11)
        pv.transcript_begin()
        if stacked == 2:          # poison what the pool hands out next: tensors that stay unwritten must not be read
            junk = [pv.from_fr(ch(7, num * m * n)) for _ in range(6)]
            del junk
        out, fin = pv.attn(pv.from_fr(Q), pv.from_fr(K), pv.from_fr(V), num, m, n, d, stacked, bs, 1, 0, 16, 16, thetas)
        pv.lib.zkp_transcript_end()
        assert (out.host() == e_out).all() and (fin == e_fin).all()
        t = pv.transcript()
        assert t.shape == e_t.shape and (t == e_t).all()
        if stacked:          # three digit planes and two mapped-value tensors
            assert pv.lib.zkp_softmax_lean_tensors_last() == (5 if stacked == 2 and num * m * n >= 1 << 17 else 0)
            assert pv.lib.zkp_softmax_scores_i64_last() == (1 if check == "i64" and m >= 32 and n >= 32 else 0)


@pytest.mark.parametrize("num,batch,n_in,n_out,bias", [(1, 4, 8, 8, False), (4, 8, 16, 4, False), (4, 8, 16, 4, True), (3, 5, 6, 7, True)])
def test_stacked_fully_connected_proof(pv, orc, num, batch, n_in, n_out, bias):
    rng = np.random.default_rng(num + batch + n_in + n_out)
    X = fr_array([int(x) % R_MOD for x in rng.integers(-1000, 1000, num * batch * n_in)])
    W = fr_array([int(x) % R_MOD for x in rng.integers(-1000, 1000, num * n_in * n_out)])
    b = fr_array([int(x) % R_MOD for x in rng.integers(-10 ** 6, 10 ** 6, num * n_out)]) if bias else None
    e_Y = np.zeros((num * batch * n_out, 8), np.uint32)
    orc.orc_seed(12)
    orc.orc_transcript_clear()
    orc_check(orc.orc_zkfc_stacked(X, W, b, num, batch, n_in, n_out, e_Y))
    e_t = orc_transcript(orc)
    pv.seed(12)
    pv.transcript_begin()
    Y = pv.zkfc_stacked(pv.from_fr(X), pv.from_fr(W), pv.from_fr(b) if bias else None, num, batch, n_in, n_out)
    pv.lib.zkp_transcript_end()
    assert (Y.host() == e_Y).all()
    t = pv.transcript()
    assert t.shape == e_t.shape and (t == e_t).all()


@pytest.mark.parametrize("k", [13, 17])
def test_hinted_lookup_job_equals_the_plain_one_whatever_the_hints(k):
    """zk_lookup_prove_begin_hinted reads 1/(S+beta) from the table's inverses where the hinted entry matches and must
    deliver what zk_lookup_prove_begin delivers for every input: right hints, wrong hints, hints outside the table,
    queries that are no table entry at all, a query with S + beta == 0 and a table entry with T + beta == 0 (pairs of
    matched invertible entries take a shortcut through (a0 + a1)(s0 + s1); every other pair must not).  2^13 queries: the inverses are written out
    before the first round; 2^17: the first round computes them on the fly."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    D, N, low = 1 << k, 64, -7
    rng = np.random.default_rng(99)
    T = ch(41, N)                                   # arbitrary table entries
    beta = ch(43, 1)[0]
    T[3] = fr_array([(-fr_ints(beta.reshape(1, 8))[0]) % R_MOD])[0]     # a table entry with T + beta == 0: its "inverse" is 0, not a unit
    pos = rng.integers(0, N, D)
    S = T[pos].copy()
    hint_int = (pos + low).astype(np.int64)         # right hints: hint - low == position
    wrong = rng.choice(D, 300, replace=False)
    hint_int[wrong[:100]] = (pos[wrong[:100]] + 1) % N + low          # another entry of the table
    hint_int[wrong[100:200]] = low + N + 5                            # outside the table
    S[wrong[200:]] = ch(42, 100)                                      # queries that are no table entries
    S[wrong[7]] = fr_array([(-fr_ints(beta.reshape(1, 8))[0]) % R_MOD])[0]
    hint = fr_array([int(x) % R_MOD for x in hint_int])
    m = fr_array([int(c) for c in np.bincount(pos, minlength=N)])
    u, v = ch(44, k - 1), ch(45, k)
    dS, dT, dm, dh = hip.upload(S), hip.upload(T), hip.upload(m), hip.upload(hint)
    res = []
    for hinted in (False, True):
        h = c_void_p()
        if hinted:
            hip.call("zk_lookup_prove_begin_hinted", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), c_void_p(dh), c_int(low), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        else:
            hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
        hip.call("zk_lookup_prove_end", h, bm, sums)
        res.append((bm, sums))
    assert (res[0][0] == res[1][0]).all() and (res[0][1] == res[1][1]).all()
    assert res[0][1].any()
    for p in (dS, dT, dm, dh):
        hip.free(p)


def test_jobs_launched_by_the_library_thread_equal_those_launched_by_the_caller():
    """zk_set_async_jobs: with it on, begin hands a job's launches to the library's launch thread and returns; off, the caller
    queues them itself.  Four lookup jobs and two Hadamard jobs begun back to back (more jobs than streams of that kind, so
    some share a stream) and ended in another order deliver the same sums both ways; the challenge arrays handed to begin are
    overwritten right after the call, which the jobs must not notice."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    assert hip.lib.zk_async_jobs() == 1
    k, N, low = 16, 256, -100
    D = 1 << k
    rng = np.random.default_rng(5)
    T = fr_array([(low + j) % R_MOD for j in range(N)])
    dT = hip.upload(T)
    jobs = []
    for j in range(4):
        pos = rng.integers(0, N, D)
        S = T[pos].copy()
        m = fr_array([int(c) for c in np.bincount(pos, minlength=N)])
        jobs.append((hip.upload(S), hip.upload(m), ch(60 + j, 1)[0], ch(70 + j, k - 1), ch(80 + j, k)))
    Xs = [hip.upload(ch(90 + j, D)) for j in range(4)]
    res = {}
    try:
        for mode in (1, 0, 1):
            hip.call("zk_set_async_jobs", c_int(mode))
            hs = []
            for j, (dS, dm, beta, u, v) in enumerate(jobs):
                h = c_void_p()
                beta_, u_, v_ = beta.copy(), u.copy(), v.copy()
                if j % 2:
                    hip.call("zk_lookup_prove_begin_hinted", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), c_void_p(dS), c_int(low), beta_, u_, v_, c_size_t(D), c_size_t(N), c_int(k), None)
                else:
                    hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), beta_, u_, v_, c_size_t(D), c_size_t(N), c_int(k), None)
                beta_[:] = 0xFFFFFFFF; u_[:] = 0xFFFFFFFF; v_[:] = 0xFFFFFFFF
                hs.append(h)
            hh = []
            for j in range(2):
                h = c_void_p()
                ptrs = (ctypes.c_void_p * 2)(Xs[2 * j], Xs[2 * j + 1])
                u_, v_ = ch(95 + j, k - 1), ch(97 + j, k)
                hip.call("zk_hadamard_prove_begin", ctypes.byref(h), ptrs, c_int(2), u_, v_, c_size_t(D), None)
                u_[:] = 0xFFFFFFFF; v_[:] = 0xFFFFFFFF
                hh.append(h)
            out = []
            for h in reversed(hh):
                coefs = np.zeros((k * 3, 8), np.uint32)
                hip.call("zk_hadamard_prove_end", h, coefs)
                out.append(coefs)
            for h in reversed(hs):
                bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
                hip.call("zk_lookup_prove_end", h, bm, sums)
                out.append(bm)
                out.append(sums)
            if mode in res:
                assert all((a == b).all() for a, b in zip(res[mode], out))
            res[mode] = out
    finally:
        hip.call("zk_set_async_jobs", c_int(1))
    assert len(res[0]) == len(res[1]) and all((a == b).all() for a, b in zip(res[0], res[1]))
    assert all(a.any() for a in res[0])
    for dS, dm, *_ in jobs:
        hip.free(dS); hip.free(dm)
    for p in Xs + [dT]:
        hip.free(p)


@pytest.mark.parametrize("k", [13, 17])
def test_mapped_lookup_job_equals_the_plain_one_on_the_combined_queries(k):
    """zk_lookup_prove_begin_mapped forms S_in + r * S_out itself (2^13 queries: written out first; 2^17: inside the first
    round) and must deliver what zk_lookup_prove_begin delivers on the combined queries computed here with big integers,
    also where an input is outside the table, an output is not the mapped value, or a combined query is -beta."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    D, N, low = 1 << k, 64, -9
    rng = np.random.default_rng(k)
    mapped = fr_ints(ch(51, N))
    r_fr, beta = ch(52, 1)[0], ch(53, 1)[0]
    r, b = fr_ints(r_fr.reshape(1, 8))[0], fr_ints(beta.reshape(1, 8))[0]
    pos = rng.integers(0, N, D)
    s_in = [(int(p) + low) % R_MOD for p in pos]
    s_out = [mapped[int(p)] for p in pos]
    odd = rng.choice(D, 200, replace=False)
    for i in odd[:100]:
        s_out[i] = (s_out[i] + 1 + int(i)) % R_MOD           # not the mapped value
    for i in odd[100:199]:
        s_in[i] = (low + N + 3 + int(i)) % R_MOD             # outside the table
    i0 = int(odd[199])
    s_out[i0] = ((-b - s_in[i0]) * pow(r, -1, R_MOD)) % R_MOD    # combined query + beta == 0
    T = fr_array([((low + j) + r * mapped[j]) % R_MOD for j in range(N)])
    S_com = fr_array([(a + r * o) % R_MOD for a, o in zip(s_in, s_out)])
    m = fr_array([int(c) for c in np.bincount(pos, minlength=N)])
    u, v = ch(54, k - 1), ch(55, k)
    dS, dT, dm, dSi, dSo = hip.upload(S_com), hip.upload(T), hip.upload(m), hip.upload(fr_array(s_in)), hip.upload(fr_array(s_out))
    res = []
    for mapped_job in (False, True):
        h = c_void_p()
        if mapped_job:
            hip.call("zk_lookup_prove_begin_mapped", ctypes.byref(h), c_void_p(dSi), c_void_p(dSo), r_fr, c_void_p(dT), c_void_p(dm), c_int(low), beta, u, v,
                     c_size_t(D), c_size_t(N), c_int(k), None)
        else:
            hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
        hip.call("zk_lookup_prove_end", h, bm, sums)
        res.append((bm, sums))
    assert (res[0][0] == res[1][0]).all() and (res[0][1] == res[1][1]).all()
    assert res[0][1].any()
    for p in (dS, dT, dm, dSi, dSo):
        hip.free(p)


@pytest.mark.parametrize("k,bad_entry", [(17, False), (17, True), (13, False), (19, False), (19, True)])
def test_mapped_lookup_over_outputs_gathered_by_their_queries(k, bad_entry):
    """Outputs made by zk_fr_gather_by_queries_ints carry where they came from; a mapped job over the same queries, outputs and
    table then reads neither outputs nor per-entry integers for queries inside the table.  Checked against the plain job on
    the combined queries (big integers), with queries outside the table (their output is entry 0's value and must be read),
    and with one table entry that is not what the integers say (the job falls back to checking every query)."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    D, N, low = 1 << k, 64, -9
    rng = np.random.default_rng(2000 + k + bad_entry)
    mapped = [int(x) for x in rng.integers(-2 ** 31, 2 ** 31, N)]
    r_fr, beta = ch(82, 1)[0], ch(83, 1)[0]
    r = fr_ints(r_fr.reshape(1, 8))[0]
    pos = rng.integers(0, N, D)
    s_in = [int(p) + low for p in pos]
    outside = rng.choice(D, 200, replace=False)
    for i in outside[:100]:
        s_in[i] = low + N + 1 + int(i % 1000)
    for i in outside[100:]:
        s_in[i] = low - 1 - int(i % 1000)
    dSi = hip.upload(fr_array([x % R_MOD for x in s_in]))
    dMp = hip.upload(fr_array([x % R_MOD for x in mapped]))
    hq, hm = c_void_p(), c_void_p()
    hip.call("zk_fr_fold_prepare", ctypes.byref(hq), c_void_p(dSi), c_size_t(D), None)
    hip.call("zk_fr_fold_prepare", ctypes.byref(hm), c_void_p(dMp), c_size_t(N), None)
    dSo = hip.malloc(32 * D)
    ho, hoq = c_void_p(), c_void_p()
    hip.call("zk_fr_fold_prepared_new", ctypes.byref(ho), ctypes.byref(hoq), c_size_t(D), None)
    hip.call("zk_fr_gather_by_queries_ints", c_void_p(dSo), ho, hq, c_int(low), hm, c_size_t(D), None)
    s_out = [mapped[x - low] if 0 <= x - low < N else mapped[0] for x in s_in]
    assert fr_ints(hip.download(dSo, (D, 8), np.uint32)) == [x % R_MOD for x in s_out]
    assert (hip.download(hoq.value, (D,), np.int32) == np.array(s_out)).all()
    Tl = [((low + j) + r * mapped[j]) % R_MOD for j in range(N)]
    if bad_entry:
        Tl[17] = (Tl[17] + 3) % R_MOD
    S_com = fr_array([(a + r * o) % R_MOD for a, o in zip(s_in, s_out)])
    index_of = {}
    for j, t in enumerate(Tl):
        index_of.setdefault(t, j)
    m_counts = np.zeros(N, np.int64)
    for q in fr_ints(S_com):
        if q in index_of:
            m_counts[index_of[q]] += 1
    dS, dT, dm = hip.upload(S_com), hip.upload(fr_array(Tl)), hip.upload(fr_array([int(c) for c in m_counts]))
    u, v = ch(84, k - 1), ch(85, k)
    res = []
    for job in ("plain", "mapped_ints"):
        h = c_void_p()
        if job == "plain":
            hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        else:
            hip.call("zk_lookup_prove_begin_mapped_ints", ctypes.byref(h), c_void_p(dSi), hq, c_void_p(dSo), ho, hm, r_fr, c_void_p(dT), c_void_p(dm), c_int(low),
                     beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
        hip.call("zk_lookup_prove_end", h, bm, sums)
        res.append((bm, sums))
        n_ok, n_tab = ctypes.c_uint32(7), ctypes.c_uint32(7)
        hip.call("zk_lookup_last_job_consistent_entries", ctypes.byref(n_ok), ctypes.byref(n_tab))
        # the entries below the first inconsistent one serve their queries from the table record alone
        assert (n_ok.value, n_tab.value) == ((0, 0) if job == "plain" else ((17 if bad_entry else N), N))
    assert (res[0][0] == res[1][0]).all() and (res[0][1] == res[1][1]).all()
    assert res[0][1].any()
    # The queries' int32 form written again and declared so (zk_fr_fold_prepared_touch): the outputs no longer count as gathered
    # by these queries, every query is compared on its own, and the job equals the plain job on the new combined queries.
    if not bad_entry:
        s_in2 = list(s_in)
        for i in range(0, D, 3):
            s_in2[i] = low + (s_in[i] - low + 1) % N if 0 <= s_in[i] - low < N else s_in[i]
        hip.lib.zk_fr_fold_prepared_ints.restype = ctypes.c_void_p
        q_ints = hip.lib.zk_fr_fold_prepared_ints(hq)
        new_ints = hip.upload(np.array(s_in2, np.int32))
        hip.lib.zk_memcpy_d2d(c_void_p(q_ints), c_void_p(new_ints), c_size_t(4 * D), None)
        hip.call("zk_fr_fold_prepared_touch", hq)
        dSi2 = hip.upload(fr_array([x % R_MOD for x in s_in2]))
        S2 = [(a + r * o) % R_MOD for a, o in zip(s_in2, s_out)]
        m2 = np.zeros(N, np.int64)
        for q in S2:
            if q in index_of:
                m2[index_of[q]] += 1
        dS2, dm2 = hip.upload(fr_array(S2)), hip.upload(fr_array([int(c) for c in m2]))
        res2 = []
        for job in ("plain", "mapped_ints"):
            h = c_void_p()
            if job == "plain":
                hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dS2), c_void_p(dT), c_void_p(dm2), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
            else:
                hip.call("zk_lookup_prove_begin_mapped_ints", ctypes.byref(h), c_void_p(dSi2), hq, c_void_p(dSo), ho, hm, r_fr, c_void_p(dT), c_void_p(dm2), c_int(low),
                         beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
            bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
            hip.call("zk_lookup_prove_end", h, bm, sums)
            res2.append((bm, sums))
        assert (res2[0][0] == res2[1][0]).all() and (res2[0][1] == res2[1][1]).all()
        assert not (res2[0][1] == res[0][1]).all()
        for q in (new_ints, dSi2, dS2, dm2):
            hip.free(q)
    for h in (hq, hm, ho):
        hip.call("zk_fr_fold_prepared_free", h)
    for q in (dSi, dMp, dSo, dS, dT, dm):
        hip.free(q)


@pytest.mark.parametrize("k,length", [(17, 48), (17, 64), (13, 37), (19, 48), (18, 64)])
def test_range_table_padded_by_repeating_its_last_value_keeps_the_short_first_round(k, length):
    """A range table of `length` entries padded to 64 by repeating its last value (zk_range_table): the entries below `length` are
    what the integers say and serve their queries from the table record alone (zk_lookup_last_job_consistent_entries reports
    `length`), queries that name a padding position or lie outside are compared on their own; the job equals the plain one."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int, c_uint
    hip = Hip()
    D, N, low = 1 << k, 64, -11
    rng = np.random.default_rng(3000 + k + length)
    dT = hip.malloc(32 * N)
    hip.call("zk_range_table", c_void_p(dT), c_int(low), c_uint(length), c_uint(N), None)
    Tl = fr_ints(hip.download(dT, (N, 8), np.uint32))
    assert Tl == [(low + min(j, length - 1)) % R_MOD for j in range(N)]
    s_in = [int(x) + low for x in rng.integers(0, length, D)]
    odd = rng.choice(D, 120, replace=False)
    for i in odd[:60]:
        s_in[i] = low + length + int(i % max(1, N - length)) if length < N else low + N + 2      # a padding position (no table value) / above the table
    for i in odd[60:]:
        s_in[i] = low - 1 - int(i % 50)
    index_of = {}
    for j, t in enumerate(Tl):
        index_of.setdefault(t, j)
    m_counts = np.zeros(N, np.int64)
    for q in s_in:
        if q % R_MOD in index_of:
            m_counts[index_of[q % R_MOD]] += 1
    dS, dm = hip.upload(fr_array([x % R_MOD for x in s_in])), hip.upload(fr_array([int(c) for c in m_counts]))
    hq = c_void_p()
    hip.call("zk_fr_fold_prepare", ctypes.byref(hq), c_void_p(dS), c_size_t(D), None)
    beta, u, v = ch(91, 1)[0], ch(92, k - 1), ch(93, k)
    res = []
    for job in ("plain", "hinted_ints"):
        h = c_void_p()
        if job == "plain":
            hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        else:
            hip.call("zk_lookup_prove_begin_hinted_ints", ctypes.byref(h), c_void_p(dS), hq, c_void_p(dT), c_void_p(dm), c_int(low), beta, u, v,
                     c_size_t(D), c_size_t(N), c_int(k), None)
        bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
        hip.call("zk_lookup_prove_end", h, bm, sums)
        res.append((bm, sums))
    n_ok, n_tab = ctypes.c_uint32(), ctypes.c_uint32()
    hip.call("zk_lookup_last_job_consistent_entries", ctypes.byref(n_ok), ctypes.byref(n_tab))
    assert (n_ok.value, n_tab.value) == (length, N)
    assert (res[0][0] == res[1][0]).all() and (res[0][1] == res[1][1]).all() and res[0][1].any()
    hip.call("zk_fr_fold_prepared_free", hq)
    for q in (dT, dS, dm):
        hip.free(q)


@pytest.mark.parametrize("k,n", [(16, 1 << 16), (17, 70001), (19, (1 << 19) - 3)])
def test_evaluations_that_never_build_the_points_eq_table_against_big_integers(k, n):
    """From 2^16 positions on zk_fr_me_multi / zk_fr_me_multi_ints evaluate through the two half tables of the point (a lane
    multiplies its elements by the high half's entry, sums unreduced, and multiplies by the low half's entry once): field
    elements through 29-bit-limb sums, int32 forms through 32-bit ones.  Checked against sum_t X[t] eq(u, t) in Python integers
    for full and ragged lengths, with the extreme values of both kinds of element present."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    rng = np.random.default_rng(k)
    u = ch(300 + k, k)
    ui = fr_ints(u)
    E = [1]
    for j in range(k):
        E = [e * (1 - ui[j]) % R_MOD for e in E] + [e * ui[j] % R_MOD for e in E]
    frs = [ch(310 + i, n) for i in range(3)]
    frs[0][0] = fr_array([R_MOD - 1])[0]
    frs[0][1] = fr_array([0])[0]
    frs[1][n - 1] = fr_array([R_MOD - 1])[0]
    ints = [rng.integers(-2 ** 31, 2 ** 31, n) for _ in range(5)]
    ints[0][:4] = [-2 ** 31, 2 ** 31 - 1, 0, -1]
    ints[1][:] = -2 ** 31                                  # every term at the largest magnitude
    ints[2][:] = 2 ** 31 - 1
    want_fr = [sum(int(x) * e for x, e in zip(fr_ints(f), E)) % R_MOD for f in frs]
    want_int = [sum(int(x) * e for x, e in zip(v, E)) % R_MOD for v in ints]
    d_fr = [hip.upload(f) for f in frs]
    d_int = [hip.upload(fr_array([int(x) % R_MOD for x in v])) for v in ints]
    hs = []
    for d in d_int:
        h = c_void_p()
        hip.call("zk_fr_fold_prepare", ctypes.byref(h), c_void_p(d), c_size_t(n), None)
        hs.append(h)
    junk = hip.upload(ch(320, n))

    def run(fr_idx, int_idx):
        K = len(fr_idx) + len(int_idx)
        ptrs = [c_void_p(d_fr[i]) for i in fr_idx] + [c_void_p(junk)] * len(int_idx)
        preps = [c_void_p(None)] * len(fr_idx) + [hs[i] for i in int_idx]
        got = np.zeros((K, 8), np.uint32)
        hip.call("zk_fr_me_multi_ints", got, (c_void_p * K)(*ptrs), (c_void_p * K)(*preps), c_int(K), c_size_t(n), u, c_int(k), None)
        exp = fr_array([want_fr[i] for i in fr_idx] + [want_int[i] for i in int_idx])
        assert (got == exp).all(), (fr_idx, int_idx)

    run([0, 1, 2], [0, 1, 2, 3, 4])       # one tensor of field elements with five forms, then two tensors of field elements
    run([0, 1], [0, 1, 2])                # two and three in one pass
    run([2], [4])
    run([], [3])
    run([], [0, 1, 2, 3, 4, 0])           # six forms in one pass
    got = np.zeros((3, 8), np.uint32)
    hip.call("zk_fr_me_multi", got, (c_void_p * 3)(*[c_void_p(d) for d in d_fr]), c_int(3), c_size_t(n), u, c_int(k), None)
    assert (got == fr_array(want_fr)).all()
    for h in hs:
        hip.call("zk_fr_fold_prepared_free", h)
    for d in d_fr + d_int + [junk]:
        hip.free(d)


def test_evaluations_of_eight_tensors_that_keep_only_their_int32_form():
    """zk_fr_me_multi_ints with eight int32 forms: every one is evaluated from that form (six, then two), never from the field
    elements passed beside it -- which hold other values here, as a tensor that keeps only its int32 form does."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    n, k = 5000, 13
    rng = np.random.default_rng(77)
    vals = [rng.integers(-2 ** 31, 2 ** 31, n) for _ in range(8)]
    devs = [hip.upload(fr_array([int(x) % R_MOD for x in v])) for v in vals]
    hs = []
    for d in devs:
        h = c_void_p()
        hip.call("zk_fr_fold_prepare", ctypes.byref(h), c_void_p(d), c_size_t(n), None)
        hs.append(h)
    junk = hip.upload(ch(78, n))
    u = ch(79, k)
    exp, got = np.zeros((8, 8), np.uint32), np.zeros((8, 8), np.uint32)
    hip.call("zk_fr_me_multi", exp, (c_void_p * 8)(*[c_void_p(d) for d in devs]), c_int(8), c_size_t(n), u, c_int(k), None)
    hip.call("zk_fr_me_multi_ints", got, (c_void_p * 8)(*[c_void_p(junk)] * 8), (c_void_p * 8)(*hs), c_int(8), c_size_t(n), u, c_int(k), None)
    assert (got == exp).all() and len({tuple(r) for r in exp}) == 8
    # seven forms and one tensor of field elements in the middle
    mixed_ptrs = [c_void_p(junk)] * 8
    mixed_ptrs[3] = c_void_p(devs[3])
    mixed_hs = list(hs)
    mixed_hs[3] = c_void_p(None)
    got2 = np.zeros((8, 8), np.uint32)
    hip.call("zk_fr_me_multi_ints", got2, (c_void_p * 8)(*mixed_ptrs), (c_void_p * 8)(*mixed_hs), c_int(8), c_size_t(n), u, c_int(k), None)
    assert (got2 == exp).all()
    for h in hs:
        hip.call("zk_fr_fold_prepared_free", h)
    for d in devs + [junk]:
        hip.free(d)


@pytest.mark.parametrize("radices", [(256, 1 << 20, 1 << 20), (100, 1000003, 999983), (7, 1 << 20, 65537)])
@pytest.mark.parametrize("rows,cols", [(5, 64), (37, 200), (64, 2048)])
def test_softmax_shift_and_decomposition_in_one_pass_equal_the_two_passes(rows, cols, radices):
    """zk_softmax_shift_decompose against zk_softmax_shift followed by zk_softmax_decompose_ints: the same shifts, shifted
    scores, digit planes and int32 planes (ragged rows: 200 columns are three full wave steps and a partial one).  The one pass
    forms the digits from 64-bit integers (a radix that is a power of two by mask and shift, any other by division), the two
    passes from the field elements; radices of both kinds, mixed.  The scores as 64-bit integers
    (zk_softmax_shift_decompose_i64) give the same again, and the digits recombine to the negated shifted scores."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    from ctypes import c_uint, c_double
    hip = Hip()
    rng = np.random.default_rng(rows * 1000 + cols)
    n = rows * cols
    scale = 65536.0 * 8.0
    X = rng.integers(-(1 << 22), 1 << 22, n).astype(np.int64)
    dX = hip.upload(fr_array([int(v) % R_MOD for v in X]))
    bs = np.array(radices, dtype=np.uint32)
    dX64 = hip.upload(X)
    out = []
    for fused in (False, True, "i64"):
        dShift, dXs = hip.malloc(32 * rows), hip.malloc(32 * n)
        planes = [hip.malloc(32 * n) for _ in range(3)]
        ints = [hip.malloc(4 * n) for _ in range(3)]
        arr = (c_void_p * 3)(*[c_void_p(x) for x in planes])
        iarr = (c_void_p * 3)(*[c_void_p(x) for x in ints])
        if fused == "i64":
            hip.call("zk_softmax_shift_decompose_i64", c_void_p(dShift), c_void_p(dXs), arr, iarr, c_void_p(dX64), c_uint(rows), c_uint(cols), c_double(scale), bs, c_int(3), None)
        elif fused:
            hip.call("zk_softmax_shift_decompose", c_void_p(dShift), c_void_p(dXs), arr, iarr, c_void_p(dX), c_uint(rows), c_uint(cols), c_double(scale), bs, c_int(3), None)
        else:
            hip.call("zk_softmax_shift", c_void_p(dShift), c_void_p(dXs), c_void_p(dX), c_uint(rows), c_uint(cols), c_double(scale), None)
            hip.call("zk_softmax_decompose_ints", arr, iarr, c_void_p(dXs), bs, c_int(3), c_size_t(n), None)
        out.append([hip.download(dShift, (rows, 8), np.uint32), hip.download(dXs, (n, 8), np.uint32)] + [hip.download(q, (n, 8), np.uint32) for q in planes]
                   + [hip.download(q, (n,), np.int32) for q in ints])
        for q in [dShift, dXs] + planes + ints:
            hip.free(q)
    for other in out[1:]:
        for a, b in zip(out[0], other):
            assert (a == b).all()
    assert out[0][2].any() and out[0][5].any()
    # the digits are those of shift - score: d0 + b0 (d1 + b1 d2)
    shift = np.array([v if v < R_MOD // 2 else v - R_MOD for v in fr_ints(out[0][0])], dtype=np.int64)
    neg = np.repeat(shift, cols) - X
    d0, d1, d2 = (out[0][5 + k].astype(np.int64) for k in range(3))
    assert (d0 + int(bs[0]) * (d1 + int(bs[1]) * d2) == neg).all()
    assert (d0 >= 0).all() and (d0 < int(bs[0])).all() and (d1 < int(bs[1])).all() and (d2 < int(bs[2])).all()
    hip.free(dX)
    hip.free(dX64)


@pytest.mark.parametrize("k", [13, 17, 19])
def test_lookup_jobs_that_read_int32_forms_equal_the_plain_one(k):
    """zk_lookup_prove_begin_mapped_ints / _hinted_ints (the first round of a large job reads the queries' int32 forms and
    takes query and inverse from the table where the entry is what the integers say) against zk_lookup_prove_begin on the
    combined queries computed here with big integers: inputs outside the table, outputs that are not the mapped value,
    the extreme integers, a table entry that is NOT low + j + r * mapped[j] (its queries must not be read from it) and one
    whose inverse does not exist.  2^13: the small-job path (the field elements serve); 2^17: the fused first round; 2^19: the
    first two rounds in one pass (k_lookup_first2_29)."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    hip = Hip()
    D, N, low = 1 << k, 64, -9
    rng = np.random.default_rng(1000 + k)
    mapped = [int(x) for x in rng.integers(-2 ** 31, 2 ** 31, N)]
    mapped[5], mapped[6] = -2 ** 31, 2 ** 31 - 1
    r_fr, beta = ch(62, 1)[0], ch(63, 1)[0]
    r, b = fr_ints(r_fr.reshape(1, 8))[0], fr_ints(beta.reshape(1, 8))[0]
    pos = rng.integers(0, N, D)
    pos[:N] = np.arange(N)                                        # every entry is queried
    s_in = [int(p) + low for p in pos]
    s_out = [mapped[int(p)] for p in pos]
    odd = rng.choice(np.arange(N, D), 300, replace=False)
    for i in odd[:100]:
        s_out[i] = int(np.int32((s_out[i] + 1 + int(i)) & 0x7FFFFFFF))      # not the mapped value
    for i in odd[100:200]:
        s_in[i] = low + N + 3 + int(i)                                      # outside the table (above)
    for i in odd[200:250]:
        s_in[i] = low - 1 - int(i)                                          # outside the table (below)
    s_in[int(odd[250])], s_in[int(odd[251])] = -2 ** 31, 2 ** 31 - 1
    s_out[int(odd[252])] = -2 ** 31
    Tl = [((low + j) + r * mapped[j]) % R_MOD for j in range(N)]
    Tl[9] = (Tl[9] + 1) % R_MOD                                   # an entry that is something else: queries at position 9 are no entries
    Tl[11] = (-b) % R_MOD                                         # T + beta == 0 (and not what the integers say)
    m_counts = np.zeros(N, np.int64)
    S_com_l = [(a + r * o) % R_MOD for a, o in zip(s_in, s_out)]
    index_of = {}
    for j, t in enumerate(Tl):
        index_of.setdefault(t, j)
    for q in S_com_l:
        if q in index_of:
            m_counts[index_of[q]] += 1
    T, S_com = fr_array(Tl), fr_array(S_com_l)
    m = fr_array([int(c) for c in m_counts])
    u, v = ch(64, k - 1), ch(65, k)
    Si, So, Mp = fr_array([x % R_MOD for x in s_in]), fr_array([x % R_MOD for x in s_out]), fr_array([x % R_MOD for x in mapped])
    dS, dT, dm, dSi, dSo, dMp = hip.upload(S_com), hip.upload(T), hip.upload(m), hip.upload(Si), hip.upload(So), hip.upload(Mp)
    hs = []
    for dev, n in ((dSi, D), (dSo, D), (dMp, N)):
        h = c_void_p()
        hip.call("zk_fr_fold_prepare", ctypes.byref(h), c_void_p(dev), c_size_t(n), None)
        assert h.value
        hs.append(h)
    # where the int32 forms suffice (zk_lookup_ints_suffice: the fused first round) the field elements beside them are never
    # read: the jobs get buffers of other values there
    suffice = hip.lib.zk_lookup_ints_suffice(c_size_t(D), c_size_t(N)) == 1
    assert suffice == (k >= 17)
    dJunk = hip.upload(ch(66, D)) if suffice else None
    fSi, fSo = (dJunk, dJunk) if suffice else (dSi, dSo)
    res = []
    for job in ("plain", "mapped_ints"):
        h = c_void_p()
        if job == "plain":
            hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dS), c_void_p(dT), c_void_p(dm), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        else:
            hip.call("zk_lookup_prove_begin_mapped_ints", ctypes.byref(h), c_void_p(fSi), hs[0], c_void_p(fSo), hs[1], hs[2], r_fr, c_void_p(dT), c_void_p(dm), c_int(low),
                     beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
        hip.call("zk_lookup_prove_end", h, bm, sums)
        res.append((bm, sums))
    assert (res[0][0] == res[1][0]).all() and (res[0][1] == res[1][1]).all()
    assert res[0][1].any()
    # a range table: the queries are their own hints
    Tr = [(low + j) % R_MOD for j in range(N)]
    Tr[13] = (Tr[13] + 5) % R_MOD                                 # not a range entry any more
    dTr = hip.upload(fr_array(Tr))
    index_of = {}
    for j, t in enumerate(Tr):
        index_of.setdefault(t, j)
    m_counts = np.zeros(N, np.int64)
    for q in s_in:
        if q % R_MOD in index_of:
            m_counts[index_of[q % R_MOD]] += 1
    dmr = hip.upload(fr_array([int(c) for c in m_counts]))
    res = []
    for job in ("plain", "hinted_ints"):
        h = c_void_p()
        if job == "plain":
            hip.call("zk_lookup_prove_begin", ctypes.byref(h), c_void_p(dSi), c_void_p(dTr), c_void_p(dmr), beta, u, v, c_size_t(D), c_size_t(N), c_int(k), None)
        else:
            hip.call("zk_lookup_prove_begin_hinted_ints", ctypes.byref(h), c_void_p(fSi), hs[0], c_void_p(dTr), c_void_p(dmr), c_int(low), beta, u, v,
                     c_size_t(D), c_size_t(N), c_int(k), None)
        bm, sums = np.zeros(8, np.uint32), np.zeros((k * 11, 8), np.uint32)
        hip.call("zk_lookup_prove_end", h, bm, sums)
        res.append((bm, sums))
    assert (res[0][0] == res[1][0]).all() and (res[0][1] == res[1][1]).all()
    for h in hs:
        hip.call("zk_fr_fold_prepared_free", h)
    for q in (dS, dT, dm, dSi, dSo, dMp, dTr, dmr) + ((dJunk,) if suffice else ()):
        hip.free(q)


@pytest.mark.parametrize("n", [3007, 1 << 16])
def test_int32_forms_written_with_the_tensors_serve_index_gather_and_evaluations(n):
    """zk_softmax_decompose_ints writes every digit plane as field elements and as int32 (both checked against divmod);
    zk_fr_gather_ints writes the gathered table values with their int32 form; zk_fr_me_multi_ints, reading the int32 forms
    where given (five of them and one tensor of full residues: the mix of a softmax proof; then seven with two residue tensors),
    returns exactly what zk_fr_me_multi returns, which is checked against the brute-force extension at small n."""
    import ctypes
    from gpuhelp import Hip, c_void_p, c_size_t, c_int
    from zkhelp import me_bruteforce
    hip = Hip()
    rng = np.random.default_rng(n)
    bs = np.array([256, 1 << 20, 1 << 20], dtype=np.uint32)
    mag = rng.integers(0, 1 << 48, n).astype(np.int64)
    mag[0], mag[1] = 0, (1 << 48) - 1
    X = fr_array([(-int(v)) % R_MOD for v in mag])
    dX = hip.upload(X)
    planes = [hip.malloc(32 * n) for _ in range(3)]
    handles, ints = [], []
    for _ in range(3):
        h, q = c_void_p(), c_void_p()
        hip.call("zk_fr_fold_prepared_new", ctypes.byref(h), ctypes.byref(q), c_size_t(n), None)
        handles.append(h)
        ints.append(q)
    hip.lib.zk_fr_fold_prepared_ints.restype = c_void_p
    for h, q in zip(handles, ints):
        assert hip.lib.zk_fr_fold_prepared_ints(h) == q.value
    arr = (c_void_p * 3)(*[c_void_p(x) for x in planes])
    iarr = (c_void_p * 3)(*ints)
    hip.call("zk_softmax_decompose_ints", arr, iarr, c_void_p(dX), bs, c_int(3), c_size_t(n), None)
    digits = []
    t = mag.astype(object)
    for b in bs:
        digits.append(np.array([int(v) % int(b) for v in t], dtype=np.int64))
        t = np.array([int(v) // int(b) for v in t], dtype=object)
    for k in range(3):
        got_fr = hip.download(planes[k], (n, 8), np.uint32)
        got_i = hip.download(ints[k].value, (n,), np.int32)
        assert (got_i == digits[k]).all(), k
        assert (got_fr[:, 0] == digits[k]).all() and not got_fr[:, 1:].any(), k
    # gather by the first plane's digits from a table of 256 integers of up to 22 bits
    tab_i = rng.integers(0, 1 << 22, 256).astype(np.int64)
    tab_i[0], tab_i[255] = (1 << 22) - 1, 0
    dT = hip.upload(fr_array([int(v) for v in tab_i]))
    th = c_void_p()
    hip.call("zk_fr_fold_prepare", ctypes.byref(th), c_void_p(dT), c_size_t(256), None)
    assert th.value
    idx = digits[0].astype(np.uint32)
    dI = hip.upload(idx)
    dG = hip.malloc(32 * n)
    gh, gq = c_void_p(), c_void_p()
    hip.call("zk_fr_fold_prepared_new", ctypes.byref(gh), ctypes.byref(gq), c_size_t(n), None)
    hip.call("zk_fr_gather_ints", c_void_p(dG), gq, c_void_p(dT), th, c_void_p(dI), c_size_t(n), None)
    got_fr = hip.download(dG, (n, 8), np.uint32)
    got_i = hip.download(gq.value, (n,), np.int32)
    assert (got_i == tab_i[idx]).all() and (got_fr[:, 0] == tab_i[idx]).all() and not got_fr[:, 1:].any()
    # the product of two tensors from their int32 forms (negative factors through a table of signed integers)
    sg_i = rng.integers(-2 ** 31, 2 ** 31, 256).astype(np.int64)
    sg_i[0], sg_i[1] = -2 ** 31, 2 ** 31 - 1
    dT2 = hip.upload(fr_array([int(v) % R_MOD for v in sg_i]))
    th2 = c_void_p()
    hip.call("zk_fr_fold_prepare", ctypes.byref(th2), c_void_p(dT2), c_size_t(256), None)
    dG2 = hip.malloc(32 * n)
    g2h, g2q = c_void_p(), c_void_p()
    hip.call("zk_fr_fold_prepared_new", ctypes.byref(g2h), ctypes.byref(g2q), c_size_t(n), None)
    hip.call("zk_fr_gather_ints", c_void_p(dG2), g2q, c_void_p(dT2), th2, c_void_p(dI), c_size_t(n), None)
    dP = hip.malloc(32 * n)
    hip.call("zk_fr_mul_ints", c_void_p(dP), g2h, g2h, c_size_t(n), None)
    sq = fr_ints(hip.download(dP, (n, 8), np.uint32))
    assert sq == [int(v) * int(v) % R_MOD for v in sg_i[idx]]
    hip.call("zk_fr_mul_ints", c_void_p(dP), g2h, gh, c_size_t(n), None)
    pr = fr_ints(hip.download(dP, (n, 8), np.uint32))
    assert pr == [int(a) * int(b) % R_MOD for a, b in zip(sg_i[idx], tab_i[idx])]
    for h in (th2, g2h):
        hip.call("zk_fr_fold_prepared_free", h)
    for q in (dT2, dG2, dP):
        hip.free(q)
    # evaluations: int32 forms where there are some, full residues elsewhere
    k = (n - 1).bit_length()
    u = ch(71, k)
    R1, R2 = ch(72, n), ch(73, n)
    dR1, dR2 = hip.upload(R1), hip.upload(R2)
    for Xs, hs in [([planes[0], planes[1], dR1, planes[2], dG, planes[0]], [handles[0], handles[1], None, handles[2], gh, handles[0]]),
                   ([dR1, planes[0], planes[1], planes[2], dG, planes[1], planes[2], dR2], [None, handles[0], handles[1], handles[2], gh, handles[1], handles[2], None]),
                   ([dR1, planes[0], dR2, planes[1]], [None, handles[0], None, handles[1]]), ([dR2, dR1, dG], [None, None, gh]),
                   ([planes[1]], [handles[1]]), ([dR1, dR2], [None, None])]:
        K = len(Xs)
        xa = (c_void_p * K)(*[c_void_p(x) for x in Xs])
        ha = (c_void_p * K)(*[h if h is not None else c_void_p(None) for h in hs])
        want, got = np.zeros((K, 8), np.uint32), np.zeros((K, 8), np.uint32)
        hip.call("zk_fr_me_multi", want, xa, c_int(K), c_size_t(n), u, c_int(k), None)
        hip.call("zk_fr_me_multi_ints", got, xa, ha, c_int(K), c_size_t(n), u, c_int(k), None)
        assert (got == want).all(), K
    if n < 5000:
        ui = fr_ints(u)
        assert fr_ints(got[:1])[0] == me_bruteforce(fr_ints(R1), ui)
        xa = (c_void_p * 1)(c_void_p(planes[1]))
        ha = (c_void_p * 1)(handles[1])
        one = np.zeros((1, 8), np.uint32)
        hip.call("zk_fr_me_multi_ints", one, xa, ha, c_int(1), c_size_t(n), u, c_int(k), None)
        assert fr_ints(one)[0] == me_bruteforce([int(v) for v in digits[1]], ui)
    for h in handles + [gh, th]:
        hip.call("zk_fr_fold_prepared_free", h)
    for q in planes + [dX, dT, dI, dG, dR1, dR2]:
        hip.free(q)


def test_config4_full_size_range_lookup_and_softmax_of_one_head(pv):
    """One attention head at sequence length 2048: 2^22 scores uniform in [-2^15, 2^15), a range table of 2^16 entries.
    Beyond what the oracle can follow, so checked through what the protocol fixes: the multiplicities are numpy's
    bincount, the inverses satisfy the LogUp identity sum_i 1/(S_i + beta) = sum_k m_k/(T_k + beta), the 22 round
    polynomials of the lookup sumcheck chain from alpha + alpha^2 to the returned claim (p(0) + p(1) = claim, claim <- p(v)),
    and zkSoftmax with the attention driver's parameters (self-attn.cu:87) proves these scores (every identity inside the
    prover holds) and returns, at scale 2^40, the softmax of the scores to 1e-6, rows summing to one."""
    n_rows = n_cols = 2048
    D, low, length = n_rows * n_cols, -(1 << 15), 1 << 16
    rng = np.random.default_rng(44)
    vals = rng.integers(low, low + length, D).astype(np.int32)
    hS = pv.from_i32(vals)
    m = pv.range_prep(hS, low, length)
    counts = np.bincount(vals.astype(np.int64) - low, minlength=length)
    mh = m.host()
    assert (mh[:, 0] == counts).all() and not mh[:, 1:].any()
    beta = ch(61, 1)[0]
    hT = pv.from_i32(np.arange(low, low + length, dtype=np.int32))
    A, B = pv.batch_inv(hS, beta), pv.batch_inv(hT, beta)
    assert (pv.sum(A) == pv.sum(pv.binop(2, m, B))).all()
    del A, B
    k, n1 = 22, 6
    alpha, u, v = ch(62, 1)[0], ch(63, k), ch(64, k)
    pv.transcript_begin()
    fin = pv.range_prove(hS, low, length, alpha, beta, u, v)
    pv.lib.zkp_transcript_end()
    t = fr_ints(pv.transcript())
    assert len(t) == 4 * k + 1 and t[-1] == fr_ints(fin)[0]
    a, vi = fr_ints(alpha)[0], fr_ints(v)
    claim = (a + a * a) % R_MOD
    for r in range(k):
        c = t[4 * r:4 * r + 4]
        assert (2 * c[0] + c[1] + c[2] + c[3]) % R_MOD == claim, r
        x = vi[n1 - 1 - r] if r < n1 else vi[k - 1 - (r - n1)]
        claim = (c[0] + c[1] * x + c[2] * x * x + c[3] * x * x * x) % R_MOD
    assert claim == t[-1]
    # zkSoftmax on the same scores
    sf_in, d = 1 << 32, 128
    pv.seed(65)
    Y, shift = pv.softmax(hS, n_rows, n_cols, d, np.array([1 << 8, 1 << 20, 1 << 20], np.uint32), 1, 0, sf_in, np.array([float(1 << 18), float(1 << 22)]), True)
    y = Y.host()
    assert not y[:, 2:].any()
    yf = (y[:, 0].astype(np.float64) + y[:, 1].astype(np.float64) * 2.0 ** 32).reshape(n_rows, n_cols) / 2.0 ** 40
    z = vals.reshape(n_rows, n_cols).astype(np.float64) / sf_in / np.sqrt(d)
    e = np.exp(z - z.max(axis=1, keepdims=True))
    ref = e / e.sum(axis=1, keepdims=True)
    assert np.abs(yf - ref).max() < 1e-6
    assert np.abs(yf.sum(axis=1) - 1.0).max() < 1e-3
    # the same head with scores spread over +-2^36 (+-1.4 after the division by sqrt(d)): the rows are far from uniform
    wide = rng.integers(-(1 << 36), 1 << 36, D)
    pv.seed(66)
    Y, shift = pv.softmax(pv.from_i64(wide), n_rows, n_cols, d, np.array([1 << 8, 1 << 20, 1 << 20], np.uint32), 1, 0, sf_in,
                          np.array([float(1 << 18), float(1 << 22)]), True)
    y = Y.host()
    yf = (y[:, 0].astype(np.float64) + y[:, 1].astype(np.float64) * 2.0 ** 32).reshape(n_rows, n_cols) / 2.0 ** 40
    z = wide.reshape(n_rows, n_cols).astype(np.float64) / sf_in / np.sqrt(d)
    e = np.exp(z - z.max(axis=1, keepdims=True))
    ref = e / e.sum(axis=1, keepdims=True)
    assert ref.max() / ref.min() > 10
    # the exponential tables are rounded at scales 2^18 and 2^22: a few 1e-4 relative on the small entries
    assert np.abs(yf - ref).max() < 5e-7 and ref.max() > 1e-3
