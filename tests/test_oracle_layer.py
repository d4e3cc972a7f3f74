"""Pins the oracle's layer-level restatement (oracle/layer_ref.hpp) by things that do not share its code:

* the SwiGLU table and the RMS statistic against their closed forms in numpy (llama-ffn.py:14-19, llama-rmsnorm.py:35-39);
* every block against an exact integer model in numpy (matrix products by numpy, rescaling as floor((x + sf/2) / sf),
  the activation as a table gather): a transposed weight, a rescale in the wrong place or by the wrong factor, a table
  offset, a wrong operand of a Hadamard product or a wrong head slice changes some output element;
* the whole layer against a float64 decoder block (RMSNorm, per-head softmax attention without mask or rotary
  embedding, output projection, skip, RMSNorm, SwiGLU FFN, skip) within a tolerance derived from the fixed-point
  scales, with negative controls showing that the tolerance separates a correct layer from a plausible mistake.
"""
import ctypes

import numpy as np
import pytest

import layercfg
from zkhelp import R_MOD, fr_array, fr_signed as signed, load_oracle, orc_check

VS_BITS = 10            # fixed-point scale of activations and weights in the mid-size configuration


def mid_cfg(swiglu_out_scale=1024.0, heads=2, head_group=0, seq=64, embed=64, hidden=64):
    """seq 64, width 64, hidden 64: tensors of 4096 elements, so that the rescaling tables (2^10, 2^12 and 2^9 entries), the
    softmax digit tables (2^10) and an activation table over [-4, 4) in steps of 2^-8 fit their tensors"""
    return layercfg.pack(seq, embed, heads, hidden, 1 << 10, 1 << 12, 1 << 9, [1 << 8, 1 << 10, 1 << 10], 1, 0, 1 << 20, [1 << 8, 1 << 10],
                         -1024, 2048, 256.0, swiglu_out_scale=swiglu_out_scale, value_scale=1024.0, open_weights=False, head_group=head_group)


def as_fr(a):
    return fr_array([int(x) % R_MOD for x in np.asarray(a).reshape(-1)])


def rescale(x, sf):
    """rescaling_kernel (rescaling.cu:8-21): remainder in [-sf/2, sf/2), i.e. round half up"""
    return np.floor_divide(x + sf // 2, sf)


class W:
    """weight handles of the oracle (no generators: these configurations do not open weights)"""

    def __init__(self, orc, mats):
        self.orc = orc
        self.h = []
        for m in mats:
            m = np.ascontiguousarray(m, dtype=np.int32)
            h = orc.orc_weight_new(m, m.shape[0], m.shape[1], None, 0, None, 0)
            assert h
            self.h.append(ctypes.c_void_p(h))

    def __del__(self):
        for h in self.h:
            self.orc.orc_weight_free(h)


@pytest.fixture(scope="module")
def orc():
    o = load_oracle()
    o.dll.orc_weight_new.restype = ctypes.c_void_p
    return o


def make_inputs(seed, cu, w_std=0.1, norm_jitter=0.2):
    rng = np.random.default_rng(seed)
    S, E, Hd = int(cu[0]), int(cu[1]), int(cu[3])
    sc = 1 << VS_BITS
    mk = lambda i, o: np.round(rng.normal(0, w_std, (i, o)) * sc).astype(np.int64)
    norm = lambda: np.round((1.0 + rng.uniform(-norm_jitter, norm_jitter, (1, E))) * sc).astype(np.int64)
    ws = [norm(), mk(E, E), mk(E, E), mk(E, E), mk(E, E), norm(), mk(E, Hd), mk(E, Hd), mk(Hd, E)]
    X = np.round(rng.normal(0, 1, (S, E)) * sc).astype(np.int64)
    return ws, X


# ---- closed forms ---------------------------------------------------------------------------------------------------
def test_swiglu_table_is_round_x_sigmoid_x_times_16_over_the_whole_table(orc):
    """llama-ffn.py:14-19 at the driver's size: Xs = arange(-512, 512, 2^-12), round(Xs * sigmoid(Xs) * 16) (the driver
    passes out_prec_num_bit = 16 itself as the factor), torch.round = half to even."""
    low, n = -(1 << 21), 1 << 22
    out = np.zeros((n, 8), np.uint32)
    orc_check(orc.orc_swiglu_table(low, n, 4096.0, 16.0, out))
    got_signed = np.array(signed(out), dtype=np.int64)
    xs = np.arange(low, low + n, dtype=np.float64) / 4096.0
    y = xs * (1.0 / (1.0 + np.exp(-xs))) * 16.0
    exp = np.rint(y).astype(np.int64)
    # Two float64 evaluations of the formula must agree except within rounding noise of a boundary k + 1/2.  Exact ties are
    # no exception: beyond |x| = 37 sigmoid(x) is exactly 0 or 1, 16 x is exact, and both sides round half to even.
    near = np.abs(y - np.floor(y) - 0.5) <= 1e-9
    exact_tie = (2.0 * y == np.rint(2.0 * y))
    must_agree = ~near | exact_tie
    assert must_agree.sum() >= n - 200 and exact_tie.sum() > 7000   # the near misses: x in (20, 37) with 16 x = k + 1/2, sigmoid(x) = 1 - tiny
    assert (got_signed[must_agree] == exp[must_agree]).all()
    assert np.abs(got_signed - exp).max() <= 1
    assert got_signed[-low] == 0 and got_signed[-1] == 8192 and got_signed[0] == 0
    assert got_signed.min() == round(-0.27846 * 16)          # minimum of x * sigmoid(x) is -0.27846...


def test_rms_inv_is_round_of_reciprocal_root_mean_square(orc):
    """llama-rmsnorm.py:35-39: X / 2^16 in float64, 1 / sqrt(mean(X^2) + eps), saved times 2^16 and rounded"""
    rng = np.random.default_rng(5)
    S, E = 24, 96
    X = np.round(rng.normal(0, 1, (S, E)) * 65536).astype(np.int64)
    X[3] = 0                                                  # an all-zero row: 1 / sqrt(eps)
    out = np.zeros((S, 8), np.uint32)
    orc_check(orc.orc_rms_inv(as_fr(X), S, E, 1e-5, 65536.0, out))
    xf = X.astype(np.float64) / 65536.0
    exp = np.rint(1.0 / np.sqrt(np.mean(xf ** 2, axis=1) + 1e-5) * 65536.0).astype(np.int64)
    assert signed(out) == list(exp)
    assert exp[3] == round(65536 / np.sqrt(1e-5))


# ---- exact integer models of the blocks ----------------------------------------------------------------------------------
def np_rmsnorm(cu, w, X, rms):
    sf = int(cu[4])
    g_ = rescale(rms.reshape(-1, 1) * w.reshape(1, -1), sf)
    return rescale(g_ * X, sf)


def np_ffn(cu, cf, up, gate, down, table, x):
    sf, sfg, low = int(cu[4]), int(cu[5]), int(cf[1])
    up_ = rescale(x @ up, sf)
    gate_ = rescale(x @ gate, sfg)
    idx = gate_ - low
    assert idx.min() >= 0 and idx.max() < len(table)
    down_in_ = rescale(table[idx] * up_, sf)
    down_out = down_in_ @ down
    return rescale(down_out, sf), down_out


def table_np(cf, n):
    xs = (cf[1] + np.arange(n, dtype=np.float64)) / cf[2]
    return np.rint(xs / (1.0 + np.exp(-xs)) * cf[3]).astype(np.int64)


@pytest.mark.parametrize("seed", [1, 2])
def test_blocks_equal_exact_integer_models(orc, seed):
    cu, cf = mid_cfg(swiglu_out_scale=16.0)                   # 16: the factor the reference's driver really uses
    ws, X = make_inputs(seed, cu)
    S, E, Hd = int(cu[0]), int(cu[1]), int(cu[3])
    hs = W(orc, ws)
    orc.orc_seed(seed)
    # RMSNorm block (rmsnorm.cu:26-49)
    rms = np.zeros((S, 8), np.uint32)
    orc_check(orc.orc_rms_inv(as_fr(X), S, E, 1e-5, 1024.0, rms))
    rms_i = np.array(signed(rms), dtype=np.int64)
    out = np.zeros((S * E, 8), np.uint32)
    orc_check(orc.orc_rmsnorm_block(cu, cf, hs.h[0], as_fr(X), rms, out))
    n1 = np_rmsnorm(cu, ws[0], X, rms_i)
    assert signed(out) == list(n1.reshape(-1))
    # Q/K/V projections (self-attn.cu:47-60)
    Q_, K_, V_ = (np.zeros((S * E, 8), np.uint32) for _ in range(3))
    orc_check(orc.orc_attn_linear_block(cu, cf, hs.h[1], hs.h[2], hs.h[3], as_fr(n1), Q_, K_, V_))
    for got, w in ((Q_, ws[1]), (K_, ws[2]), (V_, ws[3])):
        assert signed(got) == list(rescale(n1 @ w, int(cu[4])).reshape(-1))
    # output projection
    a = np.array(signed(V_), dtype=np.int64).reshape(S, E)
    orc_check(orc.orc_oproj_block(cu, cf, hs.h[4], as_fr(a), out))
    assert signed(out) == list(rescale(a @ ws[4], int(cu[4])).reshape(-1))
    # FFN block (ffn.cu:44-93); both the rescaled output and the unrescaled product that the reference executable saves
    table = table_np(cf, int(cu[9]))
    tb = np.zeros((int(cu[9]), 8), np.uint32)
    orc_check(orc.orc_swiglu_table(int(cf[1]), int(cu[9]), cf[2], cf[3], tb))
    assert signed(tb) == list(table)
    down_out = np.zeros((S * E, 8), np.uint32)
    orc_check(orc.orc_ffn_block(cu, cf, hs.h[6], hs.h[7], hs.h[8], tb, as_fr(n1), out, down_out))
    exp_out, exp_down = np_ffn(cu, cf, ws[6], ws[7], ws[8], table, n1)
    assert signed(out) == list(exp_out.reshape(-1))
    assert signed(down_out) == list(exp_down.reshape(-1))
    assert np.abs(exp_out).max() > 2                          # not a vacuous comparison


def np_attention_int(cu, cf, Q_, K_, V_, heads):
    """integer skeleton of the attention block: exact scores, then the table-based softmax rebuilt from its definition
    (zksoftmax.cu:4-32, 95-109): shift = round(s * log sum exp(x / s)), digits of shift - x in the mixed radix, output =
    product of the digit tables round(theta * exp(-B * digit / s))"""
    S, E = Q_.shape
    d = E // heads
    K = int(cu[11])
    bs = [int(b) for b in cu[12:12 + K]]
    L = int(cu[7])
    sf_in, thetas = cf[0], [cf[6 + i] for i in range(K - L)]
    s = sf_in * np.sqrt(float(d))
    out = np.zeros((S, E), dtype=np.int64)
    shifts = []
    for h in range(heads):
        q, k, v = (t[:, h * d:(h + 1) * d] for t in (Q_, K_, V_))
        X = q @ k.T
        shift = np.array([int(np.floor(s * np.log(np.sum(np.exp(row / s))) + 0.5)) for row in X.astype(np.float64)], dtype=np.int64)
        shifts.append(shift)
        Z = shift.reshape(-1, 1) - X
        assert Z.min() >= 0
        Y = np.ones(Z.shape, dtype=np.int64)
        rest = Z.copy()
        Bk = 1
        for i, b in enumerate(bs):
            dig = rest % b
            rest = rest // b
            if i >= L:
                tab = np.floor(thetas[i - L] * np.exp(-(Bk / s) * np.arange(b, dtype=np.float64)) + 0.5).astype(np.int64)
                Y = Y * tab[dig]
            Bk *= b
        assert rest.max() == 0
        out[:, h * d:(h + 1) * d] = Y @ v
    return out, shifts


@pytest.mark.parametrize("heads,head_group", [(2, 0), (2, 2), (4, 2), (1, 0)])
def test_attention_block_equals_the_integer_softmax_model(orc, heads, head_group):
    """per head and stacked: scores of each head's own columns, the table softmax, Y V, concatenation by head, two rescalings"""
    cu, cf = mid_cfg(heads=heads, head_group=head_group)
    rng = np.random.default_rng(40 + heads)
    S, E = int(cu[0]), int(cu[1])
    Q_, K_, V_ = (np.round(rng.normal(0, 1.2, (S, E)) * 1024).astype(np.int64) for _ in range(3))
    out = np.zeros((S * E, 8), np.uint32)
    orc.orc_seed(3)
    orc_check(orc.orc_attn_block(cu, cf, 0, as_fr(Q_), as_fr(K_), as_fr(V_), out, None))
    raw, _ = np_attention_int(cu, cf, Q_, K_, V_, heads)
    sfa = int(cu[6])
    exp = [int(x) for x in rescale(rescale(raw.reshape(-1), sfa), sfa)]
    got = signed(out)
    # the float steps (log-sum-exp, table entries) are evaluated by numpy here and by the oracle's own exp/log there:
    # a last-bit difference could move a rounding; none does on these inputs
    assert got == exp


def test_reference_attn_mode_is_one_head_as_wide_as_the_tensors(orc):
    """self-attn.cu:78-121: d = Q.size / seq_len, so the executable's attention is one head of the full width; it saves the
    softmax output and the twice rescaled product"""
    cu, cf = mid_cfg(heads=2)                                 # the head count of the configuration must not matter here
    rng = np.random.default_rng(77)
    S, E = int(cu[0]), int(cu[1])
    Q_, K_, V_ = (np.round(rng.normal(0, 1.0, (S, E)) * 1024).astype(np.int64) for _ in range(3))
    out, Y = np.zeros((S * E, 8), np.uint32), np.zeros((S * S, 8), np.uint32)
    orc.orc_seed(4)
    orc_check(orc.orc_attn_block(cu, cf, 1, as_fr(Q_), as_fr(K_), as_fr(V_), out, Y))
    raw, _ = np_attention_int(cu, cf, Q_, K_, V_, 1)
    sfa = int(cu[6])
    assert signed(out) == [int(x) for x in rescale(rescale(raw.reshape(-1), sfa), sfa)]
    Yi = np.array(signed(Y), dtype=np.float64).reshape(S, S)
    sm = np.exp((Q_ @ K_.T) / (cf[0] * np.sqrt(float(E))))
    sm /= sm.sum(axis=1, keepdims=True)
    assert np.abs(Yi / (cf[6] * cf[7]) - sm).max() < 0.01


# ---- the whole layer against a float64 decoder block --------------------------------------------------------------------------
def float_layer(ws, X, heads, sc, eps=1e-5, mutate=None):
    f = [w.astype(np.float64) / sc for w in ws]
    n1w, wq, wk, wv, wo, n2w, wup, wgate, wdown = f
    if mutate == "transposed_wq":
        wq = wq.T
    x = X.astype(np.float64) / sc
    rms = lambda t: t / np.sqrt(np.mean(t ** 2, axis=1, keepdims=True) + eps)
    a = rms(x) * n1w
    Q, K, V = a @ wq, a @ wk, a @ wv
    d = Q.shape[1] // heads
    att = np.zeros_like(Q)
    for h in range(heads):
        sl = slice(h * d, (h + 1) * d)
        s = Q[:, sl] @ K[:, sl].T / np.sqrt(d)
        if mutate == "no_sqrt_d":
            s = Q[:, sl] @ K[:, sl].T
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        att[:, sl] = p @ V[:, sl]
    x2 = x + att @ wo
    if mutate == "no_first_skip":
        x2 = att @ wo
    b = rms(x2) * n2w
    g = b @ wgate
    act = g / (1.0 + np.exp(-g))
    if mutate == "gate_up_swapped":
        u = b @ wup
        act, g = u / (1.0 + np.exp(-u)), None
        return x2 + (act * (b @ wgate)) @ wdown
    return x2 + (act * (b @ wup)) @ wdown


@pytest.mark.parametrize("seed,heads,head_group", [(11, 2, 0), (12, 4, 4), (13, 1, 0)])
def test_layer_is_a_decoder_block_within_the_quantisation_error(orc, seed, heads, head_group):
    cu, cf = mid_cfg(heads=heads, head_group=head_group)      # consistent scales: the activation table is saved at the value scale
    ws, X = make_inputs(seed, cu)
    S, E = int(cu[0]), int(cu[1])
    out = np.zeros((S * E, 8), np.uint32)
    orc.orc_seed(seed)
    args = [np.ascontiguousarray(w, dtype=np.int32) for w in ws]
    orc_check(orc.orc_layer(cu, cf, *args, 1, np.ascontiguousarray(X, dtype=np.int32), out, None))
    sc = float(1 << VS_BITS)
    got = np.array(signed(out), dtype=np.float64).reshape(S, E) / sc
    ref = float_layer(ws, X, heads, sc)
    # Error budget in units of the value scale 2^-10.  A rescaling rounds by at most half a unit; a matrix product passes
    # the error of its input on times about sqrt(fan_in) * |w| = 8 * 0.1, so errors neither die out nor grow along the
    # path of eight rescaled stages (two norms, four projections deep, the two Hadamard products): about two units per
    # stage in the worst element.  The table softmax adds a relative 2^-9 + 2^-11 per probability, the activation table
    # half a step of 2^-8 in its argument times a slope below 1.1.  Sum: below 16 units = 2^-6 on outputs of magnitude
    # one (measured: 7 units at most, 1.8 rms).
    tol = 16.0 / sc
    err = np.abs(got - ref).max()
    assert err < tol, err
    assert np.abs(ref).std() > 0.5
    # negative controls: each plausible mistake moves the float model away by more than twenty times the tolerance
    for mutate in ("transposed_wq", "no_sqrt_d", "no_first_skip", "gate_up_swapped"):
        wrong = float_layer(ws, X, heads, sc, mutate=mutate)
        assert np.abs(got - wrong).max() > 20 * tol, mutate
