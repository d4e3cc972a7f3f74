"""The toy configuration of the reference (zkFC 16 x 64 x 64, 6-round sumcheck, commitment of W under 64 generators and
its opening) against the committed fixture tests/golden/c1_zkfc_toy.npz.  The reference ships no vectors for this path:
the fixture was written by the CPU oracle (tests/golden/make_c1.py) and is pinned here, independently of it, by big-integer
arithmetic -- the matrix product mod r, the multilinear value the opening must return, two commitments as textbook affine
sums -- so that neither the oracle nor the fixture can drift unnoticed; the GPU test then has a fixed target."""
import importlib.util
import os

import numpy as np
import pytest

from zkhelp import (R_MOD, ROOT, ec_add, ec_mul, fr_array, fr_ints, jac_to_affine, load_oracle, me_bruteforce, orc_check)

FIXTURE = os.path.join(ROOT, "tests", "golden", "c1_zkfc_toy.npz")


def fixture():
    return dict(np.load(FIXTURE, allow_pickle=False))


def test_fixture_agrees_with_big_integer_arithmetic():
    f = fixture()
    X, W = f["X"].astype(object), f["W"].astype(object)
    assert fr_ints(f["Y"]) == [int(v) % R_MOD for v in (X @ W).reshape(-1)]
    # the opening returns the multilinear extension of the weight (64 rows x 64 columns, columns fastest) at the point
    Wm = [int(v) % R_MOD for v in f["W"].reshape(-1)]
    assert fr_ints(f["open_value"].reshape(1, 8))[0] == me_bruteforce(Wm, fr_ints(f["open_point"]))
    # com[row] = sum_j W[row, j] * gens[j] on y^2 = x^3 + 4
    gens = [jac_to_affine(g) for g in f["gens"]]
    for row in (0, 37):
        acc = None
        for j in range(64):
            acc = ec_add(acc, ec_mul(int(f["W"][row, j]) % R_MOD, gens[j]))
        assert jac_to_affine(f["com"][row]) == acc
    # the last two transcript values are X and W evaluated at the sumcheck's point, their product the final claim (zkfc.cu:77-79)
    t = fr_ints(f["transcript"])
    assert t[-2] * t[-1] % R_MOD == t[-3]
    assert fr_ints(f["claim_W"].reshape(1, 8))[0] == t[-1]


def test_oracle_reproduces_the_fixture():
    spec = importlib.util.spec_from_file_location("make_c1", os.path.join(ROOT, "tests", "golden", "make_c1.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    got, want = mod.compute(load_oracle()), fixture()
    assert sorted(got) == sorted(want)
    for k in want:
        assert got[k].shape == want[k].shape and (got[k] == want[k]).all(), k


@pytest.mark.gpu
def test_gpu_reproduces_the_fixture():
    from gpuhelp import Prover
    spec = importlib.util.spec_from_file_location("make_c1", os.path.join(ROOT, "tests", "golden", "make_c1.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    pv, orc, f = Prover(), load_oracle(), fixture()
    Y, transcript = pv.zkfc_scenario(f["X"], f["W"], seed=mod.SEED_PROOF)
    assert (Y == f["Y"]).all()
    assert transcript.shape == f["transcript"].shape and (transcript == f["transcript"]).all()

    def norm(p):
        p = np.ascontiguousarray(p, dtype=np.uint32).reshape(-1, 36)
        out = np.zeros_like(p)
        orc_check(orc.orc_g1_op(3, p, p, out, p.shape[0]))
        return out

    pv.seed(mod.SEED_GENS)
    gens = pv.commitment_random(64)
    assert (norm(gens.host()) == f["gens"]).all()
    hW = pv.from_fr(fr_array([int(v) % R_MOD for v in f["W"].reshape(-1)]))
    com = pv.commit_int(gens, hW)
    assert (norm(com.host()) == f["com"]).all()
    value, proof = pv.open(gens, hW, com, f["open_point"])
    assert (value == f["open_value"]).all()
    assert (norm(proof) == f["open_proof"]).all()
