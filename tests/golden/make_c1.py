"""Writes tests/golden/c1_zkfc_toy.npz: the reference's CPU-runnable configuration (zkFC toy: X 16 x 64, W 64 x 64, values
round(N(0, 0.02) * 2^16) embedded in Fr; Y = X W; the 6-round inner-product sumcheck of zkFC::prove under a seeded
challenge stream; Pedersen commitment of W under 64 seeded generators and its opening at a seeded point), computed by
the CPU oracle (oracle/liboracle.so).  The reference holds no vectors of its own for this path; these pin the oracle
against drift and give the GPU tests a fixed target.

    python3 tests/golden/make_c1.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from zkhelp import R_MOD, fr_array, load_oracle, mt_random_vec, orc_check, orc_transcript  # noqa: E402

SEED_DATA, SEED_PROOF, SEED_GENS, SEED_POINT = 1, 1001, 2001, 3001
B, I, O = 16, 64, 64


def inputs():
    rng = np.random.default_rng(SEED_DATA)
    X = np.round(rng.normal(0, 0.02, (B, I)) * 65536).astype(np.int32)
    W = np.round(rng.normal(0, 0.02, (I, O)) * 65536).astype(np.int32)
    return X, W


def compute(orc):
    X, W = inputs()
    Y = np.zeros((B * O, 8), np.uint32)
    claim_W = np.zeros(8, np.uint32)
    orc.orc_seed(SEED_PROOF)
    orc.orc_transcript_clear()
    orc_check(orc.orc_zkfc(X, W, B, I, O, Y, claim_W))
    transcript = orc_transcript(orc)
    orc.orc_seed(SEED_GENS)
    gens = np.zeros((O, 36), np.uint32)
    orc_check(orc.orc_commitment_random(O, gens))
    # the weight as the reference commits it: rows = input features, one generator per output feature
    Wfr = fr_array([int(v) % R_MOD for v in W.reshape(-1)])
    com = np.zeros((I, 36), np.uint32)
    orc_check(orc.orc_commit_int(gens, O, Wfr, I * O, com))
    k = 6 + 6
    u = mt_random_vec(np.random.RandomState(SEED_POINT), k)
    proof = np.zeros((3 * 6 + 1, 36), np.uint32)
    value = np.zeros(8, np.uint32)
    orc_check(orc.orc_open(gens, O, Wfr, I * O, I, u, k, proof, value))

    def norm(p):
        out = np.zeros_like(p)
        orc_check(orc.orc_g1_op(3, p, p, out, p.shape[0]))
        return out

    return dict(X=X, W=W, Y=Y, claim_W=claim_W, transcript=transcript, gens=norm(gens), com=norm(com), open_point=u, open_proof=norm(proof), open_value=value)


if __name__ == "__main__":
    out = compute(load_oracle())
    np.savez_compressed(os.path.join(HERE, "c1_zkfc_toy.npz"), **out)
    print({k: v.shape for k, v in out.items()})
