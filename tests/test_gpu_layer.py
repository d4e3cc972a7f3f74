"""GPU parity for a whole decoder layer (RMSNorm, QKV, per-head attention with zkSoftmax, output projection,
skip, RMSNorm, SwiGLU FFN, skip; every rescaling, lookup, sumcheck and weight opening): outputs and the full proof
transcript under a seeded challenge stream are bit-exact against the CPU oracle at small shapes."""
import numpy as np
import pytest

import layercfg
from zkhelp import load_oracle, orc_check, orc_transcript

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pv():
    from gpuhelp import Prover
    return Prover()


@pytest.mark.parametrize("open_weights,seed,head_group", [(True, 3, 0), (False, 4, 0), (False, 5, 2), (True, 6, 1)])
def test_tiny_layer_transcript(pv, open_weights, seed, head_group):
    orc = load_oracle()
    cu, cf = layercfg.tiny(open_weights=open_weights, head_group=head_group)
    ws = layercfg.tiny_weights(seed, cu)
    S, E = int(cu[0]), int(cu[1])
    X = np.round(np.random.default_rng(seed + 10).normal(0, 1, (S, E)) * 256).astype(np.int32)
    exp = np.zeros((S * E, 8), np.uint32)
    orc.orc_seed(seed)
    orc.orc_transcript_clear()
    orc_check(orc.orc_layer(cu, cf, *ws, 1, X, exp, None))
    exp_t = orc_transcript(orc)
    pv.seed(seed)
    layer = pv.layer_create(cu, cf, ws, 1)
    pv.transcript_begin()
    out, times = pv.layer_run(layer, pv.from_i32(X))
    pv.lib.zkp_transcript_end()
    got_t = pv.transcript()
    pv.layer_free(layer)
    assert (out.host() == exp).all()
    assert got_t.shape == exp_t.shape and (got_t == exp_t).all()
    assert times[6] > 0
