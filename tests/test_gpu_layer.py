"""GPU parity for a whole decoder layer (RMSNorm, QKV, per-head attention with zkSoftmax, output projection,
skip, RMSNorm, SwiGLU FFN, skip; every rescaling, lookup, sumcheck and weight opening): outputs and the full proof
transcript under a seeded challenge stream are bit-exact against the CPU oracle at small shapes."""
import ctypes

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


@pytest.mark.parametrize("open_weights,seed", [(True, 13), (False, 14)])
def test_tiny_layer_blocks_overlapped_and_one_after_the_other(pv, open_weights, seed):
    """With all heads as one stack every block of the layer runs in three steps, and the layer queues a block's forward pass
    and proof jobs before it collects the proofs of earlier blocks (zkp_layer_set_blocks_overlap: how many blocks may be
    begun and not yet collected; on by default).  Every order of work gives the oracle's output and transcript."""
    orc = load_oracle()
    cu, cf = layercfg.tiny(open_weights=open_weights, head_group=2)
    ws = layercfg.tiny_weights(seed, cu)
    S, E = int(cu[0]), int(cu[1])
    X = np.round(np.random.default_rng(seed + 10).normal(0, 1, (S, E)) * 256).astype(np.int32)
    exp = np.zeros((S * E, 8), np.uint32)
    orc.orc_seed(seed)
    orc.orc_transcript_clear()
    orc_check(orc.orc_layer(cu, cf, *ws, 1, X, exp, None))
    exp_t = orc_transcript(orc)
    default = pv.lib.zkp_layer_blocks_overlap()
    assert default > 0
    try:
        for overlap in (0, 1, 3, 6):
            pv.lib.zkp_layer_set_blocks_overlap(overlap)
            pv.seed(seed)
            layer = pv.layer_create(cu, cf, ws, 1)
            pv.transcript_begin()
            out, times = pv.layer_run(layer, pv.from_i32(X))
            pv.lib.zkp_transcript_end()
            got_t = pv.transcript()
            pv.layer_free(layer)
            assert (out.host() == exp).all(), overlap
            assert got_t.shape == exp_t.shape and (got_t == exp_t).all(), overlap
            assert min(times[:6]) > 0
    finally:
        pv.lib.zkp_layer_set_blocks_overlap(default)


def test_layer_run_again_starts_its_openings_ahead_and_proves_the_same(pv):
    """The first run over a set of weights learns where the nine opening points sit in the challenge stream; a second run
    starts every opening when the layer starts (batched by generator size) and must deliver the transcript of the first,
    field elements and G1 points alike, which is the oracle's.  A run under another seed (other challenges at the same
    positions) and one with the weight openings switched off and on again go through the same plan."""
    orc = load_oracle()
    cu, cf = layercfg.tiny(open_weights=True, head_group=2)
    ws = layercfg.tiny_weights(21, cu)
    S, E = int(cu[0]), int(cu[1])
    X = np.round(np.random.default_rng(31).normal(0, 1, (S, E)) * 256).astype(np.int32)
    layer = None
    for run, seed in enumerate((8, 8, 9, 8)):
        exp = np.zeros((S * E, 8), np.uint32)
        orc.orc_seed(seed)
        orc.orc_transcript_clear()
        orc_check(orc.orc_layer(cu, cf, *ws, 1, X, exp, None))
        exp_t = orc_transcript(orc)
        pv.seed(seed)
        if layer is None:
            layer = pv.layer_create(cu, cf, ws, 1)      # draws the generators from the stream seeded just above, as the oracle does
        else:
            # the generators were made at the first creation; skip the same draws
            pv.lib.zkp_challenge_skip.argtypes = [ctypes.c_ulonglong]
            pv.lib.zkp_challenge_skip(ctypes.c_ulonglong(layer_draws))
        if run == 0:
            pv.lib.zkp_challenge_position.restype = ctypes.c_ulonglong
            layer_draws = pv.lib.zkp_challenge_position()
        assert pv.lib.zkp_layer_planned_openings(ctypes.c_void_p(layer)) == (0 if run == 0 else 9)
        pv.transcript_begin()
        out, _ = pv.layer_run(layer, pv.from_i32(X))
        pv.lib.zkp_transcript_end()
        got_t = pv.transcript()
        if seed == 8:
            assert (out.host() == exp).all(), run
            assert got_t.shape == exp_t.shape and (got_t == exp_t).all(), run
            g1 = pv.transcript_g1()
            if run == 0:
                first_g1 = g1
            else:
                assert g1.shape == first_g1.shape and (g1 == first_g1).all(), run
        else:
            assert got_t.shape == exp_t.shape, run
    pv.layer_free(layer)


def test_tiny_layer_with_every_opening_started_at_its_claim(pv):
    """zkp_openings_set_only_at_claim (ZKLLM_OPEN_AHEAD=0): no plan is learned or used and nothing starts ahead inside a block;
    the openings of a block start together at its last claim, and the stacked attention proof (which opens nothing) is queued
    and collected behind the last block so that the host reaches those claims early.  Transcript and G1 points are those of
    the default run and of the oracle, also with the attention proof moved in each of the other ways and in its turn."""
    orc = load_oracle()
    cu, cf = layercfg.tiny(open_weights=True, head_group=2)
    ws = layercfg.tiny_weights(23, cu)
    S, E = int(cu[0]), int(cu[1])
    X = np.round(np.random.default_rng(33).normal(0, 1, (S, E)) * 256).astype(np.int32)
    exp = np.zeros((S * E, 8), np.uint32)
    orc.orc_seed(12)
    orc.orc_transcript_clear()
    orc_check(orc.orc_layer(cu, cf, *ws, 1, X, exp, None))
    exp_t = orc_transcript(orc)
    pv.seed(12)
    layer = pv.layer_create(cu, cf, ws, 1)
    pv.lib.zkp_challenge_position.restype = ctypes.c_ulonglong
    pv.lib.zkp_challenge_skip.argtypes = [ctypes.c_ulonglong]
    layer_draws = pv.lib.zkp_challenge_position()
    g1s, learned = [], False
    try:
        for at_claim, attention in ((1, -1), (1, -1), (0, -1), (0, -1), (1, 0), (1, 1), (1, 2), (0, 3), (0, 1)):
            pv.lib.zkp_openings_set_only_at_claim(at_claim)
            pv.lib.zkp_layer_set_attention_last(attention)
            pv.seed(12)
            pv.lib.zkp_challenge_skip(ctypes.c_ulonglong(layer_draws))
            pv.transcript_begin()
            out, _ = pv.layer_run(layer, pv.from_i32(X))
            pv.lib.zkp_transcript_end()
            got_t = pv.transcript()
            assert (out.host() == exp).all()
            assert got_t.shape == exp_t.shape and (got_t == exp_t).all()
            g1s.append(pv.transcript_g1().copy())
            # runs that only open at the claim neither learn nor use a plan: it is there once a run of the other kind has been
            learned = learned or not at_claim
            assert pv.lib.zkp_layer_planned_openings(ctypes.c_void_p(layer)) == (9 if learned else 0)
    finally:
        pv.lib.zkp_openings_set_only_at_claim(0)
        pv.lib.zkp_layer_set_attention_last(-1)
    pv.layer_free(layer)
    for g in g1s[1:]:
        assert g.shape == g1s[0].shape and (g == g1s[0]).all()


def test_full_shape_layer_gives_one_output_head_by_head_and_stacked(pv):
    """LLaMa-2-7B shape, seq 2048 (tensors of up to 2^27 elements in the stacked proof, beyond what the oracle can follow):
    every proof of the layer runs through its in-prover identities in both attention variants (a failed identity throws),
    the two variants and a group size in between give the same layer output, and the transcripts differ only in length."""
    cu, cf = layercfg.llama7b(seq=2048, open_weights=False)
    pv.seed(2024)
    layer = pv.layer_create_random(cu, cf, 7, 5)
    X = pv.from_i32(np.round(np.random.default_rng(11).normal(0, 1, (2048, 4096)) * 65536).astype(np.int32))
    outs, sizes = [], []
    for g in (0, 32, 8):
        pv.layer_set(layer, head_group=g)
        pv.seed(5)
        pv.transcript_begin()
        out, _ = pv.layer_run(layer, X)
        pv.lib.zkp_transcript_end()
        sizes.append(pv.transcript().shape[0])
        outs.append(out.host())
        del out
    pv.layer_free(layer)
    # the same layer with its nine weight openings (the benchmark's workload): each opened value must equal the claim the
    # fully connected layer's or the norm's proof left on the weight, or the prover throws; the output does not change
    cu_o, cf_o = layercfg.llama7b(seq=2048, open_weights=True)
    pv.seed(2024)
    layer = pv.layer_create_random(cu_o, cf_o, 7, 5)
    pv.layer_set(layer, head_group=32)
    # First with neither row nor cross commitments: each weight opened at its claim, every T, T0, T1 a sum over all generators
    # (commitment.cu:109-129) and every round a fold of its own.
    pv.lib.zkp_openings_use_row_commitments(0)
    try:
        pv.seed(5)
        pv.transcript_begin()
        out, _ = pv.layer_run(layer, X)
        pv.lib.zkp_transcript_end()
    finally:
        pv.lib.zkp_openings_use_row_commitments(1)
    assert pv.transcript().shape[0] == sizes[1] + 9
    assert (out.host() == outs[0]).all()
    del out
    first_t, first_g1 = pv.transcript().copy(), pv.transcript_g1().copy()
    assert pv.lib.zkp_layer_planned_openings(ctypes.c_void_p(layer)) == 9
    # The next run starts the nine openings ahead of their claims from the learned plan, batched, T / T0 / T1 of the first three
    # rounds from the weights' row and cross commitments and those rounds as one fold; the one after it starts every opening
    # at its claim (the openings of a block as one job, same commitments, same folds).  Both must deliver the field elements and
    # the G1 points of the first.
    for at_claim in (0, 1):
        pv.lib.zkp_openings_set_only_at_claim(at_claim)
        try:
            pv.seed(5)
            pv.transcript_begin()
            out, _ = pv.layer_run(layer, X)
            pv.lib.zkp_transcript_end()
        finally:
            pv.lib.zkp_openings_set_only_at_claim(0)
        assert (out.host() == outs[0]).all()
        del out
        again_t, again_g1 = pv.transcript(), pv.transcript_g1()
        assert again_t.shape == first_t.shape and (again_t == first_t).all(), at_claim
        assert again_g1.shape == first_g1.shape and first_g1.shape[0] > 9 * 30 and (again_g1 == first_g1).all(), at_claim
    # The blocks, their sumcheck jobs and the openings run on streams and host threads of their own; a missing wait between them
    # would show as a proof that changes from run to run.  Twelve more runs, every third with the openings at their claims.
    for i in range(12):
        pv.lib.zkp_openings_set_only_at_claim(1 if i % 3 == 2 else 0)
        try:
            pv.seed(5)
            pv.transcript_begin()
            out, _ = pv.layer_run(layer, X)
            pv.lib.zkp_transcript_end()
        finally:
            pv.lib.zkp_openings_set_only_at_claim(0)
        del out
        assert (pv.transcript() == first_t).all() and (pv.transcript_g1() == first_g1).all(), i
    pv.layer_free(layer)
    assert (outs[0] == outs[1]).all() and (outs[0] == outs[2]).all()
    assert np.unique(outs[0], axis=0).shape[0] > 1000
    assert sizes[1] < sizes[2] < sizes[0]
