#!/usr/bin/env python3
"""Benchmark of the MI355X zkLLM prover core.

One step = one LLaMa-2-7B-shape decoder layer at sequence length 2048, computed and proved end to end on one
GPU with weights, generators, commitments and the input already resident in HBM: RMSNorm x2, Q/K/V/O
projections, 32 attention heads (QK^T, zkSoftmax, YV), SwiGLU FFN, every rescaling / lookup / sumcheck and
the opening of all nine weight commitments.  `value` is seconds per layer.

The same JSON line also carries the layer time without the openings and with the nine commitments included, the
two throughput figures of the headline metric (G1 MSM points/s on the 4096 x 11008 commitment workload, Fr
multiplications/s) with their roofline fractions, a roofline entry for the kernel with the largest share of the
layer's GPU time (timed with HIP events around its launches inside the timed region), roofline entries of the first
lookup-sumcheck round, the generic Fr matmul and an HBM-bound fold, and a CPU baseline measured with the oracle on
this host's cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
# VALU integer peak: 256 CUs x 4 SIMDs x 16 lanes x 2.4 GHz lane-operations per second (v_mad_u64_u32 issues at
# full rate on gfx950; bench measures it as well and reports the measured figure next to this one)
VALU_PEAK_TOPS = 256 * 4 * 16 * 2.4e9 / 1e12
# HBM traffic of k_open_fold29 per generator pair in a launch of 262144 pairs, measured with rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE on the kernel alone (python3 bench.py --pmc-probe; summary in profiles/k_open_fold29_pmc_traffic.txt), each
# counter scaled by what it reads for zk_fr_add over 2^24 elements (1 GiB read, 512 MiB written).  It holds for launches of
# that size; `traffic` of the in-layer entry, whose launches are of every size, is left null and the algorithmic figure given.
FOLD_TRAFFIC_BYTES_PER_PAIR_AT_262144 = 763.5      # (53674 KiB x 2.000 fetched + 88108 KiB written) / 262144 pairs, profiles/k_open_fold29_pmc_traffic.txt
FOLD_ALGO_BYTES_PER_PAIR = 2 * 112 + 112 + 3 * 32      # two points in, one out (affine, 29-bit limbs: 112 B), two scalars in, one out
# the same for the table-driven folds, from profiles/fr_mul_fold_msm_pmc.txt (each kernel alone): k_open_fold_comb<1> at 262144 pairs
# (821668 KiB x 2 fetched + 146433 KiB written) and k_open_fold_jump at 65536 results = 7 x 65536 pairs (862752 KiB x 2 + 38100 KiB)
COMB_TRAFFIC_BYTES_PER_PAIR = (821668 * 2 + 146433) * 1024 / 262144
JUMP_TRAFFIC_BYTES_PER_PAIR = (862752 * 2 + 38100) * 1024 / (7 * 65536)
MAD_PER_FP_MUL = 300                                   # 2 * 12^2 + 12 limb products of a 381-bit Montgomery product
MAD_PER_FR_MUL = 136                                   # 2 * 8^2 + 8


def drivers_leg(seq):
    """The drop-in chain at the 7B shape: the per-block executables run as child processes over .bin files with the argument
    lists of the reference's llama-*.py scripts (README.md:60-80, llama-ppgen.py:21-31, llama-commit.py:31-46, llama-rmsnorm.py:35-45,
    llama-self-attn.py:41-81, llama-ffn.py:26-43).  Returns wall time per executable and its phases (ZKLLM_TIMING=1)."""
    import shutil
    import subprocess
    import tempfile
    E, Hd, lof = 4096, 11008, 5
    exe_dir = os.path.join(ROOT, "zkllm-ccs2024_amd", "host")
    tmp = tempfile.mkdtemp(prefix="zkllm_drivers_", dir=os.environ.get("TMPDIR", "/tmp"))
    work = os.path.join(tmp, "zkllm-workdir", "Llama-2-7b")
    os.makedirs(work)
    prefix = "layer-0"
    out = {"shape": f"seq {seq}, hidden {E}, FFN {Hd}, log_off_factor {lof}", "runs": []}

    def run(label, argv, env_extra=None):
        env = dict(os.environ, ZKLLM_TIMING="1", ZKLLM_SEED="7")
        env.update(env_extra or {})
        t0 = time.perf_counter()
        r = subprocess.run([os.path.join(exe_dir, argv[0])] + [str(a) for a in argv[1:]], cwd=tmp, env=env, capture_output=True, text=True, timeout=600)
        wall = time.perf_counter() - t0
        if r.returncode != 0:
            raise RuntimeError(f"{label}: {argv[0]} exited with {r.returncode}: {r.stderr[-800:]}")
        phases = {}
        for line in r.stderr.splitlines():
            if line.startswith("ZKLLM_TIMES "):
                phases = {k: round(v, 1) for k, v in json.loads(line[len("ZKLLM_TIMES "):]).items()}
        rec = {"run": label, "wall_s": round(wall, 3), "phases_ms": phases, "process_start_and_exit_s": round(wall - sum(phases.values()) / 1e3, 3)}
        out["runs"].append(rec)
        return rec

    try:
        rng = np.random.default_rng(7)
        params = [("input_layernorm.weight", (E,)), ("self_attn.q_proj.weight", (E, E)), ("self_attn.k_proj.weight", (E, E)), ("self_attn.v_proj.weight", (E, E)),
                  ("post_attention_layernorm.weight", (E,)), ("mlp.up_proj.weight", (E, Hd)), ("mlp.gate_proj.weight", (E, Hd)), ("mlp.down_proj.weight", (Hd, E))]
        setup = {"ppgen_s": 0.0, "commit_param_s": 0.0, "cross_commitments_ms": 0.0}
        for name, shape in params:
            pp, ib, cb = (os.path.join(work, f) for f in (f"{name}-pp.bin", f"{prefix}-{name}-int.bin", f"{prefix}-{name}-commitment.bin"))
            if len(shape) == 1:
                w = np.full(shape, 65536, np.int32)
                pp_size, dims = shape[0], (shape[0], 1)
            else:
                w = np.round(rng.normal(0, 0.02, shape) * 65536).astype(np.int32)      # in x out, as llama-commit.py saves w.T
                pp_size, dims = shape[1] << lof, shape
            w.tofile(ib)
            setup["ppgen_s"] += run(f"ppgen {name}", ["ppgen", pp_size, pp])["wall_s"]
            rec = run(f"commit-param {name}", ["commit-param", pp, ib, cb, dims[0], dims[1]])
            setup["commit_param_s"] += rec["wall_s"]
            setup["cross_commitments_ms"] += rec["phases_ms"].get("cross_commitments_ms", 0.0)
        out["setup_runs"], out["runs"] = out["runs"], []
        out["setup_s"] = {k: round(v, 3) for k, v in setup.items()}
        X = np.round(rng.normal(0, 1, (seq, E)) * 65536).astype(np.int32)
        X.tofile(os.path.join(tmp, "layer_input.bin"))

        def rms_inv_file(x_int):
            xf = x_int.astype(np.float64) / 65536.0
            np.rint(1.0 / np.sqrt(np.mean(xf ** 2, axis=1) + 1e-5) * 65536.0).astype(np.int32).tofile(os.path.join(tmp, "rms_inv_temp.bin"))
        xs = (np.arange(-(1 << 21), 1 << 21, dtype=np.float64)) / 4096.0
        np.rint(xs / (1.0 + np.exp(-xs)) * 16.0).astype(np.int32).tofile(os.path.join(tmp, "swiglu-table.bin"))      # llama-ffn.py:15-18 (save_int with 16)
        rms_inv_file(X)
        t_chain = time.perf_counter()
        run("rmsnorm input", ["rmsnorm", "input", "layer_input.bin", seq, E, work, prefix, "attn_input.bin"])
        run("self-attn linear", ["self-attn", "linear", "attn_input.bin", seq, E, work, prefix, "attn_output.bin"])
        # the attention of all 32 heads as one stack (ZKLLM_ATTN_HEADS / ZKLLM_ATTN_HEAD_GROUP, additions); the reference's attn mode
        # proves ONE head as wide as the embedding and leaves its output argument alone, so its chain cannot go on from there
        run("self-attn attn (32 heads, stacked)", ["self-attn", "attn", "attn_input.bin", seq, E, work, prefix, "attn_output.bin"],
            {"ZKLLM_ATTN_HEADS": "32", "ZKLLM_ATTN_HEAD_GROUP": "32"})
        run("skip-connection", ["skip-connection", "layer_input.bin", "attn_output.bin", "post_attn_norm_input.bin"])
        x2 = np.fromfile(os.path.join(tmp, "post_attn_norm_input.bin"), dtype=np.int32).reshape(seq, E)
        rms_inv_file(x2)
        run("rmsnorm post_attention", ["rmsnorm", "post_attention", "post_attn_norm_input.bin", seq, E, work, prefix, "ffn_input.bin"])
        run("ffn", ["ffn", "ffn_input.bin", seq, E, Hd, work, prefix, "ffn_output.bin"], {"ZKLLM_FFN_SAVE_RESCALED": "1"})
        run("skip-connection", ["skip-connection", "post_attn_norm_input.bin", "ffn_output.bin", "layer_output.bin"])
        out["chain_wall_s"] = round(time.perf_counter() - t_chain, 3)
        out["chain_prove_s"] = round(sum(r["phases_ms"].get("prove_ms", 0.0) for r in out["runs"]) / 1e3, 3)
        chain = list(out["runs"])
        # the same three blocks that open weights, without the cross-commitment side files (ZKLLM_OPEN_CROSS_ROUNDS=0: create_weight
        # ignores them): every opening sums over its generators in every round
        out["runs"] = []
        for label, argv in (("rmsnorm input", ["rmsnorm", "input", "layer_input.bin", seq, E, work, prefix, "attn_input_2.bin"]),
                            ("self-attn linear", ["self-attn", "linear", "attn_input.bin", seq, E, work, prefix, "attn_output_2.bin"]),
                            ("ffn", ["ffn", "ffn_input.bin", seq, E, Hd, work, prefix, "ffn_output_2.bin"])):
            run(label + " without cross commitments", argv, {"ZKLLM_OPEN_CROSS_ROUNDS": "0", "ZKLLM_FFN_SAVE_RESCALED": "1"})
        out["runs_without_cross_commitment_files"], out["runs"] = out["runs"], chain
        out["note"] = ("every run is a fresh process: runtime start-up, files read and uploaded (load_*), generators prepared for openings "
                       "(prepare_generators_ms: the fixed-base tables of the folds), the block's proof with its openings (prove_ms), outputs written")
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--seq", type=int, default=2048)
    ap.add_argument("--head-group", type=int, default=32,
                    help="attention proved this many heads at a time with zkAttnStacked (a divisor of 32; default: all 32 as one stack); "
                         "0 = head by head, the flow of self-attn.cu per head")
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-extras", action="store_true", help="only the layer timing (used for profiling runs)")
    ap.add_argument("--at-claim", action="store_true",
                    help="the timed layers start every weight opening at its claim (what layer_openings_at_claim_s reports); for profiling runs")
    ap.add_argument("--drivers", action="store_true", help="(default) also run the per-block executables over .bin files at the 7B shape")
    ap.add_argument("--no-drivers", action="store_true",
                    help="skip the leg that runs the per-block executables over .bin files at the 7B shape (child processes; about 8 s and 1.3 GB under TMPDIR)")
    ap.add_argument("--drivers-only", action="store_true", help="only the executables' chain (no in-process layer)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for rocprofv3 --pmc runs: three launches of the opening's fold kernel at 262144 pairs, one hinted lookup "
                         "sumcheck over 2^27 queries, the Montgomery product, the three-level fold, the commitment of config 3 and one "
                         "zk_fr_add over 2^24 elements (1 GiB read, 512 MiB written) to scale the counters by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this prover runs on one GPU; every configuration of the benchmark fits a single MI355X, "
              "so --gpus must be 1 (no multi-GPU path exists in this build)", file=sys.stderr)
        sys.exit(2)

    if args.drivers_only:
        print(json.dumps({"drivers_chain": drivers_leg(args.seq)}))
        return

    from gpuhelp import Hip, Prover, c_int, c_size_t, c_uint, c_void_p
    import layercfg
    from zkhelp import mt_random_vec

    pv = Prover()
    hip = Hip()
    lib = hip.lib

    def fold_probe_setup():
        n_big = 1 << 19
        pv.seed(6)
        gens_big = pv.commitment_random(n_big)
        pv.lib.zkp_g1_devptr.restype = ctypes.c_void_p
        gp = pv.lib.zkp_g1_devptr(c_void_p(gens_big.h))
        sc = hip.upload(mt_random_vec(np.random.RandomState(8), n_big))
        ns, ng = hip.malloc(32 * (n_big // 2)), hip.malloc(144 * (n_big // 2))
        u1 = mt_random_vec(np.random.RandomState(9), 1)
        sums3 = np.zeros((3, 36), np.uint32)
        run = lambda: hip.call("zk_g1_open_round", c_void_p(ns), c_void_p(ng), sums3, c_void_p(sc), c_void_p(gp), u1, c_size_t(n_big), None)
        return n_big, gens_big, (sc, ns, ng), run

    def prepared_opening(n_big, gens_big, scalars):
        """one opening (zk_g1_open_begin_prepared / zk_g1_open_end) of `scalars` against generators prepared once"""
        gp = pv.lib.zkp_g1_devptr(c_void_p(gens_big.h))
        prep = c_void_p()
        hip.call("zk_g1_open_prepare", ctypes.byref(prep), c_void_p(gp), c_size_t(n_big), None)
        k = (n_big - 1).bit_length()
        uk = mt_random_vec(np.random.RandomState(10), k)
        pts, fin = np.zeros((3 * k + 1, 36), np.uint32), np.zeros(8, np.uint32)

        def run():
            h = c_void_p()
            hip.call("zk_g1_open_begin_prepared", ctypes.byref(h), c_void_p(scalars), prep, uk, c_int(k), None)
            hip.call("zk_g1_open_end", h, pts, fin)
        return run

    def jump_opening(n_big, gens_big, scalars):
        """one opening whose first three rounds are one fold (k_open_fold_jump): generators prepared with the three-round tables,
        started through zk_g1_open_begin_batch_rows.  The points that stand in for the cross commitments are infinities: they only
        feed the sums T, T0, T1 of those rounds, which are not what is timed here; the folds do not read them."""
        gp = pv.lib.zkp_g1_devptr(c_void_p(gens_big.h))
        prep = c_void_p()
        hip.call("zk_g1_open_prepare_tables", ctypes.byref(prep), c_void_p(gp), c_size_t(n_big), c_int(3), None)
        k = (n_big - 1).bit_length()
        uk = mt_random_vec(np.random.RandomState(10), k)
        pts, fin = np.zeros((3 * k + 1, 36), np.uint32), np.zeros(8, np.uint32)
        rows = hip.upload(np.zeros((43, 36), np.uint32))
        sc, pp, rr = (c_void_p * 1)(c_void_p(scalars)), (c_void_p * 1)(prep), (c_void_p * 1)(c_void_p(rows))
        nr, ur, kr = np.array([1], np.uint32), (c_void_p * 1)(c_void_p(None)), np.array([0], np.int32)

        def run():
            h = c_void_p()
            hip.call("zk_g1_open_begin_batch_rows", ctypes.byref(h), c_int(1), sc, pp, uk, c_int(k), rr, nr, ur, kr, c_int(3), None)
            hip.call("zk_g1_open_end_batch", h, pts, fin)
        return run

    def lookup_probe(logD=27, logN=20):
        """one mapping-table lookup proof (tLookupRangeMapping::prove) over 2^logD uniformly spread queries into 2^logN entries"""
        D, N = 1 << logD, 1 << logN
        rng = np.random.default_rng(1)
        low = -(N // 2)
        S = pv.from_i32((rng.integers(0, N, D, dtype=np.int64) + low).astype(np.int32))
        pv.keep_for_folds(S)        # as the digit planes of the layer's softmax: the queries keep their int32 form, the outputs get theirs from the table
        mv = pv.from_i32(rng.integers(0, 1 << 22, N, dtype=np.int64).astype(np.int32))
        rs = np.random.RandomState(3)
        r, al, be = mt_random_vec(rs, 1), mt_random_vec(rs, 1), mt_random_vec(rs, 1)
        u, v = mt_random_vec(rs, logD), mt_random_vec(rs, logD)
        return (lambda: pv.mapping(S, low, N, mv, r, al, be, u, v)), (S, mv)

    if args.pmc_probe:
        n_big, gens_big, bufs, fold_round = fold_probe_setup()
        for _ in range(3):
            fold_round()
        # a whole opening over the same generators in their prepared form: the comb folds of the first two rounds on
        # 262144 and 131072 pairs, then k_open_fold29 on 65536, 32768, ... pairs
        prep_open = prepared_opening(n_big, gens_big, bufs[0])
        prep_open()
        # and one whose first three rounds are one fold (k_open_fold_jump on 65536 results, then k_open_fold29 on 32768, ... pairs)
        jump_open = jump_opening(n_big, gens_big, bufs[0])
        jump_open()
        n = 1 << 24
        dA, dB, dO = hip.malloc(32 * n), hip.malloc(32 * n), hip.malloc(32 * n)
        hip.call("zk_fr_add", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None)
        # the kernels behind the other reported rates, once each on operands of known size: the Montgomery product
        # (Fr mul/s), the fused three-level fold (HBM GB/s), the commitment of the 11008 x 4096 weight (MSM points/s)
        # and the hinted first round of a lookup sumcheck
        seed_block = mt_random_vec(np.random.RandomState(1), 1 << 16)
        src = hip.upload(seed_block)
        for i in range(n >> 16):
            lib.zk_memcpy_d2d(c_void_p(dA + i * (32 << 16)), c_void_p(src), c_size_t(32 << 16), None)
            lib.zk_memcpy_d2d(c_void_p(dB + i * (32 << 16)), c_void_p(src + 32 * 5), c_size_t((32 << 16) - 32 * 5), None)
        hip.call("zk_fr_montmul", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None)
        u3 = mt_random_vec(np.random.RandomState(2), 3)
        hip.call("zk_fr_fold_axis", c_void_p(dO), c_void_p(dA), u3, c_int(3), c_size_t(1), c_uint(2048), c_size_t(4096), None)
        pv.seed(5)
        gens = pv.commitment_random(4096)
        Wm = np.round(np.random.default_rng(12).normal(0, 0.02, (11008, 4096)) * 65536).astype(np.int32)
        com = pv.commit_int(gens, pv.from_i32(Wm))
        look, keep = lookup_probe()
        y, m, fin = look()
        hip.sync()
        print(json.dumps({"pmc_probe": {"fold_pairs_per_launch": n_big // 2, "fold_launches": 3, "copy_kernel": "k_ew<0> (zk_fr_add)",
                                        "copy_read_bytes": 64 * n, "copy_write_bytes": 32 * n, "montmul_elements": n,
                                        "fold_axis_elements_in": 2048 * 4096, "msm_pairs": 11008 * 4096,
                                        "lookup_first_round_pairs": 1 << 26, "lookup_first_round_algorithmic_bytes": (1 << 26) * 120}}))
        return

    def ev():
        e = c_void_p()
        hip.check(lib.zk_event_create(ctypes.byref(e)))
        return e

    def time_kernel(fn, reps, warm=1):
        """average duration in ms of `fn` (one launch on the default stream), HIP events on that stream"""
        for _ in range(warm):
            fn()
        e0, e1 = ev(), ev()
        hip.check(lib.zk_event_record(e0, None))
        for _ in range(reps):
            fn()
        hip.check(lib.zk_event_record(e1, None))
        ms = ctypes.c_float()
        hip.check(lib.zk_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        return ms.value / reps

    def read_fold_timer():
        fold_ms, fold_launches, fold_mults, fold_pairs = ctypes.c_double(), ctypes.c_ulonglong(), ctypes.c_double(), ctypes.c_ulonglong()
        hip.check(lib.zk_prof_fold_read(ctypes.byref(fold_ms), ctypes.byref(fold_launches), ctypes.byref(fold_mults), ctypes.byref(fold_pairs)))
        return fold_ms.value, fold_launches.value, fold_mults.value, fold_pairs.value

    def read_lookup_timer(later=False):
        ms, launches, pairs, nbytes = ctypes.c_double(), ctypes.c_ulonglong(), ctypes.c_ulonglong(), ctypes.c_double()
        fn = lib.zk_prof_lookup_later_read if later else lib.zk_prof_lookup_read
        hip.check(fn(ctypes.byref(ms), ctypes.byref(launches), ctypes.byref(pairs), ctypes.byref(nbytes)))
        return ms.value, launches.value, pairs.value, nbytes.value

    # ---- workload: the decoder layer ------------------------------------------------------------------------------
    seq = args.seq
    cu, cf = layercfg.llama7b(seq=seq, open_weights=True, head_group=args.head_group)
    t0 = time.perf_counter()
    pv.seed(2024)
    layer = pv.layer_create_random(cu, cf, 7, 5)
    pv.sync()
    setup_s = time.perf_counter() - t0

    def pool_gib():
        live_b, cached_b = ctypes.c_size_t(), ctypes.c_size_t()
        hip.check(lib.zk_pool_stats(ctypes.byref(live_b), ctypes.byref(cached_b)))
        return live_b.value / 2 ** 30, cached_b.value / 2 ** 30
    # memory: what the setup leaves resident (weights with their int32 forms and digit planes, generators, commitments, cross
    # commitments, the openings' fold tables) and what its construction used on top and gives back here
    setup_live_gib, setup_cached_gib = pool_gib()
    lib.zk_pool_trim()
    pv.lib.zkp_layer_opening_table_bytes.restype = ctypes.c_double
    tables_gib = pv.lib.zkp_layer_opening_table_bytes(c_void_p(layer)) / 2 ** 30
    setup4 = np.zeros(4)
    pv.lib.zkp_layer_setup_times(setup4.ctypes.data_as(ctypes.POINTER(ctypes.c_double)))
    pv.lib.zkp_layer_setup_cross_ms.restype = ctypes.c_double
    setup_cross_ms = pv.lib.zkp_layer_setup_cross_ms()
    X = np.round(np.random.default_rng(11).normal(0, 1, (seq, 4096)) * 65536).astype(np.int32)
    hX = pv.from_i32(X)
    devnull = os.open(os.devnull, os.O_WRONLY)
    saved_stdout = os.dup(1)
    os.dup2(devnull, 1)      # the class layer prints the reference's progress lines ("Opening complete", ...)
    try:
        parts = np.zeros(8)
        if args.at_claim:
            pv.lib.zkp_openings_set_only_at_claim(1)
        for _ in range(args.warmup):
            pv.layer_run(layer, hX)
        pv.sync()
        hip.check(lib.zk_prof_fold_begin())
        hip.check(lib.zk_prof_lookup_begin())
        t0 = time.perf_counter()
        for _ in range(args.steps):
            _, times = pv.layer_run(layer, hX)
            parts += times
        pv.sync()
        wall = time.perf_counter() - t0
        fold_ms, fold_launches, fold_mults, fold_pairs = read_fold_timer()
        m_ms, m_mults = (ctypes.c_double * 3)(), (ctypes.c_double * 3)()
        m_launches, m_pairs = (ctypes.c_ulonglong * 3)(), (ctypes.c_ulonglong * 3)()
        hip.check(lib.zk_prof_fold_methods(m_ms, m_launches, m_pairs, m_mults))
        fold_methods = {name: {"launches": int(m_launches[i]), "pairs": int(m_pairs[i]), "fp_mults": m_mults[i], "ms": m_ms[i],
                               "fp_mults_per_pair": m_mults[i] / max(1, m_pairs[i])}
                        for i, name in enumerate(("walk_k_open_fold29", "comb_k_open_fold_comb", "three_rounds_k_open_fold_jump"))}
        fold_traffic = (m_pairs[0] * FOLD_TRAFFIC_BYTES_PER_PAIR_AT_262144 + m_pairs[1] * COMB_TRAFFIC_BYTES_PER_PAIR + m_pairs[2] * JUMP_TRAFFIC_BYTES_PER_PAIR)
        lk_ms, lk_launches, lk_pairs, lk_bytes = read_lookup_timer()
        lr_ms, lr_launches, lr_pairs, lr_bytes = read_lookup_timer(later=True)
        # the same layer without its nine openings (the G1 part of verifyWeightClaim switched off), and the nine commitments alone
        noopen_s = commit_ms = nocross_s = None
        # The same layer with every opening started at its claim or later (no challenge is read before the prover has drawn it in
        # the reference's order): the openings of a block that are claimed close together run as one batched job, with the
        # same row / cross commitments and three-round folds as the planned run.
        at_claim_parts = np.zeros(8)
        at_claim_s = None
        if args.at_claim:
            at_claim_s, at_claim_parts = wall / args.steps, parts / args.steps
        elif not (args.skip_extras and args.skip_cpu):
            pv.lib.zkp_openings_set_only_at_claim(1)
            try:
                pv.layer_run(layer, hX)
                pv.sync()
                t1 = time.perf_counter()
                for _ in range(3):
                    _, times = pv.layer_run(layer, hX)
                    at_claim_parts += times
                pv.sync()
                at_claim_s = (time.perf_counter() - t1) / 3
                at_claim_parts /= 3
            finally:
                pv.lib.zkp_openings_set_only_at_claim(0)
        # ... and with every block finished before the next begins as well (no block's challenges are drawn before the block
        # before it has written its last transcript entry): the strictest reading of the reference's order of work
        in_turn_s = None
        if not args.skip_extras:
            depth = pv.lib.zkp_layer_blocks_overlap()
            pv.lib.zkp_openings_set_only_at_claim(1)
            pv.lib.zkp_layer_set_blocks_overlap(0)
            try:
                pv.layer_run(layer, hX)
                pv.sync()
                t1 = time.perf_counter()
                for _ in range(3):
                    pv.layer_run(layer, hX)
                pv.sync()
                in_turn_s = (time.perf_counter() - t1) / 3
            finally:
                pv.lib.zkp_openings_set_only_at_claim(1 if args.at_claim else 0)
                pv.lib.zkp_layer_set_blocks_overlap(depth)
        if not args.skip_extras:
            pv.layer_set(layer, open_weights=False)
            pv.layer_run(layer, hX)
            pv.sync()
            t1 = time.perf_counter()
            for _ in range(2):
                pv.layer_run(layer, hX)
            pv.sync()
            noopen_s = (time.perf_counter() - t1) / 2
            pv.layer_set(layer, open_weights=True)
            pv.lib.zkp_layer_recommit_ms.restype = ctypes.c_double
            commit_ms = pv.lib.zkp_layer_recommit_ms(c_void_p(layer))
            commit_ms = pv.lib.zkp_layer_recommit_ms(c_void_p(layer))      # second call: the tables' buffers are cached blocks now
    finally:
        os.dup2(saved_stdout, 1)
    ms_per_step = wall * 1e3 / args.steps
    parts /= args.steps
    run_live_gib, run_cached_gib = pool_gib()
    peak_gib = run_live_gib + run_cached_gib      # the allocator keeps what it once needed: live + cached behind the runs = their peak
    pv.layer_free(layer)
    lib.zk_pool_trim()
    # The layer with its openings summing over the generators in every round: no cross commitments of the weights, and the
    # generators prepared with the tables of the first two rounds (the three-round fold needs the cross commitments).  Another
    # set of prepared generators does not fit beside this one, so a child process measures it, now that this one's memory has gone back.
    if not args.skip_extras:
        import subprocess
        env = dict(os.environ, ZKLLM_OPEN_CROSS_ROUNDS="0")
        try:
            r = subprocess.run([sys.executable, os.path.abspath(__file__), "--skip-cpu", "--skip-extras", "--steps", "2", "--warmup", "1", "--seq", str(args.seq),
                                "--head-group", str(args.head_group)], env=env, capture_output=True, text=True, timeout=300)
            for line in r.stdout.splitlines():
                if line.startswith("{"):
                    nocross_s = json.loads(line)["value"]
        except Exception:
            nocross_s = None

    out = {
        "metric": "layer prove time (s), 7B shape seq 2048; G1 MSM points/s; Fr mul/s",
        "value": ms_per_step / 1e3,
        "unit": "s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32",
        "data": "synthetic",
        "config": {"workload": f"C5: LLaMa-2-7B-shape decoder layer proof, seq {seq}, hidden 4096, 32 heads x 128, FFN 11008, "
                               "random-init fixed-point weights (scale 2^16), generators of size out_features<<5, all nine weight openings included "
                               "(value: their points are read ahead from the seeded challenge stream, so all nine run from the start of the layer, batched by "
                               "generator size; layer_openings_at_claim_s: the same layer with every opening started at its claim and the attention proof, which opens nothing, queued and collected behind the last block; layer_openings_at_claim_blocks_in_turn_s: that, and every "
                               "block's proofs collected before the next block begins -- the reference's order of work, block by block; in the other two figures a block's forward pass and "
                               "proof jobs are queued while the proofs of the two blocks before it are still being collected, transcript unchanged); attention proved "
                               + (f"{args.head_group} heads at a time as head-major stacks (zkAttnStacked)" if args.head_group else "head by head"),
                   "device_pool_gib": round(peak_gib, 1),
                   "memory_gib": {"peak_during_layer_runs": round(peak_gib, 1), "fold_tables_of_the_generators": round(tables_gib, 1),
                                  "resident_weights_generators_commitments": round(setup_live_gib - tables_gib, 1),
                                  "proof_working_set": round(peak_gib - setup_live_gib, 1),
                                  "setup_scratch_given_back_before_the_runs": round(setup_cached_gib, 1)},
                   "setup_s_untimed": round(setup_s, 3),
                   "setup_parts_s": {"random_weights_host_and_upload": round(setup4[0] / 1e3, 3), "generators": round(setup4[1] / 1e3, 3),
                                     "commitments": round(setup4[2] / 1e3, 3), "generators_prepared_for_openings": round(setup4[3] / 1e3, 3),
                                     "cross_commitments_of_the_weights": round(setup_cross_ms / 1e3, 3)},
                   "setup_note": "all of it is made once per model and kept: the commitments are the public ones; the prepared generators (fixed-base tables of the "
                                 "first two fold rounds) depend on the generators alone; the cross commitments (commitments of every 2nd / 4th / 8th column of a "
                                 "weight's rows under every 2nd / 4th / 8th generator) depend on weights and generators alone and let the first three rounds of an "
                                 "opening take T, T0, T1 from sums over rows x patterns points instead of bucket sums over all generators",
                   "parts_ms": {k: round(float(v), 1) for k, v in zip(["rmsnorm1", "qkv", "attention", "oproj", "rmsnorm2", "ffn", "total", "open_wait"], parts)},
                   "parts_note": "host clock from the end of one block's proofs to the end of the next block's; the blocks overlap on the device (a block is begun "
                                 "while the two before it are being collected) and the openings run on the library's streams from the first block on, so "
                                 "a figure says when a block's proof was complete, not what it cost"},
    }
    out["layer_openings_at_claim_s"] = at_claim_s
    out["layer_openings_at_claim_blocks_in_turn_s"] = in_turn_s
    out["layer_openings_at_claim_parts_ms"] = {k: round(float(v), 1) for k, v in zip(["rmsnorm1", "qkv", "attention", "oproj", "rmsnorm2", "ffn", "total", "open_wait"], at_claim_parts)}
    if noopen_s is not None:
        out["layer_without_openings_s"] = noopen_s
        # what is made of the weights once, at commit time: the nine public commitments and their cross commitments
        out["commitments_s"] = commit_ms / 1e3 + setup_cross_ms / 1e3
        out["commitments_parts_s"] = {"row_commitments": commit_ms / 1e3, "cross_commitments": setup_cross_ms / 1e3}
        out["layer_with_commitments_s"] = ms_per_step / 1e3 + commit_ms / 1e3 + setup_cross_ms / 1e3
        out["layer_without_cross_commitments_s"] = nocross_s
        out["layer_without_cross_commitments_with_row_commitments_s"] = None if nocross_s is None else nocross_s + commit_ms / 1e3
    # roofline of the kernel with the largest share of the layer's GPU time: the generator fold of the openings
    # (one endomorphism-split scalar multiplication per pair).  It is bound by 32-bit integer multiply-adds: an
    # Fp multiplication is 2*12^2+12 = 300 of them.  Durations are HIP events around every launch inside the timed
    # region above, on the launch stream.
    fold_tops = fold_mults * MAD_PER_FP_MUL / (fold_ms * 1e-3) / 1e12 if fold_ms > 0 else 0.0
    out["roofline"] = {"kernel": "k_open_fold29, k_open_fold_comb<1> / <2> (first two rounds over prepared generators) and k_open_fold_jump (first three rounds at once, openings with cross commitments): g' = g1 + [u](g0 - g1) per generator pair, 128-bit split scalars, "
                                 "one launch per round for all openings of a size)",
                       "bound": "valu-int", "achieved": fold_tops, "peak": VALU_PEAK_TOPS, "unit": "T MAD32/s", "frac": fold_tops / VALU_PEAK_TOPS,
                       "traffic": fold_traffic / max(1, fold_launches), "algorithmic_bytes_per_launch": FOLD_ALGO_BYTES_PER_PAIR * fold_pairs / max(1, fold_launches),
                       "traffic_note": "bytes per launch from the counters of each kernel ALONE (FETCH_SIZE x 2.000 + WRITE_SIZE per pair: walk 764 B, comb 6991 B, "
                                       "three-round fold 3937 B -- the table-driven folds read their fixed-base table entries, 112 B each) times the pairs of the "
                                       "timed launches; counters of a kernel inside the layer cannot be told apart from its neighbours'",
                       "by_method": fold_methods,
                       "launches": int(fold_launches), "avg_launch_ms": fold_ms / max(1, fold_launches),
                       "total_ms_in_timed_region": fold_ms, "pairs": int(fold_pairs), "fp_mul_per_s": fold_mults / (fold_ms * 1e-3) if fold_ms > 0 else 0.0,
                       "note": "algorithmic work = Fp multiplications of the point formulas x 300 MAD32 (12-limb schoolbook product and reduction; the kernel "
                               "itself works on 14 limbs of 29 bits: 392 multiply-adds and ~110 other instructions per product, 301 per square); "
                               "peak = 256 CU x 4 SIMD x 16 lanes x 2.4 GHz.  The launches are of every size (524288 pairs in the first round of the "
                               "two 2^19 openings down to 1024 in the last halving round) and run beside the bucket sums of their own job, beside up to three other opening jobs and beside "
                               "the rest of the proof; traffic was measured for the kernel alone at 262144 pairs (roofline_fold_alone)"}
    if lk_launches:
        out["roofline_lookup_round_in_layer"] = {
            "kernel": "k_lookup_first2_29 (the first TWO rounds of the lookup sumchecks over int32 queries in one pass, 29-bit limbs; every launch of the timed layers; "
                      "pairs counts the first round's)", "bound": "hbm",
            "achieved": lk_bytes / (lk_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": lk_bytes / (lk_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "traffic": None, "launches": int(lk_launches), "pairs": int(lk_pairs), "total_ms_in_timed_region": lk_ms,
            "note": "algorithmic bytes (per quad of queries, i.e. two first-round pairs: four queries in int32 form 16 B -- a mapping table's outputs are not read when "
                    "they were gathered by these queries --, two eq weights 64 B, the second round's two folded values out 64 B, a half share of the third "
                    "round's eq table 48 B; the first round's folded values are never written) over the summed launch durations; the launches share the device "
                    "with each other, with the openings and with the main stream; alone the kernel is bound by instruction issue (4 450 lane instructions per "
                    "quad) and its table gathers, not by these bytes (profiles/layer_c5_seq2048_alone_valu_bytes.txt)"}
    if lr_launches:
        # ~1750 vector instructions per pair (profiles/fr_mul_fold_msm_pmc.txt: SQ_INSTS_VALU of the kernel alone) of which 855 are limb multiply-adds
        lr_tops = lr_pairs * 855.0 / (lr_ms * 1e-3) / 1e12
        out["roofline_lookup_later_rounds"] = {
            "kernel": "k_lookup_round29 (phase-1 rounds of the lookup sumchecks behind the first, one lane per pair, 29-bit limbs; every launch of the timed layers)",
            "bound": "hbm", "achieved": lr_bytes / (lr_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": lr_bytes / (lr_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "traffic": None, "launches": int(lr_launches), "pairs": int(lr_pairs), "total_ms_in_timed_region": lr_ms, "avg_launch_ms": lr_ms / lr_launches,
            "valu_bound": {"achieved": lr_tops, "peak": VALU_PEAK_TOPS, "unit": "T MAD32/s", "frac": lr_tops / VALU_PEAK_TOPS},
            "note": "algorithmic 240 B per pair (inverses and queries of both halves 128 B, eq weight 32 B, two folded values out 64 B, next eq table 16 B) over the "
                    "summed launch durations, and 855 limb multiply-adds per pair (four Montgomery products of 153, three unreduced ones of 81) against the "
                    "multiply-add peak; the launches share the device with each other, with the openings and with the main stream.  Alone at 2^25 pairs the "
                    "kernel takes 2.12 ms: 3.8 TB/s and 70 % of the vector issue slots -- both sides bind"}
    if args.skip_extras:
        print(json.dumps(out))
        return

    # ---- the same fold kernel alone at its largest per-opening shape in the layer: one halving of 2^19 generators ----
    n_big, gens_big, bufs, fold_round = fold_probe_setup()
    fold_round()
    hip.check(lib.zk_prof_fold_begin())
    for _ in range(3):
        fold_round()
    f_ms, f_launches, f_mults, f_pairs = read_fold_timer()
    iso_tops = f_mults * MAD_PER_FP_MUL / (f_ms * 1e-3) / 1e12
    out["roofline_fold_alone"] = {"kernel": "k_open_fold29, 262144 pairs, nothing else on the device", "bound": "valu-int", "achieved": iso_tops,
                                  "peak": VALU_PEAK_TOPS, "unit": "T MAD32/s", "frac": iso_tops / VALU_PEAK_TOPS,
                                  "traffic": FOLD_TRAFFIC_BYTES_PER_PAIR_AT_262144 * (n_big // 2), "algorithmic_bytes_per_launch": FOLD_ALGO_BYTES_PER_PAIR * (n_big // 2),
                                  "avg_launch_ms": f_ms / max(1, f_launches), "fp_mul_per_s": f_mults / (f_ms * 1e-3),
                                  "note": "4096 waves on 2048 wave slots (two per SIMD: 256 registers, most of the walk's table in LDS): two full turns.  traffic: "
                                          "FETCH_SIZE + WRITE_SIZE of this launch from profiles/k_open_fold29_pmc_traffic.txt"}
    # the fold kernels of one whole opening over the same generators prepared: the comb folds of the first two rounds
    # (262144 and 131072 pairs) and k_open_fold29 on the later rounds down to the batched last rounds
    prep_open = prepared_opening(n_big, gens_big, bufs[0])
    prep_open()
    hip.check(lib.zk_prof_fold_begin())
    t0 = time.perf_counter()
    prep_open()
    open_alone_s = time.perf_counter() - t0
    o_ms, o_launches, o_mults, o_pairs = read_fold_timer()
    o_tops = o_mults * MAD_PER_FP_MUL / (o_ms * 1e-3) / 1e12
    out["roofline_fold_opening_alone"] = {"kernel": "k_open_fold_comb<1> / <2> (first two rounds, 262144 and 131072 pairs) + k_open_fold29 (later rounds) of one opening over 2^19 prepared generators, "
                                                    "beside that opening's own bucket sums only", "bound": "valu-int", "achieved": o_tops, "peak": VALU_PEAK_TOPS,
                                          "unit": "T MAD32/s", "frac": o_tops / VALU_PEAK_TOPS, "traffic": None, "launches": int(o_launches), "pairs": int(o_pairs),
                                          "total_ms": o_ms, "fp_mul_per_pair": o_mults / max(1, o_pairs), "opening_wall_s": open_alone_s}
    for p_ in bufs:
        hip.free(p_)
    del gens_big

    # ---- G1 MSM points/s: commitment of a 4096 x 11008 weight (stored 11008 rows x 4096 against 4096 generators) -------------
    pv.seed(5)
    gens = pv.commitment_random(4096)
    Wm = np.round(np.random.default_rng(12).normal(0, 0.02, (11008, 4096)) * 65536).astype(np.int32)
    hW = pv.from_i32(Wm)
    pv.commit_int(gens, hW)
    pv.sync()
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        com = pv.commit_int(gens, hW)
    pv.sync()
    msm_s = (time.perf_counter() - t0) / reps
    out["g1_msm_points_per_s"] = 11008 * 4096 / msm_s
    out["g1_msm_ms"] = msm_s * 1e3
    # algorithmic work of the commitment: one mixed addition (11 Fp multiplications) per c-bit window of the bits the data covers
    msm_c = 8
    msm_bits = int(np.abs(Wm).max()).bit_length()
    msm_windows = (msm_bits + 1 + msm_c - 1) // msm_c      # one spare bit for the signed digits' carry, as zk_g1_commit_int counts them
    msm_tops = 11008 * 4096 * msm_windows * 11 * MAD_PER_FP_MUL / msm_s / 1e12
    out["roofline_msm"] = {"kernel": "zk_g1_commit_int (k_msm_rows and the table build, conversion and row sums around it), 11008 x 4096 scalars over 4096 generators",
                           "bound": "valu-int", "achieved": msm_tops, "peak": VALU_PEAK_TOPS, "unit": "T MAD32/s", "frac": msm_tops / VALU_PEAK_TOPS, "traffic": None,
                           "window_bits_c": msm_c, "scalar_bits_b": msm_bits, "windows": msm_windows,
                           "note": "algorithmic work = ceil((b + 1) / c) windows x 11 Fp multiplications (one mixed addition) x 300 MAD32 per (scalar, generator) pair, "
                                   "b = bits of the largest |scalar| in the data, c = 8; the time is the whole commit_int call (fixed-base table of the "
                                   "generators' multiples built and normalised, scalars range-checked, row sums) -- what g1_msm_points_per_s is quoted on"}
    del com, hW, gens

    # ---- Fr mul/s: n independent Montgomery products on resident operands ------------------------------------------------------
    n = 1 << 26
    seed_block = mt_random_vec(np.random.RandomState(1), 1 << 16)
    src = hip.upload(seed_block)
    dA, dB, dO = hip.malloc(32 * n), hip.malloc(32 * n), hip.malloc(32 * n)
    for i in range(n >> 16):
        lib.zk_memcpy_d2d(c_void_p(dA + i * (32 << 16)), c_void_p(src), c_size_t(32 << 16), None)
        lib.zk_memcpy_d2d(c_void_p(dB + i * (32 << 16)), c_void_p(src + 32 * 5), c_size_t((32 << 16) - 32 * 5), None)
    hip.sync()
    mul_ms = time_kernel(lambda: hip.call("zk_fr_montmul", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None), reps=10)
    add_ms = time_kernel(lambda: hip.call("zk_fr_add", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_size_t(n), None), reps=10)
    out["fr_mul_per_s"] = n / (mul_ms * 1e-3)
    out["fr_mul_stream_gbs"] = 96 * n / (mul_ms * 1e-3) / 1e9
    out["fr_add_stream_gbs"] = 96 * n / (add_ms * 1e-3) / 1e9
    mul_gbs = 96 * n / (mul_ms * 1e-3) / 1e9
    mul_tops = n * MAD_PER_FR_MUL / (mul_ms * 1e-3) / 1e12
    out["roofline_fr_mul"] = {"kernel": "k_ew<MONTMUL> (2^26 independent Montgomery products, operands streamed from HBM)", "bound": "hbm",
                              "achieved": mul_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": mul_gbs / HBM_PEAK_GBS, "traffic": None,
                              "valu_bound": {"achieved": mul_tops, "peak": VALU_PEAK_TOPS, "unit": "T MAD32/s", "frac": mul_tops / VALU_PEAK_TOPS},
                              "binds": "hbm", "avg_launch_ms": mul_ms,
                              "note": "96 B per product (two operands in, one out) against 136 MAD32 per product: at these rates the memory side is at "
                                      f"{mul_gbs / HBM_PEAK_GBS:.2f} of its peak and the multiply-add side at {mul_tops / VALU_PEAK_TOPS:.2f}, so HBM binds; the plain addition "
                                      f"kernel streams the same bytes at {96 * n / (add_ms * 1e-3) / 1e9:.0f} GB/s"}

    # measured VALU multiply-add peak
    peak = ctypes.c_double()
    hip.check(lib.zk_bench_mad_peak(c_uint(256 * 32), c_uint(10000), ctypes.byref(peak), None))
    out["valu_mad32_peak_measured_tops"] = peak.value / 1e12

    # ---- roofline of the kernels that dominate the layer ---------------------------------------------------------------------------
    # (1) generic Fr matmul at the projection shape: M*N*P field multiplications, 136 MAD32 each (algorithmic)
    M, N, P = 2048, 4096, 4096
    mm_ms = time_kernel(lambda: hip.call("zk_fr_matmul_generic", c_void_p(dO), c_void_p(dA), c_void_p(dB), c_uint(M), c_uint(N), c_uint(P), None), reps=1)
    # (2) fused multilinear fold (3 levels per pass) over a 2048 x 4096 tensor: 32 B read per element
    u = mt_random_vec(np.random.RandomState(2), 3)
    fold_ax_ms = time_kernel(lambda: hip.call("zk_fr_fold_axis", c_void_p(dO), c_void_p(dA), u, c_int(3), c_size_t(1), c_uint(2048), c_size_t(4096), None), reps=10)
    fold_gbs = 32 * 2048 * 4096 / (fold_ax_ms * 1e-3) / 1e9
    mm_tops = M * N * P * 72 / (mm_ms * 1e-3) / 1e12
    out["roofline_matmul"] = {"kernel": "k_matmul (generic Montgomery Fr matmul, 2048x4096x4096)", "bound": "valu-int", "achieved": mm_tops, "peak": VALU_PEAK_TOPS,
                              "unit": "T MAD32/s", "frac": mm_tops / VALU_PEAK_TOPS, "traffic": None,
                              "note": "algorithmic 72 MAD32 per field multiply-accumulate (64 limb products + 1/8 of a shared reduction); every MAD32 needs a second "
                                      "VALU instruction for its carry, so 0.5 is the ceiling of this formulation",
                              "avg_launch_ms": mm_ms, "gmac_per_s": M * N * P / (mm_ms * 1e-3) / 1e9}
    # (1b) the same shape as the layer computes it: fixed-point operands (activations to 2^20, weights N(0, 0.02) at scale 2^16) through
    # zk_fr_matmul -> digit planes -> k_gemm_i8_planes on the matrix cores
    rngm = np.random.default_rng(3)
    hXa = pv.from_i32(np.clip(np.round(rngm.normal(0, 1, (M, N)) * 65536), -(1 << 20), 1 << 20).astype(np.int32))
    hWa = pv.from_i32(np.round(rngm.normal(0, 0.02, (N, P)) * 65536).astype(np.int32))
    pv.matmul(hXa, hWa, M, N, P)
    hip.check(lib.zk_prof_gemm_begin())
    t0 = time.perf_counter()
    for _ in range(3):
        pv.matmul(hXa, hWa, M, N, P)
    pv.sync()
    mm_call_ms = (time.perf_counter() - t0) * 1e3 / 3
    g_ms, g_launches, g_macs = ctypes.c_double(), ctypes.c_ulonglong(), ctypes.c_double()
    hip.check(lib.zk_prof_gemm_read(ctypes.byref(g_ms), ctypes.byref(g_launches), ctypes.byref(g_macs)))
    if g_launches.value:
        g_tops = 2 * g_macs.value / (g_ms.value * 1e-3) / 1e12
        out["roofline_matmul_mfma"] = {"kernel": "k_gemm_i8_planes_all<3,2> (v_mfma_i32_32x32x32_i8 over base-256 digit planes: three of the activations, two of the weights; 2048x4096x4096, exact)", "bound": "mfma",
                                       "achieved": g_tops, "peak": 5000.0, "unit": "TOP/s", "frac": g_tops / 5000.0, "traffic": None,
                                       "avg_launch_ms": g_ms.value / g_launches.value, "plane_pairs": g_macs.value / g_launches.value / (M * N * P),
                                       "whole_product_ms": mm_call_ms,
                                       "note": "int8 multiply-accumulates x 2 over the kernel's launch time; whole_product_ms is zk_fr_matmul end to end (bound check on the "
                                               "device, both digit splits, the GEMM with the recombination to field elements in its epilogue)"}
    del hXa, hWa
    out["roofline_hbm"] = {"kernel": "k_fold_axis_dot<3> (fused 3-level multilinear fold, 2048x4096)", "bound": "hbm", "achieved": fold_gbs, "peak": HBM_PEAK_GBS,
                           "unit": "GB/s", "frac": fold_gbs / HBM_PEAK_GBS, "traffic": None, "avg_launch_ms": fold_ax_ms}
    for p in (dA, dB, dO, src):
        hip.free(p)

    # (3) the first round of a hinted lookup sumcheck alone: 2^26 pairs of a mapping table's 2^27 queries (the size of the stacked attention's)
    look, keep = lookup_probe()
    look()
    hip.check(lib.zk_prof_lookup_begin())
    t0 = time.perf_counter()
    look()
    pv.sync()
    look_total_ms = (time.perf_counter() - t0) * 1e3
    l_ms, l_launches, l_pairs, l_bytes = read_lookup_timer()
    if l_launches:
        out["roofline_lookup_round"] = {"kernel": "k_lookup_first2_29 alone: first two rounds of tLookupRangeMapping::prove in one pass, 2^27 queries uniformly spread over 2^20 entries",
                                        "bound": "hbm", "achieved": l_bytes / (l_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                        "frac": l_bytes / (l_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "avg_launch_ms": l_ms / l_launches, "pairs": int(l_pairs),
                                        "whole_proof_ms": look_total_ms,
                                        "note": "algorithmic 192 B per quad = 96 B per first-round pair (four queries read from their int32 form 16 B, two eq weights 64 B, the second "
                                                "round's two folded values out 64 B, a half share of the third round's eq table 48 B); the kernel also gathers a 64-byte record (table "
                                                "entry and its inverse) per query from a 64 MiB table (the outputs were gathered by these queries from this table and every entry is what "
                                                "the integers say, so nothing else is read per query) and executes about 4 450 lane instructions per quad -- bound by instruction issue and "
                                                "the gathers; as two passes (first round 4.5 ms, second 2.1 ms) the same work took 6.6 ms"}
    del keep, look

    # ---- CPU baseline: the oracle's restatement of the reference's algorithm on this host's cores ---------------------------------------
    # Measured parts, each scaled to its count in the layer: the field multiplications of the matrix products (a row sample),
    # the openings (five 255-bit scalar multiplications per generator pair; a 4096-generator opening), and the lookup arguments
    # (configuration 4 in full: multiplicities, 2^22 + 2^16 Fermat inversions, the 22-round sumcheck).  Configuration 1 runs in full.
    if not args.skip_cpu:
        from zkhelp import load_oracle, orc_check
        orc = load_oracle()
        cores = orc.dll.orc_num_threads()
        # C1: zkFC toy, forward + 6-round sumcheck
        rng1 = np.random.default_rng(7)
        X1 = np.round(rng1.normal(0, 0.02, (16, 64)) * 65536).astype(np.int32)
        W1 = np.round(rng1.normal(0, 0.02, (64, 64)) * 65536).astype(np.int32)
        orc.orc_seed(1234)
        t0 = time.perf_counter()
        orc_check(orc.orc_zkfc(X1, W1, 16, 64, 64, np.zeros((16 * 64, 8), np.uint32), np.zeros(8, np.uint32)))
        c1_s = time.perf_counter() - t0
        B = mt_random_vec(np.random.RandomState(4), 4096 * 1024)

        def mm_sample(rows):
            A = mt_random_vec(np.random.RandomState(3), rows * 4096)
            C = np.zeros((rows * 1024, 8), np.uint32)
            t0 = time.perf_counter()
            orc.orc_fr_matmul_rows(A, B, rows, 4096, 1024, rows, C)
            return time.perf_counter() - t0
        probe_rows = 2 * max(1, cores // 2)
        dt = mm_sample(probe_rows)
        rows = int(max(probe_rows, min(4096, probe_rows * 10.0 / max(dt, 1e-3)))) // max(1, cores) * max(1, cores)
        rows = max(rows, probe_rows)
        dt = mm_sample(rows)
        mm_rate = rows * 4096 * 1024 / dt                      # field multiplications per second, all cores
        # opening sample: n generators, one row
        n_open = 4096
        orc.orc_seed(99)
        gens = np.zeros((n_open, 36), np.uint32)
        orc.orc_commitment_random(n_open, gens)
        T = mt_random_vec(np.random.RandomState(6), n_open)
        k = 12
        u = mt_random_vec(np.random.RandomState(7), k)
        proof = np.zeros((3 * k + 1, 36), np.uint32)
        val = np.zeros(8, np.uint32)
        t0 = time.perf_counter()
        orc.orc_open(gens, n_open, T, n_open, 1, u, k, proof, val)
        open_s = time.perf_counter() - t0
        # C4: range lookup of 2^22 queries into 2^16 entries, in full
        D4, N4 = 1 << 22, 1 << 16
        S4 = np.zeros((D4, 8), np.uint32)
        v4 = np.random.default_rng(4).integers(-(1 << 15), 1 << 15, D4)
        orc.orc_fr_from_i64(np.ascontiguousarray(v4, dtype=np.int64), S4, D4)
        rs4 = np.random.RandomState(14)
        al4, be4 = mt_random_vec(rs4, 1), mt_random_vec(rs4, 1)
        u4, w4 = mt_random_vec(rs4, 22), mt_random_vec(rs4, 22)
        m4 = np.zeros((N4, 8), np.uint32)
        fin4 = np.zeros(8, np.uint32)
        t0 = time.perf_counter()
        orc_check(orc.orc_range_prep(S4, D4, -(1 << 15), N4, m4))
        orc_check(orc.orc_range_prove(S4, D4, -(1 << 15), N4, al4, be4, u4, w4, fin4))
        c4_s = time.perf_counter() - t0
        # C2's proof in full (zkfc.cu:61-151): the evaluation of Y, the two reductions X(u_batch, .) and W(., u_output), the 12-round
        # inner-product sumcheck over them and the closing evaluations of W and X -- on tensors of the configuration's sizes
        # (2048 x 4096, 4096 x 4096); the claim of the sumcheck is formed from the reduced vectors
        def small_fr(seed, n):
            out = np.zeros((n, 8), np.uint32)
            orc.orc_fr_from_i64(np.ascontiguousarray(np.random.default_rng(seed).integers(-(1 << 20), 1 << 20, n), dtype=np.int64), out, n)
            return out
        Bc, Ic, Oc = 2048, 4096, 4096
        Xc, Wc, Yc = small_fr(21, Bc * Ic), small_fr(22, Ic * Oc), small_fr(23, Bc * Oc)
        rs2 = np.random.RandomState(24)
        u_b, u_i, u_o = mt_random_vec(rs2, 11), mt_random_vec(rs2, 12), mt_random_vec(rs2, 12)
        lens2, one_fr = np.array([11, 12], np.uint32), np.zeros(8, np.uint32)
        n_out = ctypes.c_long()
        t0 = time.perf_counter()
        orc_check(orc.orc_fr_multi_dim_me(Yc, Bc * Oc, np.concatenate([u_b, u_o]), lens2, np.array([Bc, Oc], np.uint32), 2, one_fr))
        Xr, Wr = np.zeros((Bc * Ic, 8), np.uint32), np.zeros((Ic * Oc, 8), np.uint32)
        orc_check(orc.orc_fr_partial_me(Xc, Bc * Ic, u_b, 11, Bc, Ic, Xr, ctypes.byref(n_out)))
        assert n_out.value == Ic
        orc_check(orc.orc_fr_partial_me(Wc, Ic * Oc, u_o, 12, Oc, 1, Wr, ctypes.byref(n_out)))
        assert n_out.value == Ic
        prod, claim2 = np.zeros((Ic, 8), np.uint32), np.zeros(8, np.uint32)
        orc_check(orc.orc_fr_op(7, Xr[:Ic].copy(), Wr[:Ic].copy(), prod, Ic))
        orc_check(orc.orc_fr_sum(prod, Ic, claim2))
        orc_check(orc.orc_zkip(claim2, Xr[:Ic].copy(), Wr[:Ic].copy(), Ic, u_i, 12, np.zeros((12 * 3, 8), np.uint32), np.zeros(8, np.uint32)))
        orc_check(orc.orc_fr_multi_dim_me(Wc, Ic * Oc, np.concatenate([u_i, u_o]), np.array([12, 12], np.uint32), np.array([Ic, Oc], np.uint32), 2, one_fr))
        orc_check(orc.orc_fr_multi_dim_me(Xc, Bc * Ic, np.concatenate([u_b, u_i]), lens2, np.array([Bc, Ic], np.uint32), 2, one_fr))
        c2_prove_s = time.perf_counter() - t0
        c2_products = Bc * Oc + 2 * Bc * Ic + 2 * Ic * Oc          # one product per element folded
        del Xc, Wc, Yc, Xr, Wr
        # the softmax's Hadamard argument (multi_hadamard_sumchecks over the K = 3 table-value planes, proof.cu:191-241) for ONE
        # head: 2048 x 2048 elements, 22 rounds
        nh, kh = 2048 * 2048, 22
        Hs = np.concatenate([small_fr(31 + j, nh) for j in range(3)])
        rs3 = np.random.RandomState(34)
        u_h, v_h = mt_random_vec(rs3, kh), mt_random_vec(rs3, kh)
        p01, p012, claim3 = np.zeros((nh, 8), np.uint32), np.zeros((nh, 8), np.uint32), np.zeros(8, np.uint32)
        orc_check(orc.orc_fr_op(7, Hs[:nh], Hs[nh:2 * nh], p01, nh))
        orc_check(orc.orc_fr_op(7, p01, Hs[2 * nh:], p012, nh))
        orc_check(orc.orc_fr_me(p012, nh, u_h, kh, claim3))            # the claim the argument starts from (not timed: the prover holds it)
        del p01, p012
        t0 = time.perf_counter()
        orc_check(orc.orc_multi_hadamard(claim3, Hs, 3, nh, u_h, v_h, kh, np.zeros((kh * 4, 8), np.uint32), np.zeros(8, np.uint32)))
        hadamard_head_s = time.perf_counter() - t0
        del Hs
        layer_mm = 4.49e11                                     # field multiplications in the layer's matrix products (reference algorithm)
        # elements folded by the layer's matrix-product proofs (zkFC::prove of the seven projections: B O + 2 B I + 2 I O each) and by
        # the per-head proofs of out = Y V and X = Q K^T (self-attn.cu:97-119: Y, X of 2048 x 2048, Q, K, V, out of 2048 x 128, 32 heads)
        fc = lambda B_, I_, O_: B_ * O_ + 2 * B_ * I_ + 2 * I_ * O_
        layer_fold_products = 4 * fc(2048, 4096, 4096) + 2 * fc(2048, 4096, 11008) + fc(2048, 11008, 4096) + 32 * (2 * 2048 * 2048 + 5 * 2048 * 128)
        layer_gens = 5 * (4096 << 5) + 2 * (1 << 19) + 2 * 4096      # generators of the nine openings (11008 << 5 rounds up to 2^19); pairs over all rounds ~ the same number
        # queries of the layer's lookup arguments: three softmax segments over 32 x 2048 x 2048, the activation table and four rescalings over the
        # padded 2048 x 11008 tensors, nine rescalings over 2048 x 4096, two over 4096
        layer_queries = 3 * (1 << 27) + 4 * (1 << 25) + 9 * (1 << 23) + 2 * 4096
        parts_cpu = {"matrix_products_s": layer_mm / mm_rate, "openings_s": open_s * layer_gens / n_open, "lookup_arguments_s": c4_s * layer_queries / D4,
                     "matrix_product_proofs_s": c2_prove_s * layer_fold_products / c2_products, "softmax_hadamard_arguments_s": hadamard_head_s * 32}
        cpu_s = sum(parts_cpu.values())
        out["cpu_baseline"] = {"value": cpu_s, "unit": "s", "cores": int(cores), "kind": "port",
                               "sample": f"oracle (reference algorithm, OpenMP, {int(cores)} threads): Fr matmul {rows} x 4096 x 1024 = {rows * 4096 * 1024:.3g} multiplications in {dt:.1f} s, "
                                         f"scaled to the layer's 4.49e11; opening of {n_open} generators in {open_s:.1f} s, scaled to the layer's "
                                         f"{layer_gens} generators; configuration 4 in full (2^22 queries into 2^16 entries: multiplicities, Fermat inversions, 22 rounds) in "
                                         f"{c4_s:.1f} s, scaled to the layer's {layer_queries:.3g} queries; configuration 2's proof in full (five folds of 2048 x 4096 / "
                                         f"4096 x 4096 tensors and the 12-round inner-product sumcheck, {c2_products:.3g} products) in {c2_prove_s:.1f} s, scaled to the "
                                         f"{layer_fold_products:.3g} elements the layer's matrix-product proofs fold; the softmax's Hadamard argument of one head "
                                         f"(three planes of 2048 x 2048, 22 rounds) in {hadamard_head_s:.1f} s, times 32 heads",
                               "parts_s": {k_: round(v_, 1) for k_, v_ in parts_cpu.items()},
                               "config1_zkfc_toy_s": c1_s, "config4_lookup_s": c4_s, "config2_proof_s": c2_prove_s, "softmax_hadamard_one_head_s": hadamard_head_s,
                               "fr_mul_per_s_all_cores": mm_rate}
    if not args.no_drivers:
        del pv, hip
        lib.zk_shutdown()          # the child processes need the device memory this process held in its pool
        try:
            out["drivers_chain"] = drivers_leg(args.seq)
        except Exception as e:          # never loses the headline line
            out["drivers_chain"] = {"error": str(e)[:600]}
    print(json.dumps(out))
    lib.zk_shutdown()


if __name__ == "__main__":
    main()
